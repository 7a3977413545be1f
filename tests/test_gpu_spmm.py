"""CSR x dense SpMM parity on the GPU, through the C ABI, against the CPU oracle."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

from gpu_util import TOL, dev, from_lengths as _from_lengths
from lapis_amd import generators as gen

pytestmark = pytest.mark.gpu


def _check(gpu, oracle, A, B, C_in, dtype, what, plan=False):
    print("case", what, flush=True)
    want = C_in.copy()
    oracle.spmm(A.pos, A.crd, A.val, B, want)
    absA = sp.csr_matrix((np.abs(A.val).astype(np.float64), A.crd, A.pos), shape=(A.nrows, A.ncols))
    scale = absA @ np.abs(B).astype(np.float64) + np.abs(C_in)
    C = dev(C_in)
    dpos, dcrd = dev(A.pos), dev(A.crd)
    the_plan = gpu.CsrPlan(A.nrows, A.ncols, dpos, dcrd, value_bytes=np.dtype(dtype).itemsize) if plan else None
    gpu.spmm(A.nrows, A.ncols, dpos, dcrd, dev(A.val), dev(B), C, plan=the_plan)
    torch.cuda.synchronize()
    got = C.cpu().numpy().astype(np.float64)
    err = np.abs(got - want.astype(np.float64))
    bound = TOL[np.dtype(dtype)] * np.maximum(scale, np.finfo(np.float64).tiny)
    assert np.all(err <= bound), "%s: max excess %g" % (what, (err - bound).max())


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("k", [64, 1, 2, 3, 8, 32, 96, 100, 128, 256, 260, 512, 515])
def test_spmm_matches_oracle_over_widths(gpu, oracle, dtype, k):
    A = gen.fixed_degree_random(4096 + 3, 32, seed=4004, dtype=dtype)
    B = gen.uniform_matrix(A.ncols, k, 4005).astype(dtype)
    C_in = gen.uniform_matrix(A.nrows, k, 4006).astype(dtype)
    _check(gpu, oracle, A, B, C_in, dtype, "deg32 k=%d" % k)


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
def test_spmm_ragged_rows(gpu, oracle, dtype):
    lengths = [0, 1, 63, 64, 65, 0, 0, 200, 3, 129, 0]
    A = _from_lengths(lengths, 300, 21, dtype)
    for k in (64, 16, 5):
        B = gen.uniform_matrix(300, k, 22).astype(dtype)
        C_in = gen.uniform_matrix(len(lengths), k, 23).astype(dtype)
        _check(gpu, oracle, A, B, C_in, dtype, "ragged k=%d" % k)


def test_spmm_literal_case_of_spmm_dcsr(gpu, golden):
    g = golden["spmm_dcsr"]
    a, b = np.array(g["a_dense"]), np.array(g["b"])
    A = sp.csr_matrix(a)
    C = torch.zeros(3, 2, dtype=torch.float64, device="cuda")
    gpu.spmm(3, 4, dev(A.indptr.astype(np.int32)), dev(A.indices.astype(np.int32)), dev(A.data), dev(b), C)
    torch.cuda.synchronize()
    assert np.allclose(C.cpu().numpy(), np.matmul(a, b))


def test_spmm_strided_leading_dimensions(gpu, oracle):
    A = gen.fixed_degree_random(512, 8, seed=31, dtype=np.float32)
    k = 64
    Bfull = gen.uniform_matrix(512, 96, 32)
    Cfull = gen.uniform_matrix(512, 80, 33)
    want = Cfull[:, :k].copy()
    oracle.spmm(A.pos, A.crd, A.val, np.ascontiguousarray(Bfull[:, :k]), want)
    Bd, Cd = dev(Bfull), dev(Cfull)
    gpu.spmm(A.nrows, A.ncols, dev(A.pos), dev(A.crd), dev(A.val), Bd[:, :k], Cd[:, :k])
    torch.cuda.synchronize()
    got = Cd.cpu().numpy()
    assert np.allclose(got[:, :k], want, rtol=1e-5, atol=1e-5)
    assert np.array_equal(got[:, k:], Cfull[:, k:])  # columns beyond k are untouched


def test_batched_csrv_product_of_the_bspmm_example(gpu, oracle):
    # the shapes and sparsity of examples/bspmm.py:62-75 with a fixed seed, then a larger case
    for (m, n, b, k, pos, crd, seed) in [
            (5, 6, 8, 3, np.array([0, 1, 5, 6, 8, 8], np.int32), np.array([1, 0, 2, 3, 4, 5, 0, 1], np.int32), 12),
            (None, None, 5, 7, None, None, 13)]:
        rng = np.random.default_rng(seed)
        if m is None:
            A = gen.fixed_degree_random(300, 9, seed=41)
            m = n = 300
            pos, crd = A.pos, A.crd
        nnz = crd.shape[0]
        values = rng.uniform(1.0, 2.0, nnz * b).astype(np.float32)
        V = rng.uniform(1.0, 2.0, (n, k, b)).astype(np.float32)
        gold = np.zeros((m, k, b), np.float32)
        for i in range(b):
            gold[:, :, i] = sp.csr_matrix((values[i::b], crd, pos), (m, n)) @ V[:, :, i]
        out = torch.zeros(m, k, b, dtype=torch.float32, device="cuda")
        gpu.bspmm_csrv(m, n, dev(pos), dev(crd), dev(values), dev(V), out)
        torch.cuda.synchronize()
        assert np.allclose(gold, out.cpu().numpy())  # the example's acceptance check
        assert np.array_equal(out.cpu().numpy(), oracle.bspmm_csrv(pos, crd, values, V, m))  # same order: bit-exact


def _banded(n, offsets, seed, dtype):
    """Rows with one entry per in-range diagonal offset (a stencil's sparsity) and random values."""
    rng = np.random.default_rng(seed)
    diags = [rng.uniform(-1, 1, n - abs(o)) for o in offsets]
    A = sp.diags(diags, offsets, shape=(n, n), format="csr")
    A.sort_indices()
    return gen.CSR(n, n, A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data.astype(dtype))


@pytest.mark.parametrize("dtype,k", [(np.float32, 64), (np.float32, 16), (np.float32, 256), (np.float64, 32),
                                     (np.float64, 8), (np.float64, 128)])
def test_planned_spmm_on_banded_matrices_through_every_kernel(gpu, oracle, dtype, k, monkeypatch):
    # a 7-point stencil's pattern on 30 x 30 x 7 points: five of the seven diagonals lie inside the staged window
    n = 30 * 30 * 7
    A = _banded(n, [-900, -30, -1, 0, 1, 30, 900], 71, dtype)
    plan = gpu.CsrPlan(A.nrows, A.ncols, dev(A.pos), dev(A.crd), value_bytes=np.dtype(dtype).itemsize)
    near = plan.stats()["near_diagonal_fraction"]
    want_near = [np.mean(np.abs(A.crd - np.repeat(np.arange(n), np.diff(A.pos))) <= h) for h in (32, 64, 128, 256)]
    assert np.allclose(near, want_near, atol=1e-12)
    B = gen.uniform_matrix(n, k, 72).astype(dtype)
    C_in = gen.uniform_matrix(n, k, 73).astype(dtype)
    _check(gpu, oracle, A, B, C_in, dtype, "banded k=%d planned" % k, plan=True)  # the plan picks group per row
    lanes_per_row = k * np.dtype(dtype).itemsize // 16
    group_fits = lanes_per_row <= 32  # a row of B wider than half a wavefront leaves no room for a second group
    assert gpu.spmm_last_kernel() == ("spmm_group_row_kernel" if group_fits else "spmm_wave_row_kernel")
    # the same through both kernels explicitly: they must agree with the oracle on their own
    for which in ("lds", "wave", "group"):
        monkeypatch.setenv("LAPIS_HIP_SPMM_KERNEL", which)
        _check(gpu, oracle, A, B, C_in, dtype, "banded k=%d forced %s" % (k, which), plan=True)
        want = {"lds": "spmm_rowblock_lds_kernel", "wave": "spmm_wave_row_kernel",
                "group": "spmm_group_row_kernel" if group_fits else "spmm_wave_row_kernel"}[which]
        assert gpu.spmm_last_kernel() == want
    monkeypatch.delenv("LAPIS_HIP_SPMM_KERNEL")


@pytest.mark.parametrize("which", ["lds", "group"])
def test_staged_and_group_kernels_on_matrices_they_would_not_be_chosen_for(gpu, oracle, monkeypatch, which):
    # forced onto random columns, ragged rows, blocks cut by the matrix end and a window cut by both ends of B
    monkeypatch.setenv("LAPIS_HIP_SPMM_KERNEL", which)
    for n, deg, k in ((5000, 9, 64), (700, 3, 32), (131, 5, 128)):
        A = gen.fixed_degree_random(n, deg, seed=81 + n, dtype=np.float32)
        B = gen.uniform_matrix(A.ncols, k, 82).astype(np.float32)
        C_in = gen.uniform_matrix(A.nrows, k, 83).astype(np.float32)
        _check(gpu, oracle, A, B, C_in, np.float32, "random n=%d k=%d forced lds" % (n, k), plan=True)
    lengths = [0, 1, 63, 64, 65, 0, 0, 200, 3, 129, 0] * 30
    A = _from_lengths(lengths, 330, 84, np.float64)
    B = gen.uniform_matrix(330, 16, 85).astype(np.float64)
    C_in = gen.uniform_matrix(len(lengths), 16, 86).astype(np.float64)
    _check(gpu, oracle, A, B, C_in, np.float64, "ragged forced lds", plan=True)
    # wide and short: more columns than rows, the window follows the row index
    A = _from_lengths([7] * 600, 4000, 87, np.float32)
    B = gen.uniform_matrix(A.ncols, 64, 88).astype(np.float32)
    C_in = gen.uniform_matrix(A.nrows, 64, 89).astype(np.float32)
    _check(gpu, oracle, A, B, C_in, np.float32, "wide forced lds", plan=True)
    # tall: fewer columns than rows, the window of the last blocks lies past the end of B
    A = _from_lengths([5] * 3000, 200, 90, np.float32)
    B = gen.uniform_matrix(A.ncols, 64, 91).astype(np.float32)
    C_in = gen.uniform_matrix(A.nrows, 64, 92).astype(np.float32)
    _check(gpu, oracle, A, B, C_in, np.float32, "tall forced lds", plan=True)


def test_planned_spmm_keeps_the_wave_kernel_for_random_columns_and_checks_the_plan(gpu, oracle):
    A = gen.fixed_degree_random(20000, 32, seed=91, dtype=np.float32)
    B = gen.uniform_matrix(A.ncols, 64, 92).astype(np.float32)
    C_in = np.zeros((A.nrows, 64), np.float32)
    plan = gpu.CsrPlan(A.nrows, A.ncols, dev(A.pos), dev(A.crd), value_bytes=4)
    assert max(plan.stats()["near_diagonal_fraction"]) < 0.05
    _check(gpu, oracle, A, B, C_in, np.float32, "random planned", plan=True)
    with pytest.raises(gpu.LapisHipError) as e:  # a plan of another matrix
        gpu.spmm(A.nrows, A.ncols, dev(A.pos), dev(A.crd), dev(A.val), dev(B), dev(C_in), plan=plan)
    assert e.value.status_name == "LAPIS_HIP_ERR_PLAN_MISMATCH"
