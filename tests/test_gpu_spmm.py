"""CSR x dense SpMM parity on the GPU, through the C ABI, against the CPU oracle."""
import numpy as np
import pytest
import scipy.sparse as sp
import torch

from gpu_util import TOL, dev, from_lengths as _from_lengths
from lapis_amd import generators as gen

pytestmark = pytest.mark.gpu


def _check(gpu, oracle, A, B, C_in, dtype, what):
    print("case", what, flush=True)
    want = C_in.copy()
    oracle.spmm(A.pos, A.crd, A.val, B, want)
    absA = sp.csr_matrix((np.abs(A.val).astype(np.float64), A.crd, A.pos), shape=(A.nrows, A.ncols))
    scale = absA @ np.abs(B).astype(np.float64) + np.abs(C_in)
    C = dev(C_in)
    gpu.spmm(A.nrows, A.ncols, dev(A.pos), dev(A.crd), dev(A.val), dev(B), C)
    torch.cuda.synchronize()
    got = C.cpu().numpy().astype(np.float64)
    err = np.abs(got - want.astype(np.float64))
    bound = TOL[np.dtype(dtype)] * np.maximum(scale, np.finfo(np.float64).tiny)
    assert np.all(err <= bound), "%s: max excess %g" % (what, (err - bound).max())


@pytest.mark.parametrize("dtype", [np.float32, np.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("k", [64, 1, 2, 3, 8, 32, 100, 128, 256])
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
