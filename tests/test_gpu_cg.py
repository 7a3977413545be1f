"""Conjugate gradients on the GPU (device buffers, C ABI) against the CPU oracle."""
import numpy as np
import pytest
import torch

from conftest import read_mtx_csr
from gpu_util import dev
from lapis_amd import generators as gen

pytestmark = pytest.mark.gpu


def _solve(gpu, pos, crd, val, b, dinv, tol, maxiter, with_plan=True, with_work=False):
    n = b.shape[0]
    dpos, dcrd = dev(pos), dev(crd)
    plan = gpu.CsrPlan(n, n, dpos, dcrd) if with_plan else None
    x = torch.full((n,), 7.0, dtype=torch.float64, device="cuda")
    work = torch.empty(4 * n, dtype=torch.float64, device="cuda") if with_work else None
    iters, relres = gpu.pcg(plan, n, dpos, dcrd, dev(val), dev(b), dev(dinv) if dinv is not None else None,
                            tol, maxiter, x, work=work)
    return x.cpu().numpy(), iters, relres


def test_pcg_nos4_matches_oracle(gpu, oracle, golden):
    g = golden["pcg_solve"]
    pos, crd, val, shape = read_mtx_csr(g["matrix"])
    n = shape[0]
    import scipy.sparse as sp
    A = sp.csr_matrix((val, crd, pos), shape=shape)
    b = A @ np.ones(n)
    dinv = 1.0 / A.diagonal()
    xo, io, ro = oracle.pcg(pos, crd, val, b, dinv, g["reltol"], g["maxiter"])
    for with_plan, with_work in ((True, False), (False, True)):
        xg, ig, rg = _solve(gpu, pos, crd, val, b, dinv, g["reltol"], g["maxiter"], with_plan, with_work)
        assert ig == io, "the iteration count is an index output: it must match exactly"
        assert np.allclose(xg, xo, rtol=1e-9, atol=1e-12)
        assert abs(rg - ro) <= 1e-6 * ro + 1e-16


@pytest.mark.parametrize("maxiter", [1, 2, 5, 33, 100])
def test_unpreconditioned_fixed_iterations_on_laplace3d(gpu, oracle, maxiter):
    A, b = gen.config5(scale=(24 / 192) ** 3)
    xo, io, ro = oracle.pcg(A.pos, A.crd, A.val, b, np.ones(A.nrows), 0.0, maxiter)
    xg, ig, rg = _solve(gpu, A.pos, A.crd, A.val, b, None, 0.0, maxiter)
    assert ig == io == maxiter
    # CG amplifies rounding differences of the dot products from iteration to iteration;
    # 1e-12 relative per SpMV row grows to about 1e-9 on x over 100 iterations here
    assert np.allclose(xg, xo, rtol=1e-8, atol=1e-10)
    assert abs(rg - ro) <= 1e-7 * ro


def test_preconditioned_equals_unpreconditioned_with_unit_dinv(gpu):
    A, b = gen.config5(scale=(16 / 192) ** 3)
    x1, i1, r1 = _solve(gpu, A.pos, A.crd, A.val, b, None, 1e-8, 200)
    x2, i2, r2 = _solve(gpu, A.pos, A.crd, A.val, b, np.ones(A.nrows), 1e-8, 200)
    assert i1 == i2 and r1 <= 1e-8
    assert np.allclose(x1, x2, rtol=1e-10, atol=1e-14)


def test_convergence_stops_early_and_x_is_not_touched_afterwards(gpu, oracle):
    A, b = gen.config5(scale=(12 / 192) ** 3)
    import scipy.sparse as sp
    M = sp.csr_matrix((A.val, A.crd, A.pos), shape=(A.nrows, A.ncols))
    xs = np.linspace(-1, 1, A.nrows)
    rhs = M @ xs
    dinv = 1.0 / M.diagonal()
    xo, io, ro = oracle.pcg(A.pos, A.crd, A.val, rhs, dinv, 1e-10, 1000)
    xg, ig, rg = _solve(gpu, A.pos, A.crd, A.val, rhs, dinv, 1e-10, 1000)
    assert ig == io and ig < 1000 and rg <= 1e-10
    assert np.allclose(xg, xs, atol=1e-7)
    # kernels queued behind the converging iteration must leave x alone: the returned
    # residual is the residual of the returned x
    assert abs(np.linalg.norm(rhs - M @ xg) / np.linalg.norm(rhs) - rg) < 1e-9
    # a huge tolerance leaves after the first update, as the reference's loop does
    _, i1, _ = _solve(gpu, A.pos, A.crd, A.val, rhs, dinv, 1e30, 50)
    assert i1 == 1


@pytest.mark.parametrize("preconditioned", [False, True])
def test_odd_size_and_unaligned_buffers_take_the_elementwise_paths(gpu, oracle, preconditioned):
    """An odd n with a caller's work buffer puts two of the four work vectors on addresses that are
    not multiples of 16, and x starts one element into its allocation: the vector kernels
    then walk element by element, and must give what the 128-bit paths give."""
    A, b = gen.config5(scale=(15 / 192) ** 3)
    n = A.nrows
    assert n % 2 == 1
    import scipy.sparse as sp
    M = sp.csr_matrix((A.val, A.crd, A.pos), shape=(n, n))
    dinv = 1.0 / M.diagonal() if preconditioned else None
    xo, io, ro = oracle.pcg(A.pos, A.crd, A.val, b, dinv if preconditioned else np.ones(n), 1e-9, 500)
    dpos, dcrd = dev(A.pos), dev(A.crd)
    plan = gpu.CsrPlan(n, n, dpos, dcrd)
    xbuf = torch.full((n + 1,), 7.0, dtype=torch.float64, device="cuda")
    x = xbuf[1:]
    assert x.data_ptr() % 16 == 8
    work = torch.empty(4 * n, dtype=torch.float64, device="cuda")
    ig, rg = gpu.pcg(plan, n, dpos, dcrd, dev(A.val), dev(b), dev(dinv) if preconditioned else None, 1e-9, 500, x,
                     work=work)
    assert ig == io and rg <= 1e-9
    assert np.allclose(x.cpu().numpy(), xo, rtol=1e-7, atol=1e-10)
    assert float(xbuf[0]) == 7.0
    # the aligned run of the same system
    xa, ia, ra = _solve(gpu, A.pos, A.crd, A.val, b, dinv, 1e-9, 500)
    assert ia == ig
    assert np.allclose(x.cpu().numpy(), xa, rtol=1e-9, atol=1e-12)
    assert abs(np.linalg.norm(b - M @ x.cpu().numpy()) / np.linalg.norm(b) - rg) < 1e-9


def test_masked_cg_and_moments_match_oracle(gpu, oracle, golden):
    g = golden["hitting_times"]
    pos, crd, val, shape = read_mtx_csr("mht_A.mtx")
    n = shape[0]
    d = read_mtx_csr("mht_D.mtx")[2]
    mask = np.ones(n)
    mask[3] = 0
    dpos, dcrd, dval = dev(pos), dev(crd), dev(val)
    plan = gpu.CsrPlan(n, n, dpos, dcrd)
    m1 = torch.empty(n, dtype=torch.float64, device="cuda")
    m2 = torch.empty(n, dtype=torch.float64, device="cuda")
    gpu.mht(plan, n, dpos, dcrd, dval, dev(mask), dev(d), g["alpha"], g["tol"], g["maxiter"], m1, m2)
    assert np.array_equal(dval.cpu().numpy(), val * g["alpha"])  # scale_csr works in place, bit for bit
    vo = val.copy()
    o1, o2 = oracle.mht(pos, crd, vo, mask, d, g["alpha"], g["tol"], g["maxiter"])
    assert np.allclose(m1.cpu().numpy(), o1, rtol=1e-9, atol=1e-12)
    assert np.allclose(m2.cpu().numpy(), o2, rtol=1e-9, atol=1e-12)
    out = torch.empty(n, dtype=torch.float64, device="cuda")
    gpu.normalize_mom2(m1, m2, out)
    assert np.allclose(out.cpu().numpy(), g["mom2_gold"])
    # a larger masked system against the oracle's masked solver
    A, b = gen.config5(scale=(14 / 192) ** 3)
    nn = A.nrows
    dd = np.full(nn, 6.5)
    mk = (np.arange(nn) % 7 != 0).astype(np.float64)
    off = A.val.copy()
    off[off > 0] = 0.0
    off = -off  # adjacency part of the Laplacian: plpt applies d - A
    x = torch.empty(nn, dtype=torch.float64, device="cuda")
    dp, dc = dev(A.pos), dev(A.crd)
    it, rr = gpu.pcg_masked(gpu.CsrPlan(nn, nn, dp, dc), nn, dp, dc, dev(off), dev(b * mk), dev(mk), dev(dd), 1e-9, 300, x)
    xo, ito, _ = oracle.pcg_masked(A.pos, A.crd, off, b * mk, mk, dd, 1e-9, 300)
    assert it == ito and it < 300
    assert np.allclose(x.cpu().numpy(), xo, rtol=1e-8, atol=1e-11)


def test_iteration_counter_semantics_of_the_reference_loop(gpu, oracle):
    # examples/pcg_solve.py:74-98: i starts at 1 and the loop leaves when !(relres > tol) or i == maxiter
    A, b = gen.config5(scale=(12 / 192) ** 3)
    one = np.ones(A.nrows)
    for tol, maxiter in ((1e30, 50), (0.0, 1), (1e-3, 1000), (1e-6, 7)):
        xo, io, ro = oracle.pcg(A.pos, A.crd, A.val, b, one, tol, maxiter)
        xg, ig, rg = _solve(gpu, A.pos, A.crd, A.val, b, None, tol, maxiter)
        assert ig == io, (tol, maxiter, ig, io)
        assert np.allclose(xg, xo, rtol=1e-9, atol=1e-12)
    # a huge tolerance leaves after the first pass, with one update applied
    xg, ig, rg = _solve(gpu, A.pos, A.crd, A.val, b, None, 1e30, 50)
    assert ig == 1 and np.any(xg != 0.0)


def test_zero_right_hand_side_gives_nan_relres_and_one_pass(gpu, oracle):
    # r0 = 0: relres = 0/0 is NaN, `relres > tol` is false, the loop leaves at i = 1 (reference semantics)
    A, _ = gen.config5(scale=(10 / 192) ** 3)
    b = np.zeros(A.nrows)
    xo, io, ro = oracle.pcg(A.pos, A.crd, A.val, b, np.ones(A.nrows), 1e-10, 40)
    xg, ig, rg = _solve(gpu, A.pos, A.crd, A.val, b, None, 1e-10, 40)
    assert ig == io == 1
    assert np.isnan(rg) == np.isnan(ro)


def test_cg_with_a_column_blocked_plan(gpu, oracle):
    # an SPD matrix with random columns: A = B + B^T + diagonal shift, solved with the
    # workgroup-blocked SpMV inside the CG driver
    import scipy.sparse as sp
    R = gen.poisson_random(20000, 6.0, seed=5)
    B = sp.csr_matrix((np.abs(R.val), R.crd, R.pos), shape=(R.nrows, R.ncols))
    S = (B + B.T).tocsr()
    S = (S + sp.diags(np.asarray(S.sum(axis=1)).ravel() + 1.0)).tocsr()
    S.sort_indices()
    pos, crd, val = S.indptr.astype(np.int32), S.indices.astype(np.int32), S.data.astype(np.float64)
    n = S.shape[0]
    b = S @ np.ones(n)
    xo, io, ro = oracle.pcg(pos, crd, val, b, np.ones(n), 1e-10, 200)
    dpos, dcrd, dval = dev(pos), dev(crd), dev(val)
    plan = gpu.CsrPlan(n, n, dpos, dcrd)
    plan.build_colblock(dcrd, dval, 8, layout="group")
    x = torch.zeros(n, dtype=torch.float64, device="cuda")
    ig, rg = gpu.pcg(plan, n, dpos, dcrd, dval, dev(b), None, 1e-10, 200, x)
    assert rg <= 1e-10 and abs(ig - io) <= 1  # the sums are added in another order: the count may move by one
    assert np.allclose(x.cpu().numpy(), np.ones(n), rtol=1e-8, atol=1e-8)


def test_mht_refreshes_a_column_blocked_copy_after_scaling(gpu, oracle, golden):
    # func @mht scales val in place before its two solves (examples/hitting_times.py:153-179); a plan that
    # holds a column-blocked copy must multiply with the scaled values, not the ones it was built from
    pos, crd, val, shape = read_mtx_csr("mht_A.mtx")
    _, _, dvals, _ = read_mtx_csr("mht_D.mtx")
    n = shape[0]
    mask = np.ones(n)
    mask[3] = 0.0
    dpos, dcrd, dval = dev(pos), dev(crd), dev(val.copy())
    plan = gpu.CsrPlan(n, n, dpos, dcrd)
    plan.build_colblock(dcrd, dval, 2, layout="group")
    m1 = torch.zeros(n, dtype=torch.float64, device="cuda")
    m2 = torch.zeros(n, dtype=torch.float64, device="cuda")
    gpu.mht(plan, n, dpos, dcrd, dval, dev(mask), dev(dvals), 0.99, 1e-10, 20, m1, m2)
    o1, o2 = oracle.mht(pos, crd, val.copy(), mask, dvals, 0.99, 1e-10, 20)
    assert np.allclose(m1.cpu().numpy(), o1, rtol=1e-9, atol=1e-12)
    assert np.allclose(m2.cpu().numpy(), o2, rtol=1e-9, atol=1e-12)


def test_cg_without_a_plan_builds_the_copy_when_it_can_pay_back(gpu, oracle):
    import scipy.sparse as sp
    R = gen.poisson_random(400000, 2.0, seed=41)
    B = sp.csr_matrix((np.abs(R.val), R.crd, R.pos), shape=(R.nrows, R.ncols))
    S = (B + B.T).tocsr()
    S = (S + sp.diags(np.asarray(S.sum(axis=1)).ravel() + 1.0)).tocsr()
    S.sort_indices()
    pos, crd, val = S.indptr.astype(np.int32), S.indices.astype(np.int32), S.data.astype(np.float64)
    n = S.shape[0]
    assert S.nnz >= (1 << 20)
    b = S @ np.ones(n)
    for maxiter in (100, 20):  # with and without the copy (maxiter < 64 keeps the CSR kernel)
        x = torch.zeros(n, dtype=torch.float64, device="cuda")
        ig, rg = gpu.pcg(None, n, dev(pos), dev(crd), dev(val), dev(b), None, 1e-10, maxiter, x)
        xo, io, ro = oracle.pcg(pos, crd, val, b, np.ones(n), 1e-10, maxiter)
        assert abs(ig - io) <= 1 and np.allclose(x.cpu().numpy(), xo, rtol=1e-7, atol=1e-9)


def _arrow_spd(n, long_len, seed):
    """SPD matrix without empty rows whose first row (and column) has `long_len` entries: symmetric,
    strictly diagonally dominant with a unit diagonal, the other rows a tridiagonal band plus their entry in
    the long column."""
    import scipy.sparse as sp
    rng = np.random.Generator(np.random.PCG64(seed))
    cols = np.sort(rng.choice(np.arange(2, n), size=long_len - 2, replace=False))
    w = -rng.random(cols.shape[0]) * 0.5 - 0.1
    arrow = sp.coo_matrix((w, (np.zeros_like(cols), cols)), shape=(n, n))
    band = sp.diags([-np.ones(n - 1)], [1], shape=(n, n))
    off = sp.csr_matrix(arrow + band)
    off = off + off.T
    diag = np.asarray(abs(off).sum(axis=1)).ravel() + 1.0
    # scaled to a unit diagonal: the long row would otherwise give CG a condition number in the thousands,
    # and ten iterations would amplify rounding differences of the dot products to 1e-7
    scale = sp.diags(1.0 / np.sqrt(diag))
    A = sp.csr_matrix(scale @ (off + sp.diags(diag)) @ scale)
    A.sort_indices()
    return A


@pytest.mark.parametrize("chunk,waves", [(512, 8), (512, 4), (1024, 2), (2048, 4)])
@pytest.mark.parametrize("n,long_len", [(20011, 9000), (4099, 3000), (70001, 40000)])
def test_cg_on_the_row_split_kernel_with_rows_cut_by_many_chunks(gpu, oracle, monkeypatch, chunk, waves, n, long_len):
    # The CG driver completes the rows the row-split kernel cuts at chunk boundaries inside its p.Ap kernel.
    # A first row of thousands of entries is cut by 16 and more boundaries (the whole-wavefront branch), odd n
    # exercises the vector tail, a small matrix has fewer chunks than the p.Ap grid has blocks.
    monkeypatch.setenv("LAPIS_HIP_SPMV_CHUNK", str(chunk))
    monkeypatch.setenv("LAPIS_HIP_SPMV_WAVES", str(waves))
    A = _arrow_spd(n, long_len, 7 + n)
    pos, crd, val = A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data.astype(np.float64)
    assert (np.diff(pos) > 0).all() and np.diff(pos).max() >= long_len
    b = gen.uniform_vector(n, 5, dtype=np.float64)
    for dinv in (None, 1.0 / A.diagonal()):
        xo, io, ro = oracle.pcg(pos, crd, val, b, dinv if dinv is not None else np.ones(n), 0.0, 10)
        dpos, dcrd = dev(pos), dev(crd)
        plan = gpu.CsrPlan(n, n, dpos, dcrd)
        plan.set_kernel(3)  # NNZSPLIT whatever the statistics say
        assert plan.stats()["kernel_name"] == "nnzsplit" and plan.stats()["chunk"] == chunk
        x = torch.full((n,), 3.0, dtype=torch.float64, device="cuda")
        iters, relres = gpu.pcg(plan, n, dpos, dcrd, dev(val), dev(b), dev(dinv) if dinv is not None else None, 0.0, 10, x)
        assert iters == io == 10
        assert np.allclose(x.cpu().numpy(), xo, rtol=1e-9, atol=1e-12)
        assert abs(relres - ro) <= 1e-7 * ro
        plan.destroy()
