"""Functions the prebuilt module has no whole-function entry point for, compiled through KokkosBackend and run
operation by operation on the kernel library (lapis_amd/executor.py): tensor-level modules checked against
numpy / scipy restatements of what their text says, loop-level modules against the oracle."""
import numpy as np
import pytest
import scipy.sparse as sp

import loop_nests
import modules_mlir as M
from conftest import read_mtx_csr
from lapis_amd import generators as gen

pytestmark = pytest.mark.gpu


def _backend():
    from lapis_amd import KokkosBackend
    return KokkosBackend.KokkosBackend(decompose_tensors=True)


def _csr_args(A):
    A = sp.csr_matrix(A)
    A.sort_indices()
    m, n = A.shape
    return (A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data, ((m, n), (m + 1, A.nnz, A.nnz)))


def _spd(n, seed):
    rng = np.random.Generator(np.random.PCG64(seed))
    # six random columns per row (scipy's sp.random draws from all n*n positions: a minute for n = 40 000)
    per_row = min(n, 6)
    cols = rng.integers(0, n, (n, per_row))
    R = sp.csr_matrix((rng.random(n * per_row), cols.ravel(), np.arange(0, n * per_row + 1, per_row)), shape=(n, n))
    R.sum_duplicates()
    S = R + R.T
    return sp.csr_matrix(S + sp.diags(np.asarray(abs(S).sum(axis=1)).ravel() + 1.0)), rng


def test_spmv_followed_by_an_axpby(gpu):
    bound = _backend().bind(M.SPMV_THEN_AXPBY)
    assert bound == {"residual": ("exec", "residual")}  # no whole-function entry: operation by operation
    mod = _backend().compile(M.SPMV_THEN_AXPBY)
    for n, seed in ((5, 1), (1000, 2), (40000, 3)):
        A, rng = _spd(n, seed)
        x, z = rng.standard_normal(n), rng.standard_normal(n)
        x_before, z_before = x.copy(), z.copy()
        out = mod.residual(*_csr_args(A), x, z, 0.75, -2.5)
        assert np.allclose(out, 0.75 * (A @ x) + -2.5 * z, rtol=1e-12, atol=1e-12)
        assert np.array_equal(x, x_before) and np.array_equal(z, z_before)  # tensor arguments are values


def test_cg_with_a_fused_residual_update_matches_its_numpy_restatement_and_scipy(gpu):
    pos, crd, val, shape = read_mtx_csr("nos4.mtx")
    A = sp.csr_matrix((val, crd, pos), shape=shape)
    n = A.shape[0]
    b = A @ np.ones(n)
    mod = _backend().compile(M.CG_FUSED_UPDATE)
    for tol, maxiter in ((1e-10, 200), (1e-3, 200), (1e-12, 7), (1e-10, 0)):
        x, its, relres = mod.cg(*_csr_args(A), b, tol, maxiter)
        # what the text says, in numpy
        xr, r, p = np.zeros(n), b.copy(), b.copy()
        rr = bb = b @ b
        k = 0
        while np.sqrt(rr) / np.sqrt(bb) > tol and k < maxiter:
            Ap = A @ p
            alpha = rr / (p @ Ap)
            xr = xr + alpha * p
            r = r - alpha * Ap
            rrn = r @ r
            p = r + (rrn / rr) * p
            rr = rrn
            k += 1
        assert its == k
        # dozens of iterations on a matrix of condition 1.6e3 amplify the different summation orders of the dot
        # products: the reference's own acceptance tolerance (np.allclose defaults, examples/pcg_solve.py:134)
        assert np.allclose(x, xr, rtol=1e-5, atol=1e-7)
        # the recursive residual at convergence is made of rounding errors: its size agrees, not its digits
        assert abs(relres - np.sqrt(rr) / np.sqrt(bb)) <= 0.1 * relres + 1e-16
    x, its, relres = mod.cg(*_csr_args(A), b, 1e-10, 200)
    assert np.allclose(x, np.ones(n), rtol=1e-6, atol=1e-6) and relres <= 1e-10


def test_richardson_iteration_with_scf_for(gpu):
    mod = _backend().compile(M.RICHARDSON)
    A, rng = _spd(3000, 11)
    d = A.diagonal()
    A = sp.csr_matrix(sp.diags(1.0 / d) @ A)  # unit diagonal, strictly dominant: the iteration contracts
    b, x0 = rng.standard_normal(3000), rng.standard_normal(3000)
    for sweeps in (0, 1, 12):
        x = mod.richardson(*_csr_args(A), b, x0, 0.5, sweeps)
        xr = x0.copy()
        for _ in range(sweeps):
            xr = xr + 0.5 * (b - A @ xr)
        assert np.allclose(x, xr, rtol=1e-12, atol=1e-12)
    assert np.array_equal(x0, x0.copy())


def test_an_operand_that_is_used_again_is_not_overwritten(gpu):
    mod = _backend().compile(M.TWO_PRODUCTS)
    A, rng = _spd(777, 5)
    x = rng.standard_normal(777)
    Ax, AAx = mod.twice_plus(*_csr_args(A), x)
    assert np.allclose(Ax, A @ x + x, rtol=1e-12, atol=1e-12)           # matvec accumulates into a copy of x
    assert np.allclose(AAx, A @ (A @ x + x) + x, rtol=1e-12, atol=1e-12)  # ... and x itself is still x


def test_a_contraction_written_as_a_generic_then_scaled_fp32(gpu):
    mod = _backend().compile(M.SPMM_GENERIC_SCALED)
    rng = np.random.Generator(np.random.PCG64(9))
    A = sp.random(300, 200, density=0.05, random_state=np.random.RandomState(9), format="csr", dtype=np.float32)
    B = rng.standard_normal((200, 24)).astype(np.float32)
    C = rng.standard_normal((300, 24)).astype(np.float32)
    C_before = C.copy()
    out = mod.scaled_product(*_csr_args(A), B, C, 0.5)
    want = (C.astype(np.float64) + A.astype(np.float64) @ B.astype(np.float64)) * 0.5
    assert out.dtype == np.float32 and out.shape == (300, 24)
    assert np.allclose(out, want, rtol=2e-5, atol=2e-5)
    assert np.array_equal(C, C_before)


def test_single_precision_pcg_runs_operation_by_operation(gpu, oracle):
    # the double-precision text binds to the whole-function solver, the same text in f32 has no such entry
    assert _backend().bind(M.PCG) == {"pcg": "pcg"} and _backend().bind(M.PCG_F32) == {"pcg": ("exec", "pcg")}
    pos, crd, val, shape = read_mtx_csr("nos4.mtx")
    A = sp.csr_matrix((val, crd, pos), shape=shape)
    n = A.shape[0]
    b = (A @ np.ones(n)).astype(np.float32)
    dinv = (1.0 / A.diagonal()).astype(np.float32)
    mod = _backend().compile(M.PCG_F32)
    x, its, relres = mod.pcg(A.indptr, A.indices, A.data.astype(np.float32), ((n, n), (n + 1, A.nnz, A.nnz)), b, dinv,
                             1e-5, 200)
    assert x.dtype == np.float32 and 1 < its < 200 and relres <= 1e-5
    assert np.allclose(x, np.ones(n), rtol=2e-3, atol=2e-3)
    # the same iteration count as the double-precision oracle, give or take rounding
    xo, io, ro = oracle.pcg(A.indptr.astype(np.int32), A.indices.astype(np.int32), A.data, b.astype(np.float64),
                            dinv.astype(np.float64), 1e-5, 200)
    assert abs(its - io) <= 3


def test_a_cg_with_the_wrong_sign_computes_what_its_text_says(gpu):
    # the text differs from the catalogue's pcg in one operand: it is no longer refused, it is run as written
    mod = _backend().compile(M.PCG_WRONG_SIGN)
    pos, crd, val, shape = read_mtx_csr("nos4.mtx")
    A = sp.csr_matrix((val, crd, pos), shape=shape)
    n = A.shape[0]
    b = A @ np.ones(n)
    dinv = 1.0 / A.diagonal()
    x, its, relres = mod.pcg(A.indptr, A.indices, A.data, ((n, n), (n + 1, A.nnz, A.nnz)), b, dinv, 1e-10, 5)
    good = _backend().compile(M.PCG)
    xg, ig, rg = good.pcg(A.indptr, A.indices, A.data, ((n, n), (n + 1, A.nnz, A.nnz)), b, dinv, 1e-10, 5)
    assert its == ig == 5 and abs(relres - rg) <= 1e-9 * rg  # the residual recurrence does not see x
    assert np.allclose(x, -xg, rtol=1e-9, atol=1e-12)        # x accumulates -alpha p instead of +alpha p


def test_near_misses_outside_the_vocabulary_are_still_refused(gpu):
    b = _backend()
    for text, why in ((M.SPMV_TRANSPOSED, "linalg.vecmat"), (M.SPMV_CSC, "d1 : dense, d0 : compressed"),
                      (M.SPMV_WIDE_INDEX, "width other than 32"), (M.SPMV_THEN_EXP, "math.exp")):
        with pytest.raises(Exception, match="Lowering to Kokkos dialect failed") as e:
            b.compile(text)
        assert why in str(e.value)


# ---- loop-level modules -----------------------------------------------------------------------------------

@pytest.mark.parametrize("n", [1, 63, 5000, 1 << 20])
def test_loop_level_dot(gpu, oracle, n):
    mod = _backend().compile(loop_nests.DOT)
    u, v = gen.uniform_vector(n, 3), gen.uniform_vector(n, 4)
    got = mod.inner(u, v, 2.5)
    want = oracle.dot(u, v, 2.5)
    assert abs(got - want) <= 1e-12 * max(1.0, np.abs(u * v).sum())


@pytest.mark.parametrize("body,ref", [
    (loop_nests.AXPBY_BODY, lambda p, u, q, v: u * p + v * q),
    (loop_nests.MULT_BODY, lambda p, u, q, v: u * v),
    (loop_nests.SCALE_BODY, lambda p, u, q, v: p * u),
    (loop_nests.FILL_BODY, lambda p, u, q, v: np.full_like(u, p + q)),
])
def test_loop_level_elementwise(gpu, body, ref):
    mod = _backend().compile(loop_nests.elementwise(body))
    for n in (1, 1000, 262145):
        u, v = gen.uniform_vector(n, 6), gen.uniform_vector(n, 7)
        w = np.full(n, 99.0)
        assert mod.update(1.5, u, -0.25, v, w) is None
        assert np.array_equal(w, ref(1.5, u, -0.25, v))  # no summation order: bit for bit
    # in place: w is also an input
    w = u.copy()
    mod.update(1.5, w, -0.25, v, w)
    assert np.array_equal(w, ref(1.5, u, -0.25, v))


def test_loop_level_elementwise_the_library_has_no_kernel_for_is_refused(gpu):
    with pytest.raises(Exception, match=r"Lowering to Kokkos dialect failed[\s\S]*depth 1"):
        _backend().compile(loop_nests.elementwise(loop_nests.CUBE_BODY))
    with pytest.raises(Exception, match=r"Lowering to Kokkos dialect failed[\s\S]*depth 1"):
        _backend().compile(loop_nests.DOT_PRODUCT_REDUCTION)


@pytest.mark.parametrize("elem,dtype,tol", [("f32", np.float32, 2e-5), ("f64", np.float64, 1e-12)])
@pytest.mark.parametrize("inner", ["scf.parallel", "scf.for"])
def test_loop_level_spmm(gpu, oracle, elem, dtype, tol, inner):
    mod = _backend().compile(loop_nests.spmm_i32(elem, inner))
    rng = np.random.Generator(np.random.PCG64(21))
    for rows, cols, k in ((3, 4, 2), (500, 300, 64), (257, 1000, 33)):
        A = sp.random(rows, cols, density=min(1.0, 8.0 / cols), random_state=np.random.RandomState(rows), format="csr",
                      dtype=dtype)
        A.sort_indices()
        B = rng.standard_normal((cols, k)).astype(dtype)
        C = rng.standard_normal((rows, k)).astype(dtype)
        want = C.astype(np.float64) + A.astype(np.float64) @ B.astype(np.float64)
        # @rows_times_dense(B, ptr, idx, C, nz)
        mod.rows_times_dense(B, A.indptr.astype(np.int32), A.indices.astype(np.int32), C, A.data)
        assert np.allclose(C, want, rtol=tol, atol=tol)
    # the literal case of the reference's example (examples/spmm_dcsr_opdsl.py:139-172)
    A = sp.csr_matrix(np.array([[1.1, 0, 0, 0], [0, 2.2, 3.3, 0], [0, 0, 0, 0]], dtype=dtype))
    B = np.array([[1, 2], [4, 3], [5, 6], [8, 7]], dtype=dtype)
    C = np.zeros((3, 2), dtype)
    mod.rows_times_dense(B, A.indptr.astype(np.int32), A.indices.astype(np.int32), C, A.data)
    assert np.allclose(C, np.matmul(A.toarray(), B), rtol=tol, atol=tol)


def test_loop_level_spmv_with_more_around_it_now_runs(gpu, golden):
    # the nest plus a load and a store of single elements: no whole-function entry, but every part has one
    text = loop_nests.spmv_i32("f64").replace("    return\n", "    memref.store %x0, %y[%zero] : memref<?xf64>\n    return\n").replace(
        "%rows = memref.dim", "%x0 = memref.load %x[%zero] : memref<?xf64>\n    %rows = memref.dim")
    mod = _backend().compile(text)
    g = golden["spmv_noalloc"]
    rowptrs, colinds = np.array(g["pos"], np.int32), np.array(g["crd"], np.int32)
    values = np.array(g["val"], np.float64)
    x = np.arange(1.0, 6.0)
    y = np.zeros(5)
    mod.rowsum32(values, x, rowptrs, y, colinds)
    A = sp.csr_matrix((values, colinds, rowptrs), shape=(5, 5))
    want = A @ x
    want[0] = x[0]
    assert np.allclose(y, want, rtol=1e-14, atol=1e-14)
