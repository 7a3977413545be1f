"""The generated-module calling convention on the GPU: the reference's own example
programs (examples/spmv_noalloc.py, spmv.py, pcg_solve.py, multiple_results.py,
spmm_dcsr_opdsl.py) with only the module construction swapped."""
import subprocess
import sys
import textwrap

import numpy as np
import pytest
import scipy.sparse as sp
from scipy.sparse.linalg import cg as scipy_cg

from conftest import ROOT, read_mtx_csr
from lapis_amd import generators as gen

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def module_kokkos(gpu):
    from lapis_amd.module import LAPISModule
    return LAPISModule()


def test_spmv_noalloc_example(module_kokkos, golden):
    g = golden["spmv_noalloc"]
    rowptrs = np.array(g["pos"], dtype=np.int32)
    colinds = np.array(g["crd"], dtype=np.int32)
    values = np.array(g["val"], dtype=np.double)
    m, n = g["m"], g["n"]
    x = np.ones((n), dtype=np.double)
    ykokkos = np.zeros((m), dtype=np.double)
    ret = module_kokkos.spmv(rowptrs, colinds, values, ((m, n), (len(rowptrs), len(colinds), len(values))), x, ykokkos)
    assert np.allclose(ykokkos, g["y_expected"])  # the output argument is updated in place
    assert ret.ctypes.data == ykokkos.ctypes.data  # and the returned memref aliases it
    # a second call accumulates: linalg.matvec adds A*x to the output
    module_kokkos.spmv(rowptrs, colinds, values, ((m, n), (len(rowptrs), len(colinds), len(values))), x, ykokkos)
    assert np.allclose(ykokkos, 2 * np.array(g["y_expected"]))


def test_spmv_example_lapis_main_allocates_its_result(module_kokkos, golden):
    g = golden["spmv_noalloc"]
    rowptrs, colinds = np.array(g["pos"], np.int32), np.array(g["crd"], np.int32)
    values = np.array(g["val"], np.double)
    x = np.ones(5)
    y1 = module_kokkos.lapis_main(rowptrs, colinds, values, ((5, 5), (6, 8, 8)), x)
    y2 = module_kokkos.lapis_main(rowptrs, colinds, values, ((5, 5), (6, 8, 8)), 2 * x)
    assert np.allclose(y1, g["y_expected"]) and np.allclose(y2, 2 * np.array(g["y_expected"]))
    assert y1.ctypes.data != y2.ctypes.data  # each result stays alive until lapis_finalize


def test_wrong_dtype_inputs_are_coerced_like_the_emitted_wrapper(module_kokkos, golden):
    g = golden["spmv_noalloc"]
    y = np.zeros(5)
    module_kokkos.spmv(np.array(g["pos"], np.int64), np.array(g["crd"], np.int64), list(g["val"]),
                       ((5, 5), (6, 8, 8)), np.ones(5, np.float64), y)
    assert np.allclose(y, g["y_expected"])


def test_pcg_solve_example(module_kokkos, golden, oracle):
    g = golden["pcg_solve"]
    pos, crd, val, shape = read_mtx_csr(g["matrix"])
    A = sp.csr_matrix((val, crd, pos), shape=shape)
    n, nnz = A.shape[0], A.nnz
    xgold = np.ones((n), dtype=np.double)
    b = A @ xgold
    dinv = 1.0 / A.diagonal()
    (x, numiter, relres) = module_kokkos.pcg(A.indptr, A.indices, A.data, ((n, n), (n + 1, nnz, nnz)), b, dinv,
                                             g["reltol"], g["maxiter"])
    [x_scipy, info] = scipy_cg(A, b, np.zeros((n)), rtol=g["reltol"], maxiter=g["maxiter"], M=np.diag(dinv))
    assert np.allclose(x, x_scipy)
    _, io, _ = oracle.pcg(pos, crd, val, b, dinv, g["reltol"], g["maxiter"])
    assert int(numiter) == io and numiter.dtype == np.uint64


def test_hitting_times_example_gold_vectors(module_kokkos, golden):
    g = golden["hitting_times"]
    pos, crd, val, shape = read_mtx_csr("mht_A.mtx")
    A = sp.csr_matrix((val, crd, pos), shape=shape)
    n, nnz = A.shape[0], A.nnz
    D = read_mtx_csr("mht_D.mtx")[2]
    mask = np.ones(n)
    for s_ in g["seedset"]:
        mask[s_] = 0
    (mom1, mom2) = module_kokkos.mht(A.indptr, A.indices, A.data, ((n, n), (n + 1, nnz, nnz)), mask, D, g["alpha"],
                                     g["tol"], g["maxiter"])
    mom2_norm = module_kokkos.normalize_mom2(mom1, mom2)
    assert np.allclose(mom1, g["mom1_gold"]) and np.allclose(mom2_norm, g["mom2_gold"])  # the reference's check


def test_multiple_results_example(module_kokkos, golden):
    g = golden["multiple_results"]
    x, y = np.array(g["x"]), np.array(g["y"])
    (x_plus_y, norm) = module_kokkos.plus_norm(x, y)
    assert np.allclose(x_plus_y, x + y) and np.allclose(norm, np.linalg.norm(x + y))


def test_spmm_example(module_kokkos, golden):
    g = golden["spmm_dcsr"]
    a, b = np.array(g["a_dense"]), np.array(g["b"])
    A = sp.csr_matrix(a)
    c = np.zeros((3, 2), np.float64)
    module_kokkos.spmm(A.indptr, A.indices, A.data, ((3, 4), (4, A.nnz, A.nnz)), b, c)
    assert np.allclose(c, np.matmul(a, b))


def test_bspmm_example(module_kokkos, oracle):
    # the recipe of examples/bspmm.py:62-89 (its values are unseeded there: seeded here), checked per
    # batch against scipy as the example does, and against the oracle
    m, n, b, k, nnz = 5, 6, 8, 3, 8
    rowptrs = np.array([0, 1, 5, 6, 8, 8], dtype=np.int32)
    colinds = np.array([1, 0, 2, 3, 4, 5, 0, 1], dtype=np.int32)
    rng = np.random.default_rng(62)
    values = rng.uniform(1.0, 2.0, nnz * b).astype(np.float32)
    B = rng.uniform(1.0, 2.0, (n, k, b)).astype(np.float32)
    C_gold = np.zeros((m, k, b), dtype=np.float32)
    for i in range(b):
        Aslice = sp.csr_matrix((values[i::b], colinds, rowptrs), (m, n))
        C_gold[:, :, i] = Aslice @ B[:, :, i]
    C = module_kokkos.pte_local_bspmm(rowptrs, colinds, values, ((m, n, b), (m + 1, nnz, nnz * b)), B)
    assert C.shape == (m, k, b) and C.dtype == np.float32
    assert np.allclose(C_gold, C)
    want = oracle.bspmm_csrv(rowptrs, colinds, values, B, m)
    assert np.allclose(C, want, rtol=1e-5, atol=0)


def test_module_spmv_on_benchmark_shaped_input(module_kokkos, oracle):
    A, x = gen.config2(scale=1 / 128)
    y = np.zeros(A.nrows)
    module_kokkos.spmv(A.pos, A.crd, A.val, A.spec(), x, y)
    want = np.zeros(A.nrows)
    oracle.spmv(A.pos, A.crd, A.val, x, want)
    scale = oracle.spmv_abs_scale(A.pos, A.crd, A.val, x)
    assert np.all(np.abs(y - want) <= 1e-12 * np.maximum(scale, 1e-300))
    B, xf = gen.config3(scale=1 / 64)
    yf = np.zeros(B.nrows, np.float32)
    module_kokkos.spmv(B.pos, B.crd, B.val, B.spec(), xf, yf)
    wantf = np.zeros(B.nrows, np.float32)
    oracle.spmv(B.pos, B.crd, B.val, xf, wantf)
    scalef = oracle.spmv_abs_scale(B.pos, B.crd, B.val, xf)
    assert np.all(np.abs(yf.astype(np.float64) - wantf) <= 1e-5 * np.maximum(scalef, 1e-300))


def test_non_contiguous_memref_aborts_like_kokkos_abort():
    # the reference aborts the process (LAPISSupport.hpp:76,86); run it in a child
    code = textwrap.dedent("""
        import ctypes, numpy as np, sys
        sys.path.insert(0, %r)
        from lapis_amd.module import LAPISModule
        from lapis_amd import memref as rt
        m = LAPISModule()
        pos = np.array([0, 1, 2], np.int32); crd = np.array([0, 1], np.int32); val = np.ones(2)
        x2 = np.ones(4)[::2]          # stride 2: numpy.require(..., 'C') would copy, so call the C entry directly
        y = np.zeros(2)
        spec = np.array([2, 2, 3, 2, 2], np.int64)
        ret0 = ctypes.pointer(ctypes.pointer(rt.make_nd_memref_descriptor(1, ctypes.c_double)()))
        d = lambda a: ctypes.pointer(rt.get_ranked_memref_descriptor(a))
        m.libHandle.py_spmv(ret0, d(pos), d(crd), d(val), spec.ctypes.data_as(ctypes.c_void_p), d(x2), d(y))
        print("survived")
    """ % ROOT)
    proc = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=300)
    assert proc.returncode != 0 and "survived" not in proc.stdout
    assert "not contiguous" in proc.stderr


# ---- through KokkosBackend.compile(moduleText), as the example scripts do ----------------------------

def test_compile_binds_spmv_by_its_body_and_reproduces_the_literal_answer(gpu, golden):
    import modules_mlir as M
    from lapis_amd import KokkosBackend
    g = golden["spmv_noalloc"]
    rowptrs, colinds = np.array(g["pos"], np.int32), np.array(g["crd"], np.int32)
    values = np.array(g["val"], np.double)
    backend = KokkosBackend.KokkosBackend(decompose_tensors=True)
    module_kokkos = backend.compile(M.SPMV)
    y = np.zeros(5)
    module_kokkos.spmv(rowptrs, colinds, values, ((5, 5), (len(rowptrs), len(colinds), len(values))), np.ones(5), y)
    assert np.allclose(y, [1.1, 2.2, -19, -1, 0])  # examples/spmv_noalloc.py:31
    # the same computation under another name binds to the same kernel, under ITS name
    other = backend.compile(M.MATVEC_OTHER_NAME)
    y2 = np.zeros(5)
    other.apply_operator(rowptrs, colinds, values, ((5, 5), (6, 8, 8)), np.ones(5), y2)
    assert np.array_equal(y2, y)
    # the right name on the wrong computation never reaches a kernel
    with pytest.raises(Exception, match="Lowering to Kokkos dialect failed"):
        backend.compile(M.SPMV_TRANSPOSED)


def test_compile_binds_a_loop_level_spmv_and_routes_its_buffers_by_role(gpu, golden, oracle):
    import loop_nests
    from lapis_amd import KokkosBackend
    g = golden["spmv_noalloc"]
    rowptrs, colinds = np.array(g["pos"], np.int32), np.array(g["crd"], np.int32)
    backend = KokkosBackend.KokkosBackend(decompose_tensors=True)
    for elem, dtype, tol in (("f64", np.float64, 1e-14), ("f32", np.float32, 1e-6)):
        module_kokkos = backend.compile(loop_nests.spmv_i32(elem, name="apply"))
        values = np.array(g["val"], dtype)
        y = np.zeros(5, dtype)
        # @apply(vals, x, rowptr, y, colidx)
        module_kokkos.apply(values, np.ones(5, dtype), rowptrs, y, colinds)
        assert np.allclose(y, [1.1, 2.2, -19, -1, 0], rtol=tol, atol=tol)  # examples/spmv_noalloc.py:31
        module_kokkos.apply(values, np.ones(5, dtype), rowptrs, y, colinds)  # the nest starts from y[i]: accumulates
        assert np.allclose(y, 2 * np.array([1.1, 2.2, -19, -1, 0]), rtol=tol, atol=tol)
    # a larger matrix against the oracle
    A, x = gen.laplace2d(48), gen.uniform_vector(48 * 48, 5)
    y = np.zeros(A.nrows)
    backend.compile(loop_nests.spmv_i32("f64", name="apply")).apply(A.val, x, A.pos, y, A.crd)
    want = np.zeros(A.nrows)
    oracle.spmv(A.pos, A.crd, A.val, x, want)
    assert np.allclose(y, want, rtol=1e-13, atol=1e-13)


def test_compile_binds_pcg_and_matches_scipy_on_nos4(gpu):
    import modules_mlir as M
    from lapis_amd import KokkosBackend
    pos, crd, val, shape = read_mtx_csr("nos4.mtx")
    A = sp.csr_matrix((val, crd, pos), shape=shape)
    n = A.shape[0]
    b = A @ np.ones(n)
    dinv = 1.0 / A.diagonal()
    module_kokkos = KokkosBackend.KokkosBackend(decompose_tensors=True).compile(M.PCG)
    (x, numiter, relres) = module_kokkos.pcg(A.indptr, A.indices, A.data, ((n, n), (n + 1, A.nnz, A.nnz)), b, dinv,
                                              1e-10, 40)
    [x_scipy, info] = scipy_cg(A, b, np.zeros((n)), rtol=1e-10, maxiter=40, M=sp.diags(dinv))
    assert np.allclose(x, x_scipy)  # the acceptance check of examples/pcg_solve.py:134


def test_two_modules_share_the_library_and_outlive_each_other(gpu, golden):
    # every compile() returns a new module object over the one prebuilt library: dropping one of them must
    # neither free the results of the other nor shut the library down under it
    import gc
    import modules_mlir as M
    from lapis_amd import KokkosBackend
    g = golden["spmv_noalloc"]
    rowptrs, colinds = np.array(g["pos"], np.int32), np.array(g["crd"], np.int32)
    values = np.array(g["val"], np.double)
    backend = KokkosBackend.KokkosBackend(decompose_tensors=True)
    torch_mv = M.SPMV.replace("@spmv(%A: tensor<?x?xf64, #sparse>, %x: tensor<?xf64>, %y: tensor<?xf64>)",
                              "@main(%A: tensor<?x?xf64, #sparse>, %x: tensor<?xf64>)")
    first = backend.compile(M.SPMV)
    second = backend.compile(M.SPMV)
    kept = second.lapis_main(rowptrs, colinds, values, ((5, 5), (6, 8, 8)), np.ones(5))  # module-owned result
    want = kept.copy()
    del first
    gc.collect()
    junk = [np.full(5, 7.0) for _ in range(64)]  # reuse freed heap blocks, if any were freed
    assert np.array_equal(kept, want) and np.allclose(want, g["y_expected"])
    y = np.zeros(5)
    second.spmv(rowptrs, colinds, values, ((5, 5), (6, 8, 8)), np.ones(5), y)  # the library is still initialised
    assert np.allclose(y, g["y_expected"])
    del junk
    # the packaging arguments of examples/twomodules.py:36-39: instance k is package lapis_package_k and only the
    # last instance would have been emitted with --finalize; both run whichever goes first
    k1 = KokkosBackend.KokkosBackend(decompose_tensors=True, index_instance=0, num_instances=2).compile(M.SPMV)
    k2 = KokkosBackend.KokkosBackend(decompose_tensors=True, index_instance=1, num_instances=2).compile(M.MATVEC_OTHER_NAME)
    assert (k1.package_name, k1.finalizes_runtime) == ("lapis_package", False)
    assert (k2.package_name, k2.finalizes_runtime) == ("lapis_package_1", True)
    del k2  # the "finalizing" module goes first: the other one still runs
    gc.collect()
    y = np.zeros(5)
    k1.spmv(rowptrs, colinds, values, ((5, 5), (6, 8, 8)), np.ones(5), y)
    assert np.allclose(y, g["y_expected"])


# ---- operands that stay on the device -----------------------------------------------------------------

def test_resident_matrix_and_dual_views(gpu, oracle):
    from lapis_amd.module import LAPISModule
    mod = LAPISModule()
    A = gen.poisson_random(50000, 7.0, seed=61)
    x = gen.uniform_vector(A.ncols, 62)
    spec = ((A.nrows, A.ncols), (A.nrows + 1, A.nnz, A.nnz))
    Ad = mod.bind_csr(A.pos, A.crd, A.val, spec)
    want = np.zeros(A.nrows)
    oracle.spmv(A.pos, A.crd, A.val, x, want)
    scale = oracle.spmv_abs_scale(A.pos, A.crd, A.val, x)
    # numpy operands: copied per call, y updated in place like LAPISModule.spmv
    y = np.zeros(A.nrows)
    ret = Ad.spmv(x, y)
    assert ret is y and np.all(np.abs(y - want) <= 1e-12 * np.maximum(scale, 1e-300))
    # dual views: nothing is copied until asked for; two products accumulate on the device
    xv, yv = mod.dual_view(x.copy()), mod.dual_view(np.zeros(A.nrows))
    Ad.spmv(xv, yv)
    Ad.spmv(xv, yv)
    assert np.all(yv.host == 0.0)  # the host half is stale until sync_host
    got = yv.sync_host()
    assert np.all(np.abs(got - 2 * want) <= 2e-12 * np.maximum(scale, 1e-300))
    # a host-side change is seen only after modify_host, as with the DualView it stands for
    xv.host[:] = 2 * x
    yv.host[:] = 0.0
    yv.modify_host()
    Ad.spmv(xv, yv)
    assert np.all(np.abs(yv.sync_host() - want) <= 1e-12 * np.maximum(scale, 1e-300))  # still the old x
    xv.modify_host()
    yv.host[:] = 0.0
    yv.modify_host()
    Ad.spmv(xv, yv)
    assert np.all(np.abs(yv.sync_host() - 2 * want) <= 2e-12 * np.maximum(scale, 1e-300))
    # new values in the same pattern
    Ad.update_values(-A.val)
    y3 = np.zeros(A.nrows)
    Ad.spmv(x, y3)
    assert np.all(np.abs(y3 + want) <= 1e-12 * np.maximum(scale, 1e-300))
    Ad.release()


def test_resident_matrix_gets_the_column_blocked_copy_where_recommended(gpu, oracle):
    from lapis_amd.module import LAPISModule
    mod = LAPISModule()
    A = gen.poisson_random(600000, 4.0, seed=63)
    x = gen.uniform_vector(A.ncols, 64)
    Ad = mod.bind_csr(A.pos, A.crd, A.val, ((A.nrows, A.ncols), (A.nrows + 1, A.nnz, A.nnz)))
    y = np.zeros(A.nrows)
    Ad.spmv(x, y)
    want = np.zeros(A.nrows)
    oracle.spmv(A.pos, A.crd, A.val, x, want)
    scale = oracle.spmv_abs_scale(A.pos, A.crd, A.val, x)
    assert np.all(np.abs(y - want) <= 1e-12 * np.maximum(scale, 1e-300))
    Ad.update_values(0.5 * A.val)  # refreshes the copy through the kept permutation
    y2 = np.zeros(A.nrows)
    Ad.spmv(x, y2)
    assert np.all(np.abs(y2 - 0.5 * want) <= 1e-12 * np.maximum(scale, 1e-300))


def test_resident_fp32_matrix_spmv_and_spmm(gpu, oracle):
    # LAPIS::DualView is a template over the element type (LAPISSupport.hpp:136): resident operands exist
    # for float as for double, and for the SpMM of examples/spmm_dcsr_opdsl.py:73-110 as for SpMV
    from lapis_amd.module import LAPISModule
    mod = LAPISModule()
    A = gen.poisson_random(30000, 11.0, seed=71)
    A = gen.CSR(A.nrows, A.ncols, A.pos, A.crd, A.val.astype(np.float32))
    spec = ((A.nrows, A.ncols), (A.nrows + 1, A.nnz, A.nnz))
    Ad = mod.bind_csr(A.pos, A.crd, A.val, spec)
    assert Ad.dtype == np.float32
    x = gen.uniform_vector(A.ncols, 72, dtype=np.float32)
    want = np.zeros(A.nrows, np.float32)
    oracle.spmv(A.pos, A.crd, A.val, x, want)
    scale = oracle.spmv_abs_scale(A.pos, A.crd, A.val, x)
    y = np.zeros(A.nrows, np.float32)
    assert Ad.spmv(x, y) is y
    assert np.all(np.abs(y.astype(np.float64) - want) <= 1e-5 * np.maximum(scale, 1e-30))
    xv, yv = mod.dual_view(x.copy()), mod.dual_view(np.zeros(A.nrows, np.float32))
    assert xv.dtype == np.float32
    Ad.spmv(xv, yv)
    assert np.all(yv.host == 0.0)
    assert np.all(np.abs(yv.sync_host().astype(np.float64) - want) <= 1e-5 * np.maximum(scale, 1e-30))
    with pytest.raises(TypeError):
        Ad.spmv(mod.dual_view(np.zeros(A.ncols)), yv)  # a float64 view against a float32 matrix
    for k in (1, 7, 64):
        B = gen.uniform_matrix(A.ncols, k, 73).astype(np.float32)
        C0 = gen.uniform_matrix(A.nrows, k, 74).astype(np.float32)
        Cw = C0.copy()
        oracle.spmm(A.pos, A.crd, A.val, B, Cw)
        C = C0.copy()
        assert Ad.spmm(B, C) is C
        assert np.allclose(C, Cw, rtol=2e-5, atol=2e-5 * 11 * 1.0)
        Bv, Cv = mod.dual_view(B.copy()), mod.dual_view(C0.copy())
        Ad.spmm(Bv, Cv)
        assert np.array_equal(Cv.host, C0)  # stale until asked for
        assert np.allclose(Cv.sync_host(), Cw, rtol=2e-5, atol=2e-5 * 11 * 1.0)
    Ad.release()


def test_resident_pcg_and_the_module_entry_reach_the_column_blocked_kernel(gpu):
    # a symmetric, strictly diagonally dominant matrix with uniformly random columns and more than 2^20
    # non-zeros: the library recommends the column-blocked copy; with maxiter >= 64 py_pcg asks for it
    import scipy.sparse as sp
    import scipy.sparse.linalg as spla
    from lapis_amd.module import LAPISModule
    R = gen.poisson_random(400000, 2.0, seed=81)
    R = sp.csr_matrix((R.val, R.crd, R.pos), shape=(R.nrows, R.ncols))
    S = R + R.T
    S = S + sp.diags(np.asarray(abs(S).sum(axis=1)).ravel() + 1.0)
    S = sp.csr_matrix(S)
    S.sort_indices()
    n = S.shape[0]
    pos, crd, val = S.indptr.astype(np.int32), S.indices.astype(np.int32), S.data.astype(np.float64)
    assert val.shape[0] > (1 << 20)
    xs = gen.uniform_vector(n, 82)
    b = S @ xs
    dinv = 1.0 / S.diagonal()
    spec = ((n, n), (n + 1, val.shape[0], val.shape[0]))
    mod = LAPISModule()
    x1, it1, rr1 = mod.pcg(pos, crd, val, spec, b, dinv, 1e-10, 100)   # analysed: maxiter >= 64
    x2, it2, rr2 = mod.pcg(pos, crd, val, spec, b, dinv, 1e-10, 63)    # not analysed: plain CSR kernel
    assert rr1 <= 1e-10 and rr2 <= 1e-10 and abs(int(it1) - int(it2)) <= 1
    assert np.allclose(x1, xs, rtol=1e-7, atol=1e-9) and np.allclose(x2, xs, rtol=1e-7, atol=1e-9)
    Ad = mod.bind_csr(pos, crd, val, spec)
    x3, it3, rr3 = Ad.pcg(b, dinv, 1e-10, 100)
    assert rr3 <= 1e-10 and abs(int(it3) - int(it1)) <= 1 and np.allclose(x3, xs, rtol=1e-7, atol=1e-9)
    xv = mod.dual_view(np.zeros(n))
    out, it4, rr4 = Ad.pcg(mod.dual_view(b.copy()), None, 1e-10, 200, x=xv)   # unpreconditioned, result left on the device
    assert out is xv and rr4 <= 1e-10
    assert np.allclose(xv.sync_host(), xs, rtol=1e-7, atol=1e-9)
    assert np.linalg.norm(S @ xv.host - b) <= 2e-10 * np.linalg.norm(b)
    Ad.release()
