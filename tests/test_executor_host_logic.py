"""The executor's host logic without a GPU: lapis_amd.executor run over a numpy stand-in for the kernel library
(tests/fake_hip.py) on CPU tensors.  What is checked here is everything the executor decides itself: which buffer an
operation may overwrite, loops and calls, which entry point an operation goes to, and what it refuses."""
import re

import numpy as np
import pytest
import scipy.sparse as sp
import torch

import fake_hip
import loop_nests
import modules_mlir as M
from lapis_amd import executor as ex
from lapis_amd import mlir_text as mt


def make(text):
    e = ex.Executor(mt.Canonicalizer(text), torch_module=torch, hip_module=fake_hip, device="cpu")
    fake_hip.calls.clear()
    return e


def csr(A, dtype=np.float64):
    A = sp.csr_matrix(A)
    A.sort_indices()
    t = lambda a, d: torch.from_numpy(np.array(a, dtype=d))
    return ex.Csr(t(A.indptr, np.int32), t(A.indices, np.int32), t(A.data, dtype), A.shape[0], A.shape[1])


def vec(a, dtype=np.float64):
    return torch.from_numpy(np.array(a, dtype=dtype))


def spd(n, seed):
    R = sp.random(n, n, density=min(1.0, 5.0 / n), random_state=np.random.RandomState(seed), format="csr")
    S = R + R.T
    return sp.csr_matrix(S + sp.diags(np.asarray(abs(S).sum(axis=1)).ravel() + 1.0))


def test_spmv_then_axpby_goes_to_three_entry_points_and_leaves_its_arguments_alone():
    e = make(M.SPMV_THEN_AXPBY)
    e.check("residual")
    A = spd(50, 1)
    rng = np.random.default_rng(0)
    x, z = rng.standard_normal(50), rng.standard_normal(50)
    tx, tz = vec(x), vec(z)
    (out,) = e.run("residual", [csr(A), tx, tz, 0.75, -2.5])
    assert np.allclose(out.numpy(), 0.75 * (A @ x) - 2.5 * z)
    assert fake_hip.calls == ["fill", "spmv", "axpby"]
    assert np.array_equal(tx.numpy(), x) and np.array_equal(tz.numpy(), z)
    # the fill went into the tensor.empty, the product into the filled buffer (nothing mentions it later), and the
    # generic into the second tensor.empty: no operation needed a copy of an operand


def test_an_operand_mentioned_later_is_copied_not_overwritten():
    e = make(M.TWO_PRODUCTS)
    A = spd(40, 2)
    x = np.random.default_rng(1).standard_normal(40)
    tx = vec(x)
    Ax, AAx = e.run("twice_plus", [csr(A), tx])
    assert np.array_equal(tx.numpy(), x)                       # the argument is still x
    assert np.allclose(Ax.numpy(), A @ x + x)                  # first product accumulated into a copy of x
    assert np.allclose(AAx.numpy(), A @ (A @ x + x) + x)       # second into another copy
    assert Ax.data_ptr() != tx.data_ptr() and AAx.data_ptr() != tx.data_ptr() and Ax.data_ptr() != AAx.data_ptr()


def test_while_loop_carries_values_and_stops_as_the_text_says():
    e = make(M.CG_FUSED_UPDATE)
    e.check("cg")
    A = spd(120, 3)
    b = A @ np.ones(120)
    for tol, maxiter in ((1e-12, 500), (1e-2, 500), (1e-12, 3), (1e-12, 0)):
        x, its, relres = e.run("cg", [csr(A), vec(b), tol, maxiter])
        xr, r, p = np.zeros(120), b.copy(), b.copy()
        rr = bb = b @ b
        k = 0
        while np.sqrt(rr) / np.sqrt(bb) > tol and k < maxiter:
            Ap = A @ p
            alpha = rr / (p @ Ap)
            xr, r = xr + alpha * p, r - alpha * Ap
            rrn = r @ r
            p, rr, k = r + (rrn / rr) * p, rrn, k + 1
        assert its == k and np.allclose(x.numpy(), xr, rtol=1e-9, atol=1e-12)
    # a matrix multiplied with again and again is handed to the library's analysis once, at its sixth product
    fake_hip.calls.clear()
    A2 = csr(A)
    e.run("cg", [A2, vec(b), 1e-12, 500])
    assert fake_hip.calls.count("analyze") == 1 and fake_hip.calls.index("analyze") > fake_hip.calls.index("spmv")
    A2.release()


def test_scf_for_with_iteration_arguments():
    e = make(M.RICHARDSON)
    A = spd(60, 4)
    A = sp.csr_matrix(sp.diags(1.0 / A.diagonal()) @ A)
    rng = np.random.default_rng(2)
    b, x0 = rng.standard_normal(60), rng.standard_normal(60)
    for sweeps in (0, 1, 7):
        (x,) = e.run("richardson", [csr(A), vec(b), vec(x0), 0.5, sweeps])
        xr = x0.copy()
        for _ in range(sweeps):
            xr = xr + 0.5 * (b - A @ xr)
        assert np.allclose(x.numpy(), xr, rtol=1e-13, atol=1e-13)


def test_the_catalogue_functions_also_run_operation_by_operation():
    # the whole-function entry points are a fast path, not a different semantics
    e = make(M.PCG)
    A = spd(80, 5)
    b = A @ np.ones(80)
    dinv = 1.0 / A.diagonal()
    x, its, relres = e.run("pcg", [csr(A), vec(b), vec(dinv), 1e-10, 100])
    assert np.allclose(x.numpy(), np.ones(80), rtol=1e-7) and 1 < its < 100 and relres <= 1e-10
    e32 = make(M.PCG_F32)
    x, its, relres = e32.run("pcg", [csr(A, np.float32), vec(b, np.float32), vec(dinv, np.float32), np.float32(1e-4), 100])
    assert x.dtype == torch.float32 and isinstance(relres, np.floating) and np.allclose(x.numpy(), np.ones(80), rtol=1e-2)


def test_contraction_generic_and_elementwise_in_place():
    e = make(M.SPMM_GENERIC_SCALED)
    rng = np.random.default_rng(3)
    A = sp.random(30, 20, density=0.2, random_state=np.random.RandomState(3), format="csr", dtype=np.float32)
    B, C = rng.standard_normal((20, 6)).astype(np.float32), rng.standard_normal((30, 6)).astype(np.float32)
    tC = vec(C, np.float32)
    (out,) = e.run("scaled_product", [csr(A, np.float32), vec(B, np.float32), tC, np.float32(0.5)])
    assert np.allclose(out.numpy(), (C + A @ B) * 0.5, rtol=1e-5, atol=1e-5) and np.array_equal(tC.numpy(), C)
    assert fake_hip.calls == ["spmm", "axpby"]  # the scaling is a*x with b = 0, written over the product's own buffer


def test_loop_level_functions_update_their_memrefs_in_place():
    e = make(loop_nests.elementwise(loop_nests.AXPBY_BODY))
    e.check("update")
    u, v, w = vec(np.arange(5.0)), vec(np.ones(5)), vec(np.zeros(5))
    assert e.run("update", [2.0, u, 3.0, v, w]) == []
    assert np.array_equal(w.numpy(), 2.0 * np.arange(5.0) + 3.0)
    d = make(loop_nests.DOT)
    (got,) = d.run("inner", [vec([1.0, 2.0, 3.0]), vec([4.0, 5.0, 6.0]), 0.5])
    assert got == 32.5 and fake_hip.calls == ["dot"]
    s = make(loop_nests.spmv_i32("f64"))
    live_before = fake_hip.CsrPlan.live
    A = spd(25, 6)
    x, y = np.arange(25.0), np.ones(25)
    ty = vec(y)
    # @rowsum32(vals, x, rowptr, y, colidx)
    s.run("rowsum32", [vec(A.data), vec(x), vec(A.indptr, np.int32), ty, vec(A.indices, np.int32)])
    assert np.allclose(ty.numpy(), y + A @ x)
    assert fake_hip.CsrPlan.live == live_before + 1  # one plan for the nest's buffers ...
    s.release()
    assert fake_hip.CsrPlan.live == live_before      # ... given back


def test_refusals_name_the_operation():
    for text, fn, why in ((M.SPMV_TRANSPOSED, "spmv", "linalg.vecmat"), (M.SPMV_THEN_EXP, "residual", "math.exp"),
                          (M.SPMV_CSC, "spmv", "d1 : dense, d0 : compressed"),
                          (loop_nests.DEEP4, None, "depth 4"), (loop_nests.SPMV_INDEX, None, "memref<?xindex>"),
                          (loop_nests.elementwise(loop_nests.CUBE_BODY), "update", "depth 1")):
        e = make(text)
        name = fn or [f.name for f in e.c.public()][0]
        with pytest.raises(ex.Refused, match=re.escape(why)):
            e.check(name)
    # dense x dense and a sparse second operand are not products the library has
    gemm = ("func.func @gemm(%a: tensor<?x?xf64>, %b: tensor<?x?xf64>, %c: tensor<?x?xf64>) -> tensor<?x?xf64> {\n"
            "  %0 = linalg.matmul ins(%a, %b : tensor<?x?xf64>, tensor<?x?xf64>) outs(%c : tensor<?x?xf64>) -> tensor<?x?xf64>\n"
            "  return %0 : tensor<?x?xf64>\n}")
    with pytest.raises(ex.Refused, match="first operand is not a CSR tensor"):
        make(gemm).check("gemm")


def test_scalar_arithmetic_follows_the_types():
    text = """
    func.func @scalars(%a: f32, %b: f32, %n: index) -> (f32, i1, index, f64) {
      %s = arith.mulf %a, %b : f32
      %t = arith.addf %s, %a : f32
      %c = arith.cmpf ogt, %t, %b : f32
      %c1 = arith.constant 1 : index
      %c3 = arith.constant 3 : index
      %m = arith.muli %n, %c3 : index
      %k = arith.subi %m, %c1 : index
      %w = arith.extf %t : f32 to f64
      %r = math.sqrt %w : f64
      return %t, %c, %k, %r : f32, i1, index, f64
    }"""
    e = make(text)
    e.check("scalars")
    a, b = np.float32(1.1), np.float32(3.3)
    t, c, k, r = e.run("scalars", [a, b, 7])
    assert isinstance(t, np.float32) and t == np.float32(a * b) + a and c == bool(t > b) and k == 20
    assert r == float(np.sqrt(np.float64(t)))


def test_operands_whose_sizes_do_not_agree_stop_on_the_host():
    """The kernels take pointers and one element count: a vector that is too short would be read past its end
    on the device, so every size is compared before a call is made."""
    A = spd(30, 7)
    good = csr(A)
    # positions that do not fit the declared number of rows, values that do not fit the coordinates
    with pytest.raises(ValueError, match="positions"):
        ex.Csr(good.pos[:-1], good.crd, good.val, 30, 30)
    with pytest.raises(ValueError, match="values"):
        ex.Csr(good.pos, good.crd, good.val[:-1], 30, 30)
    # x shorter than the matrix has columns; z shorter than the product
    e = make(M.SPMV_THEN_AXPBY)
    with pytest.raises(ValueError, match="30 x 30 matrix times a vector of 29"):
        e.run("residual", [csr(A), vec(np.ones(29)), vec(np.ones(30)), 1.0, 1.0])
    assert "spmv" not in fake_hip.calls
    e = make(M.SPMV_THEN_AXPBY)
    with pytest.raises(ValueError, match="elementwise"):
        e.run("residual", [csr(A), vec(np.ones(30)), vec(np.ones(12)), 1.0, 1.0])
    assert "axpby" not in fake_hip.calls
    # loop-level: a dot over the eight elements of u against a v that holds five
    e = make(loop_nests.DOT)
    with pytest.raises(ValueError, match="shorter buffer"):
        e.run("inner", [vec(np.ones(8)), vec(np.ones(5)), 0.0])
    assert "dot_host" not in fake_hip.calls and "dot" not in fake_hip.calls


def test_host_scalars_follow_ieee_like_the_emitted_code():
    """examples/pcg_solve.py with b = 0: r.r is 0, alpha = 0/0, relres = 0/0.  The emitted C++ computes NaNs and
    leaves the loop after its first pass (NaN > tol is false); host scalars here must do the same, not raise."""
    e = make(M.PCG)
    A = spd(10, 4)
    x, its, relres = e.run("pcg", [csr(A), vec(np.zeros(10)), vec(np.ones(10)), 1e-8, 50])
    assert its == 1 and np.isnan(relres) and np.all(np.isnan(x.numpy()))
    # an integer division by zero has no value to give: it is reported as such
    e = make("""
module {
  func.func @f(%a: index, %b: index) -> index {
    %q = arith.divui %a, %b : index
    return %q : index
  }
}""")
    assert e.run("f", [7, 2]) == [3]
    with pytest.raises(RuntimeError, match="division by zero"):
        e.run("f", [7, 0])
    # an operand of the wrong kind (text that MLIR's verifier would refuse) is named, not leaked as a Python error
    e = make(M.SPMV_THEN_AXPBY.replace("ins(%A, %x", "ins(%A, %a", 1))
    with pytest.raises((RuntimeError, ex.Refused)):
        e.check("residual")
        e.run("residual", [csr(A), vec(np.ones(10)), vec(np.ones(10)), 1.0, 1.0])
