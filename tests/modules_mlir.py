"""Module texts fed to KokkosBackend.compile by the tests: the computations of the reference's examples
(examples/spmv_noalloc.py:6-15, examples/pcg_solve.py:9-103), typed out with names of their own."""

SPMV = """
#sparse = #sparse_tensor.encoding<{ map = (d0, d1) -> (d0 : dense, d1 : compressed), posWidth = 32, crdWidth = 32 }>
module {
  func.func @spmv(%A: tensor<?x?xf64, #sparse>, %x: tensor<?xf64>, %y: tensor<?xf64>) -> tensor<?xf64> {
    // y += A x
    %0 = linalg.matvec ins(%A, %x: tensor<?x?xf64, #sparse>, tensor<?xf64>) outs(%y : tensor<?xf64>) -> tensor<?xf64>
    return %0 : tensor<?xf64>
  }
}"""

# the same product under another name, with the encoding written inline and other value names
MATVEC_OTHER_NAME = """
module {
  func.func @apply_operator(%op: tensor<?x?xf64, #sparse_tensor.encoding<{ map = (r, c) -> (r : dense, c : compressed), posWidth = 32, crdWidth = 32 }>>,
                            %in: tensor<?xf64>, %inout: tensor<?xf64>) -> tensor<?xf64> {
    %res = linalg.matvec ins(%op, %in : tensor<?x?xf64, #sparse_tensor.encoding<{ map = (r, c) -> (r : dense, c : compressed), posWidth = 32, crdWidth = 32 }>>, tensor<?xf64>)
                         outs(%inout : tensor<?xf64>) -> tensor<?xf64>
    return %res : tensor<?xf64>
  }
}"""

# right name, wrong computation: x^T A
SPMV_TRANSPOSED = """
#sparse = #sparse_tensor.encoding<{ map = (d0, d1) -> (d0 : dense, d1 : compressed), posWidth = 32, crdWidth = 32 }>
module {
  func.func @spmv(%A: tensor<?x?xf64, #sparse>, %x: tensor<?xf64>, %y: tensor<?xf64>) -> tensor<?xf64> {
    %0 = linalg.vecmat ins(%x, %A: tensor<?xf64>, tensor<?x?xf64, #sparse>) outs(%y : tensor<?xf64>) -> tensor<?xf64>
    return %0 : tensor<?xf64>
  }
}"""

# right name and operation, but the operand is stored by columns
SPMV_CSC = SPMV.replace("(d0 : dense, d1 : compressed)", "(d1 : dense, d0 : compressed)")

# 64-bit positions: the module takes int32 buffers
SPMV_WIDE_INDEX = SPMV.replace("posWidth = 32", "posWidth = 64")

PCG = """
#CSR = #sparse_tensor.encoding<{ map = (d0, d1) -> (d0 : dense, d1 : compressed), posWidth = 32, crdWidth = 32 }>
#id = affine_map<(d0) -> (d0)>
module {
  func.func private @apply(%A: tensor<?x?xf64, #CSR>, %v: tensor<?xf64>, %out: tensor<?xf64>) -> tensor<?xf64> {
    %c = arith.constant 0.0 : f64
    %clean = linalg.fill ins(%c : f64) outs(%out : tensor<?xf64>) -> tensor<?xf64>
    %Av = linalg.matvec ins(%A, %v: tensor<?x?xf64, #CSR>, tensor<?xf64>) outs(%clean : tensor<?xf64>) -> tensor<?xf64>
    return %Av : tensor<?xf64>
  }
  func.func private @dotp(%a: tensor<?xf64>, %b: tensor<?xf64>) -> f64 {
    %c = arith.constant 0.0 : f64
    %acc = tensor.splat %c[] : tensor<f64>
    %d = linalg.dot ins(%a, %b : tensor<?xf64>, tensor<?xf64>) outs(%acc : tensor<f64>) -> tensor<f64>
    %s = tensor.extract %d[] : tensor<f64>
    return %s : f64
  }
  func.func private @combine(%alpha: f64, %a: tensor<?xf64>, %beta: f64, %b: tensor<?xf64>, %out: tensor<?xf64>) -> tensor<?xf64> {
    %r = linalg.generic {indexing_maps = [#id, #id, #id], iterator_types = ["parallel"]}
         ins(%a, %b : tensor<?xf64>, tensor<?xf64>) outs(%out : tensor<?xf64>) {
      ^bb0(%ea: f64, %eb: f64, %eo: f64):
        %l = arith.mulf %ea, %alpha : f64
        %m = arith.mulf %eb, %beta : f64
        %n = arith.addf %l, %m : f64
        linalg.yield %n : f64
    } -> tensor<?xf64>
    return %r : tensor<?xf64>
  }
  func.func private @hadamard(%a: tensor<?xf64>, %b: tensor<?xf64>, %out: tensor<?xf64>) -> tensor<?xf64> {
    %r = linalg.generic {indexing_maps = [#id, #id, #id], iterator_types = ["parallel"]}
         ins(%a, %b : tensor<?xf64>, tensor<?xf64>) outs(%out : tensor<?xf64>) {
      ^bb0(%ea: f64, %eb: f64, %eo: f64):
        %l = arith.mulf %ea, %eb : f64
        linalg.yield %l : f64
    } -> tensor<?xf64>
    return %r : tensor<?xf64>
  }
  // Jacobi-preconditioned conjugate gradients from a zero initial guess
  func.func @pcg(%A: tensor<?x?xf64, #CSR>, %b: tensor<?xf64>, %dinv: tensor<?xf64>, %tol: f64, %maxiter: index)
      -> (tensor<?xf64>, index, f64) {
    %c0 = arith.constant 0 : index
    %c1 = arith.constant 1 : index
    %n = tensor.dim %b, %c0 : tensor<?xf64>
    %f0 = arith.constant 0.0 : f64
    %f1 = arith.constant 1.0 : f64
    %t0 = tensor.empty(%n) : tensor<?xf64>
    %t1 = tensor.empty(%n) : tensor<?xf64>
    %t2 = tensor.empty(%n) : tensor<?xf64>
    %r0 = linalg.copy ins(%b : tensor<?xf64>) outs(%t0 : tensor<?xf64>) -> tensor<?xf64>
    %z0 = func.call @hadamard(%r0, %dinv, %t1) : (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
    %p0 = linalg.copy ins(%z0 : tensor<?xf64>) outs(%t2 : tensor<?xf64>) -> tensor<?xf64>
    %x0 = tensor.splat %f0[%n] : tensor<?xf64>
    %t3 = tensor.empty(%n) : tensor<?xf64>
    %rr0 = func.call @dotp(%r0, %r0) : (tensor<?xf64>, tensor<?xf64>) -> f64
    %nrm0 = math.sqrt %rr0 : f64
    %x, %p, %z, %r, %relres, %rz, %its = scf.while (%xi = %x0, %pi = %p0, %zi = %z0, %ri = %r0, %rzi = %f0, %i = %c1)
        : (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, index)
        -> (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, f64, index) {
      %Ap = func.call @apply(%A, %pi, %t3) : (tensor<?x?xf64, #CSR>, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
      %pAp = func.call @dotp(%pi, %Ap) : (tensor<?xf64>, tensor<?xf64>) -> f64
      %rznow = func.call @dotp(%ri, %zi) : (tensor<?xf64>, tensor<?xf64>) -> f64
      %alpha = arith.divf %rznow, %pAp : f64
      %nalpha = arith.negf %alpha : f64
      %xn = func.call @combine(%f1, %xi, %alpha, %pi, %xi) : (f64, tensor<?xf64>, f64, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
      %rn = func.call @combine(%f1, %ri, %nalpha, %Ap, %ri) : (f64, tensor<?xf64>, f64, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
      %rr = func.call @dotp(%rn, %rn) : (tensor<?xf64>, tensor<?xf64>) -> f64
      %nrm = math.sqrt %rr : f64
      %rel = arith.divf %nrm, %nrm0 : f64
      %open = arith.cmpf ogt, %rel, %tol : f64
      %more = arith.cmpi ne, %i, %maxiter : index
      %again = arith.andi %open, %more : i1
      scf.condition(%again) %xn, %pi, %zi, %rn, %rel, %rznow, %i : tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, f64, index
    } do {
    ^bb0(%xi: tensor<?xf64>, %pi: tensor<?xf64>, %zi: tensor<?xf64>, %ri: tensor<?xf64>, %ignored: f64, %rzold: f64, %i: index):
      %zn = func.call @hadamard(%ri, %dinv, %zi) : (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
      %rzn = func.call @dotp(%ri, %zn) : (tensor<?xf64>, tensor<?xf64>) -> f64
      %beta = arith.divf %rzn, %rzold : f64
      %pn = func.call @combine(%f1, %zn, %beta, %pi, %pi) : (f64, tensor<?xf64>, f64, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
      %in = arith.addi %i, %c1 : index
      scf.yield %xi, %pn, %zn, %ri, %rzn, %in : tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, index
    }
    return %x, %its, %relres : tensor<?xf64>, index, f64
  }
}"""

# the same loop with the update of x using -alpha: another iteration, refused
PCG_WRONG_SIGN = PCG.replace("@combine(%f1, %xi, %alpha, %pi, %xi)", "@combine(%f1, %xi, %nalpha, %pi, %xi)")

BSPMM = """
#csrv = #sparse_tensor.encoding<{ map = (d0, d1, d2) -> (d0 : dense, d1 : compressed, d2 : dense), posWidth = 32, crdWidth = 32}>
module {
  func.func @pte_local_bspmm(%A: tensor<?x?x?xf32, #csrv>,
    %B: tensor<?x?x?xf32>) ->  tensor<?x?x?xf32>
  {
    %i0 = arith.constant 0 : index
    %i1 = arith.constant 1 : index
    %i2 = arith.constant 2 : index
    %zero = arith.constant 0.0 : f32
    %n1 = tensor.dim %A, %i0 : tensor<?x?x?xf32, #csrv>
    %n2 = tensor.dim %A, %i1 : tensor<?x?x?xf32, #csrv>
    %nh = tensor.dim %A, %i2 : tensor<?x?x?xf32, #csrv>
    %dh = tensor.dim %B, %i1 : tensor<?x?x?xf32>
    %e = tensor.empty (%n1, %dh, %nh) : tensor<?x?x?xf32>
    %f = linalg.fill ins(%zero: f32)
      outs(%e : tensor<?x?x?xf32>)
      -> tensor<?x?x?xf32>
    %out = linalg.generic {
        indexing_maps = [affine_map<(n1, n2, dh, nh) -> (n1, n2, nh)>,
                         affine_map<(n1, n2, dh, nh) -> (n2, dh, nh)>,
                         affine_map<(n1, n2, dh, nh) -> (n1, dh, nh)>],
        iterator_types = ["parallel", "parallel", "reduction", "parallel"]}
      ins(%A, %B: tensor<?x?x?xf32, #csrv>, tensor<?x?x?xf32>)
      outs(%f: tensor<?x?x?xf32>) {
      ^bb0(%a: f32, %b: f32, %c: f32):
        %0 = arith.mulf %a, %b : f32
        %1 = arith.addf %0, %c: f32
        linalg.yield %1 : f32
    } -> tensor<?x?x?xf32>
    return %out : tensor<?x?x?xf32>
  }
  func.func @print_csrv(%A: tensor<?x?x?xf32, #csrv>)
  {
    sparse_tensor.print %A : tensor<?x?x?xf32, #csrv>
    return
  }
}"""

# ---- functions no whole-function entry point exists for: bound operation by operation ----------------------

# an SpMV followed by an axpby: alpha * (A x) + beta * z
SPMV_THEN_AXPBY = """
#CSR = #sparse_tensor.encoding<{ map = (d0, d1) -> (d0 : dense, d1 : compressed), posWidth = 32, crdWidth = 32 }>
#id = affine_map<(d0) -> (d0)>
module {
  func.func @residual(%A: tensor<?x?xf64, #CSR>, %x: tensor<?xf64>, %z: tensor<?xf64>, %alpha: f64, %beta: f64) -> tensor<?xf64> {
    %c0 = arith.constant 0 : index
    %rows = tensor.dim %A, %c0 : tensor<?x?xf64, #CSR>
    %f0 = arith.constant 0.0 : f64
    %e = tensor.empty(%rows) : tensor<?xf64>
    %clean = linalg.fill ins(%f0 : f64) outs(%e : tensor<?xf64>) -> tensor<?xf64>
    %Ax = linalg.matvec ins(%A, %x : tensor<?x?xf64, #CSR>, tensor<?xf64>) outs(%clean : tensor<?xf64>) -> tensor<?xf64>
    %e2 = tensor.empty(%rows) : tensor<?xf64>
    %out = linalg.generic {indexing_maps = [#id, #id, #id], iterator_types = ["parallel"]}
        ins(%Ax, %z : tensor<?xf64>, tensor<?xf64>) outs(%e2 : tensor<?xf64>) {
      ^bb0(%a: f64, %b: f64, %o: f64):
        %l = arith.mulf %alpha, %a : f64
        %m = arith.mulf %beta, %b : f64
        %s = arith.addf %l, %m : f64
        linalg.yield %s : f64
    } -> tensor<?xf64>
    return %out : tensor<?xf64>
  }
}"""

# unpreconditioned CG from x = 0 whose residual update r - alpha*Ap is ONE generic with a subtraction, and whose
# direction update reads its own output operand
CG_FUSED_UPDATE = """
#CSR = #sparse_tensor.encoding<{ map = (d0, d1) -> (d0 : dense, d1 : compressed), posWidth = 32, crdWidth = 32 }>
#id = affine_map<(d0) -> (d0)>
module {
  func.func private @inner(%a: tensor<?xf64>, %b: tensor<?xf64>) -> f64 {
    %c = arith.constant 0.0 : f64
    %acc = tensor.splat %c[] : tensor<f64>
    %d = linalg.dot ins(%a, %b : tensor<?xf64>, tensor<?xf64>) outs(%acc : tensor<f64>) -> tensor<f64>
    %s = tensor.extract %d[] : tensor<f64>
    return %s : f64
  }
  func.func @cg(%A: tensor<?x?xf64, #CSR>, %b: tensor<?xf64>, %tol: f64, %maxiter: index) -> (tensor<?xf64>, index, f64) {
    %c0 = arith.constant 0 : index
    %c1 = arith.constant 1 : index
    %f0 = arith.constant 0.0 : f64
    %n = tensor.dim %b, %c0 : tensor<?xf64>
    %x0 = tensor.splat %f0[%n] : tensor<?xf64>
    %e0 = tensor.empty(%n) : tensor<?xf64>
    %p0 = linalg.copy ins(%b : tensor<?xf64>) outs(%e0 : tensor<?xf64>) -> tensor<?xf64>
    %bb = func.call @inner(%b, %b) : (tensor<?xf64>, tensor<?xf64>) -> f64
    %bnorm = math.sqrt %bb : f64
    %x, %r, %p, %rr, %its = scf.while (%xi = %x0, %ri = %b, %pi = %p0, %rri = %bb, %i = %c0)
        : (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, index) -> (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, index) {
      %nrm = math.sqrt %rri : f64
      %rel = arith.divf %nrm, %bnorm : f64
      %open = arith.cmpf ogt, %rel, %tol : f64
      %more = arith.cmpi slt, %i, %maxiter : index
      %go = arith.andi %open, %more : i1
      scf.condition(%go) %xi, %ri, %pi, %rri, %i : tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, index
    } do {
    ^bb0(%xi: tensor<?xf64>, %ri: tensor<?xf64>, %pi: tensor<?xf64>, %rri: f64, %i: index):
      %e1 = tensor.empty(%n) : tensor<?xf64>
      %z = linalg.fill ins(%f0 : f64) outs(%e1 : tensor<?xf64>) -> tensor<?xf64>
      %Ap = linalg.matvec ins(%A, %pi : tensor<?x?xf64, #CSR>, tensor<?xf64>) outs(%z : tensor<?xf64>) -> tensor<?xf64>
      %pAp = func.call @inner(%pi, %Ap) : (tensor<?xf64>, tensor<?xf64>) -> f64
      %alpha = arith.divf %rri, %pAp : f64
      %xn = linalg.generic {indexing_maps = [#id, #id], iterator_types = ["parallel"]}
          ins(%pi : tensor<?xf64>) outs(%xi : tensor<?xf64>) {
        ^bb0(%pe: f64, %xe: f64):
          %t = arith.mulf %alpha, %pe : f64
          %u = arith.addf %xe, %t : f64
          linalg.yield %u : f64
      } -> tensor<?xf64>
      %rn = linalg.generic {indexing_maps = [#id, #id, #id], iterator_types = ["parallel"]}
          ins(%ri, %Ap : tensor<?xf64>, tensor<?xf64>) outs(%e1 : tensor<?xf64>) {
        ^bb0(%re: f64, %ae: f64, %oe: f64):
          %t = arith.mulf %alpha, %ae : f64
          %u = arith.subf %re, %t : f64
          linalg.yield %u : f64
      } -> tensor<?xf64>
      %rrn = func.call @inner(%rn, %rn) : (tensor<?xf64>, tensor<?xf64>) -> f64
      %beta = arith.divf %rrn, %rri : f64
      %pn = linalg.generic {indexing_maps = [#id, #id], iterator_types = ["parallel"]}
          ins(%rn : tensor<?xf64>) outs(%pi : tensor<?xf64>) {
        ^bb0(%re: f64, %pe: f64):
          %t = arith.mulf %beta, %pe : f64
          %u = arith.addf %re, %t : f64
          linalg.yield %u : f64
      } -> tensor<?xf64>
      %in = arith.addi %i, %c1 : index
      scf.yield %xn, %rn, %pn, %rrn, %in : tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, index
    }
    %nrm = math.sqrt %rr : f64
    %relres = arith.divf %nrm, %bnorm : f64
    return %x, %its, %relres : tensor<?xf64>, index, f64
  }
}"""

# Richardson iteration x <- x + omega (b - A x), a fixed number of sweeps, with named elementwise operations
RICHARDSON = """
#CSR = #sparse_tensor.encoding<{ map = (d0, d1) -> (d0 : dense, d1 : compressed), posWidth = 32, crdWidth = 32 }>
#id = affine_map<(d0) -> (d0)>
module {
  func.func @richardson(%A: tensor<?x?xf64, #CSR>, %b: tensor<?xf64>, %x0: tensor<?xf64>, %omega: f64, %sweeps: index) -> tensor<?xf64> {
    %c0 = arith.constant 0 : index
    %c1 = arith.constant 1 : index
    %f0 = arith.constant 0.0 : f64
    %n = tensor.dim %b, %c0 : tensor<?xf64>
    %x = scf.for %k = %c0 to %sweeps step %c1 iter_args(%xk = %x0) -> (tensor<?xf64>) {
      %e = tensor.empty(%n) : tensor<?xf64>
      %z = linalg.fill ins(%f0 : f64) outs(%e : tensor<?xf64>) -> tensor<?xf64>
      %Ax = linalg.matvec ins(%A, %xk : tensor<?x?xf64, #CSR>, tensor<?xf64>) outs(%z : tensor<?xf64>) -> tensor<?xf64>
      %e2 = tensor.empty(%n) : tensor<?xf64>
      %res = linalg.sub ins(%b, %Ax : tensor<?xf64>, tensor<?xf64>) outs(%e2 : tensor<?xf64>) -> tensor<?xf64>
      %e3 = tensor.empty(%n) : tensor<?xf64>
      %xn = linalg.generic {indexing_maps = [#id, #id, #id], iterator_types = ["parallel"]}
          ins(%xk, %res : tensor<?xf64>, tensor<?xf64>) outs(%e3 : tensor<?xf64>) {
        ^bb0(%xe: f64, %re: f64, %oe: f64):
          %t = arith.mulf %omega, %re : f64
          %u = arith.addf %xe, %t : f64
          linalg.yield %u : f64
      } -> tensor<?xf64>
      scf.yield %xn : tensor<?xf64>
    }
    return %x : tensor<?xf64>
  }
}"""

# two products in a row, y = A (A x), and a function whose operand it must not overwrite: %x is used again
TWO_PRODUCTS = """
#CSR = #sparse_tensor.encoding<{ map = (d0, d1) -> (d0 : dense, d1 : compressed), posWidth = 32, crdWidth = 32 }>
module {
  func.func @twice_plus(%A: tensor<?x?xf64, #CSR>, %x: tensor<?xf64>) -> (tensor<?xf64>, tensor<?xf64>) {
    %Ax = linalg.matvec ins(%A, %x : tensor<?x?xf64, #CSR>, tensor<?xf64>) outs(%x : tensor<?xf64>) -> tensor<?xf64>
    %AAx = linalg.matvec ins(%A, %Ax : tensor<?x?xf64, #CSR>, tensor<?xf64>) outs(%x : tensor<?xf64>) -> tensor<?xf64>
    return %Ax, %AAx : tensor<?xf64>, tensor<?xf64>
  }
}"""

# the CSR x dense product written as a generic (the form of examples/spmm_dcsr_opdsl.py), scaled afterwards
SPMM_GENERIC_SCALED = """
#CSR = #sparse_tensor.encoding<{ map = (d0, d1) -> (d0 : dense, d1 : compressed), posWidth = 32, crdWidth = 32 }>
#id2 = affine_map<(d0, d1) -> (d0, d1)>
module {
  func.func @scaled_product(%A: tensor<?x?xf32, #CSR>, %B: tensor<?x?xf32>, %C: tensor<?x?xf32>, %s: f32) -> tensor<?x?xf32> {
    %AB = linalg.generic {
        indexing_maps = [affine_map<(i, j, k) -> (i, k)>, affine_map<(i, j, k) -> (k, j)>, affine_map<(i, j, k) -> (i, j)>],
        iterator_types = ["parallel", "parallel", "reduction"]}
        ins(%A, %B : tensor<?x?xf32, #CSR>, tensor<?x?xf32>) outs(%C : tensor<?x?xf32>) {
      ^bb0(%a: f32, %b: f32, %c: f32):
        %p = arith.mulf %a, %b : f32
        %q = arith.addf %c, %p : f32
        linalg.yield %q : f32
    } -> tensor<?x?xf32>
    %out = linalg.generic {indexing_maps = [#id2, #id2], iterator_types = ["parallel", "parallel"]}
        ins(%AB : tensor<?x?xf32>) outs(%AB : tensor<?x?xf32>) {
      ^bb0(%e: f32, %o: f32):
        %t = arith.mulf %e, %s : f32
        linalg.yield %t : f32
    } -> tensor<?x?xf32>
    return %out : tensor<?x?xf32>
  }
}"""

# the same conjugate gradients in single precision
PCG_F32 = PCG.replace("f64", "f32")

# an operation outside the vocabulary between two that are inside it
SPMV_THEN_EXP = SPMV_THEN_AXPBY.replace("%s = arith.addf %l, %m : f64", "%s0 = arith.addf %l, %m : f64\n        %s = math.exp %s0 : f64")
