"""What the prebuilt gfx950 module implements, written down as MLIR.

Each entry names a py_<entry> of the module (include/lapis_module.h) and gives, as module text, the
function that entry computes -- the CSR SpMV / SpMM / CG computations of the reference's examples
(examples/spmv_noalloc.py, spmv.py, spmm_dcsr_opdsl.py, pcg_solve.py, multiple_results.py,
hitting_times.py, bspmm.py).  `KokkosBackend.compile` reduces a user's function and these to the
canonical form of lapis_amd/mlir_text.py and binds on equality, so what is bound is decided by what the
function does, never by what it is called.
"""

_HEADER = """
#CSR = #sparse_tensor.encoding<{ map = (i, j) -> (i : dense, j : compressed), posWidth = 32, crdWidth = 32 }>
#CSRV = #sparse_tensor.encoding<{ map = (i, j, k) -> (i : dense, j : compressed, k : dense), posWidth = 32, crdWidth = 32 }>
#same = affine_map<(i) -> (i)>
"""

# y += A x                                                       -> py_spmv / py_spmv_f32
_MATVEC = """
func.func @f(%m: tensor<?x?x{T}, #CSR>, %v: tensor<?x{T}>, %acc: tensor<?x{T}>) -> tensor<?x{T}> {
  %r = linalg.matvec ins(%m, %v : tensor<?x?x{T}, #CSR>, tensor<?x{T}>) outs(%acc : tensor<?x{T}>) -> tensor<?x{T}>
  return %r : tensor<?x{T}>
}
"""

# y = A x with y allocated and zeroed inside (the torch.mv export) -> py_lapis_main
_MV_ALLOC_NAMED = """
func.func @f(%m: tensor<?x?xf64, #CSR>, %v: tensor<?xf64>) -> tensor<?xf64> {
  %i0 = arith.constant 0 : index
  %z = arith.constant 0.0 : f64
  %rows = tensor.dim %m, %i0 : tensor<?x?xf64, #CSR>
  %e = tensor.empty(%rows) : tensor<?xf64>
  %f = linalg.fill ins(%z : f64) outs(%e : tensor<?xf64>) -> tensor<?xf64>
  %r = linalg.matvec ins(%m, %v : tensor<?x?xf64, #CSR>, tensor<?xf64>) outs(%f : tensor<?xf64>) -> tensor<?xf64>
  return %r : tensor<?xf64>
}
"""
_MV_ALLOC_STATIC = """
func.func @f(%m: tensor<5x5xf64, #CSR>, %v: tensor<5xf64>) -> tensor<5xf64> {
  %z = arith.constant 0.0 : f64
  %e = tensor.empty() : tensor<5xf64>
  %f = linalg.fill ins(%z : f64) outs(%e : tensor<5xf64>) -> tensor<5xf64>
  %r = linalg.generic {indexing_maps = [affine_map<(i, j) -> (i, j)>, affine_map<(i, j) -> (j)>, affine_map<(i, j) -> (i)>],
                       iterator_types = ["parallel", "reduction"]}
       ins(%m, %v : tensor<5x5xf64, #CSR>, tensor<5xf64>) outs(%f : tensor<5xf64>) {
    ^bb0(%a: f64, %b: f64, %c: f64):
      %p = arith.mulf %a, %b : f64
      %s = arith.addf %c, %p : f64
      linalg.yield %s : f64
  } -> tensor<5xf64>
  return %r : tensor<5xf64>
}
"""
_MV_ALLOC_STATIC_NAMED = """
func.func @f(%m: tensor<5x5xf64, #CSR>, %v: tensor<5xf64>) -> tensor<5xf64> {
  %z = arith.constant 0.0 : f64
  %e = tensor.empty() : tensor<5xf64>
  %f = linalg.fill ins(%z : f64) outs(%e : tensor<5xf64>) -> tensor<5xf64>
  %r = linalg.matvec ins(%m, %v : tensor<5x5xf64, #CSR>, tensor<5xf64>) outs(%f : tensor<5xf64>) -> tensor<5xf64>
  return %r : tensor<5xf64>
}
"""

# C += A B                                                       -> py_spmm / py_spmm_f64
_MATMUL = """
func.func @f(%m: tensor<?x?x{T}, #CSR>, %b: tensor<?x?x{T}>, %c: tensor<?x?x{T}>) -> tensor<?x?x{T}> {
  %r = linalg.matmul ins(%m, %b : tensor<?x?x{T}, #CSR>, tensor<?x?x{T}>) outs(%c : tensor<?x?x{T}>) -> tensor<?x?x{T}>
  return %r : tensor<?x?x{T}>
}
"""

_VECTOR_HELPERS = """
func.func private @matvec0(%m: tensor<?x?xf64, #CSR>, %v: tensor<?xf64>, %dst: tensor<?xf64>) -> tensor<?xf64> {
  %z = arith.constant 0.0 : f64
  %clean = linalg.fill ins(%z : f64) outs(%dst : tensor<?xf64>) -> tensor<?xf64>
  %r = linalg.matvec ins(%m, %v : tensor<?x?xf64, #CSR>, tensor<?xf64>) outs(%clean : tensor<?xf64>) -> tensor<?xf64>
  return %r : tensor<?xf64>
}
func.func private @inner(%u: tensor<?xf64>, %v: tensor<?xf64>) -> f64 {
  %z = arith.constant 0.0 : f64
  %t = tensor.splat %z[] : tensor<f64>
  %d = linalg.dot ins(%u, %v : tensor<?xf64>, tensor<?xf64>) outs(%t : tensor<f64>) -> tensor<f64>
  %s = tensor.extract %d[] : tensor<f64>
  return %s : f64
}
func.func private @lincomb(%ca: f64, %u: tensor<?xf64>, %cb: f64, %v: tensor<?xf64>, %dst: tensor<?xf64>) -> tensor<?xf64> {
  %r = linalg.generic {indexing_maps = [#same, #same, #same], iterator_types = ["parallel"]}
       ins(%u, %v : tensor<?xf64>, tensor<?xf64>) outs(%dst : tensor<?xf64>) {
    ^bb0(%eu: f64, %ev: f64, %eo: f64):
      %t0 = arith.mulf %eu, %ca : f64
      %t1 = arith.mulf %ev, %cb : f64
      %t2 = arith.addf %t0, %t1 : f64
      linalg.yield %t2 : f64
  } -> tensor<?xf64>
  return %r : tensor<?xf64>
}
func.func private @times(%u: tensor<?xf64>, %v: tensor<?xf64>, %dst: tensor<?xf64>) -> tensor<?xf64> {
  %r = linalg.generic {indexing_maps = [#same, #same, #same], iterator_types = ["parallel"]}
       ins(%u, %v : tensor<?xf64>, tensor<?xf64>) outs(%dst : tensor<?xf64>) {
    ^bb0(%eu: f64, %ev: f64, %eo: f64):
      %t = arith.mulf %eu, %ev : f64
      linalg.yield %t : f64
  } -> tensor<?xf64>
  return %r : tensor<?xf64>
}
"""

# Jacobi-preconditioned CG, x0 = 0; returns (x, iterations, relative residual)   -> py_pcg
_PCG = _VECTOR_HELPERS + """
func.func @f(%m: tensor<?x?xf64, #CSR>, %rhs: tensor<?xf64>, %jac: tensor<?xf64>, %eps: f64, %limit: index)
    -> (tensor<?xf64>, index, f64) {
  %i0 = arith.constant 0 : index
  %i1 = arith.constant 1 : index
  %len = tensor.dim %rhs, %i0 : tensor<?xf64>
  %zero = arith.constant 0.0 : f64
  %one = arith.constant 1.0 : f64
  %w0 = tensor.empty(%len) : tensor<?xf64>
  %w1 = tensor.empty(%len) : tensor<?xf64>
  %w2 = tensor.empty(%len) : tensor<?xf64>
  %res0 = linalg.copy ins(%rhs : tensor<?xf64>) outs(%w0 : tensor<?xf64>) -> tensor<?xf64>
  %pre0 = func.call @times(%res0, %jac, %w1) : (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
  %dir0 = linalg.copy ins(%pre0 : tensor<?xf64>) outs(%w2 : tensor<?xf64>) -> tensor<?xf64>
  %sol0 = tensor.splat %zero[%len] : tensor<?xf64>
  %w3 = tensor.empty(%len) : tensor<?xf64>
  %nn0 = func.call @inner(%res0, %res0) : (tensor<?xf64>, tensor<?xf64>) -> f64
  %norm0 = math.sqrt %nn0 : f64
  %sol, %dir, %pre, %res, %rel, %rho, %count = scf.while (%s = %sol0, %d = %dir0, %q = %pre0, %g = %res0, %rhoOld = %zero, %k = %i1)
      : (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, index)
      -> (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, f64, index) {
    %md = func.call @matvec0(%m, %d, %w3) : (tensor<?x?xf64, #CSR>, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
    %curv = func.call @inner(%d, %md) : (tensor<?xf64>, tensor<?xf64>) -> f64
    %rhoNow = func.call @inner(%g, %q) : (tensor<?xf64>, tensor<?xf64>) -> f64
    %step = arith.divf %rhoNow, %curv : f64
    %back = arith.negf %step : f64
    %s2 = func.call @lincomb(%one, %s, %step, %d, %s) : (f64, tensor<?xf64>, f64, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
    %g2 = func.call @lincomb(%one, %g, %back, %md, %g) : (f64, tensor<?xf64>, f64, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
    %nn = func.call @inner(%g2, %g2) : (tensor<?xf64>, tensor<?xf64>) -> f64
    %norm = math.sqrt %nn : f64
    %ratio = arith.divf %norm, %norm0 : f64
    %above = arith.cmpf ogt, %ratio, %eps : f64
    %room = arith.cmpi ne, %k, %limit : index
    %go = arith.andi %above, %room : i1
    scf.condition(%go) %s2, %d, %q, %g2, %ratio, %rhoNow, %k : tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, f64, index
  } do {
  ^bb0(%s: tensor<?xf64>, %d: tensor<?xf64>, %q: tensor<?xf64>, %g: tensor<?xf64>, %skip: f64, %rhoPrev: f64, %k: index):
    %q2 = func.call @times(%g, %jac, %q) : (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
    %rho2 = func.call @inner(%g, %q2) : (tensor<?xf64>, tensor<?xf64>) -> f64
    %mix = arith.divf %rho2, %rhoPrev : f64
    %d2 = func.call @lincomb(%one, %q2, %mix, %d, %d) : (f64, tensor<?xf64>, f64, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
    %k2 = arith.addi %k, %i1 : index
    scf.yield %s, %d2, %q2, %g, %rho2, %k2 : tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, index
  }
  return %sol, %count, %rel : tensor<?xf64>, index, f64
}
"""

# (x + y, ||x + y||)                                              -> py_plus_norm
_PLUS_NORM = """
func.func @f(%u: tensor<?xf64>, %v: tensor<?xf64>) -> (tensor<?xf64>, f64) {
  %i0 = arith.constant 0 : index
  %len = tensor.dim %v, %i0 : tensor<?xf64>
  %w = tensor.empty(%len) : tensor<?xf64>
  %sum = linalg.add ins(%u, %v : tensor<?xf64>, tensor<?xf64>) outs(%w : tensor<?xf64>) -> tensor<?xf64>
  %t = tensor.empty() : tensor<f64>
  %d = linalg.dot ins(%sum, %sum : tensor<?xf64>, tensor<?xf64>) outs(%t : tensor<f64>) -> tensor<f64>
  %sq = tensor.extract %d[] : tensor<f64>
  %nrm = math.sqrt %sq : f64
  return %sum, %nrm : tensor<?xf64>, f64
}
"""

# first two hitting-time moments: scale A in place, two masked CG solves   -> py_mht
_MHT = _VECTOR_HELPERS + """
func.func private @rescale(%m: tensor<?x?xf64, #CSR>, %factor: f64) -> tensor<?x?xf64, #CSR> {
  %r = linalg.generic {indexing_maps = [affine_map<(i, j) -> (i, j)>], iterator_types = ["parallel", "parallel"]}
       outs(%m : tensor<?x?xf64, #CSR>) {
    ^bb0(%e: f64):
      %t = sparse_tensor.unary %e : f64 to f64
        present = {
          ^bb1(%stored: f64):
            %scaled = arith.mulf %stored, %factor : f64
            sparse_tensor.yield %scaled : f64
        }
        absent = {}
      linalg.yield %t : f64
  } -> tensor<?x?xf64, #CSR>
  return %r : tensor<?x?xf64, #CSR>
}
func.func private @masked_laplacian(%m: tensor<?x?xf64, #CSR>, %v: tensor<?xf64>, %deg: tensor<?xf64>, %sel: tensor<?xf64>,
                                    %scratch: tensor<?xf64>, %dst: tensor<?xf64>) -> tensor<?xf64> {
  %sv = func.call @times(%v, %sel, %scratch) : (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
  %msv = func.call @matvec0(%m, %sv, %dst) : (tensor<?x?xf64, #CSR>, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
  %r = linalg.generic {indexing_maps = [#same, #same, #same, #same, #same], iterator_types = ["parallel"]}
       ins(%msv, %sv, %sel, %deg : tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>) outs(%dst : tensor<?xf64>) {
    ^bb0(%e0: f64, %e1: f64, %e2: f64, %e3: f64, %eo: f64):
      %t0 = arith.mulf %e3, %e1 : f64
      %t1 = arith.subf %t0, %e0 : f64
      %t2 = arith.mulf %t1, %e2 : f64
      linalg.yield %t2 : f64
  } -> tensor<?xf64>
  return %r : tensor<?xf64>
}
func.func private @masked_cg(%m: tensor<?x?xf64, #CSR>, %rhs: tensor<?xf64>, %sel: tensor<?xf64>, %deg: tensor<?xf64>, %eps: f64,
                             %limit: index) -> (tensor<?xf64>, index, f64) {
  %i0 = arith.constant 0 : index
  %i1 = arith.constant 1 : index
  %len = tensor.dim %rhs, %i0 : tensor<?xf64>
  %zero = arith.constant 0.0 : f64
  %one = arith.constant 1.0 : f64
  %scratch = tensor.empty(%len) : tensor<?xf64>
  %w0 = tensor.empty(%len) : tensor<?xf64>
  %w1 = tensor.empty(%len) : tensor<?xf64>
  %w2 = tensor.empty(%len) : tensor<?xf64>
  %res0 = linalg.copy ins(%rhs : tensor<?xf64>) outs(%w0 : tensor<?xf64>) -> tensor<?xf64>
  %pre0 = linalg.div ins(%res0, %deg : tensor<?xf64>, tensor<?xf64>) outs(%w1 : tensor<?xf64>) -> tensor<?xf64>
  %dir0 = linalg.copy ins(%pre0 : tensor<?xf64>) outs(%w2 : tensor<?xf64>) -> tensor<?xf64>
  %sol0 = tensor.splat %zero[%len] : tensor<?xf64>
  %w3 = tensor.empty(%len) : tensor<?xf64>
  %nn0 = func.call @inner(%res0, %res0) : (tensor<?xf64>, tensor<?xf64>) -> f64
  %norm0 = math.sqrt %nn0 : f64
  %sol, %dir, %pre, %res, %rel, %rho, %count = scf.while (%s = %sol0, %d = %dir0, %q = %pre0, %g = %res0, %rhoOld = %zero, %k = %i1)
      : (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, index)
      -> (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, f64, index) {
    %md = func.call @masked_laplacian(%m, %d, %deg, %sel, %scratch, %w3)
        : (tensor<?x?xf64, #CSR>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
    %curv = func.call @inner(%d, %md) : (tensor<?xf64>, tensor<?xf64>) -> f64
    %rhoNow = func.call @inner(%g, %q) : (tensor<?xf64>, tensor<?xf64>) -> f64
    %step = arith.divf %rhoNow, %curv : f64
    %back = arith.negf %step : f64
    %s2 = func.call @lincomb(%one, %s, %step, %d, %s) : (f64, tensor<?xf64>, f64, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
    %g2 = func.call @lincomb(%one, %g, %back, %md, %g) : (f64, tensor<?xf64>, f64, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
    %nn = func.call @inner(%g2, %g2) : (tensor<?xf64>, tensor<?xf64>) -> f64
    %norm = math.sqrt %nn : f64
    %ratio = arith.divf %norm, %norm0 : f64
    %above = arith.cmpf ogt, %ratio, %eps : f64
    %room = arith.cmpi ne, %k, %limit : index
    %go = arith.andi %above, %room : i1
    scf.condition(%go) %s2, %d, %q, %g2, %ratio, %rhoNow, %k : tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, f64, index
  } do {
  ^bb0(%s: tensor<?xf64>, %d: tensor<?xf64>, %q: tensor<?xf64>, %g: tensor<?xf64>, %skip: f64, %rhoPrev: f64, %k: index):
    %q2 = linalg.div ins(%g, %deg : tensor<?xf64>, tensor<?xf64>) outs(%q : tensor<?xf64>) -> tensor<?xf64>
    %rho2 = func.call @inner(%g, %q2) : (tensor<?xf64>, tensor<?xf64>) -> f64
    %mix = arith.divf %rho2, %rhoPrev : f64
    %d2 = func.call @lincomb(%one, %q2, %mix, %d, %d) : (f64, tensor<?xf64>, f64, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
    %k2 = arith.addi %k, %i1 : index
    scf.yield %s, %d2, %q2, %g, %rho2, %k2 : tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, index
  }
  return %sol, %count, %rel : tensor<?xf64>, index, f64
}
func.func @f(%m: tensor<?x?xf64, #CSR>, %sel: tensor<?xf64>, %deg: tensor<?xf64>, %factor: f64, %eps: f64, %limit: index)
    -> (tensor<?xf64>, tensor<?xf64>) {
  %i0 = arith.constant 0 : index
  %ms = func.call @rescale(%m, %factor) : (tensor<?x?xf64, #CSR>, f64) -> tensor<?x?xf64, #CSR>
  %len = tensor.dim %deg, %i0 : tensor<?xf64>
  %w = tensor.empty(%len) : tensor<?xf64>
  %rhs1 = func.call @times(%deg, %sel, %w) : (tensor<?xf64>, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
  %first, %n1, %r1 = func.call @masked_cg(%ms, %rhs1, %sel, %deg, %eps, %limit)
      : (tensor<?x?xf64, #CSR>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, index) -> (tensor<?xf64>, index, f64)
  %mf = func.call @matvec0(%ms, %first, %w) : (tensor<?x?xf64, #CSR>, tensor<?xf64>, tensor<?xf64>) -> tensor<?xf64>
  %rhs2 = linalg.generic {indexing_maps = [#same, #same, #same, #same, #same], iterator_types = ["parallel"]}
          ins(%mf, %sel, %first, %deg : tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>) outs(%w : tensor<?xf64>) {
    ^bb0(%e0: f64, %e1: f64, %e2: f64, %e3: f64, %eo: f64):
      %t0 = arith.mulf %e3, %e2 : f64
      %t1 = arith.addf %t0, %e0 : f64
      %t2 = arith.mulf %t1, %e1 : f64
      linalg.yield %t2 : f64
  } -> tensor<?xf64>
  %second, %n2, %r2 = func.call @masked_cg(%ms, %rhs2, %sel, %deg, %eps, %limit)
      : (tensor<?x?xf64, #CSR>, tensor<?xf64>, tensor<?xf64>, tensor<?xf64>, f64, index) -> (tensor<?xf64>, index, f64)
  return %first, %second : tensor<?xf64>, tensor<?xf64>
}
"""

# sqrt(mom2 - mom1^2)                                             -> py_normalize_mom2
_NORMALIZE = """
func.func @f(%first: tensor<?xf64>, %second: tensor<?xf64>) -> tensor<?xf64> {
  %i0 = arith.constant 0 : index
  %len = tensor.dim %first, %i0 : tensor<?xf64>
  %w = tensor.empty(%len) : tensor<?xf64>
  %r = linalg.generic {indexing_maps = [#same, #same, #same], iterator_types = ["parallel"]}
       ins(%first, %second : tensor<?xf64>, tensor<?xf64>) outs(%w : tensor<?xf64>) {
    ^bb0(%e0: f64, %e1: f64, %eo: f64):
      %sq = arith.mulf %e0, %e0 : f64
      %var = arith.subf %e1, %sq : f64
      %dev = math.sqrt %var : f64
      linalg.yield %dev : f64
  } -> tensor<?xf64>
  return %r : tensor<?xf64>
}
"""

# out(n1, dh, nh) = sum_n2 A(n1, n2, nh) * V(n2, dh, nh), A in CSRV        -> py_pte_local_bspmm
_BSPMM = """
func.func @f(%att: tensor<?x?x?xf32, #CSRV>, %val: tensor<?x?x?xf32>) -> tensor<?x?x?xf32> {
  %i0 = arith.constant 0 : index
  %i1 = arith.constant 1 : index
  %i2 = arith.constant 2 : index
  %z = arith.constant 0.0 : f32
  %d0 = tensor.dim %att, %i0 : tensor<?x?x?xf32, #CSRV>
  %d1 = tensor.dim %att, %i1 : tensor<?x?x?xf32, #CSRV>
  %d2 = tensor.dim %att, %i2 : tensor<?x?x?xf32, #CSRV>
  %d3 = tensor.dim %val, %i1 : tensor<?x?x?xf32>
  %e = tensor.empty(%d0, %d3, %d2) : tensor<?x?x?xf32>
  %f = linalg.fill ins(%z : f32) outs(%e : tensor<?x?x?xf32>) -> tensor<?x?x?xf32>
  %r = linalg.generic {indexing_maps = [affine_map<(a, b, c, d) -> (a, b, d)>, affine_map<(a, b, c, d) -> (b, c, d)>,
                                        affine_map<(a, b, c, d) -> (a, c, d)>],
                       iterator_types = ["parallel", "parallel", "reduction", "parallel"]}
       ins(%att, %val : tensor<?x?x?xf32, #CSRV>, tensor<?x?x?xf32>) outs(%f : tensor<?x?x?xf32>) {
    ^bb0(%x: f32, %y: f32, %o: f32):
      %p = arith.mulf %x, %y : f32
      %s = arith.addf %p, %o : f32
      linalg.yield %s : f32
  } -> tensor<?x?x?xf32>
  return %r : tensor<?x?x?xf32>
}
"""


def entries():
    """(entry point of the prebuilt module, module text whose function @f is what it computes)."""
    out = []
    for ty in ("f64", "f32"):
        out.append(("spmv", _HEADER + _MATVEC.replace("{T}", ty)))
        out.append(("spmm", _HEADER + _MATMUL.replace("{T}", ty)))
    for text in (_MV_ALLOC_NAMED, _MV_ALLOC_STATIC, _MV_ALLOC_STATIC_NAMED):
        out.append(("lapis_main", _HEADER + text))
    out.append(("pcg", _HEADER + _PCG))
    out.append(("plus_norm", _HEADER + _PLUS_NORM))
    out.append(("mht", _HEADER + _MHT))
    out.append(("normalize_mom2", _HEADER + _NORMALIZE))
    out.append(("pte_local_bspmm", _HEADER + _BSPMM))
    return out
