"""`scf.parallel` nests typed out with names of their own, in the shapes the reference's loop-mapping tests
cover (tests/Dialect/Kokkos/loop_mapping_{0,1,2,3}.mlir): a host-only two-dimensional loop, a one-level
reduction, the CSR SpMV nest and a four-deep reduction nest.  `tests/golden/loop_mapping_expected.json` holds
what the reference's gold files say those four shapes map to."""

# two induction variables; allocates inside, so it has to stay on the host       (shape of loop_mapping_0)
HOST_2D = """
module {
  func.func @scratch_per_point(%cube: memref<?x?x?xf64>, %idx: memref<?xindex>, %a: memref<?xf64>, %b: memref<?xf64>, %cols: index) {
    %zero = arith.constant 0 : index
    %one = arith.constant 1 : index
    %five = arith.constant 5 : index
    scf.parallel (%r, %c) = (%zero, %zero) to (%five, %cols) step (%one, %one) {
      %buf = memref.alloc(%five) : memref<?xf32>
      %pi = arith.constant 3.14159 : f32
      scf.for %t = %zero to %five step %one {
        memref.store %pi, %buf[%t] : memref<?xf32>
        scf.yield
      }
      scf.reduce
    }
    return
  }
}
"""

# one level, a sum                                                               (shape of loop_mapping_1)
COUNT = """
module {
  func.func @count(%n: index) -> index {
    %zero = arith.constant 0 : index
    %one = arith.constant 1 : index
    %total = scf.parallel (%i) = (%zero) to (%n) step (%one) init (%zero) -> index {
      scf.reduce(%one : index) {
      ^bb0(%lhs: index, %rhs: index):
        %s = arith.addi %lhs, %rhs : index
        scf.reduce.return %s : index
      }
    }
    return %total : index
  }
}
"""

# rows in parallel, the entries of a row reduced                                 (shape of loop_mapping_2)
SPMV_INDEX = """
module {
  func.func @rowsum(%y: memref<?xf64>, %rowptr: memref<?xindex>, %colidx: memref<?xindex>, %vals: memref<?xf64>, %x: memref<?xf64>) {
    %zero = arith.constant 0 : index
    %one = arith.constant 1 : index
    %rows = memref.dim %y, %zero : memref<?xf64>
    scf.parallel (%row) = (%zero) to (%rows) step (%one) {
      %acc0 = memref.load %y[%row] : memref<?xf64>
      %first = memref.load %rowptr[%row] : memref<?xindex>
      %next = arith.addi %row, %one : index
      %last = memref.load %rowptr[%next] : memref<?xindex>
      %len = arith.subi %last, %first : index
      %sum = scf.parallel (%k) = (%zero) to (%len) step (%one) init (%acc0) -> f64 {
        %e = arith.addi %first, %k : index
        %col = memref.load %colidx[%e] : memref<?xindex>
        %a = memref.load %vals[%e] : memref<?xf64>
        %xv = memref.load %x[%col] : memref<?xf64>
        %p = arith.mulf %a, %xv : f64
        scf.reduce(%p : f64) {
        ^bb0(%lhs: f64, %rhs: f64):
          %s = arith.addf %lhs, %rhs : f64
          scf.reduce.return %s : f64
        }
      }
      memref.store %sum, %y[%row] : memref<?xf64>
      scf.reduce
    }
    return
  }
}
"""

# the same nest over 32-bit positions and coordinates, arguments in another order, fp32 or fp64
def spmv_i32(elem="f64", name="rowsum32"):
    return """
module {
  func.func @%(name)s(%%vals: memref<?x%(t)s>, %%x: memref<?x%(t)s>, %%rowptr: memref<?xi32>, %%y: memref<?x%(t)s>, %%colidx: memref<?xi32>) {
    %%zero = arith.constant 0 : index
    %%one = arith.constant 1 : index
    %%rows = memref.dim %%y, %%zero : memref<?x%(t)s>
    scf.parallel (%%row) = (%%zero) to (%%rows) step (%%one) {
      %%acc0 = memref.load %%y[%%row] : memref<?x%(t)s>
      %%f32 = memref.load %%rowptr[%%row] : memref<?xi32>
      %%first = arith.index_cast %%f32 : i32 to index
      %%next = arith.addi %%one, %%row : index
      %%l32 = memref.load %%rowptr[%%next] : memref<?xi32>
      %%last = arith.index_cast %%l32 : i32 to index
      %%len = arith.subi %%last, %%first : index
      %%sum = scf.parallel (%%k) = (%%zero) to (%%len) step (%%one) init (%%acc0) -> %(t)s {
        %%e = arith.addi %%k, %%first : index
        %%c32 = memref.load %%colidx[%%e] : memref<?xi32>
        %%col = arith.index_cast %%c32 : i32 to index
        %%xv = memref.load %%x[%%col] : memref<?x%(t)s>
        %%a = memref.load %%vals[%%e] : memref<?x%(t)s>
        %%p = arith.mulf %%xv, %%a : %(t)s
        scf.reduce(%%p : %(t)s) {
        ^bb0(%%lhs: %(t)s, %%rhs: %(t)s):
          %%s = arith.addf %%rhs, %%lhs : %(t)s
          scf.reduce.return %%s : %(t)s
        }
      }
      memref.store %%sum, %%y[%%row] : memref<?x%(t)s>
      scf.reduce
    }
    return
  }
}
""" % {"t": elem, "name": name}


# four levels, every level reduces and stores                                      (shape of loop_mapping_3)
DEEP4 = """
module {
  func.func @deep(%t4: memref<?x?x?x?xf32>, %t3: memref<?x?x?xf32>, %t2: memref<?x?xf32>, %t1: memref<?xf32>) -> f32 {
    %i0 = arith.constant 0 : index
    %i1 = arith.constant 1 : index
    %i2 = arith.constant 2 : index
    %i3 = arith.constant 3 : index
    %f0 = arith.constant 0.000000e+00 : f32
    %n0 = memref.dim %t4, %i0 : memref<?x?x?x?xf32>
    %n1 = memref.dim %t4, %i1 : memref<?x?x?x?xf32>
    %n2 = memref.dim %t4, %i2 : memref<?x?x?x?xf32>
    %n3 = memref.dim %t4, %i3 : memref<?x?x?x?xf32>
    %r0 = scf.parallel (%a) = (%i0) to (%n0) step (%i1) init (%f0) -> f32 {
      %r1 = scf.parallel (%b) = (%i0) to (%n1) step (%i1) init (%f0) -> f32 {
        %r2 = scf.parallel (%c) = (%i0) to (%n2) step (%i1) init (%f0) -> f32 {
          %r3 = scf.parallel (%d) = (%i0) to (%n3) step (%i1) init (%f0) -> f32 {
            %v = memref.load %t4[%a, %b, %c, %d] : memref<?x?x?x?xf32>
            scf.reduce(%v : f32) {
            ^bb0(%p: f32, %q: f32):
              %s = arith.addf %p, %q : f32
              scf.reduce.return %s : f32
            }
          }
          memref.store %r3, %t3[%a, %b, %c] : memref<?x?x?xf32>
          scf.reduce(%r3 : f32) {
          ^bb0(%p: f32, %q: f32):
            %s = arith.addf %p, %q : f32
            scf.reduce.return %s : f32
          }
        }
        memref.store %r2, %t2[%a, %b] : memref<?x?xf32>
        scf.reduce(%r2 : f32) {
        ^bb0(%p: f32, %q: f32):
          %s = arith.addf %p, %q : f32
          scf.reduce.return %s : f32
        }
      }
      memref.store %r1, %t1[%a] : memref<?xf32>
      scf.reduce(%r1 : f32) {
      ^bb0(%p: f32, %q: f32):
        %s = arith.addf %p, %q : f32
        scf.reduce.return %s : f32
      }
    }
    return %r0 : f32
  }
}
"""

SHAPES = {"loop_mapping_0": HOST_2D, "loop_mapping_1": COUNT, "loop_mapping_2": SPMV_INDEX, "loop_mapping_3": DEEP4}


# ---- depth-1 loops and the SpMM nest the kernel library has entry points for ------------------------------

# a dot product as DenseLinalgToParallelLoops leaves it (the shape of linalg_to_loops_0's gold): the reduction
# starts from the value of a zero-dimensional buffer, which gets the result
DOT = """
module {
  func.func @inner(%u: memref<?xf64>, %v: memref<?xf64>, %start: f64) -> f64 {
    %zero = arith.constant 0 : index
    %one = arith.constant 1 : index
    %cell = memref.alloc() {alignment = 64 : i64} : memref<f64>
    memref.store %start, %cell[] : memref<f64>
    %count = memref.dim %u, %zero : memref<?xf64>
    %from = memref.load %cell[] : memref<f64>
    %total = scf.parallel (%k) = (%zero) to (%count) step (%one) init (%from) -> f64 {
      %a = memref.load %u[%k] : memref<?xf64>
      %b = memref.load %v[%k] : memref<?xf64>
      %prod = arith.mulf %a, %b : f64
      scf.reduce(%prod : f64) {
      ^bb0(%lhs: f64, %rhs: f64):
        %s = arith.addf %lhs, %rhs : f64
        scf.reduce.return %s : f64
      }
    }
    memref.store %total, %cell[] : memref<f64>
    %got = memref.load %cell[] : memref<f64>
    return %got : f64
  }
}
"""

# the same loop with a product reduction: no entry point
DOT_PRODUCT_REDUCTION = DOT.replace("%s = arith.addf %lhs, %rhs", "%s = arith.mulf %lhs, %rhs")


def elementwise(body, elem="f64", name="update"):
    """A depth-1 loop `w[k] = <body>(u[k], v[k], p, q)`; `body` defines %r from %a, %b, %p, %q."""
    return """
module {
  func.func @%(name)s(%%p: %(t)s, %%u: memref<?x%(t)s>, %%q: %(t)s, %%v: memref<?x%(t)s>, %%w: memref<?x%(t)s>) {
    %%zero = arith.constant 0 : index
    %%one = arith.constant 1 : index
    %%count = memref.dim %%w, %%zero : memref<?x%(t)s>
    scf.parallel (%%k) = (%%zero) to (%%count) step (%%one) {
      %%a = memref.load %%u[%%k] : memref<?x%(t)s>
      %%b = memref.load %%v[%%k] : memref<?x%(t)s>
%(body)s
      memref.store %%r, %%w[%%k] : memref<?x%(t)s>
      scf.reduce
    }
    return
  }
}
""" % {"t": elem, "name": name, "body": body.replace("%", "%%").replace("%%", "%") % {"t": elem} if "%(t)s" in body else body}


AXPBY_BODY = """      %l = arith.mulf %a, %p : f64
      %m = arith.mulf %b, %q : f64
      %r = arith.addf %l, %m : f64"""
MULT_BODY = "      %r = arith.mulf %a, %b : f64"
SCALE_BODY = "      %r = arith.mulf %p, %a : f64"
FILL_BODY = "      %r = arith.addf %p, %q : f64"
CUBE_BODY = """      %l = arith.mulf %a, %a : f64
      %r = arith.mulf %l, %b : f64"""


def spmm_i32(elem="f32", inner="scf.parallel", name="rows_times_dense"):
    """C[i, j] += sum_kk val[kk] * B[crd[kk], j]: rows parallel, the compressed loop sequential, the dense column
    loop parallel (`inner="scf.parallel"`) or sequential (`inner="scf.for"`)."""
    if inner == "scf.parallel":
        open_j, close_j = "scf.parallel (%j) = (%zero) to (%cols) step (%one) {", "          scf.reduce\n        }"
    else:
        open_j, close_j = "scf.for %j = %zero to %cols step %one {", "        }"
    return """
module {
  func.func @%(name)s(%%B: memref<?x?x%(t)s>, %%ptr: memref<?xi32>, %%idx: memref<?xi32>, %%C: memref<?x?x%(t)s>, %%nz: memref<?x%(t)s>) {
    %%zero = arith.constant 0 : index
    %%one = arith.constant 1 : index
    %%rows = memref.dim %%C, %%zero : memref<?x?x%(t)s>
    %%cols = memref.dim %%C, %%one : memref<?x?x%(t)s>
    scf.parallel (%%i) = (%%zero) to (%%rows) step (%%one) {
      %%lo32 = memref.load %%ptr[%%i] : memref<?xi32>
      %%lo = arith.index_cast %%lo32 : i32 to index
      %%inext = arith.addi %%i, %%one : index
      %%hi32 = memref.load %%ptr[%%inext] : memref<?xi32>
      %%hi = arith.index_cast %%hi32 : i32 to index
      scf.for %%kk = %%lo to %%hi step %%one {
        %%c32 = memref.load %%idx[%%kk] : memref<?xi32>
        %%c = arith.index_cast %%c32 : i32 to index
        %%a = memref.load %%nz[%%kk] : memref<?x%(t)s>
        %(open_j)s
          %%old = memref.load %%C[%%i, %%j] : memref<?x?x%(t)s>
          %%b = memref.load %%B[%%c, %%j] : memref<?x?x%(t)s>
          %%prod = arith.mulf %%a, %%b : %(t)s
          %%new = arith.addf %%old, %%prod : %(t)s
          memref.store %%new, %%C[%%i, %%j] : memref<?x?x%(t)s>
%(close_j)s
      }
      scf.reduce
    }
    return
  }
}
""" % {"t": elem, "name": name, "open_j": open_j.replace("%", "%%").replace("%%", "%"), "close_j": close_j}
