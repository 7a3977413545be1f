// RUN: %lapis-opt %s --kokkos-loop-mapping="hip-kernels" | diff %s.gold -

// CSR SpMV with 32-bit positions and coordinates (posWidth = crdWidth = 32): the nest the
// gfx950 kernel library takes over when the module is translated with --hip-kernels.
// Negative case: the reduction is a maximum, not a sum, so this is no SpMV.  The nest keeps
// its Kokkos launch and with it the vector length estimate computed from the positions.
module {
  func.func @spmv(%arg0: memref<?xf64>, %arg1: memref<?xi32>, %arg2: memref<?xi32>, %arg3: memref<?xf64>, %arg4: memref<?xf64>) {
    %c0 = arith.constant 0 : index
    %c1 = arith.constant 1 : index
    %cN = memref.dim %arg0, %c0 : memref<?xf64>
    scf.parallel (%arg5) = (%c0) to (%cN) step (%c1) {
      %0 = memref.load %arg0[%arg5] : memref<?xf64>
      %1 = memref.load %arg1[%arg5] : memref<?xi32>
      %2 = arith.index_cast %1 : i32 to index
      %3 = arith.addi %arg5, %c1 : index
      %4 = memref.load %arg1[%3] : memref<?xi32>
      %5 = arith.index_cast %4 : i32 to index
      %6 = arith.subi %5, %2 : index
      %7 = scf.parallel (%arg6) = (%c0) to (%6) step (%c1) init (%0) -> f64 {
        %8 = arith.addi %2, %arg6 : index
        %9 = memref.load %arg2[%8] : memref<?xi32>
        %10 = arith.index_cast %9 : i32 to index
        %11 = memref.load %arg3[%8] : memref<?xf64>
        %12 = memref.load %arg4[%10] : memref<?xf64>
        %13 = arith.mulf %11, %12 : f64
        scf.reduce(%13 : f64) {
        ^bb0(%arg7: f64, %arg8: f64):
          %14 = arith.maximumf %arg7, %arg8 : f64
          scf.reduce.return %14 : f64
        }
      }
      memref.store %7, %arg0[%arg5] : memref<?xf64>
      scf.reduce
    }
    return
  }
}
