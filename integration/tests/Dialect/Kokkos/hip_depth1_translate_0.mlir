// RUN: %lapis-translate --hip-kernels %s | grep -E -c "KOKKOS_LAMBDA|lapis_hip_dot_f64_host\(|lapis_hip_axpby_f64\(|lapis_hip_mult_f64\(|lapis_hip_copy_f32\(|lapis_hip_fill_f64\(|lapis_hip_init\(\)|lapis_hip_finalize\(\)" | diff %s.gold -

// Depth-1 device loops the kernel library has entry points for, translated with --hip-kernels: the dot
// product (the loop DenseLinalgToParallelLoops makes of linalg.dot), a*x + b*y, x*y, a copy (fp32) and a
// fill each become ONE library call and no KOKKOS_LAMBDA; with lapis_hip_init in lapis_initialize and
// lapis_hip_finalize in lapis_finalize that is 7 matching lines.
module {
  func.func @inner(%arg0: memref<?xf64>, %arg1: memref<?xf64>, %arg2: f64) -> f64 {
    %c0 = arith.constant 0 : index
    %dim = memref.dim %arg0, %c0 : memref<?xf64>
    %0 = kokkos.range_parallel (%arg3) -> (%dim) -> f64 {
      %1 = memref.load %arg0[%arg3] : memref<?xf64>
      %2 = memref.load %arg1[%arg3] : memref<?xf64>
      %3 = arith.mulf %1, %2 : f64
      "kokkos.update_reduction"(%3, %arg2) ({
      ^bb0(%arg4: f64, %arg5: f64):
        %4 = arith.addf %arg4, %arg5 : f64
        kokkos.yield %4 : f64
      }) : (f64, f64) -> ()
      kokkos.yield
    } {executionSpace = 1 : i64, parallelLevel = 0 : i64}
    return %0 : f64
  }
  func.func @combine(%arg0: f64, %arg1: memref<?xf64>, %arg2: f64, %arg3: memref<?xf64>, %arg4: memref<?xf64>) {
    %c0 = arith.constant 0 : index
    %dim = memref.dim %arg4, %c0 : memref<?xf64>
    kokkos.range_parallel (%arg5) -> (%dim) {
      %0 = memref.load %arg1[%arg5] : memref<?xf64>
      %1 = memref.load %arg3[%arg5] : memref<?xf64>
      %2 = arith.mulf %0, %arg0 : f64
      %3 = arith.mulf %1, %arg2 : f64
      %4 = arith.addf %2, %3 : f64
      memref.store %4, %arg4[%arg5] : memref<?xf64>
      kokkos.yield
    } {executionSpace = 1 : i64, parallelLevel = 0 : i64}
    return
  }
  func.func @hadamard(%arg0: memref<?xf64>, %arg1: memref<?xf64>, %arg2: memref<?xf64>) {
    %c0 = arith.constant 0 : index
    %dim = memref.dim %arg2, %c0 : memref<?xf64>
    kokkos.range_parallel (%arg3) -> (%dim) {
      %0 = memref.load %arg0[%arg3] : memref<?xf64>
      %1 = memref.load %arg1[%arg3] : memref<?xf64>
      %2 = arith.mulf %0, %1 : f64
      memref.store %2, %arg2[%arg3] : memref<?xf64>
      kokkos.yield
    } {executionSpace = 1 : i64, parallelLevel = 0 : i64}
    return
  }
  func.func @duplicate(%arg0: memref<?xf32>, %arg1: memref<?xf32>) {
    %c0 = arith.constant 0 : index
    %dim = memref.dim %arg1, %c0 : memref<?xf32>
    kokkos.range_parallel (%arg2) -> (%dim) {
      %0 = memref.load %arg0[%arg2] : memref<?xf32>
      memref.store %0, %arg1[%arg2] : memref<?xf32>
      kokkos.yield
    } {executionSpace = 1 : i64, parallelLevel = 0 : i64}
    return
  }
  func.func @clear(%arg0: f64, %arg1: memref<?xf64>) {
    %c0 = arith.constant 0 : index
    %dim = memref.dim %arg1, %c0 : memref<?xf64>
    kokkos.range_parallel (%arg2) -> (%dim) {
      memref.store %arg0, %arg1[%arg2] : memref<?xf64>
      kokkos.yield
    } {executionSpace = 1 : i64, parallelLevel = 0 : i64}
    return
  }
}
