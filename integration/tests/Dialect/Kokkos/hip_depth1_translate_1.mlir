// RUN: %lapis-translate --hip-kernels %s | grep -E -c "KOKKOS_LAMBDA|lapis_hip_dot_f64_host\(|lapis_hip_axpby_f64\(|lapis_hip_mult_f64\(|lapis_hip_copy_f32\(|lapis_hip_fill_f64\(|lapis_hip_init\(\)|lapis_hip_finalize\(\)" | diff %s.gold -

// Near misses stay Kokkos launches: a reduction that multiplies, an elementwise body with a product of
// three elements, a loop that runs on the host, and a scaled update whose coefficient is computed
// inside the loop. Four KOKKOS_LAMBDA-or-host-lambda launches of which three are device lambdas, plus
// lapis_hip_init / lapis_hip_finalize: 5 matching lines.
module {
  func.func @product(%arg0: memref<?xf64>, %arg1: memref<?xf64>, %arg2: f64) -> f64 {
    %c0 = arith.constant 0 : index
    %dim = memref.dim %arg0, %c0 : memref<?xf64>
    %0 = kokkos.range_parallel (%arg3) -> (%dim) -> f64 {
      %1 = memref.load %arg0[%arg3] : memref<?xf64>
      %2 = memref.load %arg1[%arg3] : memref<?xf64>
      %3 = arith.mulf %1, %2 : f64
      "kokkos.update_reduction"(%3, %arg2) ({
      ^bb0(%arg4: f64, %arg5: f64):
        %4 = arith.mulf %arg4, %arg5 : f64
        kokkos.yield %4 : f64
      }) : (f64, f64) -> ()
      kokkos.yield
    } {executionSpace = 1 : i64, parallelLevel = 0 : i64}
    return %0 : f64
  }
  func.func @cube(%arg0: memref<?xf64>, %arg1: memref<?xf64>, %arg2: memref<?xf64>) {
    %c0 = arith.constant 0 : index
    %dim = memref.dim %arg2, %c0 : memref<?xf64>
    kokkos.range_parallel (%arg3) -> (%dim) {
      %0 = memref.load %arg0[%arg3] : memref<?xf64>
      %1 = memref.load %arg1[%arg3] : memref<?xf64>
      %2 = arith.mulf %0, %0 : f64
      %3 = arith.mulf %2, %1 : f64
      memref.store %3, %arg2[%arg3] : memref<?xf64>
      kokkos.yield
    } {executionSpace = 1 : i64, parallelLevel = 0 : i64}
    return
  }
  func.func @on_the_host(%arg0: memref<?xf64>, %arg1: memref<?xf64>, %arg2: memref<?xf64>) {
    %c0 = arith.constant 0 : index
    %dim = memref.dim %arg2, %c0 : memref<?xf64>
    kokkos.range_parallel (%arg3) -> (%dim) {
      %0 = memref.load %arg0[%arg3] : memref<?xf64>
      %1 = memref.load %arg1[%arg3] : memref<?xf64>
      %2 = arith.mulf %0, %1 : f64
      memref.store %2, %arg2[%arg3] : memref<?xf64>
      kokkos.yield
    } {executionSpace = 0 : i64, parallelLevel = 0 : i64}
    return
  }
  func.func @varying_coefficient(%arg0: memref<?xf64>, %arg1: memref<?xf64>, %arg2: memref<?xf64>, %arg3: f64) {
    %c0 = arith.constant 0 : index
    %dim = memref.dim %arg2, %c0 : memref<?xf64>
    kokkos.range_parallel (%arg4) -> (%dim) {
      %0 = memref.load %arg0[%arg4] : memref<?xf64>
      %1 = memref.load %arg1[%arg4] : memref<?xf64>
      %2 = arith.addf %1, %arg3 : f64
      %3 = arith.mulf %0, %2 : f64
      %4 = arith.mulf %1, %arg3 : f64
      %5 = arith.addf %3, %4 : f64
      memref.store %5, %arg2[%arg4] : memref<?xf64>
      kokkos.yield
    } {executionSpace = 1 : i64, parallelLevel = 0 : i64}
    return
  }
}
