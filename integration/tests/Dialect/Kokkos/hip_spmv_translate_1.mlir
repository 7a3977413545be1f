// RUN: %lapis-translate --hip-kernels %s | grep -E -c "KOKKOS_LAMBDA|lapis_hip_spmv_csr_f64_i32\(lapis_hip_plan_|lapis_hip_csr_plan_create\(&lapis_hip_plan_|lapis_hip_csr_plan_matches\(lapis_hip_plan_|lapis_hip_csr_plan_analyze\(lapis_hip_plan_|lapis_hip_csr_plan_destroy\(lapis_hip_plan_|lapis_hip_init\(\)|lapis_hip_finalize\(\)" | diff %s.gold -

// Negative case (hip_spmv_1.mlir.gold): a maximum reduction is no SpMV, so the nest stays a Kokkos
// TeamPolicy launch: one KOKKOS_LAMBDA line plus lapis_hip_init / lapis_hip_finalize: 3 matching lines.
module {
  func.func @spmv(%arg0: memref<?xf64>, %arg1: memref<?xi32>, %arg2: memref<?xi32>, %arg3: memref<?xf64>, %arg4: memref<?xf64>) {
    %c0 = arith.constant 0 : index
    %c1 = arith.constant 1 : index
    %dim = memref.dim %arg0, %c0 : memref<?xf64>
    %0 = memref.load %arg1[%dim] : memref<?xi32>
    %1 = arith.index_cast %0 : i32 to index
    %2 = memref.load %arg1[%c0] : memref<?xi32>
    %3 = arith.index_cast %2 : i32 to index
    %4 = arith.subi %1, %3 : index
    %5 = arith.addi %4, %dim : index
    %6 = arith.subi %5, %c1 : index
    %7 = arith.divui %6, %dim : index
    "kokkos.thread_parallel"(%dim, %7) ({
    ^bb0(%arg5: index):
      %8 = memref.load %arg0[%arg5] : memref<?xf64>
      %9 = memref.load %arg1[%arg5] : memref<?xi32>
      %10 = arith.index_cast %9 : i32 to index
      %11 = arith.addi %arg5, %c1 : index
      %12 = memref.load %arg1[%11] : memref<?xi32>
      %13 = arith.index_cast %12 : i32 to index
      %14 = arith.subi %13, %10 : index
      %15 = kokkos.range_parallel (%arg6) -> (%14) -> f64 {
        %16 = arith.addi %10, %arg6 : index
        %17 = memref.load %arg2[%16] : memref<?xi32>
        %18 = arith.index_cast %17 : i32 to index
        %19 = memref.load %arg3[%16] : memref<?xf64>
        %20 = memref.load %arg4[%18] : memref<?xf64>
        %21 = arith.mulf %19, %20 : f64
        "kokkos.update_reduction"(%21, %8) ({
        ^bb0(%arg7: f64, %arg8: f64):
          %22 = arith.maximumf %arg7, %arg8 : f64
          kokkos.yield %22 : f64
        }) : (f64, f64) -> ()
        kokkos.yield
      } {executionSpace = 2 : i64, parallelLevel = 3 : i64}
      "kokkos.single"() <{level = 1 : i64}> ({
        memref.store %15, %arg0[%arg5] : memref<?xf64>
        kokkos.yield
      }) : () -> ()
      kokkos.yield
    }) : (index, index) -> ()
    return
  }
}
