// RUN: %lapis-translate --hip-kernels %s | grep -E -c "KOKKOS_LAMBDA|lapis_hip_spmv_csr_f64_i32\(lapis_hip_plan_|lapis_hip_csr_plan_create\(&lapis_hip_plan_|lapis_hip_csr_plan_matches\(lapis_hip_plan_|lapis_hip_csr_plan_analyze\(lapis_hip_plan_|lapis_hip_csr_plan_destroy\(lapis_hip_plan_|lapis_hip_init\(\)|lapis_hip_finalize\(\)" | diff %s.gold -

// The mapped CSR SpMV nest (hip_spmv_0.mlir.gold) translated with --hip-kernels: the kept plan is checked
// against the operands (lapis_hip_csr_plan_matches and the generation of the operands, 1 line) and
// destroyed if it was made for others, created if there is none (lapis_hip_csr_plan_create), then ONE call
// of lapis_hip_spmv_csr_f64_i32; lapis_hip_csr_plan_destroy before the rebuild and in lapis_finalize
// (2 lines), lapis_hip_init in lapis_initialize, lapis_hip_finalize in lapis_finalize -- no
// lapis_hip_csr_plan_analyze (the nest is not inside a loop) and no KOKKOS_LAMBDA: 7 matching lines.
module {
  func.func @spmv(%arg0: memref<?xf64>, %arg1: memref<?xi32>, %arg2: memref<?xi32>, %arg3: memref<?xf64>, %arg4: memref<?xf64>) {
    %c0 = arith.constant 0 : index
    %c1 = arith.constant 1 : index
    %dim = memref.dim %arg0, %c0 : memref<?xf64>
    "kokkos.thread_parallel"(%dim, %c0) ({
    ^bb0(%arg5: index):
      %0 = memref.load %arg0[%arg5] : memref<?xf64>
      %1 = memref.load %arg1[%arg5] : memref<?xi32>
      %2 = arith.index_cast %1 : i32 to index
      %3 = arith.addi %arg5, %c1 : index
      %4 = memref.load %arg1[%3] : memref<?xi32>
      %5 = arith.index_cast %4 : i32 to index
      %6 = arith.subi %5, %2 : index
      %7 = kokkos.range_parallel (%arg6) -> (%6) -> f64 {
        %8 = arith.addi %2, %arg6 : index
        %9 = memref.load %arg2[%8] : memref<?xi32>
        %10 = arith.index_cast %9 : i32 to index
        %11 = memref.load %arg3[%8] : memref<?xf64>
        %12 = memref.load %arg4[%10] : memref<?xf64>
        %13 = arith.mulf %11, %12 : f64
        "kokkos.update_reduction"(%13, %0) ({
        ^bb0(%arg7: f64, %arg8: f64):
          %14 = arith.addf %arg7, %arg8 : f64
          kokkos.yield %14 : f64
        }) : (f64, f64) -> ()
        kokkos.yield
      } {executionSpace = 2 : i64, parallelLevel = 3 : i64}
      "kokkos.single"() <{level = 1 : i64}> ({
        memref.store %7, %arg0[%arg5] : memref<?xf64>
        kokkos.yield
      }) : () -> ()
      kokkos.yield
    }) : (index, index) -> ()
    return
  }
}
