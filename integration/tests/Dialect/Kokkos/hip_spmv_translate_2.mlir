// RUN: %lapis-translate --hip-kernels %s | grep -E -c "KOKKOS_LAMBDA|lapis_hip_spmv_csr_f64_i32\(lapis_hip_plan_|lapis_hip_csr_plan_create\(&lapis_hip_plan_|lapis_hip_csr_plan_matches\(lapis_hip_plan_|lapis_hip_csr_plan_analyze\(lapis_hip_plan_|lapis_hip_csr_plan_destroy\(lapis_hip_plan_|lapis_hip_init\(\)|lapis_hip_finalize\(\)" | diff %s.gold -

// The same nest inside an scf.while (a solver's iteration): beside the 7 lines of hip_spmv_translate_0 the
// call site counts its products and hands the plan to lapis_hip_csr_plan_analyze at the eighth, where the
// library decides whether its blocked copy of the matrix pays: 8 matching lines.
module {
  func.func @repeat(%arg0: memref<?xf64>, %arg1: memref<?xi32>, %arg2: memref<?xi32>, %arg3: memref<?xf64>, %arg4: memref<?xf64>, %arg9: index) {
    %c0 = arith.constant 0 : index
    %c1 = arith.constant 1 : index
    %dim = memref.dim %arg0, %c0 : memref<?xf64>
    %15 = scf.while (%arg10 = %c0) : (index) -> index {
      %16 = arith.cmpi slt, %arg10, %arg9 : index
      scf.condition(%16) %arg10 : index
    } do {
    ^bb0(%arg10: index):
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
      %17 = arith.addi %arg10, %c1 : index
      scf.yield %17 : index
    }
    return
  }
}
