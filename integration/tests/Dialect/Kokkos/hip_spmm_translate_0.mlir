// RUN: %lapis-translate --hip-kernels %s | grep -E -c "KOKKOS_LAMBDA|lapis_hip_spmm_csr_f32_i32_plan\(lapis_hip_plan_|lapis_hip_spmm_csr_f64_i32_plan\(lapis_hip_plan_|lapis_hip_csr_plan_create\(&lapis_hip_plan_|lapis_hip_csr_plan_matches\(lapis_hip_plan_|lapis_hip_csr_plan_destroy\(lapis_hip_plan_|lapis_hip_init\(\)|lapis_hip_finalize\(\)" | diff %s.gold -

// C += A*B with A in CSR (32-bit positions and coordinates) and dense row-major B, C, in the two shapes
// that keep the compressed loop sequential: rows as a device RangePolicy loop with both inner loops
// scf.for (fp64), and rows as thread_parallel with the column loop a ThreadVector loop (fp32). Each is
// one lapis_hip_spmm_csr_*_plan call with its plan: per function the lines with
// lapis_hip_csr_plan_matches, lapis_hip_csr_plan_create, the call, and lapis_hip_csr_plan_destroy twice
// (before a rebuild, in lapis_finalize) = 5; two functions + lapis_hip_init + lapis_hip_finalize = 12,
// and no KOKKOS_LAMBDA.
module {
  func.func @rows_range(%arg0: memref<?x?xf64>, %arg1: memref<?xi32>, %arg2: memref<?xi32>, %arg3: memref<?xf64>, %arg4: memref<?x?xf64>) {
    %c0 = arith.constant 0 : index
    %c1 = arith.constant 1 : index
    %dim = memref.dim %arg0, %c0 : memref<?x?xf64>
    %dim_0 = memref.dim %arg0, %c1 : memref<?x?xf64>
    kokkos.range_parallel (%arg5) -> (%dim) {
      %0 = memref.load %arg1[%arg5] : memref<?xi32>
      %1 = arith.index_cast %0 : i32 to index
      %2 = arith.addi %arg5, %c1 : index
      %3 = memref.load %arg1[%2] : memref<?xi32>
      %4 = arith.index_cast %3 : i32 to index
      scf.for %arg6 = %1 to %4 step %c1 {
        %5 = memref.load %arg2[%arg6] : memref<?xi32>
        %6 = arith.index_cast %5 : i32 to index
        %7 = memref.load %arg3[%arg6] : memref<?xf64>
        scf.for %arg7 = %c0 to %dim_0 step %c1 {
          %8 = memref.load %arg0[%arg5, %arg7] : memref<?x?xf64>
          %9 = memref.load %arg4[%6, %arg7] : memref<?x?xf64>
          %10 = arith.mulf %7, %9 : f64
          %11 = arith.addf %8, %10 : f64
          memref.store %11, %arg0[%arg5, %arg7] : memref<?x?xf64>
        }
      }
      kokkos.yield
    } {executionSpace = 1 : i64, parallelLevel = 0 : i64}
    return
  }
  func.func @rows_threads(%arg0: memref<?x?xf32>, %arg1: memref<?xi32>, %arg2: memref<?xi32>, %arg3: memref<?xf32>, %arg4: memref<?x?xf32>) {
    %c0 = arith.constant 0 : index
    %c1 = arith.constant 1 : index
    %dim = memref.dim %arg0, %c0 : memref<?x?xf32>
    %dim_0 = memref.dim %arg0, %c1 : memref<?x?xf32>
    "kokkos.thread_parallel"(%dim, %dim_0) ({
    ^bb0(%arg5: index):
      %0 = memref.load %arg1[%arg5] : memref<?xi32>
      %1 = arith.index_cast %0 : i32 to index
      %2 = arith.addi %arg5, %c1 : index
      %3 = memref.load %arg1[%2] : memref<?xi32>
      %4 = arith.index_cast %3 : i32 to index
      scf.for %arg6 = %1 to %4 step %c1 {
        %5 = memref.load %arg2[%arg6] : memref<?xi32>
        %6 = arith.index_cast %5 : i32 to index
        %7 = memref.load %arg3[%arg6] : memref<?xf32>
        kokkos.range_parallel (%arg7) -> (%dim_0) {
          %8 = memref.load %arg0[%arg5, %arg7] : memref<?x?xf32>
          %9 = memref.load %arg4[%6, %arg7] : memref<?x?xf32>
          %10 = arith.mulf %7, %9 : f32
          %11 = arith.addf %8, %10 : f32
          memref.store %11, %arg0[%arg5, %arg7] : memref<?x?xf32>
          kokkos.yield
        } {executionSpace = 2 : i64, parallelLevel = 3 : i64}
      }
      kokkos.yield
    }) : (index, index) -> ()
    return
  }
}
