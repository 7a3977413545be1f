// RUN: %lapis-translate --hip-kernels %s | grep -E -c "KOKKOS_LAMBDA|lapis_hip_spmm_csr_f32_i32_plan\(lapis_hip_plan_|lapis_hip_spmm_csr_f64_i32_plan\(lapis_hip_plan_|lapis_hip_csr_plan_create\(&lapis_hip_plan_|lapis_hip_csr_plan_matches\(lapis_hip_plan_|lapis_hip_csr_plan_destroy\(lapis_hip_plan_|lapis_hip_init\(\)|lapis_hip_finalize\(\)" | diff %s.gold -

// Negative cases stay Kokkos launches: the same nest over 64-bit positions (the library indexes with
// int32), and a nest that multiplies by the TRANSPOSED dense operand (B[j, crd] instead of B[crd, j]).
// Two KOKKOS_LAMBDA lines + lapis_hip_init + lapis_hip_finalize: 4 matching lines.
module {
  func.func @wide_positions(%arg0: memref<?x?xf64>, %arg1: memref<?xindex>, %arg2: memref<?xi32>, %arg3: memref<?xf64>, %arg4: memref<?x?xf64>) {
    %c0 = arith.constant 0 : index
    %c1 = arith.constant 1 : index
    %dim = memref.dim %arg0, %c0 : memref<?x?xf64>
    %dim_0 = memref.dim %arg0, %c1 : memref<?x?xf64>
    kokkos.range_parallel (%arg5) -> (%dim) {
      %0 = memref.load %arg1[%arg5] : memref<?xindex>
      %1 = arith.addi %arg5, %c1 : index
      %2 = memref.load %arg1[%1] : memref<?xindex>
      scf.for %arg6 = %0 to %2 step %c1 {
        %3 = memref.load %arg2[%arg6] : memref<?xi32>
        %4 = arith.index_cast %3 : i32 to index
        %5 = memref.load %arg3[%arg6] : memref<?xf64>
        scf.for %arg7 = %c0 to %dim_0 step %c1 {
          %6 = memref.load %arg0[%arg5, %arg7] : memref<?x?xf64>
          %7 = memref.load %arg4[%4, %arg7] : memref<?x?xf64>
          %8 = arith.mulf %5, %7 : f64
          %9 = arith.addf %6, %8 : f64
          memref.store %9, %arg0[%arg5, %arg7] : memref<?x?xf64>
        }
      }
      kokkos.yield
    } {executionSpace = 1 : i64, parallelLevel = 0 : i64}
    return
  }
  func.func @transposed_operand(%arg0: memref<?x?xf64>, %arg1: memref<?xi32>, %arg2: memref<?xi32>, %arg3: memref<?xf64>, %arg4: memref<?x?xf64>) {
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
          %9 = memref.load %arg4[%arg7, %6] : memref<?x?xf64>
          %10 = arith.mulf %7, %9 : f64
          %11 = arith.addf %8, %10 : f64
          memref.store %11, %arg0[%arg5, %arg7] : memref<?x?xf64>
        }
      }
      kokkos.yield
    } {executionSpace = 1 : i64, parallelLevel = 0 : i64}
    return
  }
}
