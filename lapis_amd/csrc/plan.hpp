// The CSR plan object behind lapis_hip_csr_plan (opaque in the C ABI).
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

#include "lapis_hip.h"

struct lapis_hip_csr_plan {
  lapis_hip_csr_stats stats;
  const int32_t *pos;
  const int32_t *crd;  // the coordinates the statistics were read from (null when the plan was made without them)
  int nchunks;
  int chunk;            // non-zeros per wavefront of the row-split kernel (512, 1024 or 2048)
  int waves_per_block;  // wavefronts per workgroup of the row-split kernel
  bool nontemporal;
  int xcd_map;          // 1: contiguous ranges of blocks per XCD (see xcd_contiguous_block)
  // row-split (NNZSPLIT) metadata
  int *chunk_row;    // device, int[nchunks+1]
  void *part_first;  // device, 8 bytes * nchunks
  void *part_last;   // device, 8 bytes * nchunks
  // column-blocked (COLBLOCK) copy of the matrix, built on request
  bool colblock_built;
  int colblock_value_bytes;
  int colblock_col_bits;     // low bits of an entry hold the column, the bits above the row inside its row block
  int colblock_slice_log2;   // columns per x slice = 1 << this
  unsigned *colblock_idx;    // device, uint32[nnz]
  void *colblock_val;        // device, T[nnz]
  unsigned *colblock_perm;   // device, uint32[nnz]: CSR position of the entry stored at each position of the copy
  const void *colblock_src_crd;  // the caller's buffers the copy was made from; SpMV calls must pass the same ones
  const void *colblock_src_val;
  int colblock_steps;        // steps per wavefront trip
  int colblock_epl;          // entries per lane per step (1, 2 or 4)
  int colblock_pad;          // 1: workgroups of 8 wavefronts instead of 4
  int colblock_rows;         // rows per wavefront (512 or 1024), or per workgroup in the workgroup-blocked layout
  int colblock_threads;      // threads per workgroup of the workgroup-blocked kernel (256, 512 or 1024)
  int colblock_group;        // 1: workgroup-blocked layout (tiles in column order, row sums shared by a workgroup)
  int colblock_pc_prod;      // > 0: the workgroup kernel with this many producer wavefronts (they only stream)
  int colblock_pc_threads;   // threads per workgroup of that kernel
  int *colblock_fault;       // device int: set by a wavefront of that kernel whose bounded wait ran out
  int colblock_nblocks;      // row blocks of the workgroup-blocked layout
  int colblock_nslices;      // slices of x
  int *colblock_tile_ptr;    // device, int[nblocks * (nslices + 1)]
  // workgroup-blocked layout: work units and the rows kept apart as long rows
  int colblock_nblocks_nat;  // blocks of consecutive rows; blocks from here on hold the long rows
  int colblock_nunits;       // workgroups per launch
  int *colblock_units;       // device, int[4 * nunits]: block, first entry, one past the last, 1 if the block's only unit
  int colblock_nlong;        // rows of colblock_long_threshold entries or more
  int *colblock_long_rows;   // device, int[nlong]: their row numbers, ascending
  int colblock_long_threshold;
  unsigned colblock_pace_fp; // clock ticks per entry (16.16 fixed point) of the time-triggered pacing, 0 = off
  double colblock_free_ms;   // calibration: kernel time without pacing
  double colblock_paced_ms;  // calibration: kernel time at the chosen pace
};

namespace lapis {
constexpr int kColblockRowBits = 10;  // the per-wavefront layout keeps up to 1024 rows per wavefront

// bits needed for values 0..n-1
inline int bits_for(int64_t n) {
  int b = 0;
  while (b < 62 && (1LL << b) < n) ++b;
  return b;
}

// Workgroup-blocked layout; defined in colgroup.hip.
template <typename T>
int build_colgroup(lapis_hip_csr_plan *plan, const int32_t *crd, const T *val, int slice_log2, hipStream_t st);
template <typename T>
int launch_colgroup(const lapis_hip_csr_plan *plan, const T *x, T *y, hipStream_t st);

// Launches the column-blocked kernel; defined in colblock.hip.
template <typename T>
int launch_colblock(const lapis_hip_csr_plan *plan, const int *pos, const int *crd, const T *val, const T *x, T *y,
                    hipStream_t st);
void free_colblock(lapis_hip_csr_plan *plan);

// Sorts `nnz` 64-bit keys (bits [0, end_bit)).  On success *keys_out holds the sorted keys and
// *perm the position each sorted key had before (both device buffers, the caller frees them).
int sort_keys_with_perm(const unsigned long long *keys_in, int64_t nnz, int begin_bit, int end_bit, unsigned long long **keys_out,
                        unsigned **perm, hipStream_t st);
// out[i] = val[perm[i]]
template <typename T>
int gather_values(const unsigned *perm, const T *val, T *out, int64_t nnz, hipStream_t st);

// y = A x without reading y; defined in spmv.hip.  A caller that passes `deferred_chunk` and gets a
// non-zero chunk length back completes the rows cut at chunk boundaries itself (rowsplit_fix.hpp);
// for a square matrix `xy_chunk` (plan->nchunks doubles) then holds, per chunk, the sum of
// x[r]*y[r] over the rows that lie wholly inside the chunk.
int spmv_overwrite_f64(lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols, const int32_t *pos,
                       const int32_t *crd, const double *val, const double *x, double *y,
                       lapis_hip_stream_t stream, int *deferred_chunk = nullptr, double *xy_chunk = nullptr);
}  // namespace lapis
