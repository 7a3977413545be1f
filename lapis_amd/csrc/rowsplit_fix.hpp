// Completion of the rows the row-split SpMV kernel cuts at chunk boundaries, as a
// device function: the fix-up kernel of spmv.hip calls it, and so does the p.Ap
// kernel of the CG solver, which saves the solver one launch per iteration.
#pragma once
#include <hip/hip_runtime.h>

#include "common.hpp"

namespace lapis {

// Called by ALL 64 lanes of a wavefront, lane l for chunk boundary c (1 <= c; lanes
// with c >= nchunks take part and own nothing).  The row cut by boundary c belongs
// to the lane of the FIRST boundary that cuts it; for that lane `owner` is set, `r`
// is the row and the value returned is
//   part_last[c-1] + part_first[c] + ... + part_first[c_last]
// summed in that fixed order, so the result does not depend on scheduling.  Rows cut 16
// times or more are summed by the whole wavefront.
template <typename T, int CH>
__device__ __forceinline__ T rowsplit_row_total(long long c, int nchunks, const int *__restrict__ pos,
                                                const int *__restrict__ chunk_row,
                                                const T *__restrict__ part_first,
                                                const T *__restrict__ part_last, bool &owner, int &r) {
  const int lane = threadIdx.x & 63;
  owner = false;
  r = 0;
  int cfirst = 0, clast = -1;
  if (c < nchunks) {
    r = chunk_row[c];
    const long long ps = pos[r];
    const long long b = c * CH;
    if (ps < b && ps >= b - CH) {
      owner = true;
      cfirst = (int)c;
      clast = (pos[r + 1] - 1) / CH;
    }
  }
  const bool is_long = owner && (clast - cfirst) >= 16;
  T total = T(0);
  if (owner && !is_long) {
    total = part_last[cfirst - 1];
    for (int cc = cfirst; cc <= clast; ++cc) total = total + part_first[cc];
  }
  unsigned long long m = __ballot(is_long);
  while (m) {
    const int src = __builtin_ctzll(m);
    m &= m - 1;
    const int cs = __shfl(cfirst, src, 64);
    const int cl = __shfl(clast, src, 64);
    T part = T(0);
    for (int cc = cs + lane; cc <= cl; cc += 64) part = part + part_first[cc];
    part = group_sum<64>(part);
    if (lane == src) total = part_last[cfirst - 1] + part;
  }
  return total;
}

// The same call convention; the owner writes y[r] (+)= the row's total.
template <typename T, int CH>
__device__ __forceinline__ void rowsplit_complete_row(long long c, int nchunks, const int *__restrict__ pos,
                                                      const int *__restrict__ chunk_row,
                                                      const T *__restrict__ part_first,
                                                      const T *__restrict__ part_last, T *y, int accumulate) {
  bool owner;
  int r;
  const T total = rowsplit_row_total<T, CH>(c, nchunks, pos, chunk_row, part_first, part_last, owner, r);
  if (owner) y[r] = accumulate ? total + y[r] : total;
}

}  // namespace lapis
