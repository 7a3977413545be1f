// Column-blocked SpMV: the variant for matrices whose gathered vector x does not
// fit the 4 MB L2 of an XCD (uniformly random columns over millions of columns).
//
// A gather that misses L2 pulls a 128-byte line for 8 useful bytes, so the plain
// CSR kernels spend the HBM bandwidth on line fills.  Here the matrix is copied
// once, at plan time, into an order in which every wavefront owns 1024 consecutive
// rows and walks their non-zeros slice by slice of x (slice = 2^s consecutive
// columns, 1 MB of x by default).  All wavefronts are resident at once and start
// together, so at any moment the whole chip is gathering from the same few slices
// and they stay in L2.  Row sums are accumulated in LDS (one accumulator per row
// of the wave's block) and written to y once.
//
// Entry format: one uint32 = (row within the block << col_bits) | column, plus the
// value; 12 bytes per non-zero for fp64, exactly the CSR footprint, and `pos` is
// only read at row-block boundaries.
#include <hipcub/hipcub.hpp>

#include <algorithm>
#include <cstdlib>

#include "common.hpp"
#include "plan.hpp"

namespace lapis {



template <bool NT>
__device__ __forceinline__ void load4v(const double *p, double (&o)[4]) {
  v2d a = ldv<NT>(reinterpret_cast<const v2d *>(p));
  v2d b = ldv<NT>(reinterpret_cast<const v2d *>(p + 2));
  o[0] = a.x; o[1] = a.y; o[2] = b.x; o[3] = b.y;
}
template <bool NT>
__device__ __forceinline__ void load4v(const float *p, float (&o)[4]) {
  v4f a = ldv<NT>(reinterpret_cast<const v4f *>(p));
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
}

// One wavefront per block of RB rows.  STEPS * 256 entries are in flight per loop trip.
// Loads EPL consecutive entries (index words and values) for one lane.
template <bool NT>
__device__ __forceinline__ void load_entries(const unsigned *bi, const double *bv, long long p, unsigned (&i)[4],
                                             double (&v)[4]) {
  v4i c = ldv<NT>(reinterpret_cast<const v4i *>(bi + p));
  i[0] = (unsigned)c.x; i[1] = (unsigned)c.y; i[2] = (unsigned)c.z; i[3] = (unsigned)c.w;
  load4v<NT>(bv + p, v);
}
template <bool NT>
__device__ __forceinline__ void load_entries(const unsigned *bi, const float *bv, long long p, unsigned (&i)[4],
                                             float (&v)[4]) {
  v4i c = ldv<NT>(reinterpret_cast<const v4i *>(bi + p));
  i[0] = (unsigned)c.x; i[1] = (unsigned)c.y; i[2] = (unsigned)c.z; i[3] = (unsigned)c.w;
  load4v<NT>(bv + p, v);
}
template <bool NT, typename T>
__device__ __forceinline__ void load_entries(const unsigned *bi, const T *bv, long long p, unsigned (&i)[2], T (&v)[2]) {
  v2i c = ldv<NT>(reinterpret_cast<const v2i *>(bi + p));
  i[0] = (unsigned)c.x; i[1] = (unsigned)c.y;
  v[0] = ldv<NT>(bv + p);
  v[1] = ldv<NT>(bv + p + 1);
}
template <bool NT, typename T>
__device__ __forceinline__ void load_entries(const unsigned *bi, const T *bv, long long p, unsigned (&i)[1], T (&v)[1]) {
  i[0] = ldv<NT>(bi + p);
  v[0] = ldv<NT>(bv + p);
}

// One wavefront per block of RB rows.  A trip handles STEPS * 64 * EPL entries; the
// index words and values of the NEXT trip are already in flight while this trip's
// gathers run, so the streamed arrays keep many loads outstanding while the window
// of x a wavefront is gathering from stays small.  PAD ints of unused LDS per
// workgroup set how many workgroups fit a CU (an even spread keeps the wavefronts
// of the chip moving through x at the same pace).
template <typename T, int RB, int WAVES, int STEPS, int EPL, int PAD, bool NT>
__global__ __launch_bounds__(64 * WAVES) void spmv_colblock_kernel(int nrows, int nnz, int col_bits,
                                                                   const int *__restrict__ pos,
                                                                   const unsigned *__restrict__ bidx,
                                                                   const T *__restrict__ bval,
                                                                   const T *__restrict__ x, T *__restrict__ y,
                                                                   unsigned pace_fp) {
  // row sums are doubles for both value types: ds_add_f32 runs at a tenth of the rate
  // of ds_add_f64 on this chip
  __shared__ double lds[WAVES * RB + PAD];
  const long long t0 = wall_clock64();
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const int rb = __builtin_amdgcn_readfirstlane((int)(blockIdx.x * WAVES + wave));
  const long long row0 = (long long)rb * RB;
  if (row0 >= nrows) return;
  const int rows_here = (int)std::min<long long>(RB, nrows - row0);
  double *acc = lds + wave * RB;
  if (PAD > 0 && nrows < 0) lds[WAVES * RB + lane] = 0.0;  // keeps the padding allocated
#pragma unroll
  for (int i = 0; i < RB / 64; ++i) acc[i * 64 + lane] = 0.0;
  wave_lds_sync();

  const int start = pos[row0];
  const int end = pos[row0 + rows_here];
  const unsigned col_mask = (1u << col_bits) - 1u;
  constexpr int STEP = 64 * EPL;
  constexpr int TRIP = STEPS * STEP;
  const long long first = start & ~3;
  // entries of one trip, guarded: used for the first trip and the tail
  auto guarded_trip = [&](long long off) {
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
#pragma unroll
      for (int e = 0; e < EPL; ++e) {
        const long long p = off + s * STEP + lane * EPL + e;
        if (p >= start && p < end) {
          const unsigned ie = bidx[p];
          const T pe = bval[p] * x[ie & col_mask];
          lds_add(acc + (ie >> col_bits), (double)pe);
        }
      }
    }
  };
  long long off = first;
  if (off < end) {
    guarded_trip(off);
    off += TRIP;
  }
  // interior trips: aligned vector loads, next trip prefetched
  if (off + TRIP <= end) {
    unsigned ci[STEPS][EPL];
    T cv[STEPS][EPL];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) load_entries<NT>(bidx, bval, off + s * STEP + lane * EPL, ci[s], cv[s]);
    for (; off + TRIP <= end; off += TRIP) {
      unsigned ni[STEPS][EPL];
      T nv[STEPS][EPL];
      const bool more = off + 2 * TRIP <= end;
      if (more) {
#pragma unroll
        for (int s = 0; s < STEPS; ++s)
          load_entries<NT>(bidx, bval, off + TRIP + s * STEP + lane * EPL, ni[s], nv[s]);
      }
      if (pace_fp) {
        // time-triggered pacing: entry number k of a wavefront's range is not gathered
        // before t0 + k * pace.  Wavefronts that run ahead wait here (the loads of the
        // next trip are already in flight), so all of them cross x at the same pace and
        // the part of x in use stays small enough for L2.  The clock only moves
        // forward: the wait always ends.
        const long long target = t0 + (((off - first) * (long long)pace_fp) >> 16);
        while (wall_clock64() < target) __builtin_amdgcn_s_sleep(2);
      }
      T pr[STEPS][EPL];
#pragma unroll
      for (int s = 0; s < STEPS; ++s)
#pragma unroll
        for (int e = 0; e < EPL; ++e) pr[s][e] = cv[s][e] * x[ci[s][e] & col_mask];
#pragma unroll
      for (int s = 0; s < STEPS; ++s)
#pragma unroll
        for (int e = 0; e < EPL; ++e) lds_add(acc + (ci[s][e] >> col_bits), (double)pr[s][e]);
      if (more) {
#pragma unroll
        for (int s = 0; s < STEPS; ++s)
#pragma unroll
          for (int e = 0; e < EPL; ++e) {
            ci[s][e] = ni[s][e];
            cv[s][e] = nv[s][e];
          }
      }
    }
  }
  if (off < end) guarded_trip(off);
  wave_lds_sync();
  for (int i = lane; i < rows_here; i += 64) y[row0 + i] = T(acc[i]) + y[row0 + i];
}

// key = (row block << (32 + slice bits)) | (slice << 32) | (row in block << col_bits) | column
__global__ __launch_bounds__(256) void colblock_keys_kernel(int nrows, int rows_per_block, int col_bits,
                                                            int slice_log2, int slice_bits,
                                                            const int *__restrict__ pos,
                                                            const int *__restrict__ crd,
                                                            unsigned long long *__restrict__ keys) {
  // one wavefront per row: coalesced over the row's entries
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= nrows) return;
  const unsigned long long rb = (unsigned long long)(row / rows_per_block);
  const unsigned long long rl = (unsigned long long)(row % rows_per_block);
  const int s = pos[row], e = pos[row + 1];
  for (int j = s + lane; j < e; j += 64) {
    const unsigned long long c = (unsigned long long)(unsigned)crd[j];
    keys[j] = (rb << (32 + slice_bits)) | ((c >> slice_log2) << 32) | (rl << col_bits) | c;
  }
}

__global__ __launch_bounds__(256) void colblock_low_word_kernel(long long n, const unsigned long long *__restrict__ keys,
                                                                unsigned *__restrict__ out) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = (unsigned)keys[i];
}


namespace {
__global__ __launch_bounds__(256) void iota_kernel(long long n, unsigned *__restrict__ out) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = (unsigned)i;
}
template <typename T>
__global__ __launch_bounds__(256) void gather_values_kernel(long long n, const unsigned *__restrict__ perm,
                                                            const T *__restrict__ val, T *__restrict__ out) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < n) out[i] = val[perm[i]];
}
}  // namespace

int sort_keys_with_perm(const unsigned long long *keys_in, int64_t nnz, int begin_bit, int end_bit, unsigned long long **keys_out,
                        unsigned **perm, hipStream_t st) {
  unsigned *iota = nullptr;
  void *temp = nullptr;
  size_t temp_bytes = 0;
  *keys_out = nullptr;
  *perm = nullptr;
  auto fail = [&](hipError_t e, const char *what) {
    if (iota) (void)hipFree(iota);
    if (temp) (void)hipFree(temp);
    if (*keys_out) (void)hipFree(*keys_out);
    if (*perm) (void)hipFree(*perm);
    *keys_out = nullptr;
    *perm = nullptr;
    return set_error(LAPIS_HIP_ERR_RUNTIME, "csr_plan_build_colblock: %s failed: %s", what, hipGetErrorString(e));
  };
  hipError_t e;
  if ((e = hipMalloc(&iota, sizeof(unsigned) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(keys_out, sizeof(unsigned long long) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(perm, sizeof(unsigned) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  hipLaunchKernelGGL(iota_kernel, dim3((unsigned)ceil_div(nnz, 256)), dim3(256), 0, st, (long long)nnz, iota);
  if ((e = hipGetLastError()) != hipSuccess) return fail(e, "index kernel");
  if ((e = hipcub::DeviceRadixSort::SortPairs(nullptr, temp_bytes, keys_in, *keys_out, iota, *perm, (int)nnz, begin_bit, end_bit,
                                              st)) != hipSuccess)
    return fail(e, "radix sort sizing");
  if ((e = hipMalloc(&temp, temp_bytes ? temp_bytes : 1)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipcub::DeviceRadixSort::SortPairs(temp, temp_bytes, keys_in, *keys_out, iota, *perm, (int)nnz, begin_bit, end_bit,
                                              st)) != hipSuccess)
    return fail(e, "radix sort");
  if ((e = hipStreamSynchronize(st)) != hipSuccess) return fail(e, "synchronize");
  (void)hipFree(iota);
  (void)hipFree(temp);
  return LAPIS_HIP_OK;
}

template <typename T>
int gather_values(const unsigned *perm, const T *val, T *out, int64_t nnz, hipStream_t st) {
  if (nnz == 0) return LAPIS_HIP_OK;
  hipLaunchKernelGGL((gather_values_kernel<T>), dim3((unsigned)ceil_div(nnz, 256)), dim3(256), 0, st, (long long)nnz,
                     perm, val, out);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}
template int gather_values<double>(const unsigned *, const double *, double *, int64_t, hipStream_t);
template int gather_values<float>(const unsigned *, const float *, float *, int64_t, hipStream_t);

void free_colblock(lapis_hip_csr_plan *p) {
  if (p->colblock_idx) (void)hipFree(p->colblock_idx);
  if (p->colblock_val) (void)hipFree(p->colblock_val);
  if (p->colblock_perm) (void)hipFree(p->colblock_perm);
  p->colblock_perm = nullptr;
  p->colblock_src_crd = p->colblock_src_val = nullptr;
  if (p->colblock_tile_ptr) (void)hipFree(p->colblock_tile_ptr);
  if (p->colblock_units) (void)hipFree(p->colblock_units);
  if (p->colblock_long_rows) (void)hipFree(p->colblock_long_rows);
  if (p->colblock_fault) (void)hipFree(p->colblock_fault);
  p->colblock_fault = nullptr;
  p->colblock_pc_prod = 0;
  p->colblock_tile_ptr = nullptr;
  p->colblock_units = nullptr;
  p->colblock_long_rows = nullptr;
  p->colblock_nunits = 0;
  p->colblock_nlong = 0;
  p->colblock_idx = nullptr;
  p->colblock_val = nullptr;
  p->colblock_built = false;
}

template <typename T, int RB, int WAVES, int STEPS, int EPL>
int launch_colblock_cfg(const lapis_hip_csr_plan *p, const int *pos, const T *x, T *y, hipStream_t st) {
  const int64_t nrb = ceil_div(p->stats.nrows, RB);
  const dim3 grid((unsigned)ceil_div(nrb, WAVES)), block(64 * WAVES);
  if (p->nontemporal)
    launch_timed(spmv_colblock_kernel<T, RB, WAVES, STEPS, EPL, 0, true>, grid, block, st, (int)p->stats.nrows,
                 (int)p->stats.nnz, p->colblock_col_bits, pos, (const unsigned *)p->colblock_idx,
                 (const T *)p->colblock_val, x, y, p->colblock_pace_fp);
  else
    launch_timed(spmv_colblock_kernel<T, RB, WAVES, STEPS, EPL, 0, false>, grid, block, st, (int)p->stats.nrows,
                 (int)p->stats.nnz, p->colblock_col_bits, pos, (const unsigned *)p->colblock_idx,
                 (const T *)p->colblock_val, x, y, p->colblock_pace_fp);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}

template <typename T, int RB, int WAVES>
int launch_colblock_rb(const lapis_hip_csr_plan *p, const int *pos, const T *x, T *y, hipStream_t st) {
  switch (p->colblock_steps * 10 + p->colblock_epl) {
    case 22: return launch_colblock_cfg<T, RB, WAVES, 2, 2>(p, pos, x, y, st);
    case 12: return launch_colblock_cfg<T, RB, WAVES, 1, 2>(p, pos, x, y, st);
    case 24: return launch_colblock_cfg<T, RB, WAVES, 2, 4>(p, pos, x, y, st);
    case 14: return launch_colblock_cfg<T, RB, WAVES, 1, 4>(p, pos, x, y, st);
    default:
      return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "colblock: no kernel for steps=%d entries-per-lane=%d",
                       p->colblock_steps, p->colblock_epl);
  }
}

template <typename T>
int launch_colblock(const lapis_hip_csr_plan *p, const int *pos, const int *crd, const T *val, const T *x, T *y,
                    hipStream_t st) {
  if (p->colblock_group) return launch_colgroup<T>(p, x, y, st);
  if (p->colblock_rows == 512)
    return p->colblock_pad ? launch_colblock_rb<T, 512, 8>(p, pos, x, y, st)
                           : launch_colblock_rb<T, 512, 4>(p, pos, x, y, st);
  return p->colblock_pad ? launch_colblock_rb<T, 1024, 8>(p, pos, x, y, st)
                         : launch_colblock_rb<T, 1024, 4>(p, pos, x, y, st);
}
template int launch_colblock<double>(const lapis_hip_csr_plan *, const int *, const int *, const double *,
                                     const double *, double *, hipStream_t);
template int launch_colblock<float>(const lapis_hip_csr_plan *, const int *, const int *, const float *, const float *,
                                    float *, hipStream_t);

namespace {

// Finds the pace (clock ticks per entry) at which the paced kernel runs fastest:
// times the free-running kernel, then paced runs aimed at 50 % .. 95 % of that time,
// and keeps the best (or no pacing if nothing beats the free run by 2 %).
template <typename T>
int calibrate_pace(lapis_hip_csr_plan *p, hipStream_t st) {
  const int64_t nrows = p->stats.nrows, ncols = p->stats.ncols;
  int dev = 0, clock_khz = 0;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&clock_khz, hipDeviceAttributeWallClockRate, dev) != hipSuccess || clock_khz <= 0)
    return LAPIS_HIP_OK;  // no clock rate, no pacing
  T *x = nullptr, *y = nullptr;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  auto done = [&](int rc) {
    if (x) (void)hipFree(x);
    if (y) (void)hipFree(y);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
    return rc;
  };
  if (hipMalloc(&x, sizeof(T) * (size_t)ncols) != hipSuccess || hipMalloc(&y, sizeof(T) * (size_t)nrows) != hipSuccess ||
      hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess)
    return done(LAPIS_HIP_OK);
  (void)hipMemsetAsync(x, 0, sizeof(T) * (size_t)ncols, st);
  (void)hipMemsetAsync(y, 0, sizeof(T) * (size_t)nrows, st);
  auto time_ms = [&](unsigned pace) -> double {
    p->colblock_pace_fp = pace;
    double best = 1e30;
    for (int rep = 0; rep < 4; ++rep) {
      (void)hipEventRecord(e0, st);
      if (launch_colblock<T>(p, p->pos, nullptr, nullptr, x, y, st) != LAPIS_HIP_OK) return 1e30;
      (void)hipEventRecord(e1, st);
      if (hipEventSynchronize(e1) != hipSuccess) return 1e30;
      float ms = 0.f;
      (void)hipEventElapsedTime(&ms, e0, e1);
      if (rep > 0) best = std::min<double>(best, ms);
    }
    return best;
  };
  const double free_ms = time_ms(0);
  const double entries_per_wave = (double)p->stats.nnz / (double)ceil_div(nrows, p->colblock_rows);  // per row block
  unsigned best_pace = 0;
  int best_pct = 0;
  double best_ms = free_ms * 0.98;
  auto try_pct = [&](int pct) {
    const double target_ticks = free_ms * 1e-3 * (pct / 100.0) * (double)clock_khz * 1e3;
    const double fp = target_ticks / entries_per_wave * 65536.0;
    if (fp < 1.0 || fp > 4.0e9) return;
    const double ms = time_ms((unsigned)fp);
    if (getenv("LAPIS_HIP_VERBOSE")) fprintf(stderr, "lapis_hip:   pace target %d%% -> %.4f ms\n", pct, ms);
    if (ms < best_ms) {
      best_ms = ms;
      best_pace = (unsigned)fp;
      best_pct = pct;
    }
  };
  for (int pct = 50; pct <= 95; pct += 5) try_pct(pct);  // coarse
  if (best_pct) {
    const int centre = best_pct;
    for (int pct = centre - 4; pct <= centre + 4; ++pct)  // fine
      if (pct != centre) try_pct(pct);
  }
  p->colblock_pace_fp = best_pace;
  p->colblock_free_ms = free_ms;
  p->colblock_paced_ms = best_pace ? best_ms : free_ms;
  if (getenv("LAPIS_HIP_VERBOSE"))
    fprintf(stderr, "lapis_hip: column-blocked SpMV calibration: free %.4f ms, paced %.4f ms at %.3f ticks/entry\n",
            free_ms, p->colblock_paced_ms, best_pace / 65536.0);
  return done(LAPIS_HIP_OK);
}


template <typename T>
int build(lapis_hip_csr_plan *p, const int32_t *crd, const T *val, int slice_log2, hipStream_t st) {
  const int64_t nnz = p->stats.nnz, nrows = p->stats.nrows;
  const int col_bits = std::max(1, bits_for(p->stats.ncols));
  if (col_bits + kColblockRowBits > 32)
    return set_error(LAPIS_HIP_ERR_NO_TILING,
                     "csr_plan_build_colblock: %lld columns need %d bits, more than the %d an entry has room for",
                     (long long)p->stats.ncols, col_bits, 32 - kColblockRowBits);
  {
    const char *rows = getenv("LAPIS_HIP_COLBLOCK_ROWS");
    p->colblock_rows = (rows && atoi(rows) == 512) ? 512 : 1024;
  }
  const int rb_bits = bits_for(ceil_div(nrows, p->colblock_rows));
  // the 64-bit sort key holds row block | slice | 32-bit entry word: slices must be
  // coarse enough for all three to fit
  slice_log2 = std::max(slice_log2, col_bits - (32 - rb_bits));
  const int slice_bits = std::max(0, col_bits - slice_log2);
  const int end_bit = 32 + slice_bits + rb_bits;
  if (end_bit > 64 || slice_log2 < 0 || slice_log2 > 31)
    return set_error(LAPIS_HIP_ERR_NO_TILING, "csr_plan_build_colblock: sort key needs %d bits", end_bit);

  unsigned long long *keys_in = nullptr, *keys_out = nullptr;
  T *val_out = nullptr;
  unsigned *idx = nullptr, *perm = nullptr;
  auto fail = [&](hipError_t e, const char *what) {
    if (keys_in) (void)hipFree(keys_in);
    if (keys_out) (void)hipFree(keys_out);
    if (val_out) (void)hipFree(val_out);
    if (idx) (void)hipFree(idx);
    if (perm) (void)hipFree(perm);
    return set_error(LAPIS_HIP_ERR_RUNTIME, "csr_plan_build_colblock: %s failed: %s", what, hipGetErrorString(e));
  };
  hipError_t e;
  if ((e = hipMalloc(&keys_in, sizeof(unsigned long long) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(&val_out, sizeof(T) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(&idx, sizeof(unsigned) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  hipLaunchKernelGGL(colblock_keys_kernel, dim3((unsigned)ceil_div(nrows, 4)), dim3(256), 0, st, (int)nrows,
                     p->colblock_rows, col_bits,
                     slice_log2, slice_bits, p->pos, crd, keys_in);
  if ((e = hipGetLastError()) != hipSuccess) return fail(e, "key kernel");
  {
    const int rc = sort_keys_with_perm(keys_in, nnz, 0, end_bit, &keys_out, &perm, st);
    if (rc != LAPIS_HIP_OK) {
      (void)hipFree(keys_in);
      (void)hipFree(val_out);
      (void)hipFree(idx);
      return rc;
    }
    if (gather_values<T>(perm, val, val_out, nnz, st) != LAPIS_HIP_OK) return fail(hipGetLastError(), "value gather");
  }
  hipLaunchKernelGGL(colblock_low_word_kernel, dim3((unsigned)ceil_div(nnz, 256)), dim3(256), 0, st, (long long)nnz,
                     keys_out, idx);
  if ((e = hipGetLastError()) != hipSuccess) return fail(e, "index kernel");
  if ((e = hipStreamSynchronize(st)) != hipSuccess) return fail(e, "synchronize");
  (void)hipFree(keys_in);
  (void)hipFree(keys_out);
  free_colblock(p);
  p->colblock_group = 0;
  p->colblock_perm = perm;
  p->colblock_src_crd = crd;
  p->colblock_src_val = val;
  {
    const char *stp = getenv("LAPIS_HIP_COLBLOCK_STEPS"), *epl = getenv("LAPIS_HIP_COLBLOCK_EPL"),
               *pad = getenv("LAPIS_HIP_COLBLOCK_PAD");
    p->colblock_steps = stp ? atoi(stp) : 2;
    p->colblock_epl = epl ? atoi(epl) : 2;
    p->colblock_pad = pad ? atoi(pad) : 0;
  }
  p->colblock_idx = idx;
  p->colblock_val = val_out;
  p->colblock_value_bytes = (int)sizeof(T);
  p->colblock_col_bits = col_bits;
  p->colblock_slice_log2 = slice_log2;
  p->colblock_built = true;
  p->colblock_pace_fp = 0;
  const char *pace_env = getenv("LAPIS_HIP_COLBLOCK_PACE");
  if (pace_env && atoi(pace_env) == 0) return LAPIS_HIP_OK;
  return calibrate_pace<T>(p, st);
}
}  // namespace

}  // namespace lapis

using namespace lapis;

extern "C" int lapis_hip_csr_plan_build_colblock(lapis_hip_csr_plan *plan, const int32_t *crd, const void *val,
                                                 int value_bytes, int layout, int slice_log2_cols,
                                                 lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(plan, "csr_plan_build_colblock: null plan");
  LAPIS_REQUIRE(value_bytes == 4 || value_bytes == 8, "csr_plan_build_colblock: value_bytes must be 4 or 8");
  LAPIS_REQUIRE(layout == LAPIS_HIP_COLBLOCK_AUTO || layout == LAPIS_HIP_COLBLOCK_WAVE ||
                    layout == LAPIS_HIP_COLBLOCK_GROUP,
                "csr_plan_build_colblock: unknown layout %d", layout);
  const lapis_hip_csr_stats &s = plan->stats;
  LAPIS_REQUIRE(s.nnz > 0, "csr_plan_build_colblock: the matrix has no non-zeros");
  LAPIS_REQUIRE(crd && val, "csr_plan_build_colblock: null coordinates or values");
  // the kernels of both layouts step through the copy in trips of up to 16384 entries with int offsets,
  // and the copy is padded: keep a margin below 2^31 so that no offset wraps
  if (s.nnz > (int64_t)INT32_MAX - (1 << 20))
    return set_error(LAPIS_HIP_ERR_NO_TILING, "csr_plan_build_colblock: %lld non-zeros leave no room below 2^31",
                     (long long)s.nnz);
  if (layout == LAPIS_HIP_COLBLOCK_AUTO) layout = LAPIS_HIP_COLBLOCK_GROUP;
  int col_bits = 1;
  while ((1LL << col_bits) < s.ncols) ++col_bits;
  const bool group = layout == LAPIS_HIP_COLBLOCK_GROUP;
  // default slice: 1 MB of x for the per-wavefront layout; 2 MB of fp64 / 1 MB of fp32
  // (what an entry word has room for) for the workgroup layout
  if (slice_log2_cols <= 0) slice_log2_cols = group ? 18 : (value_bytes == 8 ? 17 : 18);
  slice_log2_cols = std::min(slice_log2_cols, col_bits);
  hipStream_t st = as_stream(stream);
  int rc;
  if (group)
    rc = value_bytes == 8 ? build_colgroup<double>(plan, crd, static_cast<const double *>(val), slice_log2_cols, st)
                          : build_colgroup<float>(plan, crd, static_cast<const float *>(val), slice_log2_cols, st);
  else
    rc = value_bytes == 8 ? build<double>(plan, crd, static_cast<const double *>(val), slice_log2_cols, st)
                          : build<float>(plan, crd, static_cast<const float *>(val), slice_log2_cols, st);
  if (rc == LAPIS_HIP_OK) {
    plan->stats.kernel = LAPIS_HIP_SPMV_COLBLOCK;
    plan->stats.colblock_layout = layout;
    plan->stats.width = 0;
    plan->stats.chunk = 0;
  }
  return rc;
}

extern "C" int lapis_hip_csr_plan_update_values(lapis_hip_csr_plan *plan, const void *val, int value_bytes,
                                                lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(plan, "csr_plan_update_values: null plan");
  if (!plan->colblock_built) return LAPIS_HIP_OK;  // the CSR kernels read the caller's values on every call
  LAPIS_REQUIRE(val, "csr_plan_update_values: null values");
  if (value_bytes != plan->colblock_value_bytes)
    return set_error(LAPIS_HIP_ERR_PLAN_MISMATCH, "csr_plan_update_values: the copy holds %d-byte values, called with %d",
                     plan->colblock_value_bytes, value_bytes);
  LAPIS_REQUIRE(plan->colblock_perm, "csr_plan_update_values: the copy was built without its permutation");
  hipStream_t st = as_stream(stream);
  const int rc = value_bytes == 8
                     ? gather_values<double>(plan->colblock_perm, static_cast<const double *>(val),
                                             static_cast<double *>(plan->colblock_val), plan->stats.nnz, st)
                     : gather_values<float>(plan->colblock_perm, static_cast<const float *>(val),
                                            static_cast<float *>(plan->colblock_val), plan->stats.nnz, st);
  if (rc == LAPIS_HIP_OK) plan->colblock_src_val = val;
  return rc;
}

extern "C" int lapis_hip_csr_plan_check(lapis_hip_csr_plan *plan, lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(plan, "csr_plan_check: null plan");
  hipStream_t st = as_stream(stream);
  LAPIS_HIP_TRY(hipStreamSynchronize(st));
  if (!plan->colblock_fault) return LAPIS_HIP_OK;
  int fault = 0;
  LAPIS_HIP_TRY(hipMemcpy(&fault, plan->colblock_fault, sizeof(int), hipMemcpyDeviceToHost));
  if (fault != 0)
    return set_error(LAPIS_HIP_ERR_RUNTIME,
                     "csr_plan_check: a wavefront of the workgroup-blocked SpMV gave up waiting for its partner");
  return LAPIS_HIP_OK;
}

namespace {
int analyze_with_layout(lapis_hip_csr_plan *plan, const int32_t *crd, const void *val, int value_bytes, int layout,
                        lapis_hip_stream_t stream);
}

extern "C" int lapis_hip_csr_plan_analyze(lapis_hip_csr_plan *plan, const int32_t *crd, const void *val, int value_bytes,
                                          lapis_hip_stream_t stream) {
  return analyze_with_layout(plan, crd, val, value_bytes, LAPIS_HIP_COLBLOCK_AUTO, stream);
}

extern "C" int lapis_hip_csr_plan_analyze_reproducible(lapis_hip_csr_plan *plan, const int32_t *crd, const void *val,
                                                       int value_bytes, lapis_hip_stream_t stream) {
  return analyze_with_layout(plan, crd, val, value_bytes, LAPIS_HIP_COLBLOCK_WAVE, stream);
}

namespace {
int analyze_with_layout(lapis_hip_csr_plan *plan, const int32_t *crd, const void *val, int value_bytes, int layout,
                        lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(plan, "csr_plan_analyze: null plan");
  LAPIS_REQUIRE(value_bytes == 4 || value_bytes == 8, "csr_plan_analyze: value_bytes must be 4 or 8");
  if (!plan->stats.colblock_recommended || plan->stats.nnz == 0) return LAPIS_HIP_OK;
  LAPIS_REQUIRE(crd && val, "csr_plan_analyze: null coordinates or values");
  const int want_group = layout == LAPIS_HIP_COLBLOCK_WAVE ? 0 : 1;
  if (plan->colblock_built && plan->colblock_value_bytes == value_bytes && plan->colblock_src_crd == crd &&
      plan->colblock_group == want_group) {
    plan->stats.kernel = LAPIS_HIP_SPMV_COLBLOCK;  // the copy is there: bring its values up to date
    return lapis_hip_csr_plan_update_values(plan, val, value_bytes, stream);
  }
  const int rc = lapis_hip_csr_plan_build_colblock(plan, crd, val, value_bytes, layout, 0, stream);
  // a matrix the tiling has no room for keeps its CSR kernel: that is an answer, not an error
  if (rc == LAPIS_HIP_ERR_NO_TILING) {
    (void)set_error(LAPIS_HIP_OK, "%s", "");
    return LAPIS_HIP_OK;
  }
  return rc;
}
}  // namespace
