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

template <bool NT, typename V>
__device__ __forceinline__ V ldv(const V *p) {
  if (NT) return load_stream(p);
  return *p;
}

__device__ __forceinline__ void lds_add(double *p, double v) { unsafeAtomicAdd(p, v); }

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


// ---- workgroup-blocked variant -------------------------------------------------
// One WORKGROUP per block of `rows_per_block` rows (16 per thread: 16384 rows for
// 1024 threads), row sums in LDS shared by the whole group.  The entries of one
// tile (row block x slice of x) are stored in COLUMN order, and the threads of the
// group take them 64 neighbours per wavefront: with about as many entries in a tile
// as the slice has 128-byte lines, neighbouring lanes fall into the same lines (the
// address unit merges them into one request) and the wavefronts of the group reuse
// each other's lines in the CU's vector cache.  Measured on a 1 MB window of
// doubles: 430 G gathers/s in this order against 205 G/s in random order, which is
// the request rate of L2.
//
// Entry word = (row within the block << slice_log2) | column within the slice;
// tile_ptr[block * (nslices + 1) + s] is where slice s of the block starts.
// Different wavefronts add to the same row sums with LDS atomics, so the order of
// the additions of one row, and with it the last bits of the result, can differ
// from run to run.
template <typename T, int THREADS, int U, bool NT>
__global__ __launch_bounds__(THREADS) void spmv_colgroup_kernel(int nrows, int rows_per_block, int nslices,
                                                                int nsplit, int slice_log2,
                                                                const int *__restrict__ tile_ptr,
                                                                const unsigned *__restrict__ bidx,
                                                                const T *__restrict__ bval, const T *__restrict__ x,
                                                                T *__restrict__ y) {
  extern __shared__ __align__(16) unsigned char colgroup_lds[];
  // Row sums are doubles for both value types: ds_add_f32 runs at a tenth of the rate of
  // ds_add_f64 on this chip (203 against 1780 G adds/s over random words, measured).
  double *acc = reinterpret_cast<double *>(colgroup_lds);
  const int tid = threadIdx.x;
  // workgroup = (row block, share of the slices): with fewer row blocks than CUs the
  // slices of a block are split over `nsplit` workgroups, which then add into y atomically
  const int block = (int)(blockIdx.x / (unsigned)nsplit);
  const int share = (int)(blockIdx.x % (unsigned)nsplit);
  const int s_first = (int)((long long)share * nslices / nsplit);
  const int s_last = (int)((long long)(share + 1) * nslices / nsplit);  // exclusive
  const long long row0 = (long long)block * rows_per_block;
  const int rows_here = (int)std::min<long long>(rows_per_block, nrows - row0);
  if (s_first >= s_last) return;  // uniform over the workgroup
  for (int i = tid; i < rows_per_block; i += THREADS) acc[i] = 0.0;
  // the tile pointers of this workgroup's slices go to LDS: read from memory at every
  // tile border they would stall the issue of the next trip's loads
  int *tp = reinterpret_cast<int *>(acc + rows_per_block) - s_first;  // indexed by slice
  {
    const int *gtp = tile_ptr + (long long)block * (nslices + 1);
    for (int i = s_first + tid; i <= s_last; i += THREADS) tp[i] = gtp[i];
  }
  __syncthreads();
  const unsigned cmask = (1u << slice_log2) - 1u;
  constexpr int TRIP = U * THREADS;
  // A trip is up to TRIP consecutive entries of ONE tile, [off, min(off + TRIP, end)):
  // the slice, and with it the base of the gathers, is uniform over the workgroup.
  // (Trips running across tile borders, and a third trip's gathers kept in flight,
  // both measured 10-30 % slower.)
  int s = s_first, off = tp[s_first], end = tp[s_first + 1];
  while (off >= end && s + 1 < s_last) {
    ++s;
    end = tp[s + 1];
  }
  bool have = off < end;
  unsigned ci[U];
  T cv[U];
  auto load_trip = [&](int o, int e, unsigned (&li)[U], T (&lv)[U]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int p = o + u * THREADS + tid;
      if (p < e) {
        li[u] = ldv<NT>(bidx + p);
        lv[u] = ldv<NT>(bval + p);
      }
    }
  };
  if (have) load_trip(off, end, ci, cv);
  while (have) {
    int ns = s, noff = off + TRIP, nend = end;
    while (noff >= nend && ns + 1 < s_last) {  // tile finished: the next one starts where it ends
      ++ns;
      noff = nend;
      nend = tp[ns + 1];
    }
    const bool more = noff < nend;
    unsigned ni[U];
    T nv[U];
    if (more) load_trip(noff, nend, ni, nv);  // in flight while this trip gathers and adds
    const T *xs = x + ((long long)s << slice_log2);
    T pr[U];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (off + u * THREADS + tid < end) pr[u] = cv[u] * xs[ci[u] & cmask];
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (off + u * THREADS + tid < end) lds_add(acc + (ci[u] >> slice_log2), (double)pr[u]);
    if (more) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        ci[u] = ni[u];
        cv[u] = nv[u];
      }
    }
    s = ns;
    off = noff;
    end = nend;
    have = more;
  }
  __syncthreads();
  if (nsplit == 1) {
    for (int i = tid; i < rows_here; i += THREADS) y[row0 + i] = T(acc[i]) + y[row0 + i];
  } else {
    for (int i = tid; i < rows_here; i += THREADS) unsafeAtomicAdd(y + row0 + i, T(acc[i]));
  }
}

// Rows of `long_threshold` entries or more stay out of the workgroup-blocked copy
// (hundreds of entries of one row in a tile would all hit one LDS word) and are
// taken from the CSR arrays in pieces, one workgroup per piece.  A piece is the part
// of one row that falls into one slice of x (columns are sorted, so it is a
// contiguous run of the row), cut to at most kLongPiece entries, and the pieces are
// listed slice by slice: the chip then gathers from one or two slices of x at a
// time, as the blocked kernel does, instead of every long row sweeping all of x.
constexpr int kLongPiece = 4096;

__global__ __launch_bounds__(256) void long_row_flag_kernel(int nrows, int long_threshold,
                                                            const int *__restrict__ pos, int *__restrict__ flag) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < nrows) flag[i] = pos[i + 1] - pos[i] >= long_threshold ? 1 : 0;
}

__global__ __launch_bounds__(256) void long_row_list_kernel(int nrows, const int *__restrict__ flag,
                                                            const int *__restrict__ rank, int *__restrict__ rows) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i < nrows && flag[i]) rows[rank[i]] = (int)i;
}

// first entry of row [s, e) whose column is >= col
__device__ __forceinline__ int lower_bound_col(const int *__restrict__ crd, int s, int e, long long col) {
  while (s < e) {
    const int mid = s + ((e - s) >> 1);
    if (crd[mid] < col) s = mid + 1; else e = mid;
  }
  return s;
}

// thread t = (slice, k-th long row).  FILL = false: counts[t] = pieces of that part of the
// row; FILL = true: writes them, pieces[3*j..3*j+2] = row, first entry, one past the last.
template <bool FILL>
__global__ __launch_bounds__(256) void long_piece_kernel(int nlong, int nslices, int slice_log2,
                                                         const int *__restrict__ rows, const int *__restrict__ pos,
                                                         const int *__restrict__ crd, int *__restrict__ counts,
                                                         const int *__restrict__ first_piece,
                                                         int *__restrict__ pieces) {
  const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
  if (t >= (long long)nlong * nslices) return;
  const int slice = (int)(t / nlong), row = rows[t % nlong];
  const int s = pos[row], e = pos[row + 1];
  const int b0 = lower_bound_col(crd, s, e, (long long)slice << slice_log2);
  const int b1 = lower_bound_col(crd, b0, e, (long long)(slice + 1) << slice_log2);
  if (!FILL) {
    counts[t] = (b1 - b0 + kLongPiece - 1) / kLongPiece;
  } else {
    int j = first_piece[t];
    for (int b = b0; b < b1; b += kLongPiece, ++j) {
      pieces[3 * j] = row;
      pieces[3 * j + 1] = b;
      pieces[3 * j + 2] = min(b + kLongPiece, b1);
    }
  }
}

// One workgroup per piece: every thread has all of its (at most kLongPiece / 256)
// entries in flight at once, first the index words and values, then the gathers.
template <typename T>
__global__ __launch_bounds__(256) void spmv_long_piece_kernel(const int *__restrict__ pieces,
                                                              const int *__restrict__ crd,
                                                              const T *__restrict__ val, const T *__restrict__ x,
                                                              T *__restrict__ y) {
  __shared__ T lds4[4];
  constexpr int U = kLongPiece / 256;
  const int row = pieces[3 * blockIdx.x], first = pieces[3 * blockIdx.x + 1], last = pieces[3 * blockIdx.x + 2];
  int c[U];
  T a[U], g[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const int j = first + u * 256 + (int)threadIdx.x;
    if (j < last) {
      c[u] = load_stream(crd + j);
      a[u] = load_stream(val + j);
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (first + u * 256 + (int)threadIdx.x < last) g[u] = x[c[u]];
  T sum[4] = {T(0), T(0), T(0), T(0)};
#pragma unroll
  for (int u = 0; u < U; ++u)
    if (first + u * 256 + (int)threadIdx.x < last) sum[u & 3] = sum[u & 3] + a[u] * g[u];
  T v = (sum[0] + sum[1]) + (sum[2] + sum[3]);
  v = group_sum<64>(v);
  if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = v;
  __syncthreads();
  if (threadIdx.x == 0) unsafeAtomicAdd(y + row, (lds4[0] + lds4[1]) + (lds4[2] + lds4[3]));
}

// key = (row block << (col_bits + row_bits)) | (column << row_bits) | row in block:
// sorted, the entries of a row block come slice by slice and by column inside a slice
__global__ __launch_bounds__(256) void colgroup_keys_kernel(int nrows, int row_bits, int col_bits, int nblocks,
                                                            int long_threshold, const int *__restrict__ pos,
                                                            const int *__restrict__ crd,
                                                            unsigned long long *__restrict__ keys) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= nrows) return;
  const int s = pos[row], e = pos[row + 1];
  // entries of a long row sort behind every block: the copy ends where they begin
  const unsigned long long rb = e - s >= long_threshold ? (unsigned long long)nblocks : (unsigned long long)(row >> row_bits);
  const unsigned long long rl = (unsigned long long)(row & ((1LL << row_bits) - 1));
  for (int j = s + lane; j < e; j += 64) {
    const unsigned long long c = (unsigned long long)(unsigned)crd[j];
    keys[j] = (rb << (col_bits + row_bits)) | (c << row_bits) | rl;
  }
}

__global__ __launch_bounds__(256) void colgroup_entry_kernel(long long n, int row_bits, int slice_log2,
                                                             const unsigned long long *__restrict__ keys,
                                                             unsigned *__restrict__ out) {
  const long long i = (long long)blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const unsigned long long k = keys[i];
  const unsigned rl = (unsigned)(k & ((1ull << row_bits) - 1ull));
  const unsigned cs = (unsigned)((k >> row_bits) & ((1ull << slice_log2) - 1ull));
  out[i] = (rl << slice_log2) | cs;
}

// tile_ptr[b * (nslices + 1) + s] = first sorted entry whose key is >= (block b, slice s)
__global__ __launch_bounds__(256) void colgroup_tile_ptr_kernel(long long nnz, int nblocks, int nslices, int row_bits,
                                                                int col_bits, int slice_log2,
                                                                const unsigned long long *__restrict__ keys,
                                                                int *__restrict__ tile_ptr) {
  const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
  if (t >= (long long)nblocks * (nslices + 1)) return;
  const unsigned long long b = (unsigned long long)(t / (nslices + 1));
  const int s = (int)(t % (nslices + 1));
  const unsigned long long target =
      s == nslices ? ((b + 1) << (col_bits + row_bits))
                   : ((b << (col_bits + row_bits)) | (((unsigned long long)s << slice_log2) << row_bits));
  long long lo = 0, hi = nnz;
  while (lo < hi) {
    const long long mid = (lo + hi) >> 1;
    if (keys[mid] < target) lo = mid + 1; else hi = mid;
  }
  tile_ptr[t] = (int)lo;
}

void free_colblock(lapis_hip_csr_plan *p) {
  if (p->colblock_idx) (void)hipFree(p->colblock_idx);
  if (p->colblock_val) (void)hipFree(p->colblock_val);
  if (p->colblock_tile_ptr) (void)hipFree(p->colblock_tile_ptr);
  if (p->colblock_pieces) (void)hipFree(p->colblock_pieces);
  p->colblock_tile_ptr = nullptr;
  p->colblock_pieces = nullptr;
  p->colblock_npieces = 0;
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

template <typename T, int THREADS, int U, bool NT>
int launch_colgroup_cfg(const lapis_hip_csr_plan *p, const int *crd, const T *val, const T *x, T *y, hipStream_t st) {
  auto kernel = spmv_colgroup_kernel<T, THREADS, U, NT>;
  const int slices_per_group = (int)ceil_div(p->colblock_nslices, p->colblock_nsplit) + 2;
  const size_t lds_bytes = sizeof(double) * (size_t)p->colblock_rows + sizeof(int) * (size_t)slices_per_group;
  static bool attribute_set = false;  // one per instantiation; more than 64 KB of dynamic LDS has to be asked for
  if (!attribute_set) {
    LAPIS_HIP_TRY(hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
    attribute_set = true;
  }
  const dim3 grid((unsigned)(p->colblock_nblocks * p->colblock_nsplit)), block(THREADS);
  const bool pieces = p->colblock_npieces > 0;
  if (pieces) LAPIS_REQUIRE(crd && val, "spmv: this plan takes its long rows from crd/val, which are null");
  // kernel timing covers the whole product: from the start of the blocked kernel to the
  // end of the long-row kernel when there is one
  hipEvent_t e0 = nullptr, e1 = nullptr;
  const bool timed = timing_next_events(&e0, &e1);
  if (timed)
    hipExtLaunchKernelGGL(kernel, grid, block, lds_bytes, st, e0, pieces ? nullptr : e1, 0, (int)p->stats.nrows,
                          p->colblock_rows, p->colblock_nslices, p->colblock_nsplit, p->colblock_slice_log2,
                          (const int *)p->colblock_tile_ptr, (const unsigned *)p->colblock_idx,
                          (const T *)p->colblock_val, x, y);
  else
    hipLaunchKernelGGL(kernel, grid, block, lds_bytes, st, (int)p->stats.nrows, p->colblock_rows,
                       p->colblock_nslices, p->colblock_nsplit, p->colblock_slice_log2,
                       (const int *)p->colblock_tile_ptr, (const unsigned *)p->colblock_idx,
                       (const T *)p->colblock_val, x, y);
  LAPIS_LAUNCH_CHECK();
  if (pieces) {
    const dim3 pgrid((unsigned)p->colblock_npieces), pblock(256);
    if (timed)
      hipExtLaunchKernelGGL(spmv_long_piece_kernel<T>, pgrid, pblock, 0, st, nullptr, e1, 0,
                            (const int *)p->colblock_pieces, crd, val, x, y);
    else
      hipLaunchKernelGGL(spmv_long_piece_kernel<T>, pgrid, pblock, 0, st, (const int *)p->colblock_pieces, crd, val, x,
                         y);
    LAPIS_LAUNCH_CHECK();
  }
  return LAPIS_HIP_OK;
}

template <typename T, int THREADS>
int launch_colgroup_threads(const lapis_hip_csr_plan *p, const int *crd, const T *val, const T *x, T *y,
                            hipStream_t st) {
  const bool nt = p->nontemporal;
  if (p->colblock_epl == 4)
    return nt ? launch_colgroup_cfg<T, THREADS, 4, true>(p, crd, val, x, y, st)
              : launch_colgroup_cfg<T, THREADS, 4, false>(p, crd, val, x, y, st);
  return nt ? launch_colgroup_cfg<T, THREADS, 8, true>(p, crd, val, x, y, st)
            : launch_colgroup_cfg<T, THREADS, 8, false>(p, crd, val, x, y, st);
}

template <typename T>
int launch_colgroup(const lapis_hip_csr_plan *p, const int *crd, const T *val, const T *x, T *y, hipStream_t st) {
  switch (p->colblock_rows) {
    case 16384: return launch_colgroup_threads<T, 1024>(p, crd, val, x, y, st);
    case 8192: return launch_colgroup_threads<T, 512>(p, crd, val, x, y, st);
    case 4096: return launch_colgroup_threads<T, 256>(p, crd, val, x, y, st);
    default:
      return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "colblock: no workgroup kernel for %d rows per block",
                       p->colblock_rows);
  }
}

template <typename T>
int launch_colblock(const lapis_hip_csr_plan *p, const int *pos, const int *crd, const T *val, const T *x, T *y,
                    hipStream_t st) {
  if (p->colblock_group) return launch_colgroup<T>(p, crd, val, x, y, st);
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
int bits_for(int64_t n) {  // bits needed for values 0..n-1
  int b = 0;
  while (b < 62 && (1LL << b) < n) ++b;
  return b;
}

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


// Builds the workgroup-blocked layout (see spmv_colgroup_kernel) and the list of
// long-row pieces.
template <typename T>
int build_group(lapis_hip_csr_plan *p, const int32_t *crd, const T *val, int slice_log2, hipStream_t st) {
  const int64_t nnz = p->stats.nnz, nrows = p->stats.nrows;
  const int col_bits = std::max(1, bits_for(p->stats.ncols));
  auto env_or = [](const char *name, int fallback) {
    const char *v = getenv(name);
    return v ? atoi(v) : fallback;
  };
  // 16 rows per thread.  The more rows share a tile, the more lanes fall into one line
  // of x, so the block is as large as LDS allows unless the matrix is smaller.
  int rows = env_or("LAPIS_HIP_COLBLOCK_ROWS", 0);
  if (rows != 4096 && rows != 8192 && rows != 16384) rows = nrows > 8192 ? 16384 : (nrows > 4096 ? 8192 : 4096);
  const int row_bits = bits_for(rows);
  slice_log2 = std::min(slice_log2, 32 - row_bits);  // an entry word holds row in block | column in slice
  const int nblocks = (int)ceil_div(nrows, rows);
  const int64_t nslices64 = ceil_div(p->stats.ncols, 1LL << slice_log2);
  const int end_bit = bits_for((int64_t)nblocks + 1) + col_bits + row_bits;
  if (end_bit > 64 || slice_log2 < 1 || nslices64 * nblocks > (1LL << 26))
    return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT,
                     "csr_plan_build_colblock: %d row blocks x %lld slices of 2^%d columns is not a usable tiling",
                     nblocks, (long long)nslices64, slice_log2);
  const int nslices = (int)nslices64;
  // fewer row blocks than CUs: several workgroups share a block, each with a share of its slices
  int nsplit = env_or("LAPIS_HIP_COLBLOCK_SPLIT", 0);
  if (nsplit < 1) nsplit = (int)ceil_div(device_cu_count(), nblocks);
  nsplit = std::max(1, std::min(nsplit, nslices));
  if (ceil_div(nslices, nsplit) > 6000)  // their tile pointers sit in LDS beside 128 KB of row sums
    return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT,
                     "csr_plan_build_colblock: %d slices of 2^%d columns per workgroup; use larger slices", nslices,
                     slice_log2);
  const int long_threshold = std::max(64, env_or("LAPIS_HIP_COLBLOCK_LONG", 32768));

  unsigned long long *keys_in = nullptr, *keys_out = nullptr;
  T *val_out = nullptr;
  unsigned *idx = nullptr;
  int *tile_ptr = nullptr, *piece_count = nullptr, *piece_first = nullptr, *pieces = nullptr, *long_rows = nullptr;
  void *temp = nullptr, *scan_temp = nullptr;
  size_t temp_bytes = 0, scan_bytes = 0;
  auto release = [&](bool all) {
    if (keys_in) (void)hipFree(keys_in);
    if (keys_out) (void)hipFree(keys_out);
    if (temp) (void)hipFree(temp);
    if (scan_temp) (void)hipFree(scan_temp);
    if (piece_count) (void)hipFree(piece_count);
    if (piece_first) (void)hipFree(piece_first);
    if (long_rows) (void)hipFree(long_rows);
    if (all) {
      if (val_out) (void)hipFree(val_out);
      if (idx) (void)hipFree(idx);
      if (tile_ptr) (void)hipFree(tile_ptr);
      if (pieces) (void)hipFree(pieces);
    }
  };
  auto fail = [&](hipError_t e, const char *what) {
    release(true);
    return set_error(LAPIS_HIP_ERR_RUNTIME, "csr_plan_build_colblock: %s failed: %s", what, hipGetErrorString(e));
  };
  hipError_t e;

  // long rows: their list, then their pieces slice by slice
  int npieces = 0;
  if (p->stats.max_row_len >= long_threshold) {
    const dim3 row_grid((unsigned)ceil_div(nrows, 256));
    auto scan = [&](int *in, int *out, int64_t n) -> hipError_t {
      size_t need = 0;
      hipError_t se = hipcub::DeviceScan::ExclusiveSum(nullptr, need, in, out, (int)n, st);
      if (se != hipSuccess) return se;
      if (need > scan_bytes) {
        if (scan_temp) (void)hipFree(scan_temp);
        scan_temp = nullptr;
        if ((se = hipMalloc(&scan_temp, need)) != hipSuccess) return se;
        scan_bytes = need;
      }
      return hipcub::DeviceScan::ExclusiveSum(scan_temp, need, in, out, (int)n, st);
    };
    auto total_of = [&](const int *count, const int *first, int64_t n, int *total) -> hipError_t {
      int tail[2] = {0, 0};
      hipError_t ce = hipMemcpyAsync(&tail[0], count + (n - 1), sizeof(int), hipMemcpyDeviceToHost, st);
      if (ce == hipSuccess) ce = hipMemcpyAsync(&tail[1], first + (n - 1), sizeof(int), hipMemcpyDeviceToHost, st);
      if (ce == hipSuccess) ce = hipStreamSynchronize(st);
      *total = tail[0] + tail[1];
      return ce;
    };
    int nlong = 0;
    if ((e = hipMalloc(&piece_count, sizeof(int) * (size_t)nrows)) != hipSuccess) return fail(e, "hipMalloc");
    if ((e = hipMalloc(&piece_first, sizeof(int) * (size_t)nrows)) != hipSuccess) return fail(e, "hipMalloc");
    hipLaunchKernelGGL(long_row_flag_kernel, row_grid, dim3(256), 0, st, (int)nrows, long_threshold, p->pos,
                       piece_count);
    if ((e = hipGetLastError()) != hipSuccess) return fail(e, "long row flag kernel");
    if ((e = scan(piece_count, piece_first, nrows)) != hipSuccess) return fail(e, "scan");
    if ((e = total_of(piece_count, piece_first, nrows, &nlong)) != hipSuccess) return fail(e, "copy");
    if (nlong > 0) {
      const int64_t nparts = (int64_t)nlong * nslices;
      if (nparts > (1LL << 28))
        return fail(hipErrorInvalidValue, "listing the long rows (too many rows x slices)");
      if ((e = hipMalloc(&long_rows, sizeof(int) * (size_t)nlong)) != hipSuccess) return fail(e, "hipMalloc");
      hipLaunchKernelGGL(long_row_list_kernel, row_grid, dim3(256), 0, st, (int)nrows, piece_count, piece_first,
                         long_rows);
      if ((e = hipGetLastError()) != hipSuccess) return fail(e, "long row list kernel");
      (void)hipFree(piece_count);
      (void)hipFree(piece_first);
      piece_count = piece_first = nullptr;
      if ((e = hipMalloc(&piece_count, sizeof(int) * (size_t)nparts)) != hipSuccess) return fail(e, "hipMalloc");
      if ((e = hipMalloc(&piece_first, sizeof(int) * (size_t)nparts)) != hipSuccess) return fail(e, "hipMalloc");
      const dim3 part_grid((unsigned)ceil_div(nparts, 256));
      hipLaunchKernelGGL(long_piece_kernel<false>, part_grid, dim3(256), 0, st, nlong, nslices, slice_log2, long_rows,
                         p->pos, crd, piece_count, (const int *)nullptr, (int *)nullptr);
      if ((e = hipGetLastError()) != hipSuccess) return fail(e, "piece count kernel");
      if ((e = scan(piece_count, piece_first, nparts)) != hipSuccess) return fail(e, "scan");
      if ((e = total_of(piece_count, piece_first, nparts, &npieces)) != hipSuccess) return fail(e, "copy");
      if (npieces > 0) {
        if ((e = hipMalloc(&pieces, sizeof(int) * 3 * (size_t)npieces)) != hipSuccess) return fail(e, "hipMalloc");
        hipLaunchKernelGGL(long_piece_kernel<true>, part_grid, dim3(256), 0, st, nlong, nslices, slice_log2, long_rows,
                           p->pos, crd, (int *)nullptr, piece_first, pieces);
        if ((e = hipGetLastError()) != hipSuccess) return fail(e, "piece fill kernel");
      }
    }
  }

  const size_t ntiles = (size_t)nblocks * ((size_t)nslices + 1);
  if ((e = hipMalloc(&keys_in, sizeof(unsigned long long) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(&keys_out, sizeof(unsigned long long) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(&val_out, sizeof(T) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(&idx, sizeof(unsigned) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(&tile_ptr, sizeof(int) * ntiles)) != hipSuccess) return fail(e, "hipMalloc");
  hipLaunchKernelGGL(colgroup_keys_kernel, dim3((unsigned)ceil_div(nrows, 4)), dim3(256), 0, st, (int)nrows, row_bits,
                     col_bits, nblocks, long_threshold, p->pos, crd, keys_in);
  if ((e = hipGetLastError()) != hipSuccess) return fail(e, "key kernel");
  if ((e = hipcub::DeviceRadixSort::SortPairs(nullptr, temp_bytes, keys_in, keys_out, val, val_out, (int)nnz, 0,
                                              end_bit, st)) != hipSuccess)
    return fail(e, "radix sort sizing");
  if ((e = hipMalloc(&temp, temp_bytes ? temp_bytes : 1)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipcub::DeviceRadixSort::SortPairs(temp, temp_bytes, keys_in, keys_out, val, val_out, (int)nnz, 0, end_bit,
                                              st)) != hipSuccess)
    return fail(e, "radix sort");
  hipLaunchKernelGGL(colgroup_entry_kernel, dim3((unsigned)ceil_div(nnz, 256)), dim3(256), 0, st, (long long)nnz,
                     row_bits, slice_log2, keys_out, idx);
  if ((e = hipGetLastError()) != hipSuccess) return fail(e, "entry kernel");
  hipLaunchKernelGGL(colgroup_tile_ptr_kernel, dim3((unsigned)ceil_div((int64_t)ntiles, 256)), dim3(256), 0, st,
                     (long long)nnz, nblocks, nslices, row_bits, col_bits, slice_log2, keys_out, tile_ptr);
  if ((e = hipGetLastError()) != hipSuccess) return fail(e, "tile pointer kernel");
  if ((e = hipStreamSynchronize(st)) != hipSuccess) return fail(e, "synchronize");
  release(false);
  free_colblock(p);
  p->colblock_group = 1;
  p->colblock_epl = env_or("LAPIS_HIP_COLBLOCK_EPL", 8);  // entries per thread and trip
  p->colblock_rows = rows;
  p->colblock_nblocks = nblocks;
  p->colblock_nslices = nslices;
  p->colblock_nsplit = nsplit;
  p->colblock_long_threshold = long_threshold;
  p->colblock_npieces = npieces;
  p->colblock_pieces = pieces;
  p->colblock_tile_ptr = tile_ptr;
  p->colblock_idx = idx;
  p->colblock_val = val_out;
  p->colblock_value_bytes = (int)sizeof(T);
  p->colblock_col_bits = col_bits;
  p->colblock_slice_log2 = slice_log2;
  p->colblock_built = true;
  p->colblock_pace_fp = 0;  // the workgroups keep pace by themselves: pacing measured no gain here
  p->colblock_free_ms = p->colblock_paced_ms = 0.0;
  if (getenv("LAPIS_HIP_VERBOSE"))
    fprintf(stderr,
            "lapis_hip: workgroup-blocked copy: %d blocks of %d rows x %d slices of 2^%d columns, %d workgroups per "
            "block, %d pieces of rows with >= %d entries\n",
            nblocks, rows, nslices, slice_log2, nsplit, npieces, long_threshold);
  return LAPIS_HIP_OK;
}

template <typename T>
int build(lapis_hip_csr_plan *p, const int32_t *crd, const T *val, int slice_log2, hipStream_t st) {
  const int64_t nnz = p->stats.nnz, nrows = p->stats.nrows;
  const int col_bits = std::max(1, bits_for(p->stats.ncols));
  if (col_bits + kColblockRowBits > 32)
    return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT,
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
    return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "csr_plan_build_colblock: sort key needs %d bits", end_bit);

  unsigned long long *keys_in = nullptr, *keys_out = nullptr;
  T *val_out = nullptr;
  unsigned *idx = nullptr;
  void *temp = nullptr;
  size_t temp_bytes = 0;
  auto fail = [&](hipError_t e, const char *what) {
    if (keys_in) (void)hipFree(keys_in);
    if (keys_out) (void)hipFree(keys_out);
    if (val_out) (void)hipFree(val_out);
    if (idx) (void)hipFree(idx);
    if (temp) (void)hipFree(temp);
    return set_error(LAPIS_HIP_ERR_RUNTIME, "csr_plan_build_colblock: %s failed: %s", what, hipGetErrorString(e));
  };
  hipError_t e;
  if ((e = hipMalloc(&keys_in, sizeof(unsigned long long) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(&keys_out, sizeof(unsigned long long) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(&val_out, sizeof(T) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipMalloc(&idx, sizeof(unsigned) * (size_t)nnz)) != hipSuccess) return fail(e, "hipMalloc");
  hipLaunchKernelGGL(colblock_keys_kernel, dim3((unsigned)ceil_div(nrows, 4)), dim3(256), 0, st, (int)nrows,
                     p->colblock_rows, col_bits,
                     slice_log2, slice_bits, p->pos, crd, keys_in);
  if ((e = hipGetLastError()) != hipSuccess) return fail(e, "key kernel");
  if ((e = hipcub::DeviceRadixSort::SortPairs(nullptr, temp_bytes, keys_in, keys_out, val, val_out, (int)nnz, 0,
                                              end_bit, st)) != hipSuccess)
    return fail(e, "radix sort sizing");
  if ((e = hipMalloc(&temp, temp_bytes ? temp_bytes : 1)) != hipSuccess) return fail(e, "hipMalloc");
  if ((e = hipcub::DeviceRadixSort::SortPairs(temp, temp_bytes, keys_in, keys_out, val, val_out, (int)nnz, 0, end_bit,
                                              st)) != hipSuccess)
    return fail(e, "radix sort");
  hipLaunchKernelGGL(colblock_low_word_kernel, dim3((unsigned)ceil_div(nnz, 256)), dim3(256), 0, st, (long long)nnz,
                     keys_out, idx);
  if ((e = hipGetLastError()) != hipSuccess) return fail(e, "index kernel");
  if ((e = hipStreamSynchronize(st)) != hipSuccess) return fail(e, "synchronize");
  (void)hipFree(keys_in);
  (void)hipFree(keys_out);
  (void)hipFree(temp);
  free_colblock(p);
  p->colblock_group = 0;
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
    rc = value_bytes == 8 ? build_group<double>(plan, crd, static_cast<const double *>(val), slice_log2_cols, st)
                          : build_group<float>(plan, crd, static_cast<const float *>(val), slice_log2_cols, st);
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
