// CSR SpMV for gfx950: the plan (row-length statistics -> kernel choice) and the
// three kernel families it chooses from.
//
//   y[i] = y[i] + sum_{j in [pos[i], pos[i+1])} val[j] * x[crd[j]]
//
// replaces the TeamPolicy / ThreadVectorRange lambda the reference emits for
// tests/Dialect/Kokkos/loop_mapping_2.mlir.gold:12-37.
#include <algorithm>
#include <cmath>
#include <cstdlib>
#include <cstring>

#include "common.hpp"
#include "plan.hpp"
#include "rowsplit_fix.hpp"

namespace lapis {

// ------------------------------------------------------------------------------
// Device helpers
// ------------------------------------------------------------------------------
template <bool NT, typename V>
__device__ __forceinline__ V ld(const V *p) {
  if (NT) return load_stream(p);
  return *p;
}

template <bool NT>
__device__ __forceinline__ void load4(const double *p, double (&o)[4]) {
  v2d a = ld<NT>(reinterpret_cast<const v2d *>(p));
  v2d b = ld<NT>(reinterpret_cast<const v2d *>(p + 2));
  o[0] = a.x; o[1] = a.y; o[2] = b.x; o[3] = b.y;
}
template <bool NT>
__device__ __forceinline__ void load4(const float *p, float (&o)[4]) {
  v4f a = ld<NT>(reinterpret_cast<const v4f *>(p));
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
}
__device__ __forceinline__ void store4_lds(double *p, const double (&v)[4]) {
  v2d a, b;
  a.x = v[0]; a.y = v[1]; b.x = v[2]; b.y = v[3];
  *reinterpret_cast<v2d *>(p) = a;
  *reinterpret_cast<v2d *>(p + 2) = b;
}
__device__ __forceinline__ void store4_lds(float *p, const float (&v)[4]) {
  v4f a;
  a.x = v[0]; a.y = v[1]; a.z = v[2]; a.w = v[3];
  *reinterpret_cast<v4f *>(p) = a;
}

// Stage val[j]*x[crd[j]] for j in [g0, g0+count) into buf[0..count): 4 consecutive
// non-zeros per lane, 256 per wavefront step.  `g0` is a multiple of 4 so that the
// 128-bit loads are aligned when VEC is set; `avail` = number of array elements
// that exist from g0 on (loads never touch anything at or beyond g0+avail).
template <typename T, int CAP, bool VEC, bool NT>
__device__ __forceinline__ void stage_products(T *buf, int lane, const int *__restrict__ crd,
                                               const T *__restrict__ val, const T *__restrict__ x,
                                               int g0, int count, int avail) {
  constexpr int STEPS = CAP / 256;
  if (VEC && count == CAP && avail >= CAP) {
    // full tile: no guards, all index/value loads can be issued before the gathers
    v4i cc[STEPS];
    T vv[STEPS][4];
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int k = s * 256 + lane * 4;
      cc[s] = ld<NT>(reinterpret_cast<const v4i *>(crd + g0 + k));
      load4<NT>(val + g0 + k, vv[s]);
    }
#pragma unroll
    for (int s = 0; s < STEPS; ++s) {
      const int k = s * 256 + lane * 4;
      T pr[4];
      pr[0] = vv[s][0] * x[cc[s].x];
      pr[1] = vv[s][1] * x[cc[s].y];
      pr[2] = vv[s][2] * x[cc[s].z];
      pr[3] = vv[s][3] * x[cc[s].w];
      store4_lds(buf + k, pr);
    }
    return;
  }
#pragma unroll
  for (int s = 0; s < STEPS; ++s) {
    const int k = s * 256 + lane * 4;
    if (k >= count) continue;
    if (VEC && k + 4 <= avail) {
      v4i c4 = ld<NT>(reinterpret_cast<const v4i *>(crd + g0 + k));
      T v4[4], pr[4];
      load4<NT>(val + g0 + k, v4);
      pr[0] = v4[0] * x[c4.x];
      pr[1] = v4[1] * x[c4.y];
      pr[2] = v4[2] * x[c4.z];
      pr[3] = v4[3] * x[c4.w];
      store4_lds(buf + k, pr);
    } else {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        if (k + e < count && k + e < avail) {
          const int cj = ld<NT>(crd + g0 + k + e);
          const T vj = ld<NT>(val + g0 + k + e);
          buf[k + e] = vj * x[cj];
        }
      }
    }
  }
}

// One row piece per lane out of the staged tile: buf[lo..hi) summed in ascending
// order by the owning lane; pieces longer than LONG_PIECE are summed by the whole
// wavefront instead (strided partial sums + DPP reduction).
constexpr int kLongPiece = 48;

template <typename T>
__device__ __forceinline__ T sum_piece(const T *buf, int lane, int lo, int hi) {
  const int len = hi - lo;
  const bool is_long = len > kLongPiece;
  T acc = T(0);
  if (!is_long) {
    for (int j = lo; j < hi; ++j) acc = acc + buf[j];
  }
  unsigned long long m = __ballot(is_long);
  while (m) {
    const int src = __builtin_ctzll(m);
    m &= m - 1;
    const int llo = __shfl(lo, src, 64);
    const int lhi = __shfl(hi, src, 64);
    T part = T(0);
    for (int j = llo + lane; j < lhi; j += 64) part = part + buf[j];
    part = group_sum<64>(part);
    if (lane == src) acc = part;
  }
  return acc;
}

// ------------------------------------------------------------------------------
// Kernel family 1: W lanes per row
// ------------------------------------------------------------------------------
template <typename T, int W, bool NT>
__global__ __launch_bounds__(256) void spmv_subwarp_kernel(int nrows, const int *__restrict__ pos,
                                                           const int *__restrict__ crd,
                                                           const T *__restrict__ val,
                                                           const T *__restrict__ x, T *__restrict__ y) {
  const long long gid = (long long)blockIdx.x * 256 + threadIdx.x;
  const long long row = gid / W;
  const int sub = (int)(gid % W);
  int j = 0, end = 0;
  if (row < nrows) {
    j = pos[row] + sub;
    end = pos[row + 1];
  }
  T acc = T(0);
  for (; j < end; j += W) {
    const int cj = ld<NT>(crd + j);
    const T vj = ld<NT>(val + j);
    acc = acc + vj * x[cj];
  }
  acc = group_sum<W>(acc);
  if (sub == 0 && row < nrows) y[row] = acc + y[row];
}

// ------------------------------------------------------------------------------
// Kernel family 2: 64 consecutive rows per wavefront, products staged in LDS
// ------------------------------------------------------------------------------
template <typename T, int CAP, int WAVES, bool VEC, bool NT>
__global__ __launch_bounds__(64 * WAVES) void spmv_rowblock_kernel(
    int nrows, int nnz, const int *__restrict__ pos, const int *__restrict__ crd,
    const T *__restrict__ val, const T *__restrict__ x, T *__restrict__ y, int xcd_map) {
  __shared__ T lds[WAVES * CAP];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const unsigned blk = xcd_map ? xcd_contiguous_block(blockIdx.x, gridDim.x) : blockIdx.x;
  const long long row0 = ((long long)blk * WAVES + wave) * 64;
  if (row0 >= nrows) return;
  T *buf = lds + wave * CAP;
  const long long row = row0 + lane;
  const bool valid = row < nrows;
  int ps = nnz, pe = nnz;
  if (valid) {
    ps = pos[row];
    pe = pos[row + 1];
  }
  const int base = __shfl(ps, 0, 64);
  const int end = __shfl(pe, 63, 64);
  T acc = T(0);
  for (long long off = base & ~3; off < end; off += CAP) {
    const int g0 = (int)off;
    const int count = (int)std::min<long long>(CAP, end - off);
    const int avail = (int)std::min<long long>(CAP, (long long)nnz - off);
    stage_products<T, CAP, VEC, NT>(buf, lane, crd, val, x, g0, count, avail);
    wave_lds_sync();
    const int lo = std::max(ps, g0) - g0;
    const int hi = (int)(std::min<long long>(pe, off + CAP) - off);
    const T part = sum_piece(buf, lane, lo, hi);
    acc = acc + part;
    wave_lds_sync();
  }
  if (valid) y[row] = acc + y[row];
}

// ------------------------------------------------------------------------------
// Kernel family 3: CH consecutive non-zeros per wavefront (row split)
// ------------------------------------------------------------------------------
// chunk_row[c] = row owning non-zero c*CH (c < nchunks), chunk_row[nchunks] = nrows.
// A row piece that is a whole row is written to y at once; a piece of a row that
// started in an earlier chunk goes to part_first[c], a piece of a row that
// continues into the next chunk to part_last[c]; the fix-up kernel adds them up.
// With `xy_chunk` (square matrices) the wavefront also leaves xy_chunk[c] = sum of
// x[r] * (A x)[r] over the rows r that lie wholly inside its chunk, lanes summed in a
// fixed order: the p.Ap of a CG iteration without a second pass over the vectors.
template <typename T, int CH, int WAVES, bool VEC, bool NT>
__global__ __launch_bounds__(64 * WAVES) void spmv_nnzsplit_kernel(
    int nrows, int nnz, int nchunks, const int *__restrict__ pos, const int *__restrict__ crd,
    const T *__restrict__ val, const T *__restrict__ x, T *__restrict__ y,
    const int *__restrict__ chunk_row, T *__restrict__ part_first, T *__restrict__ part_last, int accumulate,
    int xcd_map, double *__restrict__ xy_chunk) {
  __shared__ T lds[WAVES * CH];
  const int lane = threadIdx.x & 63;
  const int wave = threadIdx.x >> 6;
  const unsigned blk = xcd_map ? xcd_contiguous_block(blockIdx.x, gridDim.x) : blockIdx.x;
  const int c = __builtin_amdgcn_readfirstlane((int)(blk * WAVES + wave));
  if (c >= nchunks) return;
  T *buf = lds + wave * CH;
  const int e0 = c * CH;
  const int len = std::min(CH, nnz - e0);
  const long long e1 = (long long)e0 + len;
  const int r0 = chunk_row[c];
  const int r1 = std::min(chunk_row[c + 1], nrows - 1);

  stage_products<T, CH, VEC, NT>(buf, lane, crd, val, x, e0, len, len);
  wave_lds_sync();

  double xy = 0.0;
  for (long long rb = r0; rb <= r1;) {
    const long long r = rb + lane;
    int ps = 0, pe = 0;
    T xr = T(0);  // asked for together with the positions, so that its latency hides behind the row sums
    if (r <= r1) {
      ps = ld<NT>(pos + r);
      pe = ld<NT>(pos + r + 1);
      if (xy_chunk) xr = x[r];
    }
    const int lo = std::max(ps, e0) - e0;
    const int hi = (int)(std::min<long long>(pe, e1) - e0);
    const T acc = sum_piece(buf, lane, lo, hi);
    if (hi > lo) {
      const bool starts = ps >= e0;
      const bool ends = pe <= e1;
      if (starts && ends) {
        y[r] = accumulate ? acc + y[r] : acc;
        xy = xy + (double)xr * (double)acc;
      } else if (!starts)
        part_first[c] = acc;
      else
        part_last[c] = acc;
    }
    // Runs of empty rows must not cost a trip per 64 of them: after 64 rows without a
    // single entry the next row that has one is found by bisection (positions are
    // sorted), and rows that start at or behind the end of the chunk end the walk.
    const int ps_first = __shfl(ps, 0, 64);
    const int pe_last = __shfl(pe, 63, 64);
    if (ps_first >= e1) break;
    long long next = rb + 64;
    if (next <= r1 && pe_last == ps_first) {
      long long lo_r = next, hi_r = r1;  // first row in [next, r1] with pos[row + 1] > pe_last, else r1
      while (lo_r < hi_r) {
        const long long mid = (lo_r + hi_r) >> 1;
        if (pos[mid + 1] > pe_last) hi_r = mid; else lo_r = mid + 1;
      }
      next = lo_r;
    }
    rb = next;
  }
  if (xy_chunk) {
    xy = group_sum<64>(xy);
    if (lane == 0) xy_chunk[c] = xy;
  }
}

// One thread per chunk boundary c (1 <= c < nchunks); see rowsplit_complete_row.
template <typename T, int CH>
__global__ __launch_bounds__(256) void spmv_nnzsplit_fixup_kernel(
    int nchunks, const int *__restrict__ pos, const int *__restrict__ chunk_row,
    const T *__restrict__ part_first, const T *__restrict__ part_last, T *__restrict__ y, int accumulate) {
  const long long c = (long long)blockIdx.x * 256 + threadIdx.x + 1;
  rowsplit_complete_row<T, CH>(c, nchunks, pos, chunk_row, part_first, part_last, y, accumulate);
}

// ------------------------------------------------------------------------------
// Plan analysis kernels
// ------------------------------------------------------------------------------
struct DeviceStats {
  int min_len;
  int max_len;
  int bad;  // bit 0: positions decrease; bit 1: coordinate out of range
  int pad;
  unsigned long long empty_rows;
  double sum_sq;
  unsigned long long span_sum;  // sum over 1024-non-zero chunks of (max column - min column)
  unsigned long long near[4];   // non-zeros with |column - row| <= 32, 64, 128, 256
};

// Every statistic is first reduced over the block and reaches the one DeviceStats with one
// atomic per block and field: tens of thousands of atomics on the same few words would take
// longer than reading the matrix.
__global__ __launch_bounds__(256) void row_stats_kernel(int nrows, const int *__restrict__ pos,
                                                        DeviceStats *st) {
  __shared__ int s_mn[4], s_mx[4], s_bad[4];
  __shared__ unsigned long long s_empt[4];
  __shared__ double s_sq[4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int mn = INT32_MAX, mx = 0, bad = 0;
  unsigned long long empt = 0;
  double sq = 0.0;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nrows;
       i += (long long)gridDim.x * 256) {
    const int len = pos[i + 1] - pos[i];
    if (len < 0) bad = 1;
    mn = std::min(mn, len);
    mx = std::max(mx, len);
    empt += (len == 0);
    sq += (double)len * (double)len;
  }
  for (int o = 32; o > 0; o >>= 1) {
    mn = std::min(mn, __shfl_xor(mn, o, 64));
    mx = std::max(mx, __shfl_xor(mx, o, 64));
    bad |= __shfl_xor(bad, o, 64);
    empt += __shfl_xor(empt, o, 64);
    sq += __shfl_xor(sq, o, 64);
  }
  if (lane == 0) {
    s_mn[wave] = mn;
    s_mx[wave] = mx;
    s_bad[wave] = bad;
    s_empt[wave] = empt;
    s_sq[wave] = sq;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) {
      mn = std::min(mn, s_mn[w]);
      mx = std::max(mx, s_mx[w]);
      bad |= s_bad[w];
      empt += s_empt[w];
      sq += s_sq[w];
    }
    atomicMin(&st->min_len, mn);
    atomicMax(&st->max_len, mx);
    if (bad) atomicOr(&st->bad, 1);
    if (empt) atomicAdd(&st->empty_rows, empt);
    atomicAdd(&st->sum_sq, sq);
  }
}

// One wavefront per 1024 consecutive non-zeros, wavefronts striding over the chunks:
//  * range check of the coordinates;
//  * the column span (max - min) of the chunk, summed over chunks: the mean span says how
//    much of x a wavefront's gathers wander over, small for stencils and bands, the whole
//    vector for uniformly random columns;
//  * how much of the matrix lies in a band around the diagonal (|column - row| <= 32 ... 256).
// The rows of a chunk's entries come from the positions (rows_of_chunk).  The work is by entries, so a
// row of a million entries costs what a million short rows cost.
__global__ __launch_bounds__(256) void entry_stats_kernel(int nrows, long long nnz, int ncols,
                                                          const int *__restrict__ pos,
                                                          const int *__restrict__ crd, DeviceStats *st) {
  __shared__ unsigned long long s_span[4], s_near[4][4];
  __shared__ int s_bad[4];
  __shared__ int s_rows[4][1024];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const long long nchunks = (nnz + 1023) / 1024;
  unsigned cnt[4] = {0u, 0u, 0u, 0u};
  unsigned long long span = 0ull;
  int bad = 0;
  for (long long chunk = (long long)blockIdx.x * 4 + wave; chunk < nchunks; chunk += (long long)gridDim.x * 4) {
    const long long j0 = chunk * 1024;
    const long long j1 = std::min(nnz, j0 + 1024);
    rows_of_chunk(pos, nrows, j0, j1, s_rows[wave]);
    int mn = INT32_MAX, mx = INT32_MIN;
    for (long long j = j0 + lane; j < j1; j += 64) {
      const int cj = crd[j];
      if (cj < 0 || cj >= ncols) bad = 1;
      mn = std::min(mn, cj);
      mx = std::max(mx, cj);
      const long long d = (long long)cj - s_rows[wave][j - j0];
      const long long a = d < 0 ? -d : d;
      cnt[0] += a <= 32;
      cnt[1] += a <= 64;
      cnt[2] += a <= 128;
      cnt[3] += a <= 256;
    }
    for (int o = 32; o > 0; o >>= 1) {
      mn = std::min(mn, __shfl_xor(mn, o, 64));
      mx = std::max(mx, __shfl_xor(mx, o, 64));
    }
    span += (unsigned long long)((long long)mx - (long long)mn);  // the same in every lane
    wave_lds_sync();  // the next chunk's rows go into the same LDS
  }
  unsigned long long near[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    near[i] = cnt[i];
    for (int o = 32; o > 0; o >>= 1) near[i] += __shfl_xor(near[i], o, 64);
  }
  for (int o = 32; o > 0; o >>= 1) bad |= __shfl_xor(bad, o, 64);
  if (lane == 0) {
    s_span[wave] = span;
    s_bad[wave] = bad;
    for (int i = 0; i < 4; ++i) s_near[wave][i] = near[i];
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < 4; ++w) {
      span += s_span[w];
      bad |= s_bad[w];
      for (int i = 0; i < 4; ++i) near[i] += s_near[w][i];
    }
    if (bad) atomicOr(&st->bad, 2);
    if (span) atomicAdd(&st->span_sum, span);
    for (int i = 0; i < 4; ++i)
      if (near[i]) atomicAdd(&st->near[i], near[i]);
  }
}

template <int CH>
__global__ __launch_bounds__(256) void chunk_row_kernel(int nrows, int nchunks,
                                                        const int *__restrict__ pos,
                                                        int *__restrict__ chunk_row) {
  const long long r = (long long)blockIdx.x * 256 + threadIdx.x;
  if (r == 0) chunk_row[nchunks] = nrows;
  if (r >= nrows) return;
  const long long ps = pos[r], pe = pos[r + 1];
  if (pe <= ps) return;
  const long long first = (ps + CH - 1) / CH;
  const long long last = (pe - 1) / CH;
  for (long long c = first; c <= last; ++c) chunk_row[c] = (int)r;
}

}  // namespace lapis

// ------------------------------------------------------------------------------
// Host side
// ------------------------------------------------------------------------------
using namespace lapis;

namespace {
constexpr int kRowblockCap = 1024;  // staged non-zeros per wavefront tile in the row-block kernel
constexpr int kWavesPerBlock = 4;

int env_int(const char *name, int dflt) {
  const char *s = getenv(name);
  return (s && *s) ? atoi(s) : dflt;
}

// LAPIS::threadParallelVectorLength (LAPISSupport.hpp:428-435) with the wave64
// vector_length_max, including the "no hint -> 8" case (emitter :2013-2019).
int reference_vector_length(int64_t hint) {
  if (hint == 0) return 8;
  int par = (int)std::min<int64_t>(hint, INT32_MAX);
  if (par < 1) return 1;
  int v = 1;
  while (v < kWave && v * 6 < par) v *= 2;
  return v;
}

int64_t reference_hint(int64_t nrows, int64_t pos_first, int64_t pos_last) {
  if (nrows <= 0) return 0;
  return (pos_last - pos_first + nrows - 1) / nrows;
}
}  // namespace

namespace {

void choose_kernel(lapis_hip_csr_plan *p) {
  lapis_hip_csr_stats &s = p->stats;
  s.chunk = 0;
  s.width = 0;
  if (s.nnz == 0 || s.nrows == 0) {
    s.kernel = LAPIS_HIP_SPMV_SUBWARP;
    s.width = 1;
    return;
  }
  // Measured on MI355X (fp64): the row-split kernel streams at 4.2-4.9 TB/s on
  // stencil and FEM-like matrices with 7 to 80 non-zeros per row and is the only one
  // that balances power-law rows; below a few million non-zeros its second (fix-up)
  // launch costs more than it gains and the single-launch row-block kernel wins.
  const double mean = s.mean_row_len;
  const bool skewed = (double)s.max_row_len > 8.0 * std::max(mean, 32.0);
  if (s.nnz < (3 << 20) && !skewed && mean < 512.0) {
    s.kernel = LAPIS_HIP_SPMV_ROWBLOCK;
    return;
  }
  if (skewed || mean < 2048.0) {
    s.kernel = LAPIS_HIP_SPMV_NNZSPLIT;
    s.chunk = p->chunk;
    return;
  }
  // very long, even rows: a whole wavefront per row
  s.kernel = LAPIS_HIP_SPMV_SUBWARP;
  s.width = 64;
}

template <typename T, int W, bool NT>
int launch_subwarp_w(int64_t nrows, const int *pos, const int *crd, const T *val, const T *x, T *y,
                     hipStream_t st) {
  const int64_t blocks = ceil_div(nrows * W, 256);
  if (blocks > 0x7fffffffLL)
    return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "spmv: %lld rows with %d lanes per row exceed the grid limit",
                     (long long)nrows, W);
  launch_timed(spmv_subwarp_kernel<T, W, NT>, dim3((unsigned)blocks), dim3(256), st, (int)nrows, pos, crd, val, x,
               y);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}

template <typename T, bool NT>
int launch_subwarp(int width, int64_t nrows, const int *pos, const int *crd, const T *val, const T *x,
                   T *y, hipStream_t st) {
  switch (width) {
    case 1: return launch_subwarp_w<T, 1, NT>(nrows, pos, crd, val, x, y, st);
    case 2: return launch_subwarp_w<T, 2, NT>(nrows, pos, crd, val, x, y, st);
    case 4: return launch_subwarp_w<T, 4, NT>(nrows, pos, crd, val, x, y, st);
    case 8: return launch_subwarp_w<T, 8, NT>(nrows, pos, crd, val, x, y, st);
    case 16: return launch_subwarp_w<T, 16, NT>(nrows, pos, crd, val, x, y, st);
    case 32: return launch_subwarp_w<T, 32, NT>(nrows, pos, crd, val, x, y, st);
    case 64: return launch_subwarp_w<T, 64, NT>(nrows, pos, crd, val, x, y, st);
    default:
      return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "spmv: lanes per row must be a power of two <= 64, got %d",
                       width);
  }
}

template <typename T, bool VEC, bool NT>
int launch_rowblock(int64_t nrows, int64_t nnz, const int *pos, const int *crd, const T *val, const T *x,
                    T *y, hipStream_t st, int xcd_map) {
  const int64_t blocks = ceil_div(nrows, 64 * kWavesPerBlock);
  launch_timed(spmv_rowblock_kernel<T, kRowblockCap, kWavesPerBlock, VEC, NT>, dim3((unsigned)blocks),
               dim3(64 * kWavesPerBlock), st, (int)nrows, (int)nnz, pos, crd, val, x, y, xcd_map);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}

template <typename T, bool VEC, bool NT, int CH, int WPB>
int launch_nnzsplit_cfg(const lapis_hip_csr_plan *p, const int *pos, const int *crd, const T *val, const T *x,
                        T *y, hipStream_t st, int accumulate, bool defer_fixup, double *xy_chunk) {
  const int nchunks = p->nchunks;
  const int blocks = (int)ceil_div(nchunks, WPB);
  launch_timed(spmv_nnzsplit_kernel<T, CH, WPB, VEC, NT>, dim3(blocks), dim3(64 * WPB),
               st, (int)p->stats.nrows, (int)p->stats.nnz, nchunks, pos, crd, val, x, y,
               (const int *)p->chunk_row, static_cast<T *>(p->part_first), static_cast<T *>(p->part_last), accumulate,
               p->xcd_map, xy_chunk);
  LAPIS_LAUNCH_CHECK();
  if (nchunks > 1 && !defer_fixup) {
    const int fblocks = (int)ceil_div(nchunks - 1, 256);
    hipLaunchKernelGGL((spmv_nnzsplit_fixup_kernel<T, CH>), dim3(fblocks), dim3(256), 0, st, nchunks, pos,
                       p->chunk_row, static_cast<const T *>(p->part_first),
                       static_cast<const T *>(p->part_last), y, accumulate);
    LAPIS_LAUNCH_CHECK();
  }
  return LAPIS_HIP_OK;
}

template <typename T, bool VEC, bool NT>
int launch_nnzsplit(const lapis_hip_csr_plan *p, const int *pos, const int *crd, const T *val, const T *x,
                    T *y, hipStream_t st, int accumulate = 1, bool defer_fixup = false,
                    double *xy_chunk = nullptr) {
  switch (p->stats.chunk * 16 + p->waves_per_block) {
    case 512 * 16 + 4: return launch_nnzsplit_cfg<T, VEC, NT, 512, 4>(p, pos, crd, val, x, y, st, accumulate, defer_fixup, xy_chunk);
    case 512 * 16 + 8: return launch_nnzsplit_cfg<T, VEC, NT, 512, 8>(p, pos, crd, val, x, y, st, accumulate, defer_fixup, xy_chunk);
    case 1024 * 16 + 2: return launch_nnzsplit_cfg<T, VEC, NT, 1024, 2>(p, pos, crd, val, x, y, st, accumulate, defer_fixup, xy_chunk);
    case 1024 * 16 + 4: return launch_nnzsplit_cfg<T, VEC, NT, 1024, 4>(p, pos, crd, val, x, y, st, accumulate, defer_fixup, xy_chunk);
    case 1024 * 16 + 8: return launch_nnzsplit_cfg<T, VEC, NT, 1024, 8>(p, pos, crd, val, x, y, st, accumulate, defer_fixup, xy_chunk);
    case 2048 * 16 + 2: return launch_nnzsplit_cfg<T, VEC, NT, 2048, 2>(p, pos, crd, val, x, y, st, accumulate, defer_fixup, xy_chunk);
    case 2048 * 16 + 4: return launch_nnzsplit_cfg<T, VEC, NT, 2048, 4>(p, pos, crd, val, x, y, st, accumulate, defer_fixup, xy_chunk);
    default:
      return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "spmv: no row-split kernel for %d non-zeros per wavefront, %d wavefronts per block",
                       p->stats.chunk, p->waves_per_block);
  }
}

template <typename T>
int spmv_impl(lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols, const int32_t *pos, const int32_t *crd,
              const T *val, const T *x, T *y, lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(nrows >= 0 && ncols >= 0, "spmv: negative dimension (%lld x %lld)", (long long)nrows,
                (long long)ncols);
  LAPIS_REQUIRE(nrows <= INT32_MAX - 64 && ncols <= INT32_MAX, "spmv: dimensions exceed the int32 index range");
  if (nrows == 0) return LAPIS_HIP_OK;
  LAPIS_REQUIRE(pos && y, "spmv: null positions or output with %lld rows", (long long)nrows);
  hipStream_t st = as_stream(stream);

  if (!plan) {
    // The reference's own rule: read pos[n] and pos[0] on the host at every call
    // (KokkosLoopMapping.cpp:290-322), turn the mean row length into a vector length.
    int32_t ends[2] = {0, 0};
    LAPIS_HIP_TRY(hipMemcpyAsync(&ends[0], pos, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    LAPIS_HIP_TRY(hipMemcpyAsync(&ends[1], pos + nrows, sizeof(int32_t), hipMemcpyDeviceToHost, st));
    LAPIS_HIP_TRY(hipStreamSynchronize(st));
    const int64_t nnz = (int64_t)ends[1] - ends[0];
    LAPIS_REQUIRE(nnz >= 0, "spmv: pos[n] < pos[0]");
    if (nnz == 0) return LAPIS_HIP_OK;
    LAPIS_REQUIRE(crd && val && x, "spmv: null coordinates, values or x with %lld non-zeros", (long long)nnz);
    const int w = reference_vector_length(reference_hint(nrows, ends[0], ends[1]));
    return launch_subwarp<T, true>(w, nrows, pos, crd, val, x, y, st);
  }

  const lapis_hip_csr_stats &s = plan->stats;
  if (s.nrows != nrows || s.ncols != ncols || plan->pos != pos)
    return set_error(LAPIS_HIP_ERR_PLAN_MISMATCH,
                     "spmv: plan was built for a %lld x %lld matrix at positions %p, called with %lld x %lld at %p",
                     (long long)s.nrows, (long long)s.ncols, (const void *)plan->pos, (long long)nrows,
                     (long long)ncols, (const void *)pos);
  if (s.nnz == 0) return LAPIS_HIP_OK;
  LAPIS_REQUIRE(x && crd && val, "spmv: null coordinates, values or x with %lld non-zeros", (long long)s.nnz);
  const bool vec = aligned16(crd) && aligned16(val);
  const bool nt = plan->nontemporal;
  switch (s.kernel) {
    case LAPIS_HIP_SPMV_SUBWARP:
      return nt ? launch_subwarp<T, true>(s.width, nrows, pos, crd, val, x, y, st)
                : launch_subwarp<T, false>(s.width, nrows, pos, crd, val, x, y, st);
    case LAPIS_HIP_SPMV_ROWBLOCK:
      if (vec)
        return nt ? launch_rowblock<T, true, true>(nrows, s.nnz, pos, crd, val, x, y, st, plan->xcd_map)
                  : launch_rowblock<T, true, false>(nrows, s.nnz, pos, crd, val, x, y, st, plan->xcd_map);
      return launch_rowblock<T, false, true>(nrows, s.nnz, pos, crd, val, x, y, st, plan->xcd_map);
    case LAPIS_HIP_SPMV_NNZSPLIT:
      if (vec)
        return nt ? launch_nnzsplit<T, true, true>(plan, pos, crd, val, x, y, st)
                  : launch_nnzsplit<T, true, false>(plan, pos, crd, val, x, y, st);
      return launch_nnzsplit<T, false, true>(plan, pos, crd, val, x, y, st);
    case LAPIS_HIP_SPMV_COLBLOCK:
      if (!plan->colblock_built || plan->colblock_value_bytes != (int)sizeof(T))
        return set_error(LAPIS_HIP_ERR_PLAN_MISMATCH, "spmv: the plan holds no column-blocked copy for %d-byte values",
                         (int)sizeof(T));
      // the copy stands in for crd/val: refuse buffers it was not made from (new values in the same
      // buffer are brought in with lapis_hip_csr_plan_update_values)
      if (crd != plan->colblock_src_crd || val != plan->colblock_src_val)
        return set_error(LAPIS_HIP_ERR_PLAN_MISMATCH,
                         "spmv: the column-blocked copy was made from coordinates %p and values %p, called with %p and %p "
                         "(lapis_hip_csr_plan_update_values takes new values)",
                         plan->colblock_src_crd, plan->colblock_src_val, (const void *)crd, (const void *)val);
      return launch_colblock<T>(plan, pos, crd, val, x, y, st);
    default:
      return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "spmv: plan holds unknown kernel %d", s.kernel);
  }
}

}  // namespace

namespace lapis {
// y = A x (y is not read).  The row-split kernel writes every non-empty row itself;
// any other case zero-fills y and accumulates.
//
// With `deferred_chunk` the caller offers to complete the rows cut at chunk boundaries
// itself (rowsplit_complete_row over boundaries 1..nchunks-1 with the plan's chunk_row,
// part_first and part_last, accumulate = 0): when the row-split kernel runs, its fix-up
// launch is left out and *deferred_chunk is the chunk length, otherwise it is 0 and y is complete.
// In that case, and only then, `xy_chunk` (plan->nchunks doubles, square matrices) receives per
// chunk the sum of x[r]*y[r] over the rows that lie wholly inside the chunk; the rows the caller
// completes are missing from it.
int spmv_overwrite_f64(lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols, const int32_t *pos,
                       const int32_t *crd, const double *val, const double *x, double *y,
                       lapis_hip_stream_t stream, int *deferred_chunk, double *xy_chunk) {
  if (deferred_chunk) *deferred_chunk = 0;
  if (plan && plan->stats.kernel == LAPIS_HIP_SPMV_NNZSPLIT && plan->stats.empty_rows == 0 && plan->stats.nnz > 0 &&
      plan->stats.nrows == nrows && plan->stats.ncols == ncols && plan->pos == pos && aligned16(crd) &&
      aligned16(val)) {
    LAPIS_CHECK_INIT();
    hipStream_t st = as_stream(stream);
    const bool defer = deferred_chunk && plan->nchunks > 1;
    double *xy = (defer && nrows == ncols) ? xy_chunk : nullptr;
    const int rc = plan->nontemporal
                       ? launch_nnzsplit<double, true, true>(plan, pos, crd, val, x, y, st, 0, defer, xy)
                       : launch_nnzsplit<double, true, false>(plan, pos, crd, val, x, y, st, 0, defer, xy);
    if (rc == LAPIS_HIP_OK && defer) *deferred_chunk = plan->stats.chunk;
    return rc;
  }
  const int rc = lapis_hip_fill_f64(nrows, 0.0, y, stream);
  if (rc != LAPIS_HIP_OK) return rc;
  return lapis_hip_spmv_csr_f64_i32(plan, nrows, ncols, pos, crd, val, x, y, stream);
}
}  // namespace lapis

namespace {
void free_plan_buffers(lapis_hip_csr_plan *p) {
  if (p->chunk_row) (void)hipFree(p->chunk_row);
  if (p->part_first) (void)hipFree(p->part_first);
  if (p->part_last) (void)hipFree(p->part_last);
  p->chunk_row = nullptr;
  p->part_first = p->part_last = nullptr;
  free_colblock(p);
}

}  // namespace

extern "C" int lapis_hip_csr_plan_create(lapis_hip_csr_plan **out, int64_t nrows, int64_t ncols, int64_t nnz,
                                         const int32_t *pos, const int32_t *crd, int value_bytes,
                                         lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(out, "csr_plan_create: null output");
  *out = nullptr;
  LAPIS_REQUIRE(nrows >= 0 && ncols >= 0 && nnz >= 0, "csr_plan_create: negative size");
  LAPIS_REQUIRE(nrows <= INT32_MAX - 64 && ncols <= INT32_MAX && nnz <= INT32_MAX,
                "csr_plan_create: sizes exceed the int32 index range");
  LAPIS_REQUIRE(value_bytes == 4 || value_bytes == 8, "csr_plan_create: value_bytes must be 4 or 8");
  LAPIS_REQUIRE(pos, "csr_plan_create: null positions (a CSR matrix with n rows has n+1 positions)");
  hipStream_t st = as_stream(stream);

  int32_t ends[2] = {0, 0};
  LAPIS_HIP_TRY(hipMemcpyAsync(&ends[0], pos, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  LAPIS_HIP_TRY(hipMemcpyAsync(&ends[1], pos + nrows, sizeof(int32_t), hipMemcpyDeviceToHost, st));
  LAPIS_HIP_TRY(hipStreamSynchronize(st));
  if (ends[0] != 0 || ends[1] != nnz)
    return set_error(LAPIS_HIP_ERR_BAD_CSR, "csr_plan_create: pos[0]=%d pos[n]=%d, expected 0 and nnz=%lld",
                     ends[0], ends[1], (long long)nnz);

  DeviceStats init{INT32_MAX, 0, 0, 0, 0ull, 0.0, 0ull, {0ull, 0ull, 0ull, 0ull}};
  DeviceStats host = init;
  if (nrows > 0) {
    DeviceStats *dstats = nullptr;
    LAPIS_HIP_TRY(hipMalloc(&dstats, sizeof(DeviceStats)));
    hipError_t e = hipMemcpyAsync(dstats, &init, sizeof(init), hipMemcpyHostToDevice, st);
    if (e == hipSuccess) {
      const int blocks = (int)std::min<int64_t>(ceil_div(nrows, 256), 1024);
      hipLaunchKernelGGL(row_stats_kernel, dim3(blocks), dim3(256), 0, st, (int)nrows, pos, dstats);
      e = hipGetLastError();
    }
    if (e == hipSuccess && crd && nnz > 0) {
      const int blocks = (int)std::min<int64_t>(ceil_div(ceil_div(nnz, 1024), 4), 2048);
      hipLaunchKernelGGL(entry_stats_kernel, dim3(blocks), dim3(256), 0, st, (int)nrows, (long long)nnz, (int)ncols,
                         pos, crd, dstats);
      e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipMemcpyAsync(&host, dstats, sizeof(host), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    (void)hipFree(dstats);
    if (e != hipSuccess)
      return set_error(LAPIS_HIP_ERR_RUNTIME, "csr_plan_create: analysis failed: %s", hipGetErrorString(e));
  } else {
    host.min_len = 0;
  }
  if (host.bad & 1) return set_error(LAPIS_HIP_ERR_BAD_CSR, "csr_plan_create: positions are not non-decreasing");
  if (host.bad & 2)
    return set_error(LAPIS_HIP_ERR_BAD_CSR, "csr_plan_create: a coordinate lies outside [0, %lld)", (long long)ncols);

  lapis_hip_csr_plan *p = new lapis_hip_csr_plan();
  memset(p, 0, sizeof(*p));
  lapis_hip_csr_stats &s = p->stats;
  s.nrows = nrows;
  s.ncols = ncols;
  s.nnz = nnz;
  s.min_row_len = host.min_len;
  s.max_row_len = host.max_len;
  s.empty_rows = (int64_t)host.empty_rows;
  s.mean_row_len = nrows ? (double)nnz / (double)nrows : 0.0;
  s.var_row_len = nrows ? std::max(0.0, host.sum_sq / (double)nrows - s.mean_row_len * s.mean_row_len) : 0.0;
  s.mean_chunk_col_span = (crd && nnz > 0) ? (double)host.span_sum / (double)ceil_div(nnz, 1024) : -1.0;
  for (int i = 0; i < 4; ++i) s.near_diagonal_fraction[i] = (crd && nnz > 0) ? (double)host.near[i] / (double)nnz : -1.0;
  // The column-blocked copy pays when the gathers of a chunk wander over more of x
  // than an XCD's L2 keeps (4 MB, shared with the streamed arrays) and the matrix is
  // large enough for the extra launch work not to matter.
  s.colblock_recommended = (s.mean_chunk_col_span * value_bytes > 2.0 * 1024 * 1024 && nnz >= (1 << 20)) ? 1 : 0;
  s.reference_hint = reference_hint(nrows, ends[0], ends[1]);
  s.reference_vector_length = reference_vector_length(s.reference_hint);
  p->pos = pos;
  p->crd = crd;
  // Non-temporal loads of the streamed arrays pay when x does not fit L2 anyway (they
  // keep the stream from evicting what little of x is cached); when the gathers of a
  // chunk stay inside a window L2 can hold, plain loads are 10-15 % faster.
  p->nontemporal = env_int("LAPIS_HIP_SPMV_NONTEMPORAL", s.mean_chunk_col_span * value_bytes > 2.0 * 1024 * 1024) != 0;
  // Contiguous block ranges per XCD measured no better than the hardware's round-robin
  // (7-point stencil, n = 7.1M: 0.284 against 0.275 ms per CG iteration; neutral on the
  // others), so it stays an opt-in.
  p->xcd_map = env_int("LAPIS_HIP_SPMV_XCD_MAP", 0) != 0;
  // Measured: 512 non-zeros per wavefront in workgroups of 8 for short rows (7-point
  // stencil: +4 to +8 % over 1024 x 4), 1024 in workgroups of 2 from about 32 per row on.
  p->chunk = env_int("LAPIS_HIP_SPMV_CHUNK", s.mean_row_len < 32.0 ? 512 : 1024);
  if (p->chunk != 512 && p->chunk != 2048) p->chunk = 1024;
  p->waves_per_block = env_int("LAPIS_HIP_SPMV_WAVES", p->chunk == 512 ? 8 : 2);
  if (p->waves_per_block != 2 && p->waves_per_block != 4 && p->waves_per_block != 8) p->waves_per_block = 4;
  if (p->chunk == 2048 && p->waves_per_block == 8) p->waves_per_block = 4;
  if (p->chunk == 512 && p->waves_per_block == 2) p->waves_per_block = 4;
  p->nchunks = (int)ceil_div(nnz, p->chunk);
  choose_kernel(p);

  // Row-split metadata is built whatever the choice, so that set_kernel can switch to it.
  if (p->nchunks > 0) {
    hipError_t e = hipMalloc(&p->chunk_row, sizeof(int) * ((size_t)p->nchunks + 1));
    if (e == hipSuccess) e = hipMalloc(&p->part_first, 8 * (size_t)p->nchunks);
    if (e == hipSuccess) e = hipMalloc(&p->part_last, 8 * (size_t)p->nchunks);
    if (e == hipSuccess) {
      const dim3 g((unsigned)ceil_div(nrows, 256));
      if (p->chunk == 512)
        hipLaunchKernelGGL((chunk_row_kernel<512>), g, dim3(256), 0, st, (int)nrows, p->nchunks, pos, p->chunk_row);
      else if (p->chunk == 2048)
        hipLaunchKernelGGL((chunk_row_kernel<2048>), g, dim3(256), 0, st, (int)nrows, p->nchunks, pos, p->chunk_row);
      else
        hipLaunchKernelGGL((chunk_row_kernel<1024>), g, dim3(256), 0, st, (int)nrows, p->nchunks, pos, p->chunk_row);
      e = hipGetLastError();
    }
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) {
      free_plan_buffers(p);
      delete p;
      return set_error(LAPIS_HIP_ERR_RUNTIME, "csr_plan_create: building row-split metadata failed: %s",
                       hipGetErrorString(e));
    }
  }
  *out = p;
  return LAPIS_HIP_OK;
}

extern "C" const char *lapis_hip_csr_plan_kernel_name(const lapis_hip_csr_plan *plan) {
  if (!plan) return "";
  switch (plan->stats.kernel) {
    case LAPIS_HIP_SPMV_SUBWARP: return "spmv_subwarp_kernel";
    case LAPIS_HIP_SPMV_ROWBLOCK: return "spmv_rowblock_kernel";
    case LAPIS_HIP_SPMV_NNZSPLIT: return "spmv_nnzsplit_kernel";
    case LAPIS_HIP_SPMV_COLBLOCK:
      if (!plan->colblock_group) return "spmv_colblock_kernel";
      return plan->colblock_pc_prod > 0 ? "spmv_colgroup_pc_kernel" : "spmv_colgroup_kernel";
    default: return "";
  }
}

extern "C" int lapis_hip_csr_plan_matches(const lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols, int64_t nnz,
                                          const int32_t *pos, const int32_t *crd) {
  if (!plan) return 0;
  const lapis_hip_csr_stats &s = plan->stats;
  return (s.nrows == nrows && s.ncols == ncols && s.nnz == nnz && plan->pos == pos && plan->crd == crd) ? 1 : 0;
}

extern "C" int lapis_hip_csr_plan_set_kernel(lapis_hip_csr_plan *plan, int kernel, int width) {
  LAPIS_REQUIRE(plan, "csr_plan_set_kernel: null plan");
  lapis_hip_csr_stats &s = plan->stats;
  switch (kernel) {
    case LAPIS_HIP_SPMV_AUTO:
      choose_kernel(plan);
      return LAPIS_HIP_OK;
    case LAPIS_HIP_SPMV_SUBWARP: {
      const int w = width == 0 ? s.reference_vector_length : width;
      LAPIS_REQUIRE(w >= 1 && w <= 64 && (w & (w - 1)) == 0,
                    "csr_plan_set_kernel: lanes per row must be a power of two <= 64, got %d", w);
      s.kernel = kernel;
      s.width = w;
      s.chunk = 0;
      return LAPIS_HIP_OK;
    }
    case LAPIS_HIP_SPMV_ROWBLOCK:
      s.kernel = kernel;
      s.width = 0;
      s.chunk = 0;
      return LAPIS_HIP_OK;
    case LAPIS_HIP_SPMV_NNZSPLIT:
      s.kernel = kernel;
      s.width = 0;
      s.chunk = plan->chunk;
      return LAPIS_HIP_OK;
    case LAPIS_HIP_SPMV_COLBLOCK:
      if (!plan->colblock_built)
        return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT,
                         "csr_plan_set_kernel: call lapis_hip_csr_plan_build_colblock first");
      s.kernel = kernel;
      s.width = 0;
      s.chunk = 0;
      return LAPIS_HIP_OK;
    default:
      return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "csr_plan_set_kernel: unknown kernel %d", kernel);
  }
}

extern "C" int lapis_hip_csr_plan_get_stats(const lapis_hip_csr_plan *plan, lapis_hip_csr_stats *stats) {
  LAPIS_REQUIRE(plan && stats, "csr_plan_get_stats: null argument");
  *stats = plan->stats;
  return LAPIS_HIP_OK;
}

extern "C" int lapis_hip_csr_plan_destroy(lapis_hip_csr_plan *plan) {
  if (!plan) return LAPIS_HIP_OK;
  free_plan_buffers(plan);
  delete plan;
  return LAPIS_HIP_OK;
}

extern "C" int lapis_hip_spmv_csr_f64_i32(lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols,
                                          const int32_t *pos, const int32_t *crd, const double *val,
                                          const double *x, double *y, lapis_hip_stream_t stream) {
  return spmv_impl<double>(plan, nrows, ncols, pos, crd, val, x, y, stream);
}

extern "C" int lapis_hip_spmv_csr_f32_i32(lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols,
                                          const int32_t *pos, const int32_t *crd, const float *val,
                                          const float *x, float *y, lapis_hip_stream_t stream) {
  return spmv_impl<float>(plan, nrows, ncols, pos, crd, val, x, y, stream);
}
