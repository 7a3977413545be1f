// CSR x dense SpMM for gfx950:  C[i,:] = C[i,:] + sum_kk val[kk] * B[crd[kk],:]
// (row-major B and C).  Replaces the i -> kk -> j nest the sparsifier emits for
// CSR x dense linalg.matmul (examples/spmm_dcsr_opdsl.py:73-110).
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <mutex>
#include <type_traits>

#include "common.hpp"
#include "plan.hpp"

namespace lapis {

template <typename T>
struct RowVec;
template <>
struct RowVec<float> {
  typedef v4f type;
  static constexpr int width = 4;
};
template <>
struct RowVec<double> {
  typedef v2d type;
  static constexpr int width = 2;
};

// One wavefront per row of A and per chunk of LPR * VW columns of B (blockIdx.y).  The
// chunk of a B row is covered by LPR lanes with one 128-bit load each, so the 64 lanes
// take G = 64/LPR non-zeros of the row per step: every gathered B row is one fully
// coalesced read.  The row's crd/val are read once, 64 at a time and coalesced, then
// handed to the lane groups by bpermute.  The G partial rows are added up with xor
// shuffles.  VEC = false is the same kernel with element-wise guarded accesses, for k
// that is no multiple of the vector width and for buffers that are not 16-byte aligned.
template <typename T, int LPR, bool VEC, bool DEEP>
__global__ __launch_bounds__(256) void spmm_wave_row_kernel(int nrows, int k, const int *__restrict__ pos,
                                                            const int *__restrict__ crd,
                                                            const T *__restrict__ val, const T *__restrict__ B,
                                                            long long ldb, T *__restrict__ C, long long ldc) {
  typedef typename RowVec<T>::type V;
  constexpr int VW = RowVec<T>::width;
  constexpr int G = 64 / LPR;
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= nrows) return;
  const int g = lane / LPR;
  const int l = lane % LPR;
  const int col = (int)blockIdx.y * (LPR * VW) + l * VW;  // first of this lane's VW columns
  const int start = pos[row];
  const int end = pos[row + 1];
  V acc = {};
  for (int base = start; base < end; base += 64) {
    const int cnt = min(64, end - base);
    int c_l = 0;
    T a_l = T(0);
    if (lane < cnt) {
      c_l = load_stream(crd + base + lane);
      a_l = load_stream(val + base + lane);
    }
    // Every lane runs every step (the bpermutes need their source lanes active).  With DEEP, steps go
    // together in batches of 8, 4, 2 and 1: the B rows of a batch are loaded first, without any condition
    // -- a lane group past the row end reads the row of a lane that holds column 0 and value 0, a lane
    // past the last column of B reads column 0 -- and then added in order, so a lane keeps up to 8
    // gathered rows in flight.  (Loads inside the `t < cnt` test are not unrolled by the compiler and
    // are waited for one by one, which is what !DEEP does: better where B comes from HBM anyway.)
    const int colc = col < k ? col : 0;
    auto batch = [&](int t0, auto unr) {
      constexpr int UNR = decltype(unr)::value;
      T a[UNR];
      if (VEC) {
        V b[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          const int t = t0 + u * G + g;
          const int cj = __shfl(c_l, t & 63, 64);
          a[u] = __shfl(a_l, t & 63, 64);
          b[u] = *reinterpret_cast<const V *>(B + (long long)cj * ldb + colc);
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          if (t0 + u * G + g < cnt && col < k) {
#pragma unroll
            for (int e = 0; e < VW; ++e) acc[e] = acc[e] + a[u] * b[u][e];
          }
        }
      } else {
        T b[UNR][VW];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          const int t = t0 + u * G + g;
          const int cj = __shfl(c_l, t & 63, 64);
          a[u] = __shfl(a_l, t & 63, 64);
          const T *bp = B + (long long)cj * ldb;
#pragma unroll
          for (int e = 0; e < VW; ++e) b[u][e] = bp[col + e < k ? col + e : 0];
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          if (t0 + u * G + g < cnt) {
#pragma unroll
            for (int e = 0; e < VW; ++e)
              if (col + e < k) acc[e] = acc[e] + a[u] * b[u][e];
          }
        }
      }
    };
    int t0 = 0;
    if (DEEP) {
      for (; t0 + 7 * G < cnt; t0 += 8 * G) batch(t0, std::integral_constant<int, 8>());
      if (t0 + 3 * G < cnt) {
        batch(t0, std::integral_constant<int, 4>());
        t0 += 4 * G;
      }
      if (t0 + G < cnt) {
        batch(t0, std::integral_constant<int, 2>());
        t0 += 2 * G;
      }
    }
    for (; t0 < cnt; t0 += G) batch(t0, std::integral_constant<int, 1>());
  }
#pragma unroll
  for (int o = LPR; o < 64; o <<= 1) {
#pragma unroll
    for (int e = 0; e < VW; ++e) acc[e] = acc[e] + __shfl_xor(acc[e], o, 64);
  }
  if (g == 0 && col < k) {
    T *cp = C + row * ldc + col;
    if (VEC) {
      V cin = load_stream(reinterpret_cast<V *>(cp));
#pragma unroll
      for (int e = 0; e < VW; ++e) cin[e] = acc[e] + cin[e];
      store_stream(reinterpret_cast<V *>(cp), cin);
    } else {
#pragma unroll
      for (int e = 0; e < VW; ++e)
        if (col + e < k) cp[e] = acc[e] + cp[e];
    }
  }
}

// One group of LPR lanes per row of A: a wavefront works on G = 64/LPR rows at a time,
// ROUNDS times over (once by default).  Each group walks its own row, LPR non-zeros per coalesced read of
// crd/val, one B row (LPR 128-bit loads) per non-zero, and keeps the row of C in its own
// registers: no reduction across lanes, G rows of loads in flight per instruction, and
// the G rows of C a wavefront writes are neighbours.  For short, even rows (stencils,
// meshes, fixed-degree graphs) this does the work of the kernel above with a quarter of
// the wavefronts and none of its shuffles; one very long row would leave the other
// groups of its wavefront idle, so skewed matrices stay with the kernel above.
template <typename T, int LPR, int ROUNDS, bool XCD>
__global__ __launch_bounds__(256) void spmm_group_row_kernel(int nrows, const int *__restrict__ pos,
                                                             const int *__restrict__ crd,
                                                             const T *__restrict__ val, const T *__restrict__ B,
                                                             long long ldb, T *__restrict__ C, long long ldc) {
  typedef typename RowVec<T>::type V;
  constexpr int VW = RowVec<T>::width;
  constexpr int G = 64 / LPR;
  const int lane = threadIdx.x & 63;
  const int g = lane / LPR;
  const int l = lane % LPR;
  // Workgroups go to the 8 XCDs round-robin; mapped like this each XCD works on one contiguous eighth of
  // the rows, so with local columns its L2 fetches an eighth of B instead of all of it.
  const unsigned block = XCD ? xcd_contiguous_block(blockIdx.x, gridDim.x) : blockIdx.x;
  const long long wave_row0 = ((long long)block * 4 + (threadIdx.x >> 6)) * (G * ROUNDS);
#pragma unroll 1
  for (int r = 0; r < ROUNDS; ++r) {
    const long long row = wave_row0 + r * G + g;
    int start = 0, end = 0;
    if (row < nrows) {
      start = pos[row];
      end = pos[row + 1];
    }
    V acc = {};
    for (int base = start; base < end; base += LPR) {
      const int cnt = min(LPR, end - base);
      int c_l = 0;
      T a_l = T(0);
      if (l < cnt) {
        c_l = load_stream(crd + base + l);
        a_l = load_stream(val + base + l);
      }
      // Non-zeros go together in batches of 8, 4, 2 and 1: the B rows of a batch are loaded first, then
      // added in order, so a lane keeps up to 8 gathered rows in flight (a loop that loads and adds one
      // non-zero per trip is not unrolled by the compiler and waits for every row before it asks for the next)
      auto batch = [&](int t0, auto unr) {
        constexpr int UNR = decltype(unr)::value;
        T a[UNR];
        V b[UNR];
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
          const int src = g * LPR + t0 + u;  // a lane of this group: it runs the same trip
          const int cj = __shfl(c_l, src, 64);
          a[u] = __shfl(a_l, src, 64);
          b[u] = *reinterpret_cast<const V *>(B + (long long)cj * ldb + l * VW);
        }
#pragma unroll
        for (int u = 0; u < UNR; ++u) {
#pragma unroll
          for (int e = 0; e < VW; ++e) acc[e] = acc[e] + a[u] * b[u][e];
        }
      };
      int t0 = 0;
      for (; t0 + 8 <= cnt; t0 += 8) batch(t0, std::integral_constant<int, 8>());
      if (t0 + 4 <= cnt) {
        batch(t0, std::integral_constant<int, 4>());
        t0 += 4;
      }
      if (t0 + 2 <= cnt) {
        batch(t0, std::integral_constant<int, 2>());
        t0 += 2;
      }
      if (t0 < cnt) batch(t0, std::integral_constant<int, 1>());
    }
    if (row < nrows) {
      V *cp = reinterpret_cast<V *>(C + row * ldc + l * VW);
      V cin = load_stream(cp);
#pragma unroll
      for (int e = 0; e < VW; ++e) cin[e] = acc[e] + cin[e];
      store_stream(cp, cin);
    }
  }
}

// LDS-staged row blocks, for matrices with a band around the diagonal.  A workgroup of
// 16 wavefronts owns `rb` consecutive rows of A.  It first copies the rows
// [row0 - halo, row0 + rb + halo) of B into LDS, LPR 128-bit vectors per row, fully
// coalesced; then every wavefront walks its rows as the kernel above does, and a
// non-zero whose column lies in the staged window reads its B row from LDS, any other
// from global memory.  A B row that several rows of the block use crosses the L2 -> CU
// path once instead of once per use; on this chip that path, not HBM, is what bounds a
// stencil SpMM (about 260 G lines per second for the whole chip).  k = LPR * VW exactly.
template <typename T, int LPR>
__global__ __launch_bounds__(1024) void spmm_rowblock_lds_kernel(int nrows, int ncols, int rb, int halo,
                                                                 const int *__restrict__ pos,
                                                                 const int *__restrict__ crd,
                                                                 const T *__restrict__ val, const T *__restrict__ B,
                                                                 long long ldb, T *__restrict__ C, long long ldc) {
  typedef typename RowVec<T>::type V;
  constexpr int VW = RowVec<T>::width;
  constexpr int G = 64 / LPR;
  extern __shared__ __align__(16) unsigned char spmm_lds[];
  V *tile = reinterpret_cast<V *>(spmm_lds);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const long long row0 = (long long)blockIdx.x * rb;
  const int wlo = (int)std::max<long long>(0, row0 - halo);
  const int whi = (int)std::min<long long>(ncols, row0 + rb + halo);
  const int nvec = (whi - wlo) * LPR;
  for (int v = tid; v < nvec; v += 1024) {
    const int r = v / LPR, c = v % LPR;
    tile[v] = *reinterpret_cast<const V *>(B + (long long)(wlo + r) * ldb + c * VW);
  }
  __syncthreads();
  const int g = lane / LPR;
  const int l = lane % LPR;
  const long long row_end = std::min<long long>(nrows, row0 + rb);
  for (long long row = row0 + wave; row < row_end; row += 16) {
    const int start = pos[row];
    const int end = pos[row + 1];
    V acc = {};
    for (int base = start; base < end; base += 64) {
      const int cnt = min(64, end - base);
      int c_l = 0;
      T a_l = T(0);
      if (lane < cnt) {
        c_l = load_stream(crd + base + lane);
        a_l = load_stream(val + base + lane);
      }
      for (int t0 = 0; t0 < cnt; t0 += G) {
        const int t = t0 + g;
        const int cj = __shfl(c_l, t & 63, 64);
        const T aj = __shfl(a_l, t & 63, 64);
        if (t < cnt) {
          V b;
          if (cj >= wlo && cj < whi)
            b = tile[(cj - wlo) * LPR + l];
          else
            b = *reinterpret_cast<const V *>(B + (long long)cj * ldb + l * VW);
#pragma unroll
          for (int e = 0; e < VW; ++e) acc[e] = acc[e] + aj * b[e];
        }
      }
    }
#pragma unroll
    for (int o = LPR; o < 64; o <<= 1) {
#pragma unroll
      for (int e = 0; e < VW; ++e) acc[e] = acc[e] + __shfl_xor(acc[e], o, 64);
    }
    if (g == 0) {
      V *cp = reinterpret_cast<V *>(C + row * ldc + l * VW);
      V cin = *cp;
#pragma unroll
      for (int e = 0; e < VW; ++e) cin[e] = acc[e] + cin[e];
      *cp = cin;
    }
  }
}

// Batched CSRV product of examples/bspmm.py:22-50: A is CSR over (n1, n2) and every
// non-zero carries nh values (a trailing dense batch); out(i, d, h) += A(i, c, h) * V(c, d, h).
// One wavefront per row; lanes walk the dh*nh values of an output row, so the read of
// a V row is coalesced and the nh batch values of a non-zero are read contiguously.
__global__ __launch_bounds__(256) void bspmm_csrv_kernel(int n1, int dh, int nh, const int *__restrict__ pos,
                                                         const int *__restrict__ crd,
                                                         const float *__restrict__ val,
                                                         const float *__restrict__ V, float *__restrict__ out) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= n1) return;
  const int start = pos[row], end = pos[row + 1];
  const long long K = (long long)dh * nh;
  for (long long j = lane; j < K; j += 64) {
    const int h = (int)(j % nh);
    float acc = out[row * K + j];
    for (int e = start; e < end; ++e) {
      const float prod = val[(long long)e * nh + h] * V[(long long)crd[e] * K + j];
      acc = prod + acc;
    }
    out[row * K + j] = acc;
  }
}

template <typename T, int LPR, bool VEC>
void launch_wave_row(int64_t nrows, int64_t k, const int *pos, const int *crd, const T *val, const T *B, int64_t ldb,
                     T *C, int64_t ldc, hipStream_t st, bool deep) {
  constexpr int VW = RowVec<T>::width;
  const dim3 grid((unsigned)ceil_div(nrows, 4), (unsigned)ceil_div(k, LPR * VW));
  if (deep)
    launch_timed(spmm_wave_row_kernel<T, LPR, VEC, true>, grid, dim3(256), st, (int)nrows, (int)k, pos, crd, val, B,
                 (long long)ldb, C, (long long)ldc);
  else
    launch_timed(spmm_wave_row_kernel<T, LPR, VEC, false>, grid, dim3(256), st, (int)nrows, (int)k, pos, crd, val, B,
                 (long long)ldb, C, (long long)ldc);
}

template <typename T, bool VEC>
void launch_wave_row_any(int64_t nrows, int64_t k, const int *pos, const int *crd, const T *val, const T *B, int64_t ldb,
                         T *C, int64_t ldc, hipStream_t st, bool deep) {
  constexpr int VW = RowVec<T>::width;
  // lanes per chunk of a B row: the smallest power of two that covers k, at most a wavefront
  int lpr = 1;
  while (lpr < 64 && (int64_t)lpr * VW < k) lpr *= 2;
  switch (lpr) {
    case 1: launch_wave_row<T, 1, VEC>(nrows, k, pos, crd, val, B, ldb, C, ldc, st, deep); break;
    case 2: launch_wave_row<T, 2, VEC>(nrows, k, pos, crd, val, B, ldb, C, ldc, st, deep); break;
    case 4: launch_wave_row<T, 4, VEC>(nrows, k, pos, crd, val, B, ldb, C, ldc, st, deep); break;
    case 8: launch_wave_row<T, 8, VEC>(nrows, k, pos, crd, val, B, ldb, C, ldc, st, deep); break;
    case 16: launch_wave_row<T, 16, VEC>(nrows, k, pos, crd, val, B, ldb, C, ldc, st, deep); break;
    case 32: launch_wave_row<T, 32, VEC>(nrows, k, pos, crd, val, B, ldb, C, ldc, st, deep); break;
    default: launch_wave_row<T, 64, VEC>(nrows, k, pos, crd, val, B, ldb, C, ldc, st, deep); break;
  }
}

template <typename T, int LPR, int ROUNDS>
void launch_group_row_r(int64_t nrows, const int *pos, const int *crd, const T *val, const T *B, int64_t ldb, T *C,
                        int64_t ldc, hipStream_t st) {
  constexpr int rows_per_block = 4 * (64 / LPR) * ROUNDS;
  const char *xcd = getenv("LAPIS_HIP_SPMM_XCD_MAP");
  if (xcd && atoi(xcd) == 0)
    launch_timed(spmm_group_row_kernel<T, LPR, ROUNDS, false>, dim3((unsigned)ceil_div(nrows, rows_per_block)), dim3(256),
                 st, (int)nrows, pos, crd, val, B, (long long)ldb, C, (long long)ldc);
  else
    launch_timed(spmm_group_row_kernel<T, LPR, ROUNDS, true>, dim3((unsigned)ceil_div(nrows, rows_per_block)), dim3(256),
                 st, (int)nrows, pos, crd, val, B, (long long)ldb, C, (long long)ldc);
}

template <typename T, int LPR>
void launch_group_row(int64_t nrows, const int *pos, const int *crd, const T *val, const T *B, int64_t ldb, T *C,
                      int64_t ldc, hipStream_t st) {
  // Rounds of rows per wavefront.  One is fastest now that a lane keeps several B rows in flight (Laplace3D_100
  // k = 64: 0.195 / 0.196 / 0.209 ms with 1 / 2 / 4 rounds; Elasticity3D_60: 0.606 / 0.623 / 0.649 ms): the fewer
  // rows an XCD has in flight, the smaller the part of B its L2 has to hold.  LAPIS_HIP_SPMM_ROUNDS = 2, 4 for tuning.
  const int rounds = getenv("LAPIS_HIP_SPMM_ROUNDS") ? atoi(getenv("LAPIS_HIP_SPMM_ROUNDS")) : 1;
  if (rounds == 4) launch_group_row_r<T, LPR, 4>(nrows, pos, crd, val, B, ldb, C, ldc, st);
  else if (rounds == 2) launch_group_row_r<T, LPR, 2>(nrows, pos, crd, val, B, ldb, C, ldc, st);
  else launch_group_row_r<T, LPR, 1>(nrows, pos, crd, val, B, ldb, C, ldc, st);
}

constexpr int kSpmmLdsBytes = 128 * 1024;  // staged rows of B per workgroup of the LDS kernel

// Row block and halo of the LDS kernel for rows of `row_bytes` bytes: a quarter of the
// staged rows on either side of the block, from the halo widths the plan has statistics for.
void lds_block_shape(int64_t row_bytes, int *rb, int *halo, int *halo_index) {
  const int64_t rows = kSpmmLdsBytes / row_bytes;
  const int widths[4] = {32, 64, 128, 256};
  int i = 0;
  while (i + 1 < 4 && widths[i + 1] * 4 <= rows) ++i;
  *halo = widths[i];
  *halo_index = i;
  *rb = (int)std::max<int64_t>(16, rows - 2 * widths[i]);
}

template <typename T, int LPR>
int launch_rowblock_lds(int64_t nrows, int64_t ncols, int rb, int halo, const int *pos, const int *crd, const T *val,
                        const T *B, int64_t ldb, T *C, int64_t ldc, hipStream_t st) {
  auto kernel = spmm_rowblock_lds_kernel<T, LPR>;
  static std::once_flag attribute_once;
  static hipError_t attribute_status = hipSuccess;
  std::call_once(attribute_once, [&] {
    attribute_status = hipFuncSetAttribute(reinterpret_cast<const void *>(kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  });
  LAPIS_HIP_TRY(attribute_status);
  const size_t lds = (size_t)(rb + 2 * halo) * LPR * 16;
  const dim3 grid((unsigned)ceil_div(nrows, rb)), block(1024);
  hipEvent_t e0, e1;
  if (timing_next_events(&e0, &e1))
    hipExtLaunchKernelGGL(kernel, grid, block, lds, st, e0, e1, 0, (int)nrows, (int)ncols, rb, halo, pos, crd, val, B,
                          (long long)ldb, C, (long long)ldc);
  else
    hipLaunchKernelGGL(kernel, grid, block, lds, st, (int)nrows, (int)ncols, rb, halo, pos, crd, val, B, (long long)ldb, C,
                       (long long)ldc);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}

// name of the kernel the calling thread's last SpMM ran (lapis_hip_spmm_last_kernel)
static thread_local const char *g_last_spmm_kernel = "";

template <typename T>
int spmm_impl(const char *what, const lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols, int64_t k,
              const int32_t *pos, const int32_t *crd, const T *val, const T *B, int64_t ldb, T *C, int64_t ldc,
              lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(nrows >= 0 && ncols >= 0 && k >= 0, "%s: negative dimension", what);
  LAPIS_REQUIRE(nrows <= INT32_MAX - 64 && ncols <= INT32_MAX && k <= INT32_MAX, "%s: dimension exceeds int32", what);
  LAPIS_REQUIRE(ldb >= k && ldc >= k, "%s: leading dimension smaller than k=%lld", what, (long long)k);
  if (plan && (plan->stats.nrows != nrows || plan->stats.ncols != ncols || plan->pos != pos))
    return set_error(LAPIS_HIP_ERR_PLAN_MISMATCH, "%s: plan was built for a %lld x %lld matrix at positions %p", what,
                     (long long)plan->stats.nrows, (long long)plan->stats.ncols, (const void *)plan->pos);
  if (nrows == 0 || k == 0) return LAPIS_HIP_OK;
  LAPIS_REQUIRE(pos && C, "%s: null positions or C", what);
  LAPIS_REQUIRE(ncols == 0 || (crd && val && B), "%s: null coordinates, values or B", what);
  if (ncols == 0) return LAPIS_HIP_OK;  // a matrix without columns has no non-zeros
  hipStream_t st = as_stream(stream);
  constexpr int VW = RowVec<T>::width;
  const bool vec = aligned16(B) && aligned16(C) && (ldb % VW == 0) && (ldc % VW == 0) && (k % VW == 0);
  // The LDS-staged kernel: whole B rows of a power-of-two number of vectors, between 64 bytes and 1 KB,
  // and at least three non-zeros per row inside the window it would stage.
  const int64_t lpr = vec ? k / VW : 0;
  const char *force = getenv("LAPIS_HIP_SPMM_KERNEL");  // "lds" / "wave": tuning and tests
  bool use_lds = false;
  int rb = 0, halo = 0, hi = 0;
  if (vec && lpr >= 4 && lpr <= 64 && (lpr & (lpr - 1)) == 0) {
    lds_block_shape(k * (int64_t)sizeof(T), &rb, &halo, &hi);
    // Never chosen automatically: measured on MI355X it loses to the kernels below wherever it applies
    // (7-point stencil 100^3, k = 64 fp32: 0.625 ms against 0.259 ms; 27-point x 3 unknowns 60^3: 1.55 against
    // 0.94 ms).  The window a block stages is read from L2 once per block, halo included (twice B in
    // all), the block cannot start on its rows before the window is in, and the reuse it serves -- a
    // B row used by neighbouring rows -- is reuse the 32 KB vector cache of the CU already catches.
    if (force && !strcmp(force, "lds")) use_lds = true;
  }
  if (force && !strcmp(force, "wave")) use_lds = false;
  // Group-per-row: whole B rows of up to 32 vectors (a wavefront holds at least two rows), rows short and
  // even enough that the groups of a wavefront finish together.
  bool use_group = false;
  if (vec && lpr >= 1 && lpr <= 32 && (lpr & (lpr - 1)) == 0 && plan) {
    const lapis_hip_csr_stats &ps = plan->stats;
    // ... and the B rows a stretch of 1024 non-zeros touches fit the L2s (matrices with column locality:
    // 7-point stencil, k = 64 fp32: 0.259 ms against 0.433 ms for the wavefront-per-row kernel, k = 16: 0.080
    // against 0.310; 81 per row FEM: 0.94 against 1.01).  With columns all over B every gather goes to HBM
    // and the wavefront-per-row kernel, which keeps more of them in flight, is 6-30 % faster.
    use_group = ps.mean_row_len <= 256.0 && (double)ps.max_row_len <= 4.0 * std::max(ps.mean_row_len, 8.0) &&
                ps.mean_chunk_col_span >= 0.0 && ps.mean_chunk_col_span * (double)(k * sizeof(T)) <= 32.0 * 1024 * 1024;
  }
  if (force) {
    use_group = !strcmp(force, "group") && vec && lpr >= 1 && lpr <= 32 && (lpr & (lpr - 1)) == 0;
    if (use_group) use_lds = false;
  }
  if (use_group && !use_lds) {
    g_last_spmm_kernel = "spmm_group_row_kernel";
    switch (lpr) {
      case 1: launch_group_row<T, 1>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
      case 2: launch_group_row<T, 2>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
      case 4: launch_group_row<T, 4>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
      case 8: launch_group_row<T, 8>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
      case 16: launch_group_row<T, 16>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
      default: launch_group_row<T, 32>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
    }
    LAPIS_LAUNCH_CHECK();
    return LAPIS_HIP_OK;
  }
  if (use_lds) {
    g_last_spmm_kernel = "spmm_rowblock_lds_kernel";
    switch (lpr) {
      case 4: return launch_rowblock_lds<T, 4>(nrows, ncols, rb, halo, pos, crd, val, B, ldb, C, ldc, st);
      case 8: return launch_rowblock_lds<T, 8>(nrows, ncols, rb, halo, pos, crd, val, B, ldb, C, ldc, st);
      case 16: return launch_rowblock_lds<T, 16>(nrows, ncols, rb, halo, pos, crd, val, B, ldb, C, ldc, st);
      case 32: return launch_rowblock_lds<T, 32>(nrows, ncols, rb, halo, pos, crd, val, B, ldb, C, ldc, st);
      default: return launch_rowblock_lds<T, 64>(nrows, ncols, rb, halo, pos, crd, val, B, ldb, C, ldc, st);
    }
  }
  g_last_spmm_kernel = "spmm_wave_row_kernel";
  // Several gathered B rows in flight per lane pay where B rows come from L2 (columns of a chunk of A within
  // 32 MB of B, or no plan to say otherwise); where every gather goes to HBM they only get in each other's way
  // (config 4 of the benchmarks: 1.21 ms one at a time, 1.26 ms eight at a time).
  bool deep = true;
  if (plan) deep = plan->stats.mean_chunk_col_span * (double)k * sizeof(T) <= 32.0 * 1024 * 1024;
  if (const char *d = getenv("LAPIS_HIP_SPMM_DEEP")) deep = atoi(d) != 0;
  if (vec)
    launch_wave_row_any<T, true>(nrows, k, pos, crd, val, B, ldb, C, ldc, st, deep);
  else
    launch_wave_row_any<T, false>(nrows, k, pos, crd, val, B, ldb, C, ldc, st, deep);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}

}  // namespace lapis

using namespace lapis;

extern "C" const char *lapis_hip_spmm_last_kernel(void) { return g_last_spmm_kernel; }

extern "C" int lapis_hip_spmm_csr_f32_i32(int64_t nrows, int64_t ncols, int64_t k, const int32_t *pos,
                                          const int32_t *crd, const float *val, const float *B, int64_t ldb,
                                          float *C, int64_t ldc, lapis_hip_stream_t stream) {
  return spmm_impl<float>("spmm_csr_f32", nullptr, nrows, ncols, k, pos, crd, val, B, ldb, C, ldc, stream);
}
extern "C" int lapis_hip_spmm_csr_f32_i32_plan(const lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols, int64_t k,
                                               const int32_t *pos, const int32_t *crd, const float *val, const float *B,
                                               int64_t ldb, float *C, int64_t ldc, lapis_hip_stream_t stream) {
  return spmm_impl<float>("spmm_csr_f32_plan", plan, nrows, ncols, k, pos, crd, val, B, ldb, C, ldc, stream);
}
extern "C" int lapis_hip_spmm_csr_f64_i32(int64_t nrows, int64_t ncols, int64_t k, const int32_t *pos,
                                          const int32_t *crd, const double *val, const double *B, int64_t ldb,
                                          double *C, int64_t ldc, lapis_hip_stream_t stream) {
  return spmm_impl<double>("spmm_csr_f64", nullptr, nrows, ncols, k, pos, crd, val, B, ldb, C, ldc, stream);
}
extern "C" int lapis_hip_spmm_csr_f64_i32_plan(const lapis_hip_csr_plan *plan, int64_t nrows, int64_t ncols, int64_t k,
                                               const int32_t *pos, const int32_t *crd, const double *val,
                                               const double *B, int64_t ldb, double *C, int64_t ldc,
                                               lapis_hip_stream_t stream) {
  return spmm_impl<double>("spmm_csr_f64_plan", plan, nrows, ncols, k, pos, crd, val, B, ldb, C, ldc, stream);
}

extern "C" int lapis_hip_bspmm_csrv_f32_i32(int64_t n1, int64_t n2, int64_t dh, int64_t nh, const int32_t *pos,
                                            const int32_t *crd, const float *val, const float *V, float *out,
                                            lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(n1 >= 0 && n2 >= 0 && dh >= 0 && nh >= 0, "bspmm_csrv: negative dimension");
  LAPIS_REQUIRE(n1 <= INT32_MAX - 64 && n2 <= INT32_MAX && dh <= INT32_MAX && nh <= INT32_MAX,
                "bspmm_csrv: dimension exceeds int32");
  if (n1 == 0 || dh == 0 || nh == 0) return LAPIS_HIP_OK;
  LAPIS_REQUIRE(pos && out, "bspmm_csrv: null positions or output");
  LAPIS_REQUIRE(n2 == 0 || (crd && val && V), "bspmm_csrv: null coordinates, values or V");
  if (n2 == 0) return LAPIS_HIP_OK;
  hipLaunchKernelGGL(bspmm_csrv_kernel, dim3((unsigned)ceil_div(n1, 4)), dim3(256), 0, as_stream(stream), (int)n1,
                     (int)dh, (int)nh, pos, crd, val, V, out);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}
