// CSR x dense SpMM for gfx950:  C[i,:] = C[i,:] + sum_kk val[kk] * B[crd[kk],:]
// (row-major B and C).  Replaces the i -> kk -> j nest the sparsifier emits for
// CSR x dense linalg.matmul (examples/spmm_dcsr_opdsl.py:73-110).
#include "common.hpp"

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

// One wavefront per row of A.  A row of B (k = LPR * VW values) is covered by LPR
// lanes with one 128-bit load each, so the 64 lanes take G = 64/LPR non-zeros of
// the row per step: every gathered B row is one fully coalesced k*sizeof(T) read.
// The row's crd/val are read once, 64 at a time and coalesced, then handed to the
// lane groups by bpermute.  The G partial rows are added up with xor shuffles.
template <typename T, int LPR>
__global__ __launch_bounds__(256) void spmm_wave_row_kernel(int nrows, const int *__restrict__ pos,
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
    // every lane runs every round (the bpermutes need their source lanes active);
    // a group whose non-zero index falls past the row end sits the round out
#pragma unroll 8
    for (int t0 = 0; t0 < cnt; t0 += G) {
      const int t = t0 + g;
      const int cj = __shfl(c_l, t & 63, 64);
      const T aj = __shfl(a_l, t & 63, 64);
      if (t < cnt) {
        const V b = *reinterpret_cast<const V *>(B + (long long)cj * ldb + l * VW);
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

// Any k, any alignment: one wavefront per row, lane j takes columns j, j+64, ...
template <typename T>
__global__ __launch_bounds__(256) void spmm_wave_row_generic_kernel(int nrows, int k, const int *__restrict__ pos,
                                                                    const int *__restrict__ crd,
                                                                    const T *__restrict__ val,
                                                                    const T *__restrict__ B, long long ldb,
                                                                    T *__restrict__ C, long long ldc) {
  const int lane = threadIdx.x & 63;
  const long long row = (long long)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= nrows) return;
  const int start = pos[row];
  const int end = pos[row + 1];
  for (int jb = 0; jb < k; jb += 64) {
    const int j = jb + lane;
    T acc = T(0);
    for (int base = start; base < end; base += 64) {
      const int cnt = min(64, end - base);
      int c_l = 0;
      T a_l = T(0);
      if (lane < cnt) {
        c_l = crd[base + lane];
        a_l = val[base + lane];
      }
      for (int t = 0; t < cnt; ++t) {
        const int cj = __shfl(c_l, t, 64);
        const T aj = __shfl(a_l, t, 64);
        if (j < k) acc = acc + aj * B[(long long)cj * ldb + j];
      }
    }
    if (j < k) C[row * ldc + j] = acc + C[row * ldc + j];
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

template <typename T, int LPR>
void launch_wave_row(int64_t nrows, const int *pos, const int *crd, const T *val, const T *B, int64_t ldb, T *C,
                     int64_t ldc, hipStream_t st) {
  launch_timed(spmm_wave_row_kernel<T, LPR>, dim3((unsigned)ceil_div(nrows, 4)), dim3(256), st, (int)nrows, pos,
               crd, val, B, (long long)ldb, C, (long long)ldc);
}

template <typename T>
int spmm_impl(const char *what, int64_t nrows, int64_t ncols, int64_t k, const int32_t *pos, const int32_t *crd,
              const T *val, const T *B, int64_t ldb, T *C, int64_t ldc, lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(nrows >= 0 && ncols >= 0 && k >= 0, "%s: negative dimension", what);
  LAPIS_REQUIRE(nrows <= INT32_MAX - 64 && ncols <= INT32_MAX && k <= INT32_MAX, "%s: dimension exceeds int32", what);
  LAPIS_REQUIRE(ldb >= k && ldc >= k, "%s: leading dimension smaller than k=%lld", what, (long long)k);
  if (nrows == 0 || k == 0) return LAPIS_HIP_OK;
  LAPIS_REQUIRE(pos && C, "%s: null positions or C", what);
  LAPIS_REQUIRE(ncols == 0 || (crd && val && B), "%s: null coordinates, values or B", what);
  if (ncols == 0) return LAPIS_HIP_OK;  // a matrix without columns has no non-zeros
  hipStream_t st = as_stream(stream);
  constexpr int VW = RowVec<T>::width;
  const bool vec = aligned16(B) && aligned16(C) && (ldb % VW == 0) && (ldc % VW == 0) && (k % VW == 0);
  const int64_t lpr = vec ? k / VW : 0;
  switch (lpr) {
    case 1: launch_wave_row<T, 1>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
    case 2: launch_wave_row<T, 2>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
    case 4: launch_wave_row<T, 4>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
    case 8: launch_wave_row<T, 8>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
    case 16: launch_wave_row<T, 16>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
    case 32: launch_wave_row<T, 32>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
    case 64: launch_wave_row<T, 64>(nrows, pos, crd, val, B, ldb, C, ldc, st); break;
    default:
      launch_timed(spmm_wave_row_generic_kernel<T>, dim3((unsigned)ceil_div(nrows, 4)), dim3(256), st, (int)nrows,
                   (int)k, pos, crd, val, B, (long long)ldb, C, (long long)ldc);
  }
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}

}  // namespace lapis

using namespace lapis;

extern "C" int lapis_hip_spmm_csr_f32_i32(int64_t nrows, int64_t ncols, int64_t k, const int32_t *pos,
                                          const int32_t *crd, const float *val, const float *B, int64_t ldb,
                                          float *C, int64_t ldc, lapis_hip_stream_t stream) {
  return spmm_impl<float>("spmm_csr_f32", nrows, ncols, k, pos, crd, val, B, ldb, C, ldc, stream);
}
extern "C" int lapis_hip_spmm_csr_f64_i32(int64_t nrows, int64_t ncols, int64_t k, const int32_t *pos,
                                          const int32_t *crd, const double *val, const double *B, int64_t ldb,
                                          double *C, int64_t ldc, lapis_hip_stream_t stream) {
  return spmm_impl<double>("spmm_csr_f64", nrows, ncols, k, pos, crd, val, B, ldb, C, ldc, stream);
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
