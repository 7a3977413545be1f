// Dense vector kernels of the CG path: dot, axpby, mult, div, fill, copy, scale.
// They replace the RangePolicy parallel_for / parallel_reduce launches the
// reference emits for the linalg.generic / linalg.dot ops of
// examples/pcg_solve.py:22-47.
#include <mutex>

#include "blas1.hpp"
#include "common.hpp"

namespace lapis {

// ---- elementwise ----------------------------------------------------------------
// One pass; each thread takes VW consecutive elements with one 128-bit access when
// every buffer is 16-byte aligned, the last n % VW elements go to the tail threads.
template <typename T>
struct VecOf;
template <>
struct VecOf<double> {
  typedef v2d type;
  static constexpr int width = 2;
};
template <>
struct VecOf<float> {
  typedef v4f type;
  static constexpr int width = 4;
};

template <typename T, typename F, int NIN>
__global__ __launch_bounds__(256) void elementwise_kernel(long long n, long long nvec, const T *a, const T *b,
                                                          T *dst, F f) {
  typedef typename VecOf<T>::type V;
  constexpr int VW = VecOf<T>::width;
  const long long t = (long long)blockIdx.x * 256 + threadIdx.x;
  if (t < nvec) {
    V va = {}, vb = {}, vo;
    if (NIN >= 1) va = reinterpret_cast<const V *>(a)[t];
    if (NIN >= 2) vb = reinterpret_cast<const V *>(b)[t];
#pragma unroll
    for (int e = 0; e < VW; ++e) vo[e] = f(va[e], vb[e]);
    reinterpret_cast<V *>(dst)[t] = vo;
  } else {
    const long long i = nvec * VW + (t - nvec);
    if (i < n) {
      const T xa = NIN >= 1 ? a[i] : T(0);
      const T xb = NIN >= 2 ? b[i] : T(0);
      dst[i] = f(xa, xb);
    }
  }
}

template <typename T, int NIN, typename F>
int launch_elementwise(const char *what, int64_t n, const T *a, const T *b, T *dst, F f, hipStream_t st) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(n >= 0, "%s: negative length", what);
  if (n == 0) return LAPIS_HIP_OK;
  LAPIS_REQUIRE(dst && (NIN < 1 || a) && (NIN < 2 || b), "%s: null buffer with n=%lld", what, (long long)n);
  constexpr int VW = VecOf<T>::width;
  const bool vec = aligned16(dst) && (NIN < 1 || aligned16(a)) && (NIN < 2 || aligned16(b));
  const long long nvec = vec ? n / VW : 0;
  const long long threads = nvec + (n - nvec * VW);
  const long long blocks = ceil_div(threads, 256);
  LAPIS_REQUIRE(blocks <= 0x7fffffffLL, "%s: n=%lld exceeds the grid limit", what, (long long)n);
  hipLaunchKernelGGL((elementwise_kernel<T, F, NIN>), dim3((unsigned)blocks), dim3(256), 0, st, (long long)n,
                     nvec, a, b, dst, f);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}

template <typename T>
struct AxpbyOp {
  T a, b;
  // x*a and y*b are rounded separately, then added (examples/pcg_solve.py:33-35)
  __device__ T operator()(T x, T y) const {
    const T t0 = x * a;
    const T t1 = y * b;
    return t0 + t1;
  }
};
template <typename T>
struct MultOp {
  __device__ T operator()(T x, T y) const { return x * y; }
};
template <typename T>
struct DivOp {
  __device__ T operator()(T x, T y) const { return x / y; }
};
template <typename T>
struct FillOp {
  T v;
  __device__ T operator()(T, T) const { return v; }
};
template <typename T>
struct CopyOp {
  __device__ T operator()(T x, T) const { return x; }
};
template <typename T>
struct ScaleOp {
  T a;
  __device__ T operator()(T x, T) const { return x * a; }
};

// ---- dot --------------------------------------------------------------------------
// Two launches: each block sums a grid-strided slice (per-thread partial, DPP wave
// sum, LDS across the four waves in wave order) into partials[block]; a one-block
// kernel behind it adds the partials in index order and writes init + total.  The
// order is fixed, so the result is the same from run to run, and the kernel boundary
// does the ordering: no device-scope fence, which on a multi-XCD part would write
// back and invalidate L2 once per block.
template <typename T>
__device__ __forceinline__ T block_sum_256(T v, T *lds4) {
  v = group_sum<64>(v);
  const int wave = threadIdx.x >> 6;
  if ((threadIdx.x & 63) == 0) lds4[wave] = v;
  __syncthreads();
  const T total = ((lds4[0] + lds4[1]) + lds4[2]) + lds4[3];
  __syncthreads();
  return total;
}

template <typename T>
__global__ __launch_bounds__(256) void dot_partial_kernel(long long n, const T *__restrict__ x,
                                                          const T *__restrict__ y, T *__restrict__ partials,
                                                          int vec) {
  typedef typename VecOf<T>::type V;
  constexpr int VW = VecOf<T>::width;
  __shared__ T lds4[4];
  T acc = T(0);
  const long long nv = vec ? n / VW : 0;  // 128-bit accesses when both vectors are 16-byte aligned
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nv; i += (long long)gridDim.x * 256) {
    const V a = reinterpret_cast<const V *>(x)[i], b = reinterpret_cast<const V *>(y)[i];
#pragma unroll
    for (int e = 0; e < VW; ++e) acc = acc + a[e] * b[e];
  }
  for (long long i = nv * VW + (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256)
    acc = acc + x[i] * y[i];
  const T total = block_sum_256(acc, lds4);
  if (threadIdx.x == 0) partials[blockIdx.x] = total;
}

template <typename T>
__global__ __launch_bounds__(256) void dot_final_kernel(int count, const T *__restrict__ partials, T init,
                                                        T *__restrict__ result) {
  __shared__ T lds4[4];
  T s = T(0);
  for (int i = threadIdx.x; i < count; i += 256) s = s + partials[i];
  const T all = block_sum_256(s, lds4);
  if (threadIdx.x == 0) *result = all + init;
}


// dst = a*x + b*y and the partial sums of dst . z in one pass (z == nullptr: dst . dst).  Element order,
// grid and the order of the additions are those of elementwise_kernel and dot_partial_kernel, so the pair
// of results has the bits the two separate calls give.
template <typename T>
__global__ __launch_bounds__(256) void axpby_dot_partial_kernel(long long n, T a, const T *x, T b, const T *y, T *dst,
                                                                const T *z, T *__restrict__ partials, int vec) {
  typedef typename VecOf<T>::type V;
  constexpr int VW = VecOf<T>::width;
  __shared__ T lds4[4];
  T acc = T(0);
  const long long nv = vec ? n / VW : 0;
  for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < nv; i += (long long)gridDim.x * 256) {
    const V vx = reinterpret_cast<const V *>(x)[i], vy = reinterpret_cast<const V *>(y)[i];
    V vd;
#pragma unroll
    for (int e = 0; e < VW; ++e) vd[e] = a * vx[e] + b * vy[e];
    const V vz = z ? reinterpret_cast<const V *>(z)[i] : vd;
    reinterpret_cast<V *>(dst)[i] = vd;
#pragma unroll
    for (int e = 0; e < VW; ++e) acc = acc + vd[e] * vz[e];
  }
  for (long long i = nv * VW + (long long)blockIdx.x * 256 + threadIdx.x; i < n; i += (long long)gridDim.x * 256) {
    const T d = a * x[i] + b * y[i];
    const T w = z ? z[i] : d;
    dst[i] = d;
    acc = acc + d * w;
  }
  const T total = block_sum_256(acc, lds4);
  if (threadIdx.x == 0) partials[blockIdx.x] = total;
}

int dot_grid(int64_t n) {
  const int64_t want = ceil_div(n, 256 * 8);
  const int64_t cap = std::max(1, device_cu_count()) * 8;
  return (int)std::max<int64_t>(1, std::min<int64_t>(std::min<int64_t>(want, cap), kDotMaxBlocks));
}

template <typename T>
int launch_dot(int64_t n, const T *x, const T *y, T init, T *result, T *partials, hipStream_t st) {
  const int grid = dot_grid(n);
  hipLaunchKernelGGL((dot_partial_kernel<T>), dim3(grid), dim3(256), 0, st, (long long)n, x, y, partials,
                     (aligned16(x) && aligned16(y)) ? 1 : 0);
  hipLaunchKernelGGL((dot_final_kernel<T>), dim3(1), dim3(256), 0, st, grid, (const T *)partials, init, result);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}
template int launch_dot<double>(int64_t, const double *, const double *, double, double *, double *, hipStream_t);
template int launch_dot<float>(int64_t, const float *, const float *, float, float *, float *, hipStream_t);

// Scratch for the stand-alone dot entry points: a ring of slots, one per call, so
// that dots queued on different streams do not share partials unless more than
// kSlots of them are in flight at once.
namespace {
constexpr int kSlots = 64;
std::mutex g_scratch_mutex;
char *g_scratch = nullptr;  // kSlots * kDotMaxBlocks * 8 bytes
unsigned g_next_slot = 0;
constexpr size_t kSlotBytes = ((size_t)kDotMaxBlocks + 2) * 8;  // the partials, then one result for the *_host entries

int take_slot(void **partials) {
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch) LAPIS_HIP_TRY(hipMalloc(&g_scratch, kSlots * kSlotBytes));
  *partials = g_scratch + (size_t)(g_next_slot++ % kSlots) * kSlotBytes;
  return LAPIS_HIP_OK;
}

// ---- the dot that allocates nothing ------------------------------------------------
// Partials of lapis_hip_dot_f64_noalloc: a fixed array in the code object instead of the
// ring above, so the entry point never calls hipMalloc.  Every GPU holds its own copy at
// its own address; host code uses the address hipGetSymbolAddress returns for the
// current device, never the array's name.
static __device__ __align__(256) double g_dot_noalloc_scratch[kDotMaxBlocks];
constexpr int kMaxDevices = 64;
std::mutex g_noalloc_mutex;
double *g_noalloc_ptr[kMaxDevices] = {};

int noalloc_scratch(double **out) {
  int dev = 0;
  LAPIS_HIP_TRY(hipGetDevice(&dev));
  LAPIS_REQUIRE(dev >= 0 && dev < kMaxDevices, "dot_f64_noalloc: device ordinal %d outside [0, %d)", dev, kMaxDevices);
  std::lock_guard<std::mutex> lock(g_noalloc_mutex);
  if (!g_noalloc_ptr[dev]) {
    void *p = nullptr;
    LAPIS_HIP_TRY(hipGetSymbolAddress(&p, HIP_SYMBOL(g_dot_noalloc_scratch)));
    g_noalloc_ptr[dev] = static_cast<double *>(p);
  }
  *out = g_noalloc_ptr[dev];
  return LAPIS_HIP_OK;
}

template <typename T>
int dot_entry(const char *what, int64_t n, const T *x, const T *y, T init, T *result, lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(n >= 0, "%s: negative length", what);
  LAPIS_REQUIRE(result, "%s: null result", what);
  LAPIS_REQUIRE(n == 0 || (x && y), "%s: null vector with n=%lld", what, (long long)n);
  void *partials = nullptr;
  const int rc = take_slot(&partials);
  if (rc != LAPIS_HIP_OK) return rc;
  return launch_dot<T>(n, x, y, init, result, static_cast<T *>(partials), as_stream(stream));
}
}  // namespace

// Resolves the no-alloc scratch of the current device (called by lapis_hip_init, so that
// the first lapis_hip_dot_f64_noalloc call does no set-up work either).
int dot_noalloc_setup() {
  double *p = nullptr;
  return noalloc_scratch(&p);
}

// Gives the ring of partials back (lapis_hip_finalize at reference count zero).
void dot_release_scratch() {
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch) (void)hipFree(g_scratch);
  g_scratch = nullptr;
  g_next_slot = 0;
}

}  // namespace lapis

using namespace lapis;

extern "C" int lapis_hip_dot_f64_noalloc(int64_t n, const double *x, const double *y, double init, double *result,
                                         lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(n >= 0, "dot_f64_noalloc: negative length");
  if (n > LAPIS_HIP_DOT_NOALLOC_MAX_N)
    return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "dot_f64_noalloc: n=%lld exceeds the maximum of %lld elements",
                     (long long)n, (long long)LAPIS_HIP_DOT_NOALLOC_MAX_N);
  LAPIS_REQUIRE(result, "dot_f64_noalloc: null result");
  LAPIS_REQUIRE(n == 0 || (x && y), "dot_f64_noalloc: null vector with n=%lld", (long long)n);
  double *partials = nullptr;
  const int rc = noalloc_scratch(&partials);
  if (rc != LAPIS_HIP_OK) return rc;
  // dot_partial_kernel writes every partial the final kernel reads (dot_grid(n) of them):
  // nothing of the previous call's contents is read, so nothing has to be cleared.
  return launch_dot<double>(n, x, y, init, result, partials, as_stream(stream));
}


namespace {
// dot with the result on the host: what the reference's parallel_reduce into a host scalar gives
// (TranslateToKokkosCpp.cpp:1696-1705,1838), blocking included.
template <typename T>
int dot_host_entry(const char *what, int64_t n, const T *x, const T *y, T init, T *host_result, lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(n >= 0, "%s: negative length", what);
  LAPIS_REQUIRE(host_result, "%s: null result", what);
  LAPIS_REQUIRE(n == 0 || (x && y), "%s: null vector with n=%lld", what, (long long)n);
  void *partials = nullptr;
  int rc = take_slot(&partials);
  if (rc != LAPIS_HIP_OK) return rc;
  T *device_result = reinterpret_cast<T *>(static_cast<char *>(partials) + (size_t)kDotMaxBlocks * 8);
  hipStream_t st = as_stream(stream);
  rc = launch_dot<T>(n, x, y, init, device_result, static_cast<T *>(partials), st);
  if (rc != LAPIS_HIP_OK) return rc;
  LAPIS_HIP_TRY(hipMemcpyAsync(host_result, device_result, sizeof(T), hipMemcpyDeviceToHost, st));
  LAPIS_HIP_TRY(hipStreamSynchronize(st));
  return LAPIS_HIP_OK;
}

template <typename T>
int axpby_dot_entry(const char *what, int64_t n, T a, const T *x, T b, const T *y, T *dst, const T *z, T init, T *result,
                    lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(n >= 0, "%s: negative length", what);
  LAPIS_REQUIRE(result, "%s: null result", what);
  LAPIS_REQUIRE(n == 0 || (x && y && dst), "%s: null vector with n=%lld", what, (long long)n);
  void *slot = nullptr;
  const int rc = take_slot(&slot);
  if (rc != LAPIS_HIP_OK) return rc;
  T *partials = static_cast<T *>(slot);
  hipStream_t st = as_stream(stream);
  const int grid = dot_grid(n);
  const int vec = (aligned16(x) && aligned16(y) && aligned16(dst) && (!z || aligned16(z))) ? 1 : 0;
  hipLaunchKernelGGL((axpby_dot_partial_kernel<T>), dim3(grid), dim3(256), 0, st, (long long)n, a, x, b, y, dst, z,
                     partials, vec);
  hipLaunchKernelGGL((dot_final_kernel<T>), dim3(1), dim3(256), 0, st, grid, (const T *)partials, init, result);
  LAPIS_LAUNCH_CHECK();
  return LAPIS_HIP_OK;
}
}  // namespace

extern "C" int lapis_hip_dot_f64_host(int64_t n, const double *x, const double *y, double init, double *host_result,
                                      lapis_hip_stream_t stream) {
  return dot_host_entry<double>("dot_f64_host", n, x, y, init, host_result, stream);
}
extern "C" int lapis_hip_dot_f32_host(int64_t n, const float *x, const float *y, float init, float *host_result,
                                      lapis_hip_stream_t stream) {
  return dot_host_entry<float>("dot_f32_host", n, x, y, init, host_result, stream);
}
extern "C" int lapis_hip_axpby_dot_f64(int64_t n, double a, const double *x, double b, const double *y, double *dst,
                                       const double *z, double init, double *result, lapis_hip_stream_t stream) {
  return axpby_dot_entry<double>("axpby_dot_f64", n, a, x, b, y, dst, z, init, result, stream);
}
extern "C" int lapis_hip_axpby_dot_f32(int64_t n, float a, const float *x, float b, const float *y, float *dst,
                                       const float *z, float init, float *result, lapis_hip_stream_t stream) {
  return axpby_dot_entry<float>("axpby_dot_f32", n, a, x, b, y, dst, z, init, result, stream);
}

extern "C" int lapis_hip_dot_f64(int64_t n, const double *x, const double *y, double init, double *result,
                                 lapis_hip_stream_t stream) {
  return dot_entry<double>("dot_f64", n, x, y, init, result, stream);
}
extern "C" int lapis_hip_dot_f32(int64_t n, const float *x, const float *y, float init, float *result,
                                 lapis_hip_stream_t stream) {
  return dot_entry<float>("dot_f32", n, x, y, init, result, stream);
}
extern "C" int lapis_hip_axpby_f64(int64_t n, double a, const double *x, double b, const double *y, double *dst,
                                   lapis_hip_stream_t stream) {
  return launch_elementwise<double, 2>("axpby_f64", n, x, y, dst, AxpbyOp<double>{a, b}, as_stream(stream));
}
extern "C" int lapis_hip_axpby_f32(int64_t n, float a, const float *x, float b, const float *y, float *dst,
                                   lapis_hip_stream_t stream) {
  return launch_elementwise<float, 2>("axpby_f32", n, x, y, dst, AxpbyOp<float>{a, b}, as_stream(stream));
}
extern "C" int lapis_hip_mult_f64(int64_t n, const double *x, const double *y, double *dst,
                                  lapis_hip_stream_t stream) {
  return launch_elementwise<double, 2>("mult_f64", n, x, y, dst, MultOp<double>{}, as_stream(stream));
}
extern "C" int lapis_hip_div_f64(int64_t n, const double *x, const double *y, double *dst,
                                 lapis_hip_stream_t stream) {
  return launch_elementwise<double, 2>("div_f64", n, x, y, dst, DivOp<double>{}, as_stream(stream));
}
extern "C" int lapis_hip_fill_f64(int64_t n, double v, double *dst, lapis_hip_stream_t stream) {
  return launch_elementwise<double, 0>("fill_f64", n, (const double *)nullptr, (const double *)nullptr, dst,
                                       FillOp<double>{v}, as_stream(stream));
}
extern "C" int lapis_hip_fill_f32(int64_t n, float v, float *dst, lapis_hip_stream_t stream) {
  return launch_elementwise<float, 0>("fill_f32", n, (const float *)nullptr, (const float *)nullptr, dst,
                                      FillOp<float>{v}, as_stream(stream));
}
extern "C" int lapis_hip_mult_f32(int64_t n, const float *x, const float *y, float *dst, lapis_hip_stream_t stream) {
  return launch_elementwise<float, 2>("mult_f32", n, x, y, dst, MultOp<float>{}, as_stream(stream));
}
extern "C" int lapis_hip_div_f32(int64_t n, const float *x, const float *y, float *dst, lapis_hip_stream_t stream) {
  return launch_elementwise<float, 2>("div_f32", n, x, y, dst, DivOp<float>{}, as_stream(stream));
}
extern "C" int lapis_hip_copy_f32(int64_t n, const float *src, float *dst, lapis_hip_stream_t stream) {
  return launch_elementwise<float, 1>("copy_f32", n, src, (const float *)nullptr, dst, CopyOp<float>{},
                                      as_stream(stream));
}
extern "C" int lapis_hip_copy_f64(int64_t n, const double *src, double *dst, lapis_hip_stream_t stream) {
  return launch_elementwise<double, 1>("copy_f64", n, src, (const double *)nullptr, dst, CopyOp<double>{},
                                       as_stream(stream));
}
extern "C" int lapis_hip_scale_f64(int64_t n, double alpha, double *val, lapis_hip_stream_t stream) {
  return launch_elementwise<double, 1>("scale_f64", n, val, (const double *)nullptr, val, ScaleOp<double>{alpha},
                                       as_stream(stream));
}
