// Measurement kernels behind `bench.py --calibrate-gather`: what one launch of a
// gather-heavy kernel can cost at best on this chip.
//
// Every compute unit runs one workgroup that, per step, streams 16-byte vectors
// (the crd/val stream of an SpMV: 12 bytes per non-zero = three vectors per four
// gathers) and/or gathers doubles from a window of x.  The window size decides where
// the gathers hit (16 KB: the vector cache of the CU; 1 MB: L2; 64 MB: HBM), and
// `lanes_per_line` consecutive lanes of a wave instruction share one 128-byte line,
// which the address unit merges into one request.  Measured on MI355X: a streamed
// line and an L2-hit gather line each take their own time and the two ADD UP
// (805 MB stream 0.122 ms; 67 M single-line gathers 0.255 ms; both 0.424 ms), as if
// every CU could keep a fixed number of line requests in flight whatever they are.
// bench.py turns the two rates into the floor of the column-blocked SpMV kernels.
#include <algorithm>
#include <cstdlib>

#include "common.hpp"

namespace lapis {
namespace {

__device__ __forceinline__ unsigned mix32(unsigned a) {
  a ^= a >> 16;
  a *= 0x7feb352dU;
  a ^= a >> 15;
  a *= 0x846ca68bU;
  a ^= a >> 16;
  return a;
}

// GPT = 4 gathers with a chosen cache policy on the load (gfx950 `sc0`, `sc1`, `nt` bits): the probe for
// whether a policy changes the rate at which L2 serves line requests.  It does not (256-269 G lines/s for
// every combination, 4- and 8-byte elements alike), which is why the SpMV kernels use plain loads.
template <int POLICY>
__device__ __forceinline__ void gather4(const double *const (&p)[4], double (&g)[4]) {
  if (POLICY == 0) {
#pragma unroll
    for (int j = 0; j < 4; ++j) g[j] = *p[j];
    return;
  }
#define LAPIS_GATHER4(BITS)                                                                                        \
  asm volatile("global_load_dwordx2 %0, %4, off " BITS "\n global_load_dwordx2 %1, %5, off " BITS                  \
               "\n global_load_dwordx2 %2, %6, off " BITS "\n global_load_dwordx2 %3, %7, off " BITS               \
               "\n s_waitcnt vmcnt(0)"                                                                             \
               : "=&v"(g[0]), "=&v"(g[1]), "=&v"(g[2]), "=&v"(g[3])                                                \
               : "v"(p[0]), "v"(p[1]), "v"(p[2]), "v"(p[3])                                                        \
               : "memory")
  if (POLICY == 1) LAPIS_GATHER4("nt");
  if (POLICY == 2) LAPIS_GATHER4("sc0");
  if (POLICY == 3) LAPIS_GATHER4("sc1");
  if (POLICY == 4) LAPIS_GATHER4("sc0 sc1");
#undef LAPIS_GATHER4
}

template <int THREADS, int GPT, int SB, bool GATHER, int POLICY>
__global__ __launch_bounds__(THREADS) void calibrate_kernel(const v2d *__restrict__ stream, long long vecs_per_group,
                                                            const double *__restrict__ x, unsigned window_lines,
                                                            int share_log2, int steps, double *__restrict__ sink) {
  const int tid = threadIdx.x;
  const unsigned wave = (blockIdx.x * THREADS + tid) >> 6, lane = tid & 63;
  const v2d *sp = stream + (long long)blockIdx.x * vecs_per_group;
  double acc = 0.0;
  for (int s = 0; s < steps; ++s) {
    double g[GPT];
    v2d sv[SB > 0 ? SB : 1];
    if (SB > 0) {
#pragma unroll
      for (int j = 0; j < SB; ++j) sv[j] = load_stream(sp + ((long long)s * SB + j) * THREADS + tid);
    }
    if (GATHER) {
      static_assert(GPT == 4, "gather4 takes four addresses");
      const double *gp[GPT];
#pragma unroll
      for (int j = 0; j < GPT; ++j) {
        const unsigned line =
            mix32((wave * 4099u + (unsigned)s) * 64u * GPT + j * 64u + (lane >> share_log2)) % window_lines;
        gp[j] = x + (size_t)line * 16 + (lane & 15);
      }
      gather4<POLICY>(gp, g);
#pragma unroll
      for (int j = 0; j < GPT; ++j) acc += g[j];
    }
    if (SB > 0) {
#pragma unroll
      for (int j = 0; j < SB; ++j) acc += sv[j].x + sv[j].y;
    }
  }
  if (acc == 1.2345e300) sink[blockIdx.x] = acc;  // keeps the loads alive; never true for finite inputs
}

template <bool GATHER, int SB>
int run(const double *x, int64_t window_bytes, int share_log2, const void *stream, int64_t stream_bytes, int64_t gathers,
        double *sink, double *elapsed_ms, double *gathers_done, double *stream_bytes_done, hipStream_t st) {
  constexpr int THREADS = 512, GPT = 4;
  const int groups = std::max(1, device_cu_count());
  const long long per_step = (long long)groups * THREADS * GPT;
  const int steps = (int)std::max<long long>(1, gathers / per_step);
  const long long vecs_per_group = (long long)steps * SB * THREADS;
  if (SB > 0 && vecs_per_group * groups * 16 > stream_bytes)
    return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "calibrate_gather: the stream buffer holds %lld bytes, %lld are needed",
                     (long long)stream_bytes, vecs_per_group * groups * 16);
  const unsigned window_lines = (unsigned)std::max<int64_t>(1, window_bytes / 128);
  hipEvent_t e0, e1;
  LAPIS_HIP_TRY(hipEventCreate(&e0));
  LAPIS_HIP_TRY(hipEventCreate(&e1));
  float best = 0.f;
  hipError_t err = hipSuccess;
  // LAPIS_HIP_CALIBRATE_POLICY = 1 (nt), 2 (sc0), 3 (sc1), 4 (sc0 sc1): cache policy of the gathers
  const char *pol = GATHER ? getenv("LAPIS_HIP_CALIBRATE_POLICY") : nullptr;
  const int policy = pol ? atoi(pol) : 0;
  if (policy < 0 || policy > 4)
    return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "calibrate_gather: LAPIS_HIP_CALIBRATE_POLICY must be 0..4, got %d", policy);
  for (int rep = 0; rep < 6 && err == hipSuccess; ++rep) {
    const dim3 grid(groups), block(THREADS);
    const v2d *sv = static_cast<const v2d *>(stream);
#define LAPIS_CAL_LAUNCH(P)                                                                                       \
  hipExtLaunchKernelGGL((calibrate_kernel<THREADS, GPT, SB, GATHER, P>), grid, block, 0, st, e0, e1, 0, sv,      \
                        vecs_per_group, x, window_lines, share_log2, steps, sink)
    switch (policy) {
      case 1: LAPIS_CAL_LAUNCH(1); break;
      case 2: LAPIS_CAL_LAUNCH(2); break;
      case 3: LAPIS_CAL_LAUNCH(3); break;
      case 4: LAPIS_CAL_LAUNCH(4); break;
      default: LAPIS_CAL_LAUNCH(0); break;
    }
#undef LAPIS_CAL_LAUNCH
    err = hipGetLastError();
    if (err == hipSuccess) err = hipEventSynchronize(e1);
    float ms = 0.f;
    if (err == hipSuccess) err = hipEventElapsedTime(&ms, e0, e1);
    if (rep > 0 && (best == 0.f || ms < best)) best = ms;  // the first launch warms the caches
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (err != hipSuccess) return set_error(LAPIS_HIP_ERR_RUNTIME, "calibrate_gather: %s", hipGetErrorString(err));
  *elapsed_ms = best;
  if (gathers_done) *gathers_done = GATHER ? (double)steps * per_step : 0.0;
  if (stream_bytes_done) *stream_bytes_done = (double)vecs_per_group * groups * 16;
  return LAPIS_HIP_OK;
}

}  // namespace
}  // namespace lapis

using namespace lapis;

extern "C" int lapis_hip_calibrate_gather(const double *x, int64_t window_bytes, int lanes_per_line, const void *stream_buf,
                                          int64_t stream_bytes, int64_t gathers, double *sink, double *elapsed_ms,
                                          double *gathers_done, double *stream_bytes_done, lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(elapsed_ms && sink, "calibrate_gather: null output");
  LAPIS_REQUIRE(gathers > 0, "calibrate_gather: nothing to do");
  LAPIS_REQUIRE(lanes_per_line == 0 || (lanes_per_line >= 1 && lanes_per_line <= 16 &&
                                        (lanes_per_line & (lanes_per_line - 1)) == 0),
                "calibrate_gather: lanes per line must be 0 (no gathers) or a power of two up to 16");
  LAPIS_REQUIRE(lanes_per_line == 0 || (x && window_bytes >= 128), "calibrate_gather: gathers need a window of x");
  LAPIS_REQUIRE(lanes_per_line != 0 || stream_buf, "calibrate_gather: neither gathers nor a stream");
  int share_log2 = 0;
  while ((1 << share_log2) < lanes_per_line) ++share_log2;
  hipStream_t st = as_stream(stream);
  if (lanes_per_line == 0)
    return run<false, 3>(x, 128, 0, stream_buf, stream_bytes, gathers, sink, elapsed_ms, gathers_done, stream_bytes_done, st);
  if (stream_buf)
    return run<true, 3>(x, window_bytes, share_log2, stream_buf, stream_bytes, gathers, sink, elapsed_ms, gathers_done,
                        stream_bytes_done, st);
  return run<true, 0>(x, window_bytes, share_log2, nullptr, 0, gathers, sink, elapsed_ms, gathers_done, stream_bytes_done,
                      st);
}
