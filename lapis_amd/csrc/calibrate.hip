// Measurement kernels behind `bench.py --calibrate-gather`: what one launch of a
// gather-heavy kernel can cost at best on this chip.
//
// Every compute unit runs one workgroup that, per step, streams 16-byte vectors
// (the crd/val stream of an SpMV: 12 bytes per non-zero = three vectors per four
// gathers) and/or gathers doubles from a window of x.  The window size decides where
// the gathers hit (16 KB: the vector cache of the CU; 1 MB: L2; 64 MB: HBM), and
// `lanes_per_line` consecutive lanes of a wave instruction share one 128-byte line,
// which the address unit merges into one request.  Measured on MI355X with wavefronts
// that do both: a streamed line and an L2-hit gather line each take their own time and
// the two ADD UP (805 MB stream 0.118 ms; 67 M single-line gathers 0.246 ms; both
// 0.417 ms).  Wavefronts or workgroups with one role each overlap the two by about a
// fifth (lapis_hip_calibrate_mix: 42 M gather lines + 805 MB in 0.215-0.23 ms against
// 0.277 ms for the sum of the parts and 0.262-0.295 ms for wavefronts that do both).
// bench.py turns the two rates into the floor of the column-blocked SpMV kernels.
//
// lapis_hip_calibrate_mix varies the arrangement: wavefronts per CU, loads in flight,
// streaming and gathering split between wavefronts or between workgroups of a CU, the
// stream issued behind the gathers, the cache policy of the stream, the stream sent
// straight to LDS, the stream kept in L2 (what a perfect prefetch would give), and the
// stream read or touched through the scalar cache.
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

// start/stop events of one timed launch, destroyed on every way out
struct EventPair {
  hipEvent_t start = nullptr, stop = nullptr;
  hipError_t create() {
    hipError_t e = hipEventCreate(&start);
    if (e == hipSuccess) e = hipEventCreate(&stop);
    return e;
  }
  ~EventPair() {
    if (start) (void)hipEventDestroy(start);
    if (stop) (void)hipEventDestroy(stop);
  }
};

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
  // LAPIS_HIP_CALIBRATE_POLICY = 1 (nt), 2 (sc0), 3 (sc1), 4 (sc0 sc1): cache policy of the gathers
  const char *pol = GATHER ? getenv("LAPIS_HIP_CALIBRATE_POLICY") : nullptr;
  const int policy = pol ? atoi(pol) : 0;
  if (policy < 0 || policy > 4)
    return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "calibrate_gather: LAPIS_HIP_CALIBRATE_POLICY must be 0..4, got %d", policy);
  EventPair ev;
  LAPIS_HIP_TRY(ev.create());
  const hipEvent_t e0 = ev.start, e1 = ev.stop;
  float best = 0.f;
  hipError_t err = hipSuccess;
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
  if (err != hipSuccess) return set_error(LAPIS_HIP_ERR_RUNTIME, "calibrate_gather: %s", hipGetErrorString(err));
  *elapsed_ms = best;
  if (gathers_done) *gathers_done = GATHER ? (double)steps * per_step : 0.0;
  if (stream_bytes_done) *stream_bytes_done = (double)vecs_per_group * groups * 16;
  return LAPIS_HIP_OK;
}


// ---- arrangements of the same two kinds of load (lapis_hip_calibrate_mix) ----------------------

struct MixArgs {
  const v4i *stream;      // 16-byte vectors; every streaming wavefront has a contiguous region of its own
  long long region_vecs;
  const double *x;
  unsigned window_lines;
  int share_log2;
  int roles;              // 0: every wavefront streams and gathers; 1: wavefronts [0, producers) of a workgroup
                          // stream, the others gather; 2: by arrival order of the workgroup on its CU
  int producers;
  int s_steps, g_steps;   // steps of a streaming / of a gathering wavefront
  int wrap;               // > 0: the stream's step index wraps after this many steps (the stream stays in L2)
  int nt;                 // non-temporal stream loads (policy 1)
  int *cu_count;          // [16 * 256] arrival counters, zero at launch (roles 2)
  double *sink;
};

// which CU this workgroup runs on: XCC id and the SE / SH / CU fields of HW_ID
__device__ __forceinline__ unsigned cu_key() {
  unsigned hw, xcc;
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
  asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
  return ((xcc & 15u) << 8) | ((hw >> 8) & 255u);
}

__device__ __forceinline__ void mix_roles(const MixArgs &a, int *role_lds, int &ns, int &ng, unsigned &swave) {
  const unsigned wave_in_wg = threadIdx.x >> 6, waves_per_wg = blockDim.x >> 6;
  ns = a.s_steps;
  ng = a.g_steps;
  swave = blockIdx.x * waves_per_wg + wave_in_wg;
  if (a.roles == 1) {
    if ((int)wave_in_wg < a.producers) ng = 0; else ns = 0;
    swave = blockIdx.x * a.producers + wave_in_wg;
  } else if (a.roles == 2) {
    if (threadIdx.x == 0) *role_lds = atomicAdd(a.cu_count + cu_key(), 1) & 1;
    __syncthreads();
    if (*role_lds == 0) ng = 0; else ns = 0;
  }
}

__device__ __forceinline__ const double *mix_gather_address(const MixArgs &a, unsigned wave, int s, int j, int gpt,
                                                            unsigned lane) {
  const unsigned line =
      mix32((wave * 4099u + (unsigned)s) * 64u * gpt + j * 64u + (lane >> a.share_log2)) % a.window_lines;
  return a.x + (size_t)line * 16 + (lane & 15);
}

// BEHIND = false: the step's stream loads, then its gathers, one wait for all.  BEHIND = true: the gathers
// first, then the stream loads of the NEXT step, so that the wait for the gathers leaves them in flight.
template <int SB, int GPT, bool BEHIND>
__global__ void calibrate_mix_kernel(MixArgs a) {
  __shared__ int role_lds;
  const unsigned lane = threadIdx.x & 63;
  const unsigned wave = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  int ns, ng;
  unsigned swave;
  mix_roles(a, &role_lds, ns, ng, swave);
  const v4i *sp = a.stream + (long long)swave * a.region_vecs + lane;
  double acc = 0;
  int iacc = 0;
  const int steps = max(ns, ng);
  v4i sv[SB > 0 ? SB : 1];
  auto load_step = [&](int s, v4i (&dst)[SB > 0 ? SB : 1]) {
    const int ss = a.wrap > 0 ? s % a.wrap : s;
#pragma unroll
    for (int j = 0; j < SB; ++j) {
      const v4i *q = sp + ((long long)ss * SB + j) * 64;
      dst[j] = a.nt ? __builtin_nontemporal_load(q) : *q;
    }
  };
  if (BEHIND && SB > 0 && ns > 0) load_step(0, sv);
  for (int s = 0; s < steps; ++s) {
    double g[GPT > 0 ? GPT : 1];
    v4i nv[SB > 0 ? SB : 1];
    if (!BEHIND && SB > 0 && s < ns) load_step(s, sv);
    if (GPT > 0 && s < ng) {
#pragma unroll
      for (int j = 0; j < GPT; ++j) g[j] = *mix_gather_address(a, wave, s, j, GPT, lane);
    }
    if (BEHIND && SB > 0 && s + 1 < ns) load_step(s + 1, nv);
    if (GPT > 0 && s < ng) {
#pragma unroll
      for (int j = 0; j < GPT; ++j) acc += g[j];
    }
    if (SB > 0 && s < ns) {
#pragma unroll
      for (int j = 0; j < SB; ++j) iacc += sv[j].x ^ sv[j].y ^ sv[j].z ^ sv[j].w;
    }
    if (BEHIND && SB > 0 && s + 1 < ns) {
#pragma unroll
      for (int j = 0; j < SB; ++j) sv[j] = nv[j];
    }
  }
  if (acc == 1.2345e300 || iacc == 0x7fffff13) a.sink[blockIdx.x] = acc + iacc;
}

// The stream loads written out with their cache policy bits (POLICY 2: sc0 sc1, 3: sc0 sc1 nt), or
// sent straight to LDS without passing through registers (POLICY 4; every wavefront has SB KB of LDS).
template <int SB, int GPT, int POLICY>
__global__ void calibrate_mix_policy_kernel(MixArgs a) {
  extern __shared__ __align__(16) unsigned char mix_lds[];
  __shared__ int role_lds;
  const unsigned lane = threadIdx.x & 63, wave_in_wg = threadIdx.x >> 6;
  const unsigned wave = blockIdx.x * (blockDim.x >> 6) + wave_in_wg;
  int ns, ng;
  unsigned swave;
  mix_roles(a, &role_lds, ns, ng, swave);
  const v4i *sp = a.stream + (long long)swave * a.region_vecs + lane;
  typedef __attribute__((address_space(3))) unsigned char lds_byte;
  lds_byte *mine = (lds_byte *)mix_lds + wave_in_wg * SB * 1024;
  double acc = 0;
  int iacc = 0;
  const int steps = max(ns, ng);
  for (int s = 0; s < steps; ++s) {
    v4i sv[SB];
    double g[GPT > 0 ? GPT : 1];
    if (s < ns) {
#pragma unroll
      for (int j = 0; j < SB; ++j) {
        const v4i *q = sp + ((long long)s * SB + j) * 64;
        if (POLICY == 2) asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1" : "=v"(sv[j]) : "v"(q) : "memory");
        if (POLICY == 3) asm volatile("global_load_dwordx4 %0, %1, off sc0 sc1 nt" : "=v"(sv[j]) : "v"(q) : "memory");
        if (POLICY == 4)
          __builtin_amdgcn_global_load_lds((const void __attribute__((address_space(1))) *)q,
                                           (void __attribute__((address_space(3))) *)(mine + j * 1024), 16, 0, 2);
      }
    }
    if (GPT > 0 && s < ng) {
#pragma unroll
      for (int j = 0; j < GPT; ++j) g[j] = *mix_gather_address(a, wave, s, j, GPT, lane);
#pragma unroll
      for (int j = 0; j < GPT; ++j) acc += g[j];
    }
    // the compiler does not count loads issued from inline assembly: wait for everything by hand
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    if (s < ns) {
      if (POLICY == 4) {
        iacc += *(__attribute__((address_space(3))) int *)(mine + lane * 16);
      } else {
#pragma unroll
        for (int j = 0; j < SB; ++j) {
          asm volatile("" : "+v"(sv[j]));
          iacc += sv[j].x ^ sv[j].y ^ sv[j].z ^ sv[j].w;
        }
      }
    }
  }
  if (acc == 1.2345e300 || iacc == 0x7fffff13) a.sink[blockIdx.x] = acc + iacc;
}

// ---- the scalar cache as a second way into the CU ----------------------------------------------
typedef int v16i __attribute__((ext_vector_type(16)));

// every wavefront reads its region with 64-byte scalar loads, four in flight
__global__ void calibrate_scalar_stream_kernel(const int *base, long long region_bytes, int steps, double *sink) {
  const unsigned wave = __builtin_amdgcn_readfirstlane((blockIdx.x * blockDim.x + threadIdx.x) >> 6);
  const char *q = (const char *)base + (long long)wave * region_bytes;
  int iacc = 0;
  for (int s = 0; s < steps; ++s) {
    v16i r[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const char *p = q + ((long long)s * 4 + d) * 64;
      asm volatile("s_load_dwordx16 %0, %1, 0x0" : "=s"(r[d]) : "s"(p));
    }
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(r[0]), "+s"(r[1]), "+s"(r[2]), "+s"(r[3]));
#pragma unroll
    for (int d = 0; d < 4; ++d) iacc += r[d][0] ^ r[d][7] ^ r[d][15];
  }
  if (iacc == 0x7fffff13) sink[blockIdx.x] = iacc;
}

// Wavefronts [0, cons) stream and gather as in calibrate_mix_kernel and post their step in LDS; wavefront
// cons + w touches, `ahead` steps in front of wavefront w, the lines that one will stream: one 4-byte
// scalar load per `touch_stride` bytes, never looked at -- a prefetch into L2 that does not pass through
// the vector cache.  The helper's wait is bounded and the consumers wait for nobody.
template <int SB, int GPT>
__global__ void calibrate_scalar_prefetch_kernel(MixArgs a, int cons, int ahead, int touch_stride) {
  __shared__ int progress[16];
  const int tid = threadIdx.x;
  const unsigned lane = tid & 63, wave_in_wg = tid >> 6;
  if (tid < 16) progress[tid] = -1;
  __syncthreads();
  volatile int *prog = progress;
  if ((int)wave_in_wg < cons) {
    const unsigned wave = blockIdx.x * cons + wave_in_wg;
    const v4i *sp = a.stream + (long long)wave * a.region_vecs + lane;
    double acc = 0;
    int iacc = 0;
    for (int s = 0; s < a.s_steps; ++s) {
      v4i sv[SB];
      double g[GPT > 0 ? GPT : 1];
      if (lane == 0) prog[wave_in_wg] = s;
#pragma unroll
      for (int j = 0; j < SB; ++j) sv[j] = __builtin_nontemporal_load(sp + ((long long)s * SB + j) * 64);
      if (GPT > 0) {
#pragma unroll
        for (int j = 0; j < GPT; ++j) g[j] = *mix_gather_address(a, wave, s, j, GPT, lane);
#pragma unroll
        for (int j = 0; j < GPT; ++j) acc += g[j];
      }
#pragma unroll
      for (int j = 0; j < SB; ++j) iacc += sv[j].x ^ sv[j].y ^ sv[j].z ^ sv[j].w;
    }
    if (lane == 0) prog[wave_in_wg] = 0x3fffffff;  // done: the helper never waits again
    if (acc == 1.2345e300 || iacc == 0x7fffff13) a.sink[blockIdx.x] = acc + iacc;
  } else if ((int)wave_in_wg < 2 * cons) {
    const int w = wave_in_wg - cons;
    const unsigned wave = __builtin_amdgcn_readfirstlane(blockIdx.x * cons + w);
    const char *q = (const char *)(a.stream + (long long)wave * a.region_vecs);
    const int step_bytes = SB * 64 * 16;
    int junk = 0;
    for (int s = 0; s < a.s_steps; ++s) {
      int spins = 0;
      while (s > prog[w] + ahead && spins < (1 << 20)) {
        __builtin_amdgcn_s_sleep(2);
        ++spins;
      }
      for (int o = 0; o < step_bytes; o += touch_stride) {
        const char *p = q + (long long)s * step_bytes + o;
        // in-out: the register stays reserved while loads into it are in flight
        asm volatile("s_load_dword %0, %1, 0x0" : "+s"(junk) : "s"(p));
      }
    }
    asm volatile("s_waitcnt lgkmcnt(0)" : "+s"(junk));
    if (junk == 0x7fffff13) a.sink[blockIdx.x] = junk;
  }
}

template <typename Launch>
int time_best_of(Launch launch, int *cu_count, hipStream_t st, double *elapsed_ms) {
  EventPair ev;
  LAPIS_HIP_TRY(ev.create());
  float best = 0.f;
  for (int rep = 0; rep < 6; ++rep) {
    if (cu_count) LAPIS_HIP_TRY(hipMemsetAsync(cu_count, 0, 16 * 256 * sizeof(int), st));
    LAPIS_HIP_TRY(hipEventRecord(ev.start, st));
    launch();
    LAPIS_LAUNCH_CHECK();
    LAPIS_HIP_TRY(hipEventRecord(ev.stop, st));
    LAPIS_HIP_TRY(hipEventSynchronize(ev.stop));
    float ms = 0.f;
    LAPIS_HIP_TRY(hipEventElapsedTime(&ms, ev.start, ev.stop));
    if (rep > 0 && (best == 0.f || ms < best)) best = ms;  // the first launch warms the caches
  }
  *elapsed_ms = best;
  return LAPIS_HIP_OK;
}

template <int SB, int GPT>
int launch_mix(const lapis_hip_calibrate_mode &m, const MixArgs &a, dim3 grid, dim3 block, int *cu_count, hipStream_t st,
               double *elapsed_ms) {
  const size_t lds = (size_t)(block.x / 64) * SB * 1024;
  if (m.scalar == 2)
    return time_best_of(
        [&] {
          hipLaunchKernelGGL((calibrate_scalar_prefetch_kernel<(SB > 0 ? SB : 1), GPT>), grid, dim3(2 * block.x), 0, st, a,
                             (int)(block.x / 64), m.scalar_ahead, m.scalar_stride);
        },
        nullptr, st, elapsed_ms);
  switch (m.stream_policy) {
    case 0:
    case 1:
      if (m.stream_behind)
        return time_best_of([&] { hipLaunchKernelGGL((calibrate_mix_kernel<SB, GPT, true>), grid, block, 0, st, a); },
                            cu_count, st, elapsed_ms);
      return time_best_of([&] { hipLaunchKernelGGL((calibrate_mix_kernel<SB, GPT, false>), grid, block, 0, st, a); },
                          cu_count, st, elapsed_ms);
    case 2:
      return time_best_of(
          [&] { hipLaunchKernelGGL((calibrate_mix_policy_kernel<(SB > 0 ? SB : 1), GPT, 2>), grid, block, 0, st, a); },
          cu_count, st, elapsed_ms);
    case 3:
      return time_best_of(
          [&] { hipLaunchKernelGGL((calibrate_mix_policy_kernel<(SB > 0 ? SB : 1), GPT, 3>), grid, block, 0, st, a); },
          cu_count, st, elapsed_ms);
    default:
      return time_best_of(
          [&] { hipLaunchKernelGGL((calibrate_mix_policy_kernel<(SB > 0 ? SB : 1), GPT, 4>), grid, block, lds, st, a); },
          cu_count, st, elapsed_ms);
  }
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

extern "C" int lapis_hip_calibrate_mix(const lapis_hip_calibrate_mode *mode, const double *x, int64_t window_bytes,
                                       const void *stream_buf, int64_t stream_buf_bytes, int64_t stream_bytes,
                                       int64_t gathers, int *cu_count, double *sink, double *elapsed_ms,
                                       double *gathers_done, double *stream_bytes_done, int *cus_with_both_roles,
                                       lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(mode && elapsed_ms && sink, "calibrate_mix: null mode or output");
  const lapis_hip_calibrate_mode m = *mode;
  LAPIS_REQUIRE(m.threads >= 64 && m.threads <= 1024 && m.threads % 64 == 0, "calibrate_mix: threads must be 64..1024");
  const int sb = m.stream_in_flight, gpt = m.gathers_in_flight;
  LAPIS_REQUIRE(sb == 0 || sb == 3 || sb == 6 || sb == 12, "calibrate_mix: stream loads in flight must be 0, 3, 6 or 12");
  LAPIS_REQUIRE(gpt == 0 || gpt == 2 || gpt == 4 || gpt == 8, "calibrate_mix: gathers in flight must be 0, 2, 4 or 8");
  LAPIS_REQUIRE(sb > 0 || gpt > 0, "calibrate_mix: neither gathers nor a stream");
  LAPIS_REQUIRE(m.roles >= 0 && m.roles <= 2, "calibrate_mix: roles must be 0, 1 or 2");
  LAPIS_REQUIRE(m.stream_policy >= 0 && m.stream_policy <= 4, "calibrate_mix: stream policy must be 0..4");
  LAPIS_REQUIRE(m.scalar >= 0 && m.scalar <= 2, "calibrate_mix: scalar must be 0, 1 or 2");
  LAPIS_REQUIRE(m.lanes_per_line >= 1 && m.lanes_per_line <= 16 && (m.lanes_per_line & (m.lanes_per_line - 1)) == 0,
                "calibrate_mix: lanes per line must be a power of two up to 16");
  LAPIS_REQUIRE(gpt == 0 || (x && window_bytes >= 128), "calibrate_mix: gathers need a window of x");
  LAPIS_REQUIRE(sb == 0 || stream_buf, "calibrate_mix: a stream needs its buffer");
  LAPIS_REQUIRE(m.roles != 2 || cu_count, "calibrate_mix: roles by workgroup need the arrival counters (16 * 256 ints)");
  const int wpw = m.threads / 64;
  LAPIS_REQUIRE(m.roles != 1 || (m.producers >= 1 && m.producers < wpw && sb > 0 && gpt > 0),
                "calibrate_mix: roles by wavefront need 1 <= producers < wavefronts per workgroup, a stream and gathers");
  LAPIS_REQUIRE(m.roles != 2 || (sb > 0 && gpt > 0), "calibrate_mix: roles by workgroup need a stream and gathers");
  LAPIS_REQUIRE(m.scalar == 0 || (m.roles == 0 && m.stream_policy <= 1 && !m.stream_behind && m.stream_in_l2 == 0),
                "calibrate_mix: the scalar modes go with no other option");
  LAPIS_REQUIRE(m.scalar != 2 || (wpw <= 8 && sb > 0 && m.scalar_ahead >= 1 &&
                                  (m.scalar_stride == 64 || m.scalar_stride == 128)),
                "calibrate_mix: scalar prefetch needs at most 512 threads, a stream, ahead >= 1 and a stride of 64 or 128");
  LAPIS_REQUIRE(m.stream_policy <= 1 || (sb > 0 && !m.stream_behind && m.stream_in_l2 == 0),
                "calibrate_mix: stream policies 2..4 go with a plain in-order stream");
  hipStream_t st = as_stream(stream);
  const int nwg = m.workgroups > 0 ? m.workgroups : std::max(1, device_cu_count());
  long long swaves, gwaves;
  if (m.roles == 0) swaves = gwaves = (long long)nwg * wpw;
  else if (m.roles == 1) { swaves = (long long)nwg * m.producers; gwaves = (long long)nwg * (wpw - m.producers); }
  else swaves = gwaves = std::max(1LL, (long long)nwg * wpw / 2);

  if (m.scalar == 1) {  // the stream alone, through the scalar cache
    const long long waves = (long long)nwg * wpw;
    const int steps = (int)std::max<long long>(1, stream_bytes / (waves * 256));
    const long long region = (long long)steps * 256;
    if (waves * region > stream_buf_bytes)
      return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "calibrate_mix: the stream buffer is too small");
    const int rc = time_best_of(
        [&] {
          hipLaunchKernelGGL(calibrate_scalar_stream_kernel, dim3(nwg), dim3(m.threads), 0, st, (const int *)stream_buf,
                             region, steps, sink);
        },
        nullptr, st, elapsed_ms);
    if (gathers_done) *gathers_done = 0.0;
    if (stream_bytes_done) *stream_bytes_done = (double)waves * region;
    if (cus_with_both_roles) *cus_with_both_roles = -1;
    return rc;
  }

  MixArgs a{};
  a.stream = static_cast<const v4i *>(stream_buf);
  a.x = x;
  a.window_lines = (unsigned)std::max<int64_t>(1, window_bytes / 128);
  while ((1 << a.share_log2) < m.lanes_per_line) ++a.share_log2;
  a.roles = m.roles;
  a.producers = m.producers;
  a.s_steps = sb > 0 && stream_bytes > 0 ? (int)std::max<long long>(1, stream_bytes / (swaves * sb * 1024)) : 0;
  a.g_steps = gpt > 0 && gathers > 0 ? (int)std::max<long long>(1, gathers / (gwaves * gpt * 64)) : 0;
  if (m.scalar == 2) a.g_steps = gpt > 0 ? a.s_steps : 0;  // the consumers do both in every step
  // 48 KB per workgroup, read round and round: more than the vector cache holds, and 32 workgroups' worth fit an L2
  a.wrap = m.stream_in_l2 ? std::max(1, 48 / std::max(1, wpw * sb)) : 0;
  a.nt = m.stream_policy == 1;
  a.cu_count = cu_count;
  a.sink = sink;
  a.region_vecs = sb > 0 ? (a.wrap > 0 ? (long long)a.wrap : (long long)a.s_steps) * sb * 64 : 0;
  const long long region_owners = m.roles == 1 ? (long long)nwg * m.producers : (long long)nwg * wpw;
  if (sb > 0 && region_owners * a.region_vecs * 16 > stream_buf_bytes)
    return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "calibrate_mix: the stream buffer holds %lld bytes, %lld are needed",
                     (long long)stream_buf_bytes, region_owners * a.region_vecs * 16);
  const dim3 grid(nwg), block(m.threads);
  int *cc = m.roles == 2 ? cu_count : nullptr;
  int rc = LAPIS_HIP_ERR_INVALID_ARGUMENT;
#define LAPIS_MIX_CASE(SB, GPT) \
  case SB * 16 + GPT: rc = launch_mix<SB, GPT>(m, a, grid, block, cc, st, elapsed_ms); break
  switch (sb * 16 + gpt) {
    LAPIS_MIX_CASE(3, 0);
    LAPIS_MIX_CASE(6, 0);
    LAPIS_MIX_CASE(12, 0);
    LAPIS_MIX_CASE(0, 4);
    LAPIS_MIX_CASE(0, 8);
    LAPIS_MIX_CASE(3, 2);
    LAPIS_MIX_CASE(3, 4);
    LAPIS_MIX_CASE(6, 4);
    LAPIS_MIX_CASE(6, 8);
    LAPIS_MIX_CASE(12, 4);
    LAPIS_MIX_CASE(12, 8);
    default:
      return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "calibrate_mix: no kernel with %d stream loads and %d gathers in flight",
                       sb, gpt);
  }
#undef LAPIS_MIX_CASE
  if (rc != LAPIS_HIP_OK) return rc;
  if (gathers_done) *gathers_done = (double)a.g_steps * gwaves * gpt * 64;
  if (m.scalar == 2 && gathers_done) *gathers_done = (double)a.g_steps * nwg * wpw * gpt * 64;
  if (stream_bytes_done) *stream_bytes_done = (double)a.s_steps * swaves * sb * 1024;
  if (cus_with_both_roles) {
    *cus_with_both_roles = -1;
    if (m.roles == 2) {
      static int host[16 * 256];
      LAPIS_HIP_TRY(hipMemcpy(host, cu_count, sizeof(host), hipMemcpyDeviceToHost));
      int both = 0;
      for (int v : host) both += v == 2;
      *cus_with_both_roles = both;
    }
  }
  return LAPIS_HIP_OK;
}
