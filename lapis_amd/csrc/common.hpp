// Shared host/device helpers of the gfx950 kernel library.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>

#include "lapis_hip.h"

namespace lapis {

constexpr int kWave = 64;  // CDNA wavefront width

// ---- host: status and error text ---------------------------------------------
int set_error(int status, const char *fmt, ...);
bool is_initialized();

#define LAPIS_CHECK_INIT()                                                          \
  do {                                                                              \
    if (!::lapis::is_initialized())                                                 \
      return ::lapis::set_error(LAPIS_HIP_ERR_NOT_INITIALIZED,                      \
                                "%s: lapis_hip_init() has not been called", __func__); \
  } while (0)

#define LAPIS_HIP_TRY(expr)                                                         \
  do {                                                                              \
    hipError_t e_ = (expr);                                                         \
    if (e_ != hipSuccess)                                                           \
      return ::lapis::set_error(LAPIS_HIP_ERR_RUNTIME, "%s: %s failed: %s", __func__, #expr, \
                                hipGetErrorString(e_));                             \
  } while (0)

#define LAPIS_LAUNCH_CHECK() LAPIS_HIP_TRY(hipGetLastError())

#define LAPIS_REQUIRE(cond, ...)                                                    \
  do {                                                                              \
    if (!(cond)) return ::lapis::set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, __VA_ARGS__); \
  } while (0)

inline hipStream_t as_stream(lapis_hip_stream_t s) { return reinterpret_cast<hipStream_t>(s); }
inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

int device_cu_count();

// Event pair for the next launch of a dominant kernel while kernel timing is on
// (see lapis_hip_kernel_timing_start); false when timing is off or the ring is full.
bool timing_next_events(hipEvent_t *start, hipEvent_t *stop);

// Launches `kernel`, attaching a start/stop event pair to the dispatch when kernel
// timing is on.
template <typename... KArgs, typename... Args>
inline void launch_timed(void (*kernel)(KArgs...), dim3 grid, dim3 block, hipStream_t st, Args... args) {
  hipEvent_t e0, e1;
  if (timing_next_events(&e0, &e1))
    hipExtLaunchKernelGGL(kernel, grid, block, 0, st, e0, e1, 0, args...);
  else
    hipLaunchKernelGGL(kernel, grid, block, 0, st, args...);
}

// ---- device: vector types, streaming loads ------------------------------------
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef double v2d __attribute__((ext_vector_type(2)));

// Streamed-once data (crd, val, pos) is loaded non-temporally so that it does not
// displace the gathered vector x from L2.
template <typename V>
__device__ __forceinline__ V load_stream(const V *p) {
  return __builtin_nontemporal_load(p);
}
template <typename V>
__device__ __forceinline__ void store_stream(V *p, V v) {
  __builtin_nontemporal_store(v, p);
}

template <bool NT, typename V>
__device__ __forceinline__ V ldv(const V *p) {
  if (NT) return load_stream(p);
  return *p;
}

// Largest row r in [lo, hi] with pos[r] <= j: the row that holds non-zero j when the positions
// ascend.  The structure has not been validated when this runs: whatever pos holds, the
// search ends after log2(hi - lo) steps and stays inside [lo, hi].
__device__ __forceinline__ int row_of_entry(const int *__restrict__ pos, long long j, int lo, int hi) {
  while (lo < hi) {
    const int mid = (int)(((long long)lo + hi + 1) >> 1);
    if (pos[mid] <= j) lo = mid; else hi = mid - 1;
  }
  return lo;
}

// Row sums in LDS are doubles for every value type: ds_add_f32 runs at a tenth of the
// rate of ds_add_f64 on this chip (203 against 1780 G adds/s over random words, measured).
__device__ __forceinline__ void lds_add(double *p, double v) { unsafeAtomicAdd(p, v); }

// ---- device: DPP wavefront reductions -------------------------------------------
template <int CTRL>
__device__ __forceinline__ int dpp_mov(int v) {
  return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, false);
}
template <int CTRL>
__device__ __forceinline__ float dpp_get(float v) {
  return __builtin_bit_cast(float, dpp_mov<CTRL>(__builtin_bit_cast(int, v)));
}
template <int CTRL>
__device__ __forceinline__ double dpp_get(double v) {
  v2i w = __builtin_bit_cast(v2i, v);
  w.x = dpp_mov<CTRL>(w.x);
  w.y = dpp_mov<CTRL>(w.y);
  return __builtin_bit_cast(double, w);
}

// Sum over aligned groups of W consecutive lanes; every lane of a group ends with
// the group's total.  Steps inside a 16-lane DPP row use quad_perm / row mirrors
// (no LDS traffic); the 32- and 64-lane steps cross rows with a bpermute.
template <int W, typename T>
__device__ __forceinline__ T group_sum(T v) {
  static_assert(W >= 1 && W <= 64 && (W & (W - 1)) == 0, "W must be a power of two <= 64");
  if (W >= 2) v = v + dpp_get<0xB1>(v);   // quad_perm [1,0,3,2]
  if (W >= 4) v = v + dpp_get<0x4E>(v);   // quad_perm [2,3,0,1]
  if (W >= 8) v = v + dpp_get<0x141>(v);  // row_half_mirror
  if (W >= 16) v = v + dpp_get<0x140>(v); // row_mirror
  if (W >= 32) v = v + __shfl_xor(v, 16, 64);
  if (W >= 64) v = v + __shfl_xor(v, 32, 64);
  return v;
}

// Workgroups are handed to the 8 XCDs round-robin (workgroup b runs on XCD b % 8), and
// each XCD has its own L2.  With this map XCD k works on the k-th contiguous eighth
// of the logical blocks instead of every eighth one, so neighbouring blocks, which
// gather from overlapping parts of x, share an L2.  A bijection on [0, nblocks).
constexpr int kXcds = 8;
__device__ __forceinline__ unsigned xcd_contiguous_block(unsigned b, unsigned nblocks) {
  const unsigned xcd = b % kXcds, idx = b / kXcds;
  const unsigned q = nblocks / kXcds, r = nblocks % kXcds;
  return xcd * q + (xcd < r ? xcd : r) + idx;
}

// Orders LDS traffic between the lanes of ONE wavefront (no s_barrier): LDS
// operations of a wave execute in issue order, the fences stop the compiler from
// moving accesses across this point.
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// rows[k] = row of non-zero j0 + k for the up to 1024 consecutive non-zeros [j0, j1) of one wavefront
// (`rows` is that wavefront's own 1024 ints of LDS; all 64 lanes call).  Lanes 0 and 1 bisect the
// positions for the rows of the first and last entry; every row in between that starts inside the
// chunk leaves its number at its starting entry, and a running maximum over the chunk spreads the
// numbers to the entries that follow (empty rows start at the entry of the next row that has one, which
// wins the maximum).  A chunk that spans more than 2048 rows bisects entry by entry instead.  Works on
// positions nobody has validated yet: every LDS index is checked, every row stays in [0, nrows).
__device__ __forceinline__ void rows_of_chunk(const int *__restrict__ pos, int nrows, long long j0, long long j1,
                                              int *rows) {
  const int lane = threadIdx.x & 63;
  const int n = (int)(j1 - j0);
  int edge = 0;
  if (lane < 2) edge = row_of_entry(pos, lane == 0 ? j0 : j1 - 1, 0, nrows - 1);
  const int r_lo = __shfl(edge, 0, 64), r_hi = __shfl(edge, 1, 64);
  if (r_hi - r_lo > 2048 || r_hi < r_lo) {
    for (int k = lane; k < n; k += 64) rows[k] = row_of_entry(pos, j0 + k, r_lo, r_hi < r_lo ? r_lo : r_hi);
    wave_lds_sync();
    return;
  }
  for (int k = lane; k < 1024; k += 64) rows[k] = 0;
  wave_lds_sync();
  for (int r = r_lo + 1 + lane; r <= r_hi; r += 64) {
    const long long at = (long long)pos[r] - j0;
    if (at >= 0 && at < n) atomicMax(rows + at, r - r_lo);
  }
  wave_lds_sync();
  int local[16];
  int m = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    m = max(m, rows[lane * 16 + i]);
    local[i] = m;
  }
  int incl = m;
  for (int o = 1; o < 64; o <<= 1) {
    const int t = __shfl_up(incl, o, 64);
    if (lane >= o) incl = max(incl, t);
  }
  int before = __shfl_up(incl, 1, 64);
  if (lane == 0) before = 0;
#pragma unroll
  for (int i = 0; i < 16; ++i) rows[lane * 16 + i] = r_lo + max(local[i], before);
  wave_lds_sync();
}

}  // namespace lapis
