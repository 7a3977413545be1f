// Library life cycle, status text and error reporting.
#include <algorithm>
#include <cstring>
#include <mutex>
#include <vector>

#include "blas1.hpp"
#include "common.hpp"

namespace lapis {
namespace {
thread_local char g_error[512] = "";
std::mutex g_mutex;
int g_refcount = 0;
int g_cu_count = 0;

// kernel timing: a ring of event pairs handed out to dominant-kernel launches
std::mutex g_timing_mutex;
std::vector<hipEvent_t> g_timing_events;  // 2 * capacity
int g_timing_used = 0;
bool g_timing_on = false;

void timing_release() {
  for (hipEvent_t e : g_timing_events) (void)hipEventDestroy(e);
  g_timing_events.clear();
  g_timing_used = 0;
  g_timing_on = false;
}
}  // namespace

bool timing_next_events(hipEvent_t *start, hipEvent_t *stop) {
  if (!g_timing_on) return false;
  std::lock_guard<std::mutex> lock(g_timing_mutex);
  if (!g_timing_on || 2 * (size_t)g_timing_used + 1 >= g_timing_events.size()) return false;
  *start = g_timing_events[2 * (size_t)g_timing_used];
  *stop = g_timing_events[2 * (size_t)g_timing_used + 1];
  ++g_timing_used;
  return true;
}

int set_error(int status, const char *fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_error, sizeof(g_error), fmt, ap);
  va_end(ap);
  return status;
}

bool is_initialized() { return g_refcount > 0; }
int device_cu_count() { return g_cu_count; }
}  // namespace lapis

using namespace lapis;

extern "C" int lapis_hip_init(void) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g_refcount > 0) {
    ++g_refcount;
    return LAPIS_HIP_OK;
  }
  int dev = 0;
  LAPIS_HIP_TRY(hipGetDevice(&dev));
  hipDeviceProp_t prop;
  LAPIS_HIP_TRY(hipGetDeviceProperties(&prop, dev));
  if (strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return set_error(LAPIS_HIP_ERR_UNSUPPORTED_DEVICE,
                     "lapis_hip_init: device %d is %s; this library holds gfx950 code only", dev,
                     prop.gcnArchName);
  if (prop.warpSize != kWave)
    return set_error(LAPIS_HIP_ERR_UNSUPPORTED_DEVICE, "lapis_hip_init: wavefront size %d, expected 64",
                     prop.warpSize);
  g_cu_count = prop.multiProcessorCount;
  const int rc = dot_noalloc_setup();
  if (rc != LAPIS_HIP_OK) return rc;
  g_refcount = 1;
  return LAPIS_HIP_OK;
}

extern "C" int lapis_hip_finalize(void) {
  std::lock_guard<std::mutex> lock(g_mutex);
  if (g_refcount <= 0)
    return set_error(LAPIS_HIP_ERR_NOT_INITIALIZED, "lapis_hip_finalize: not initialized");
  if (--g_refcount == 0) dot_release_scratch();
  return LAPIS_HIP_OK;
}

static double g_timing_median = 0.0;  // of the launches the last kernel_timing_stop read

extern "C" int lapis_hip_kernel_timing_start(int capacity) {
  LAPIS_CHECK_INIT();
  LAPIS_REQUIRE(capacity > 0 && capacity <= (1 << 20), "kernel_timing_start: capacity %d outside [1, 2^20]", capacity);
  std::lock_guard<std::mutex> lock(g_timing_mutex);
  timing_release();
  g_timing_events.reserve(2 * (size_t)capacity);
  for (int i = 0; i < 2 * capacity; ++i) {
    hipEvent_t e;
    hipError_t err = hipEventCreate(&e);
    if (err != hipSuccess) {
      timing_release();
      return set_error(LAPIS_HIP_ERR_RUNTIME, "kernel_timing_start: hipEventCreate failed: %s", hipGetErrorString(err));
    }
    g_timing_events.push_back(e);
  }
  g_timing_on = true;
  return LAPIS_HIP_OK;
}

extern "C" int lapis_hip_kernel_timing_stop(int *count, double *mean_ms, double *min_ms, double *max_ms) {
  LAPIS_CHECK_INIT();
  std::lock_guard<std::mutex> lock(g_timing_mutex);
  if (!g_timing_on) return set_error(LAPIS_HIP_ERR_INVALID_ARGUMENT, "kernel_timing_stop: timing was not started");
  hipError_t err = hipDeviceSynchronize();
  double sum = 0.0, mn = 0.0, mx = 0.0;
  int n = 0;
  std::vector<float> all;
  for (int i = 0; err == hipSuccess && i < g_timing_used; ++i) {
    float ms = 0.f;
    err = hipEventElapsedTime(&ms, g_timing_events[2 * (size_t)i], g_timing_events[2 * (size_t)i + 1]);
    if (err != hipSuccess) break;
    all.push_back(ms);
    sum += ms;
    mn = (n == 0) ? ms : std::min<double>(mn, ms);
    mx = (n == 0) ? ms : std::max<double>(mx, ms);
    ++n;
  }
  timing_release();
  if (err != hipSuccess)
    return set_error(LAPIS_HIP_ERR_RUNTIME, "kernel_timing_stop: %s", hipGetErrorString(err));
  g_timing_median = 0.0;
  if (n) {
    std::sort(all.begin(), all.end());
    g_timing_median = (n & 1) ? all[n / 2] : 0.5 * ((double)all[n / 2 - 1] + all[n / 2]);
  }
  if (count) *count = n;
  if (mean_ms) *mean_ms = n ? sum / n : 0.0;
  if (min_ms) *min_ms = mn;
  if (max_ms) *max_ms = mx;
  return LAPIS_HIP_OK;
}

extern "C" double lapis_hip_kernel_timing_median_ms(void) {
  std::lock_guard<std::mutex> lock(g_timing_mutex);
  return g_timing_median;
}

extern "C" const char *lapis_hip_last_error(void) { return g_error; }

extern "C" const char *lapis_hip_status_name(int status) {
  switch (status) {
    case LAPIS_HIP_OK: return "LAPIS_HIP_OK";
    case LAPIS_HIP_ERR_INVALID_ARGUMENT: return "LAPIS_HIP_ERR_INVALID_ARGUMENT";
    case LAPIS_HIP_ERR_RUNTIME: return "LAPIS_HIP_ERR_RUNTIME";
    case LAPIS_HIP_ERR_NOT_INITIALIZED: return "LAPIS_HIP_ERR_NOT_INITIALIZED";
    case LAPIS_HIP_ERR_BAD_CSR: return "LAPIS_HIP_ERR_BAD_CSR";
    case LAPIS_HIP_ERR_UNSUPPORTED_DEVICE: return "LAPIS_HIP_ERR_UNSUPPORTED_DEVICE";
    case LAPIS_HIP_ERR_PLAN_MISMATCH: return "LAPIS_HIP_ERR_PLAN_MISMATCH";
    case LAPIS_HIP_ERR_NO_TILING: return "LAPIS_HIP_ERR_NO_TILING";
    default: return "LAPIS_HIP_ERR_UNKNOWN";
  }
}

extern "C" int lapis_hip_stream_synchronize(lapis_hip_stream_t stream) {
  LAPIS_CHECK_INIT();
  LAPIS_HIP_TRY(hipStreamSynchronize(as_stream(stream)));
  return LAPIS_HIP_OK;
}
