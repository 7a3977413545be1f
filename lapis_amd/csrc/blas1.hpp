// Internal interface of the dot kernel, shared with the CG driver.
#pragma once
#include <hip/hip_runtime.h>

#include <cstdint>

namespace lapis {

constexpr int kDotMaxBlocks = 2048;  // upper bound of dot_grid(); sizes the partials scratch

// Number of blocks (= partial sums) a dot over n elements uses.
int dot_grid(int64_t n);

// *result = init + sum x[i]*y[i].  `partials` holds kDotMaxBlocks elements of T.
template <typename T>
int launch_dot(int64_t n, const T *x, const T *y, T init, T *result, T *partials, hipStream_t st);

// Per-device set-up of lapis_hip_dot_f64_noalloc (address of its fixed scratch array) and
// release of the allocated ring of partials the other dot entry points use.
int dot_noalloc_setup();
void dot_release_scratch();

}  // namespace lapis
