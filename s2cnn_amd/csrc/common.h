// Shared host-side helpers for the C-ABI entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "s2cnn_hip.h"

namespace s2cnn {

// Status of the launches an entry point has just made.  hipGetLastError returns (and clears) the last error of
// this host thread, whoever caused it: entry points call clear_stale_error() before their first launch so that an
// error left behind by other code on the thread is not reported as theirs.
inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? S2CNN_OK : static_cast<int>(e);
}
inline void clear_stale_error() { (void)hipGetLastError(); }

inline bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline long so3_nspec(long b) { return b * (4 * b * b - 1) / 3; }

__host__ __device__ inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

// max(v, 0) that keeps a NaN, and the factor by which the gradient of that function passes where its OUTPUT is m
__device__ __forceinline__ float relu_f(float v) { return v < 0.f ? 0.f : v; }
__device__ __forceinline__ float relu_pass(float g, float m) { return m <= 0.f ? 0.f : g; }

}  // namespace s2cnn
