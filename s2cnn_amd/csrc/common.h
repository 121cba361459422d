// Shared host-side helpers for the C-ABI entry points.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include "s2cnn_hip.h"

namespace s2cnn {

inline int launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? S2CNN_OK : static_cast<int>(e);
}

inline bool aligned8(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; }
inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

inline long so3_nspec(long b) { return b * (4 * b * b - 1) / 3; }

__host__ __device__ inline int ceil_div(int a, int b) { return (a + b - 1) / b; }

}  // namespace s2cnn
