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

// What an analysis does to its input as it loads it (the signal v that is transformed):
//   NONE            v = x
//   MASK            v = x where w > 0, else 0                       (w: a tensor of the shape of x)
//   BITS            the same with one bit per sample in w           (per-volume kernels of the 64^3 grid only)
//   AFFINE_RELU     v = max(a x + b, 0)                             (a, b: per feature, params [2][nfeature])
//   BN_RELU_GRAD    v = a (a w + b > 0 ? x : 0) + p + q w           (x: incoming gradient, w: the tensor the forward
//                   pass normalised; a, b, p, q per feature, params [4][nfeature]: the gradient of a batch normalisation
//                   followed by max(., 0) with respect to its input)
// The feature of volume z is z % nfeature.
enum Prologue { PRO_NONE = 0, PRO_MASK = 1, PRO_BITS = 2, PRO_AFFINE_RELU = 3, PRO_BN_RELU_GRAD = 4 };
struct Input {
  const float* x;
  const float* w = nullptr;
  int kind = PRO_NONE;
  const float* params = nullptr;
  int nfeature = 1;
  bool second_tensor() const { return kind == PRO_MASK || kind == PRO_BN_RELU_GRAD; }
};
__device__ __forceinline__ float affine_relu(float x, float a, float b) { return relu_f(fmaf(a, x, b)); }
__device__ __forceinline__ float bn_relu_grad(float g, float w, float a, float b, float p, float q) {
  return fmaf(q, w, p) + relu_pass(a * g, fmaf(a, w, b));
}

// Accesses with the non-temporal hint, for data that is streamed: written once and not found in a cache by its reader
// anyway (hundreds of megabytes), or read once.  On this chip such stores run at up to 1.5 times the rate of plain ones.
typedef float ext2_t __attribute__((ext_vector_type(2)));
typedef float ext4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ void stream_store(float v, float* p) { __builtin_nontemporal_store(v, p); }
__device__ __forceinline__ void stream_store(float2 v, float2* p) { __builtin_nontemporal_store(ext2_t{v.x, v.y}, reinterpret_cast<ext2_t*>(p)); }
__device__ __forceinline__ void stream_store(float4 v, float4* p) { __builtin_nontemporal_store(ext4_t{v.x, v.y, v.z, v.w}, reinterpret_cast<ext4_t*>(p)); }
__device__ __forceinline__ float stream_load(const float* p) { return __builtin_nontemporal_load(p); }
__device__ __forceinline__ float2 stream_load(const float2* p) {
  const ext2_t v = __builtin_nontemporal_load(reinterpret_cast<const ext2_t*>(p));
  return make_float2(v.x, v.y);
}
__device__ __forceinline__ float4 stream_load(const float4* p) {
  const ext4_t v = __builtin_nontemporal_load(reinterpret_cast<const ext4_t*>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}

// The hint chosen at run time by a uniform flag.  Tensors of at least STREAM_BYTES are streamed: they pass no cache on
// their way to their reader (256 MB of memory-side cache); smaller ones are left to the caches.
constexpr size_t STREAM_BYTES = (size_t)256 << 20;
template <class V> __device__ __forceinline__ void store_policy(V v, V* p, bool stream) {
  if (stream) stream_store(v, p);
  else *p = v;
}
template <class V> __device__ __forceinline__ V load_policy(const V* p, bool stream) { return stream ? stream_load(p) : *p; }

}  // namespace s2cnn
