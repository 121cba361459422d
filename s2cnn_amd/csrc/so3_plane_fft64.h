// 64x64 (alpha, gamma) plane transforms for bandwidth 32, held entirely in LDS.
//
// Two real planes a, b of the same workgroup are transformed as ONE complex plane a + i b
// (forward), or two Hermitian half spectra are combined into one complex spectrum whose inverse
// is a + i b (inverse); the planes are separated / combined with the Hermitian symmetry of real
// signals.  Each 64-point line transform is 8 x 8: a thread does an 8-point butterfly in registers,
// lines are exchanged through LDS.  With j = 8 j1 + j2 in, k = k1 + 8 k2 out:
//   X[k1 + 8 k2] = sum_{j2} w8^{j2 k2} ( w64^{j2 k1} sum_{j1} x[8 j1 + j2] w8^{j1 k1} )
// pass A (thread = (line, j2)) does the inner sum and the twiddle in place (slots 8 j1 + j2 ->
// 8 k1 + j2), pass B (thread = (line, k1)) the outer sum in place (slots 8 k1 + j2 -> 8 k1 + k2).
// Output bin k therefore sits at slot sigma(k) = 8 (k % 8) + k / 8; consumers index through sigma.
#pragma once
#include <hip/hip_runtime.h>
#include "common.h"

namespace fft64 {

constexpr int N = 64;
constexpr int PITCH = 65;                 // row pitch in complex elements (odd: conflict-free columns and rows)
constexpr int LDS_ELEMS = N * PITCH;      // float2 elements per complex plane
constexpr int THREADS = 256;

__device__ __forceinline__ int sigma(int k) { return 8 * (k & 7) + (k >> 3); }

__device__ __forceinline__ float2 cadd(float2 a, float2 b) { return make_float2(a.x + b.x, a.y + b.y); }
__device__ __forceinline__ float2 csub(float2 a, float2 b) { return make_float2(a.x - b.x, a.y - b.y); }
__device__ __forceinline__ float2 cmul(float2 a, float2 b) { return make_float2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x); }
// multiply by -i (forward) or +i (inverse)
template <bool INV> __device__ __forceinline__ float2 rot90(float2 a) { return INV ? make_float2(-a.y, a.x) : make_float2(a.y, -a.x); }

// 4-point DFT, natural order in and out; sign of the exponent: - (forward) / + (INV)
template <bool INV>
__device__ __forceinline__ void fft4(float2& y0, float2& y1, float2& y2, float2& y3) {
  const float2 b0 = cadd(y0, y2), b1 = csub(y0, y2), b2 = cadd(y1, y3), b3 = rot90<INV>(csub(y1, y3));
  y0 = cadd(b0, b2); y2 = csub(b0, b2); y1 = cadd(b1, b3); y3 = csub(b1, b3);
}

// 8-point DFT in registers, natural order in and out
template <bool INV>
__device__ __forceinline__ void fft8(float2 (&v)[8]) {
  constexpr float R = 0.70710678118654752440f;
  float2 e0 = cadd(v[0], v[4]), e1 = cadd(v[1], v[5]), e2 = cadd(v[2], v[6]), e3 = cadd(v[3], v[7]);
  float2 o0 = csub(v[0], v[4]), o1 = csub(v[1], v[5]), o2 = csub(v[2], v[6]), o3 = csub(v[3], v[7]);
  // o_n *= w8^n:  w8 = e^{-i pi/4} (forward), e^{+i pi/4} (inverse)
  o1 = INV ? make_float2(R * (o1.x - o1.y), R * (o1.x + o1.y)) : make_float2(R * (o1.x + o1.y), R * (o1.y - o1.x));
  o2 = rot90<INV>(o2);
  o3 = INV ? make_float2(-R * (o3.x + o3.y), R * (o3.x - o3.y)) : make_float2(R * (o3.y - o3.x), -R * (o3.x + o3.y));
  fft4<INV>(e0, e1, e2, e3);
  fft4<INV>(o0, o1, o2, o3);
  v[0] = e0; v[2] = e1; v[4] = e2; v[6] = e3;
  v[1] = o0; v[3] = o1; v[5] = o2; v[7] = o3;
}

// In-place 2-D transform of a 64x64 complex plane in LDS (row pitch PITCH), natural order in,
// sigma order out on both axes.  tw[k] = w64^(j2 k) for this thread's j2 = threadIdx.x / 32.
// All 256 threads must call; ends with a barrier.
template <bool INV>
__device__ __forceinline__ void transform_2d(float2* buf, const float2 (&tw)[8]) {
  const int lo = threadIdx.x & 31;   // line within a half
  const int d = threadIdx.x >> 5;    // j2 in pass A, k1 in pass B
  float2 v[8];
  // ---- rows (contiguous lines): line = alpha
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    float2* line = buf + (lo + 32 * half) * PITCH;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = line[8 * j + d];
    fft8<INV>(v);
#pragma unroll
    for (int j = 1; j < 8; ++j) v[j] = cmul(v[j], tw[j]);
#pragma unroll
    for (int j = 0; j < 8; ++j) line[8 * j + d] = v[j];
  }
  __syncthreads();
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    float2* line = buf + (lo + 32 * half) * PITCH + 8 * d;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = line[j];
    fft8<INV>(v);
#pragma unroll
    for (int j = 0; j < 8; ++j) line[j] = v[j];
  }
  __syncthreads();
  // ---- columns (stride PITCH): line = gamma slot
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    float2* line = buf + (lo + 32 * half);
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = line[(8 * j + d) * PITCH];
    fft8<INV>(v);
#pragma unroll
    for (int j = 1; j < 8; ++j) v[j] = cmul(v[j], tw[j]);
#pragma unroll
    for (int j = 0; j < 8; ++j) line[(8 * j + d) * PITCH] = v[j];
  }
  __syncthreads();
#pragma unroll
  for (int half = 0; half < 2; ++half) {
    float2* line = buf + (lo + 32 * half) + 8 * d * PITCH;
#pragma unroll
    for (int j = 0; j < 8; ++j) v[j] = line[j * PITCH];
    fft8<INV>(v);
#pragma unroll
    for (int j = 0; j < 8; ++j) line[j * PITCH] = v[j];
  }
  __syncthreads();
}

template <bool INV>
__device__ __forceinline__ void make_twiddles(float2 (&tw)[8]) {
  const int d = threadIdx.x >> 5;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    float s, c;
    sincospif((float)(d * k) / 32.0f, &s, &c);   // angle 2 pi d k / 64
    tw[k] = make_float2(c, INV ? s : -s);
  }
}

// Forward: planes 2q, 2q+1 of x ([planes][64][64] real) -> X ([planes][mw][nb] complex), the bins
// m = -(nb-1)..nb-1, n = 0..nb-1 of each plane's 2-D DFT.  Grid-stride over plane pairs.
// ztile = 0: X is [plane][mi][n];  ztile = Z > 0: X is [z / Z][mi][beta][z % Z][n] (plane = z * 64 + beta),
// the order in which the tiled Wigner contraction streams it.
// mask: NULL, or a tensor of the shape of x; samples of x where it is not positive count as zero.
__global__ __launch_bounds__(THREADS) void plane_fft64_fwd(const float* __restrict__ x, float2* __restrict__ X,
                                                           long npairs, int nb, int ztile, const float* __restrict__ mask) {
  __shared__ float2 buf[LDS_ELEMS];
  float2 tw[8];
  make_twiddles<false>(tw);
  const int MW = 2 * nb - 1;
  for (long pair = blockIdx.x; pair < npairs; pair += gridDim.x) {
    const float4* pa = reinterpret_cast<const float4*>(x + pair * 2 * (N * N));
    const float4* pb = pa + N * N / 4;
    float4 a[4], b[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {                    // float4 index q: row q/16, cols 4*(q%16)..
      a[i] = pa[threadIdx.x + THREADS * i];
      b[i] = pb[threadIdx.x + THREADS * i];
    }
    if (mask) {
      const float4* ma = reinterpret_cast<const float4*>(mask + pair * 2 * (N * N));
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float4 u = ma[threadIdx.x + THREADS * i], v = ma[threadIdx.x + THREADS * i + N * N / 4];
        a[i] = make_float4(s2cnn::relu_pass(a[i].x, u.x), s2cnn::relu_pass(a[i].y, u.y), s2cnn::relu_pass(a[i].z, u.z), s2cnn::relu_pass(a[i].w, u.w));
        b[i] = make_float4(s2cnn::relu_pass(b[i].x, v.x), s2cnn::relu_pass(b[i].y, v.y), s2cnn::relu_pass(b[i].z, v.z), s2cnn::relu_pass(b[i].w, v.w));
      }
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = threadIdx.x + THREADS * i;
      float2* dst = buf + (q >> 4) * PITCH + 4 * (q & 15);
      dst[0] = make_float2(a[i].x, b[i].x); dst[1] = make_float2(a[i].y, b[i].y);
      dst[2] = make_float2(a[i].z, b[i].z); dst[3] = make_float2(a[i].w, b[i].w);
    }
    __syncthreads();
    transform_2d<false>(buf, tw);
    // Z = A + iB with A, B Hermitian:  A[m,n] = (Z[m,n] + conj Z[-m,-n]) / 2,  B[m,n] = (Z[m,n] - conj Z[-m,-n]) / (2i)
    // element (mi, n) of plane a at Xa[mi * mstride + n]; plane b (the next beta) at + bstride
    float2* Xa;
    size_t mstride, bstride;
    if (ztile > 0) {
      const long z = pair >> 5;
      const int beta = (int)(pair & 31) * 2;
      Xa = X + ((size_t)(z / ztile) * MW * N + beta) * ztile * nb + (size_t)(z % ztile) * nb;
      mstride = (size_t)N * ztile * nb;
      bstride = (size_t)ztile * nb;
    } else {
      Xa = X + pair * 2 * (size_t)(MW * nb);
      mstride = nb;
      bstride = (size_t)MW * nb;
    }
    for (int o = threadIdx.x; o < MW * nb; o += THREADS) {
      const int mi = o / nb, n = o - mi * nb;
      const int m = mi - (nb - 1);
      const float2 z1 = buf[sigma(m & 63) * PITCH + sigma(n)];
      const float2 z2 = buf[sigma((-m) & 63) * PITCH + sigma((-n) & 63)];
      float2* d = Xa + mi * mstride + n;
      d[0] = make_float2(0.5f * (z1.x + z2.x), 0.5f * (z1.y - z2.y));
      d[bstride] = make_float2(0.5f * (z1.y + z2.y), 0.5f * (z2.x - z1.x));
    }
    __syncthreads();
  }
}

// Inverse: half spectra S ([planes][mw][nb] complex, Hermitian completion implied) of planes 2q, 2q+1
// -> y ([planes][64][64] real), unnormalised:  y[alpha,gamma] = sum_{m,n} e^{+i(m alpha + n gamma)} G[m,n].
__global__ __launch_bounds__(THREADS) void plane_fft64_inv(const float2* __restrict__ S, float* __restrict__ y,
                                                           long npairs, int nb) {
  __shared__ float2 buf[LDS_ELEMS];
  float2 tw[8];
  make_twiddles<true>(tw);
  const int MW = 2 * nb - 1;
  for (long pair = blockIdx.x; pair < npairs; pair += gridDim.x) {
    for (int i = threadIdx.x; i < LDS_ELEMS; i += THREADS) buf[i] = make_float2(0.f, 0.f);
    __syncthreads();
    const float2* Sa = S + pair * 2 * (size_t)(MW * nb);
    const float2* Sb = Sa + (size_t)MW * nb;
    for (int o = threadIdx.x; o < MW * nb; o += THREADS) {
      const int mi = o / nb, n = o - mi * nb;
      const int m = mi - (nb - 1);
      const float2 a = Sa[o], b = Sb[o];
      buf[(m & 63) * PITCH + n] = make_float2(a.x - b.y, a.y + b.x);                       // A + iB
      if (n > 0) buf[((-m) & 63) * PITCH + (64 - n)] = make_float2(a.x + b.y, b.x - a.y);  // conj A + i conj B
    }
    __syncthreads();
    transform_2d<true>(buf, tw);
    float4* pa = reinterpret_cast<float4*>(y + pair * 2 * (N * N));
    float4* pb = pa + N * N / 4;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int q = threadIdx.x + THREADS * i;
      const float2* row = buf + sigma(q >> 4) * PITCH;
      const int c = 4 * (q & 15);
      const float2 v0 = row[sigma(c)], v1 = row[sigma(c + 1)], v2 = row[sigma(c + 2)], v3 = row[sigma(c + 3)];
      pa[q] = make_float4(v0.x, v1.x, v2.x, v3.x);
      pb[q] = make_float4(v0.y, v1.y, v2.y, v3.y);
    }
    __syncthreads();
  }
}

}  // namespace fft64
