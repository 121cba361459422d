// S^2 x S^2 -> SO(3) spectral outer product for spectra of REAL signals held in the real basis, and its adjoints.
//
// The spectrum of a real signal on the sphere obeys x[l,-m] = (-1)^m conj(x[l,m]); in the basis of so3_real_basis.hip
// (row +m: sqrt2 Re x[l,m], row -m: sqrt2 Im x[l,m], row 0: x[l,0]) it is a real vector per degree, and the complex
// outer product z[l,m,n] = x[l,m] conj(y[l,n]) of two such spectra becomes the real outer product of the vectors,
// which IS the real-basis form of the SO(3) spectrum z:
//
//   fwd   : z [l,r,s,i,j] = sum_k x[l,r,i,k] * y[l,s,k,j]
//   gradx : gx[l,r,i,k]   = sum_{s,j} gz[l,r,s,i,j] * y[l,s,k,j]
//   grady : gy[l,s,k,j]   = sum_{r,i} gz[l,r,s,i,j] * x[l,r,i,k]
//
// x [nl^2, B, F_in], y [nl^2, F_in, F_out], z [nspec(nl), B, F_out]: half the bytes of the complex product, and all
// three kernels are bound by streaming z / gz once (4 nspec B F_out bytes).  Lanes run along j in groups of VEC
// consecutive output features (16-byte accesses when F_out is a multiple of 4), the small operands come from L1/L2,
// input features are taken KC at a time in registers.
#include "common.h"

namespace {

constexpr int KC = 8;       // input features per register pass
constexpr int NSPLIT = 8;   // forward: workgroups along n per (l, r)
constexpr int IPT = 2;      // forward: batch items per thread
constexpr int IB = 4;       // grad x: batch items per workgroup

template <int VEC> struct Pack;
template <> struct Pack<1> {
  typedef float type;
  static __device__ __forceinline__ float zero() { return 0.f; }
  static __device__ __forceinline__ void fma(float a, float b, float& c) { c = fmaf(a, b, c); }
  static __device__ __forceinline__ float dot(float a, float b) { return a * b; }
};
template <> struct Pack<2> {
  typedef float2 type;
  static __device__ __forceinline__ float2 zero() { return make_float2(0.f, 0.f); }
  static __device__ __forceinline__ void fma(float a, float2 b, float2& c) { c.x = fmaf(a, b.x, c.x); c.y = fmaf(a, b.y, c.y); }
  static __device__ __forceinline__ float dot(float2 a, float2 b) { return fmaf(a.x, b.x, a.y * b.y); }
};
template <> struct Pack<4> {
  typedef float4 type;
  static __device__ __forceinline__ float4 zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
  static __device__ __forceinline__ void fma(float a, float4 b, float4& c) {
    c.x = fmaf(a, b.x, c.x); c.y = fmaf(a, b.y, c.y); c.z = fmaf(a, b.z, c.z); c.w = fmaf(a, b.w, c.w);
  }
  static __device__ __forceinline__ float dot(float4 a, float4 b) { return fmaf(a.x, b.x, fmaf(a.y, b.y, fmaf(a.z, b.z, a.w * b.w))); }
};

__device__ inline int isqrt_floor(int v) {
  int l = (int)sqrtf((float)v);
  while (l * l > v) --l;
  while ((l + 1) * (l + 1) <= v) ++l;
  return l;
}

// ---- forward.  grid.x = nl^2 (l, r), grid.y = part of the s range, grid.z = tile of 256 (item group, j group) outputs.
// A thread owns IPT batch items (ngroup apart, so that the lanes of a store cover whole rows of z) and VEC output
// features: x[l,r,i,:] stays in registers while it walks s, so per s it reads KC pieces of the row y[l,s] once for all
// its items and writes IPT pieces of the row z[l,r,s].
template <int VEC>
__global__ __launch_bounds__(256) void s2_mm_real_fwd_kernel(const float* __restrict__ x, const float* __restrict__ y,
                                                             float* __restrict__ z, int nl, int nbatch, int fi, int fo) {
  typedef typename Pack<VEC>::type vec_t;
  const int lr = blockIdx.x;
  const int l = isqrt_floor(lr), r = lr - l * l - l;
  const int L = 2 * l + 1;
  const int s_lo = (int)((long)blockIdx.y * L / NSPLIT), s_hi = (int)((long)(blockIdx.y + 1) * L / NSPLIT);
  const int fov = fo / VEC, ngroup = (nbatch + IPT - 1) / IPT;
  const int o = blockIdx.z * 256 + threadIdx.x;
  if (o >= ngroup * fov || s_lo >= s_hi) return;
  const int ip = o / fov, jv = o - ip * fov;
  int item[IPT];
#pragma unroll
  for (int q = 0; q < IPT; ++q) item[q] = ip + q * ngroup < nbatch ? ip + q * ngroup : -1;    // item[0] always exists
  const size_t zrow = (size_t)l * (4 * l * l - 1) / 3 + (size_t)(l + r) * L;
  const bool stream = (size_t)nl * (4 * nl * nl - 1) / 3 * nbatch * fo * 4 >= s2cnn::STREAM_BYTES;     // z passes no cache: uniform
  for (int k0 = 0; k0 < fi; k0 += KC) {
    float xa[IPT][KC];
#pragma unroll
    for (int q = 0; q < IPT; ++q) {
      const float* xq = x + ((size_t)lr * nbatch + (item[q] < 0 ? ip : item[q])) * fi;
#pragma unroll
      for (int u = 0; u < KC; ++u) xa[q][u] = k0 + u < fi ? xq[k0 + u] : 0.f;
    }
    for (int s = s_lo; s < s_hi; ++s) {
      const vec_t* ys = reinterpret_cast<const vec_t*>(y + ((size_t)(l * l + s) * fi + k0) * fo) + jv;
      vec_t* zs = reinterpret_cast<vec_t*>(z + (zrow + s) * nbatch * fo) + jv;
      vec_t acc[IPT];
#pragma unroll
      for (int q = 0; q < IPT; ++q) acc[q] = (k0 > 0 && item[q] >= 0) ? zs[(size_t)item[q] * fov] : Pack<VEC>::zero();   // later feature passes accumulate
#pragma unroll
      for (int u = 0; u < KC; ++u) {
        if (k0 + u < fi) {
          const vec_t b = ys[(size_t)u * fov];
#pragma unroll
          for (int q = 0; q < IPT; ++q) Pack<VEC>::fma(xa[q][u], b, acc[q]);
        }
      }
#pragma unroll
      for (int q = 0; q < IPT; ++q)
        if (item[q] >= 0) s2cnn::store_policy(acc[q], zs + (size_t)item[q] * fov, stream);
    }
  }
}

// ---- grad x.  grid.x = nl^2 (l, r), grid.y = group of IB batch items, grid.z = feature pass.  The (s, j group) pairs of
// the row block gz[l,r,:,i,:] are spread over the threads; a thread accumulates IB x KC partial sums (one piece of y
// serves the IB items), then lanes and waves are reduced.
template <int VEC>
__global__ __launch_bounds__(256) void s2_mm_real_gradx_kernel(const float* __restrict__ gz, const float* __restrict__ y,
                                                               float* __restrict__ gx, int nl, int nbatch, int fi, int fo) {
  typedef typename Pack<VEC>::type vec_t;
  __shared__ float part[4][IB][KC];
  const int lr = blockIdx.x, i0 = blockIdx.y * IB, k0 = blockIdx.z * KC;
  const int l = isqrt_floor(lr), r = lr - l * l - l;
  const int L = 2 * l + 1;
  const size_t zrow = (size_t)l * (4 * l * l - 1) / 3 + (size_t)(l + r) * L;
  const int fov = fo / VEC;
  float acc[IB][KC];
#pragma unroll
  for (int q = 0; q < IB; ++q)
#pragma unroll
    for (int u = 0; u < KC; ++u) acc[q][u] = 0.f;
  int s = threadIdx.x / fov, jv = threadIdx.x - s * fov;           // walks (s, jv) with stride 256
  const int ds = 256 / fov, dj = 256 - ds * fov;
  for (; s < L; ) {
    const vec_t* g = reinterpret_cast<const vec_t*>(gz + ((zrow + s) * nbatch + i0) * fo) + jv;
    vec_t a[IB];
#pragma unroll
    for (int q = 0; q < IB; ++q) a[q] = i0 + q < nbatch ? g[(size_t)q * fov] : Pack<VEC>::zero();
    const vec_t* yy = reinterpret_cast<const vec_t*>(y + ((size_t)(l * l + s) * fi + k0) * fo) + jv;
#pragma unroll
    for (int u = 0; u < KC; ++u) {
      if (k0 + u < fi) {
        const vec_t b = yy[(size_t)u * fov];
#pragma unroll
        for (int q = 0; q < IB; ++q) acc[q][u] += Pack<VEC>::dot(a[q], b);
      }
    }
    s += ds; jv += dj;
    if (jv >= fov) { jv -= fov; ++s; }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int q = 0; q < IB; ++q)
#pragma unroll
    for (int u = 0; u < KC; ++u) {
      float v = acc[q][u];
#pragma unroll
      for (int sh = 32; sh > 0; sh >>= 1) v += __shfl_down(v, sh, 64);
      if (lane == 0) part[wave][q][u] = v;
    }
  __syncthreads();
  if (threadIdx.x < IB * KC) {
    const int q = threadIdx.x / KC, u = threadIdx.x - q * KC;
    if (i0 + q < nbatch && k0 + u < fi)
      gx[((size_t)lr * nbatch + i0 + q) * fi + k0 + u] = (part[0][q][u] + part[1][q][u]) + (part[2][q][u] + part[3][q][u]);
  }
}

// ---- grad y.  grid.x = nl^2 (l, s), grid.y = tile of JT j groups, grid.z = feature pass.  The threads form
// SL = 256 / JT slices of JT lanes; slice q takes the (r, i) pairs q, q + SL, ...; a lane accumulates KC pieces (x is
// uniform over a slice), then the slices are reduced through LDS.
template <int VEC, int JT>
__global__ __launch_bounds__(256) void s2_mm_real_grady_kernel(const float* __restrict__ gz, const float* __restrict__ x,
                                                               float* __restrict__ gy, int nl, int nbatch, int fi, int fo) {
  typedef typename Pack<VEC>::type vec_t;
  constexpr int SL = 256 / JT;
  __shared__ float part[SL][KC][JT * VEC];
  const int ls = blockIdx.x, k0 = blockIdx.z * KC;
  const int l = isqrt_floor(ls), sn = ls - l * l - l;
  const int L = 2 * l + 1;
  const size_t zcol = (size_t)l * (4 * l * l - 1) / 3 + (size_t)(l + sn);
  const int fov = fo / VEC;
  const int slice = threadIdx.x / JT, jl = threadIdx.x - slice * JT;
  const int jv = blockIdx.y * JT + jl;
  vec_t acc[KC];
#pragma unroll
  for (int u = 0; u < KC; ++u) acc[u] = Pack<VEC>::zero();
  const int total = L * nbatch;                                    // (r, i) pairs
  int rr = slice / nbatch, i = slice - rr * nbatch;                // walks the pairs with stride SL
  const int dr = SL / nbatch, di = SL - dr * nbatch;
  for (int p = slice; p < total; p += SL) {
    const vec_t a = jv < fov ? reinterpret_cast<const vec_t*>(gz + ((zcol + (size_t)rr * L) * nbatch + i) * fo)[jv] : Pack<VEC>::zero();
    const float* xx = x + ((size_t)(l * l + rr) * nbatch + i) * fi + k0;
#pragma unroll
    for (int u = 0; u < KC; ++u)
      if (k0 + u < fi) Pack<VEC>::fma(xx[u], a, acc[u]);
    rr += dr; i += di;
    if (i >= nbatch) { i -= nbatch; ++rr; }
  }
#pragma unroll
  for (int u = 0; u < KC; ++u) reinterpret_cast<vec_t*>(&part[slice][u][0])[jl] = acc[u];
  __syncthreads();
  for (int o = threadIdx.x; o < KC * JT * VEC; o += 256) {
    const int u = o / (JT * VEC), jj = o - u * (JT * VEC);
    const int j = blockIdx.y * JT * VEC + jj;
    if (k0 + u < fi && j < fo) {
      float v = 0.f;
#pragma unroll
      for (int q = 0; q < SL; ++q) v += part[q][u][jj];
      gy[((size_t)ls * fi + k0 + u) * fo + j] = v;
    }
  }
}

int check(const void* a, const void* b, const void* c, int nl, int nbatch, int fi, int fo) {
  if (!a || !b || !c || nl < 1 || nl > 255 || nbatch < 1 || nbatch > 65535 * IB || fi < 1 || fo < 1) return S2CNN_EINVAL;
  if ((long)nbatch * fo >= (1L << 31) || (long)nbatch * fi >= (1L << 31) || (long)fi * fo >= (1L << 31)) return S2CNN_EINVAL;
  if ((fi + KC - 1) / KC > 65535 || fo / 16 + 1 > 65535 || ((long)nbatch * fo + 255) / 256 > 65535) return S2CNN_EINVAL;
  if ((reinterpret_cast<uintptr_t>(a) | reinterpret_cast<uintptr_t>(b) | reinterpret_cast<uintptr_t>(c)) & 3u) return S2CNN_EALIGN;
  return S2CNN_OK;
}

// 16-byte (8-byte) accesses need rows of z, y that start on 16-byte (8-byte) boundaries
bool vec4(const void* a, const void* b, const void* c, int fo) {
  return fo % 4 == 0 && s2cnn::aligned16(a) && s2cnn::aligned16(b) && s2cnn::aligned16(c);
}
bool vec2(const void* a, const void* b, const void* c, int fo) {
  return fo % 2 == 0 && s2cnn::aligned8(a) && s2cnn::aligned8(b) && s2cnn::aligned8(c);
}

}  // namespace

extern "C" int s2cnn_s2_mm_real_fwd(const float* x, const float* y, float* z, int nl, int nbatch, int f_in, int f_out, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(x, y, z, nl, nbatch, f_in, f_out)) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int npair = (nbatch + IPT - 1) / IPT;      // item groups of the forward kernel
  if (vec4(y, z, z, f_out)) {
    const dim3 grid(nl * nl, NSPLIT, (unsigned)(((long)npair * (f_out / 4) + 255) / 256));
    hipLaunchKernelGGL(s2_mm_real_fwd_kernel<4>, grid, dim3(256), 0, st, x, y, z, nl, nbatch, f_in, f_out);
  } else if (vec2(y, z, z, f_out)) {
    const dim3 grid(nl * nl, NSPLIT, (unsigned)(((long)npair * (f_out / 2) + 255) / 256));
    hipLaunchKernelGGL(s2_mm_real_fwd_kernel<2>, grid, dim3(256), 0, st, x, y, z, nl, nbatch, f_in, f_out);
  } else {
    const dim3 grid(nl * nl, NSPLIT, (unsigned)(((long)npair * f_out + 255) / 256));
    hipLaunchKernelGGL(s2_mm_real_fwd_kernel<1>, grid, dim3(256), 0, st, x, y, z, nl, nbatch, f_in, f_out);
  }
  return s2cnn::launch_status();
}

extern "C" int s2cnn_s2_mm_real_gradx(const float* gz, const float* y, float* gx, int nl, int nbatch, int f_in, int f_out, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(gz, y, gx, nl, nbatch, f_in, f_out)) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const dim3 grid(nl * nl, (nbatch + IB - 1) / IB, (f_in + KC - 1) / KC);
  if (vec4(gz, y, y, f_out))
    hipLaunchKernelGGL(s2_mm_real_gradx_kernel<4>, grid, dim3(256), 0, st, gz, y, gx, nl, nbatch, f_in, f_out);
  else if (vec2(gz, y, y, f_out))
    hipLaunchKernelGGL(s2_mm_real_gradx_kernel<2>, grid, dim3(256), 0, st, gz, y, gx, nl, nbatch, f_in, f_out);
  else
    hipLaunchKernelGGL(s2_mm_real_gradx_kernel<1>, grid, dim3(256), 0, st, gz, y, gx, nl, nbatch, f_in, f_out);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_s2_mm_real_grady(const float* gz, const float* x, float* gy, int nl, int nbatch, int f_in, int f_out, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(gz, x, gy, nl, nbatch, f_in, f_out)) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (vec4(gz, gz, gy, f_out)) {
    const dim3 grid(nl * nl, (f_out / 4 + 15) / 16, (f_in + KC - 1) / KC);
    hipLaunchKernelGGL((s2_mm_real_grady_kernel<4, 16>), grid, dim3(256), 0, st, gz, x, gy, nl, nbatch, f_in, f_out);
  } else if (vec2(gz, gz, gy, f_out)) {
    const dim3 grid(nl * nl, (f_out / 2 + 31) / 32, (f_in + KC - 1) / KC);
    hipLaunchKernelGGL((s2_mm_real_grady_kernel<2, 32>), grid, dim3(256), 0, st, gz, x, gy, nl, nbatch, f_in, f_out);
  } else {
    const dim3 grid(nl * nl, (f_out + 63) / 64, (f_in + KC - 1) / KC);
    hipLaunchKernelGGL((s2_mm_real_grady_kernel<1, 64>), grid, dim3(256), 0, st, gz, x, gy, nl, nbatch, f_in, f_out);
  }
  return s2cnn::launch_status();
}
