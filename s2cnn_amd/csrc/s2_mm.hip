// S^2 x S^2 -> SO(3) spectral outer product and its two adjoints.
//
//   fwd   : z [l,m,n,i,j] = sum_k x[l,m,i,k] * conj(y[l,n,k,j])
//   gradx : gx[l,m,i,k]   = sum_{n,j} gz[l,m,n,i,j] * y[l,n,k,j]
//   grady : gy[l,n,k,j]   = sum_{m,i} conj(gz[l,m,n,i,j]) * x[l,m,i,k]
//
// The contraction of the forward product runs over the input features only (a handful in a first
// layer), so all three are bound by streaming the big tensor z / gz once: 8 nspec B F_out bytes.
// Lanes always run along j, the fastest index of z, so every access to z is a full coalesced row;
// the small operands are re-read through L1/L2.  Input features are handled KC at a time in registers.
#include "common.h"

namespace {

constexpr int KC = 8;   // input features per register pass

__device__ inline int isqrt_floor(int v) {
  int l = (int)sqrtf((float)v);
  while (l * l > v) --l;
  while ((l + 1) * (l + 1) <= v) ++l;
  return l;
}

// CV complex numbers per lane along j: 2 (16-byte accesses) when F_out is even and the rows start on 16-byte boundaries
template <int CV> struct CPack;
template <> struct CPack<1> {
  typedef float2 type;
  static __device__ __forceinline__ float2 zero() { return make_float2(0.f, 0.f); }
  // acc += sum over the lane's entries of a * b (complex)
  static __device__ __forceinline__ void dot(float2 a, float2 b, float2& acc) {
    acc.x = fmaf(a.x, b.x, fmaf(-a.y, b.y, acc.x));
    acc.y = fmaf(a.x, b.y, fmaf(a.y, b.x, acc.y));
  }
  // acc[entry] += s * conj(b[entry]) for a complex scalar s
  static __device__ __forceinline__ void scal_conj(float2 s, float2 b, float2& acc) {
    acc.x = fmaf(s.x, b.x, fmaf(s.y, b.y, acc.x));
    acc.y = fmaf(s.y, b.x, fmaf(-s.x, b.y, acc.y));
  }
  // acc[entry] += conj(a[entry]) * s for a complex scalar s
  static __device__ __forceinline__ void conj_axpy(float2 a, float2 s, float2& acc) {
    acc.x = fmaf(a.x, s.x, fmaf(a.y, s.y, acc.x));
    acc.y = fmaf(a.x, s.y, fmaf(-a.y, s.x, acc.y));
  }
};
template <> struct CPack<2> {
  typedef float4 type;
  static __device__ __forceinline__ float4 zero() { return make_float4(0.f, 0.f, 0.f, 0.f); }
  static __device__ __forceinline__ void dot(float4 a, float4 b, float2& acc) {
    acc.x = fmaf(a.x, b.x, fmaf(-a.y, b.y, fmaf(a.z, b.z, fmaf(-a.w, b.w, acc.x))));
    acc.y = fmaf(a.x, b.y, fmaf(a.y, b.x, fmaf(a.z, b.w, fmaf(a.w, b.z, acc.y))));
  }
  static __device__ __forceinline__ void scal_conj(float2 s, float4 b, float4& acc) {
    acc.x = fmaf(s.x, b.x, fmaf(s.y, b.y, acc.x));
    acc.y = fmaf(s.y, b.x, fmaf(-s.x, b.y, acc.y));
    acc.z = fmaf(s.x, b.z, fmaf(s.y, b.w, acc.z));
    acc.w = fmaf(s.y, b.z, fmaf(-s.x, b.w, acc.w));
  }
  static __device__ __forceinline__ void conj_axpy(float4 a, float2 s, float4& acc) {
    acc.x = fmaf(a.x, s.x, fmaf(a.y, s.y, acc.x));
    acc.y = fmaf(a.x, s.y, fmaf(-a.y, s.x, acc.y));
    acc.z = fmaf(a.z, s.x, fmaf(a.w, s.y, acc.z));
    acc.w = fmaf(a.z, s.y, fmaf(-a.w, s.x, acc.w));
  }
};

// ---- forward: grid.x = nl^2 (l,m), grid.y = part of the n range, grid.z = tile of 256 (item group, j group) outputs.
// A thread owns IPT batch items (ngroup apart, so that the lanes of a store cover whole rows of z) and CV output
// features: x[l,m,i,:] stays in registers while it walks n, so per n it reads KC pieces of the row y[l,n] once for all
// its items and writes IPT pieces of the row z[l,m,n]; consecutive n are consecutive blocks of z.
constexpr int NSPLIT = 8;
constexpr int IPT = 2;

template <int CV>
__global__ __launch_bounds__(256) void s2_mm_fwd_kernel(const float2* __restrict__ x, const float2* __restrict__ y,
                                                        float2* __restrict__ z, int nl, int nbatch, int fi, int fo) {
  typedef typename CPack<CV>::type vec_t;
  const int lm = blockIdx.x;
  const int l = isqrt_floor(lm), m = lm - l * l - l;
  const int L = 2 * l + 1;
  const int n_lo = (int)((long)blockIdx.y * L / NSPLIT), n_hi = (int)((long)(blockIdx.y + 1) * L / NSPLIT);
  const int fov = fo / CV, ngroup = (nbatch + IPT - 1) / IPT;
  const int o = blockIdx.z * 256 + threadIdx.x;
  if (o >= ngroup * fov || n_lo >= n_hi) return;
  const int ip = o / fov, jv = o - ip * fov;
  int item[IPT];
#pragma unroll
  for (int q = 0; q < IPT; ++q) item[q] = ip + q * ngroup < nbatch ? ip + q * ngroup : -1;    // item[0] always exists
  const size_t zbase = (size_t)l * (4 * l * l - 1) / 3 + (size_t)(l + m) * L;
  const bool stream = (size_t)nl * (4 * nl * nl - 1) / 3 * nbatch * fo * 8 >= s2cnn::STREAM_BYTES;     // z passes no cache: uniform
  for (int k0 = 0; k0 < fi; k0 += KC) {
    float2 xr[IPT][KC];
#pragma unroll
    for (int q = 0; q < IPT; ++q) {
      const float2* xs = x + ((size_t)lm * nbatch + (item[q] < 0 ? ip : item[q])) * fi;
#pragma unroll
      for (int u = 0; u < KC; ++u) xr[q][u] = k0 + u < fi ? xs[k0 + u] : make_float2(0.f, 0.f);
    }
    for (int nn = n_lo; nn < n_hi; ++nn) {
      const vec_t* ys = reinterpret_cast<const vec_t*>(y + ((size_t)(l * l + nn) * fi + k0) * fo) + jv;
      vec_t* zs = reinterpret_cast<vec_t*>(z + (zbase + nn) * nbatch * fo) + jv;
      vec_t acc[IPT];
#pragma unroll
      for (int q = 0; q < IPT; ++q) acc[q] = (k0 > 0 && item[q] >= 0) ? zs[(size_t)item[q] * fov] : CPack<CV>::zero();   // later feature passes accumulate
#pragma unroll
      for (int u = 0; u < KC; ++u) {
        if (k0 + u < fi) {
          const vec_t b = ys[(size_t)u * fov];
#pragma unroll
          for (int q = 0; q < IPT; ++q) CPack<CV>::scal_conj(xr[q][u], b, acc[q]);
        }
      }
#pragma unroll
      for (int q = 0; q < IPT; ++q)
        if (item[q] >= 0) s2cnn::store_policy(acc[q], zs + (size_t)item[q] * fov, stream);
    }
  }
}

constexpr int IB = 4;   // grad x: batch items per workgroup

// ---- grad x.  grid.x = nl^2 (l, m), grid.y = group of IB batch items, grid.z = feature pass.  The (n, j group) pairs of
// the row block gz[l,m,:,i,:] are spread over the threads (consecutive threads read consecutive 8 CV bytes of a row); a
// thread accumulates IB x KC partial sums (one piece of y serves the IB items), then lanes and waves are reduced.
template <int CV>
__global__ __launch_bounds__(256) void s2_mm_gradx_kernel(const float2* __restrict__ gz, const float2* __restrict__ y,
                                                          float2* __restrict__ gx, int nl, int nbatch, int fi, int fo) {
  typedef typename CPack<CV>::type vec_t;
  __shared__ float2 part[4][IB][KC];
  const int lm = blockIdx.x, i0 = blockIdx.y * IB, k0 = blockIdx.z * KC;
  const int l = isqrt_floor(lm), m = lm - l * l - l;
  const int L = 2 * l + 1;
  const size_t base = (size_t)l * (4 * l * l - 1) / 3 + (size_t)(l + m) * L;
  const int fov = fo / CV;
  float2 acc[IB][KC];
#pragma unroll
  for (int q = 0; q < IB; ++q)
#pragma unroll
    for (int u = 0; u < KC; ++u) acc[q][u] = make_float2(0.f, 0.f);
  int nn = threadIdx.x / fov, jv = threadIdx.x - nn * fov;          // walks (n, jv) with stride 256
  const int dn = 256 / fov, dj = 256 - dn * fov;
  for (; nn < L; ) {
    const vec_t* g = reinterpret_cast<const vec_t*>(gz + ((base + nn) * nbatch + i0) * fo) + jv;
    vec_t a[IB];
#pragma unroll
    for (int q = 0; q < IB; ++q) a[q] = i0 + q < nbatch ? g[(size_t)q * fov] : CPack<CV>::zero();
    const vec_t* yy = reinterpret_cast<const vec_t*>(y + ((size_t)(l * l + nn) * fi + k0) * fo) + jv;
#pragma unroll
    for (int u = 0; u < KC; ++u) {
      if (k0 + u < fi) {
        const vec_t b = yy[(size_t)u * fov];
#pragma unroll
        for (int q = 0; q < IB; ++q) CPack<CV>::dot(a[q], b, acc[q][u]);
      }
    }
    nn += dn; jv += dj;
    if (jv >= fov) { jv -= fov; ++nn; }
  }
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
  for (int q = 0; q < IB; ++q)
#pragma unroll
    for (int u = 0; u < KC; ++u) {
      float2 v = acc[q][u];
#pragma unroll
      for (int sh = 32; sh > 0; sh >>= 1) { v.x += __shfl_down(v.x, sh, 64); v.y += __shfl_down(v.y, sh, 64); }
      if (lane == 0) part[wave][q][u] = v;
    }
  __syncthreads();
  if (threadIdx.x < IB * KC) {
    const int q = threadIdx.x / KC, u = threadIdx.x - q * KC;
    if (i0 + q < nbatch && k0 + u < fi) {
      const float2 a = part[0][q][u], b = part[1][q][u], c = part[2][q][u], d = part[3][q][u];
      gx[((size_t)lm * nbatch + i0 + q) * fi + k0 + u] = make_float2((a.x + b.x) + (c.x + d.x), (a.y + b.y) + (c.y + d.y));
    }
  }
}

// ---- grad y.  grid.x = nl^2 (l, n), grid.y = tile of JT j groups, grid.z = feature pass.  The threads form
// SL = 256 / JT slices of JT lanes; slice q takes the (m, i) pairs q, q + SL, ...; a lane accumulates KC pieces (x is
// uniform over a slice), then the slices are reduced through LDS in a fixed order.
template <int CV, int JT>
__global__ __launch_bounds__(256) void s2_mm_grady_kernel(const float2* __restrict__ gz, const float2* __restrict__ x,
                                                          float2* __restrict__ gy, int nl, int nbatch, int fi, int fo) {
  typedef typename CPack<CV>::type vec_t;
  constexpr int SL = 256 / JT;
  __shared__ float2 part[SL][KC][JT * CV];
  const int ln = blockIdx.x, k0 = blockIdx.z * KC;
  const int l = isqrt_floor(ln), n = ln - l * l - l;
  const int L = 2 * l + 1;
  const size_t base = (size_t)l * (4 * l * l - 1) / 3 + (size_t)(l + n);
  const int fov = fo / CV;
  const int slice = threadIdx.x / JT, jl = threadIdx.x - slice * JT;
  const int jv = blockIdx.y * JT + jl;
  vec_t acc[KC];
#pragma unroll
  for (int u = 0; u < KC; ++u) acc[u] = CPack<CV>::zero();
  const int total = L * nbatch;                                    // (m, i) pairs
  int mm = slice / nbatch, i = slice - mm * nbatch;                // walks the pairs with stride SL
  const int dm = SL / nbatch, di = SL - dm * nbatch;
  for (int p = slice; p < total; p += SL) {
    const vec_t a = jv < fov ? reinterpret_cast<const vec_t*>(gz + ((base + (size_t)mm * L) * nbatch + i) * fo)[jv] : CPack<CV>::zero();
    const float2* xx = x + ((size_t)(l * l + mm) * nbatch + i) * fi + k0;
#pragma unroll
    for (int u = 0; u < KC; ++u)
      if (k0 + u < fi) CPack<CV>::conj_axpy(a, xx[u], acc[u]);
    mm += dm; i += di;
    if (i >= nbatch) { i -= nbatch; ++mm; }
  }
#pragma unroll
  for (int u = 0; u < KC; ++u) reinterpret_cast<vec_t*>(&part[slice][u][0])[jl] = acc[u];
  __syncthreads();
  for (int o = threadIdx.x; o < KC * JT * CV; o += 256) {
    const int u = o / (JT * CV), jj = o - u * (JT * CV);
    const int j = blockIdx.y * JT * CV + jj;
    if (k0 + u < fi && j < fo) {
      float2 v = make_float2(0.f, 0.f);
#pragma unroll
      for (int q = 0; q < SL; ++q) { v.x += part[q][u][jj].x; v.y += part[q][u][jj].y; }
      gy[((size_t)ln * fi + k0 + u) * fo + j] = v;
    }
  }
}

int check(const void* a, const void* b, const void* c, int nl, int nbatch, int fi, int fo) {
  if (!a || !b || !c || nl < 1 || nl > 255 || nbatch < 1 || nbatch > 65535 || fi < 1 || fo < 1) return S2CNN_EINVAL;   // grid.y of grad x: ceil(nbatch / IB)
  if ((long)nbatch * fo >= (1L << 31) || (long)nbatch * fi >= (1L << 31) || (long)fi * fo >= (1L << 31)) return S2CNN_EINVAL;
  if ((fi + KC - 1) / KC > 65535 || (fo + 63) / 64 > 65535 || ((long)nbatch * fo + 255) / 256 > 65535) return S2CNN_EINVAL;
  if (!s2cnn::aligned8(a) || !s2cnn::aligned8(b) || !s2cnn::aligned8(c)) return S2CNN_EALIGN;
  return S2CNN_OK;
}

}  // namespace

extern "C" int s2cnn_s2_mm_fwd(const float* x, const float* y, float* z, int nl, int nbatch, int f_in, int f_out, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(x, y, z, nl, nbatch, f_in, f_out)) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const float2 *x2 = reinterpret_cast<const float2*>(x), *y2 = reinterpret_cast<const float2*>(y);
  const long ngroup = (nbatch + IPT - 1) / IPT;
  if (f_out % 2 == 0 && s2cnn::aligned16(y) && s2cnn::aligned16(z))
    hipLaunchKernelGGL(s2_mm_fwd_kernel<2>, dim3(nl * nl, NSPLIT, (unsigned)((ngroup * (f_out / 2) + 255) / 256)), dim3(256), 0, st,
                       x2, y2, reinterpret_cast<float2*>(z), nl, nbatch, f_in, f_out);
  else
    hipLaunchKernelGGL(s2_mm_fwd_kernel<1>, dim3(nl * nl, NSPLIT, (unsigned)((ngroup * f_out + 255) / 256)), dim3(256), 0, st,
                       x2, y2, reinterpret_cast<float2*>(z), nl, nbatch, f_in, f_out);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_s2_mm_gradx(const float* gz, const float* y, float* gx, int nl, int nbatch, int f_in, int f_out, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(gz, y, gx, nl, nbatch, f_in, f_out)) return rc;
  const dim3 grid(nl * nl, (nbatch + IB - 1) / IB, (f_in + KC - 1) / KC);
  hipStream_t st = static_cast<hipStream_t>(stream);
  const float2 *g2 = reinterpret_cast<const float2*>(gz), *y2 = reinterpret_cast<const float2*>(y);
  if (f_out % 2 == 0 && s2cnn::aligned16(gz) && s2cnn::aligned16(y))
    hipLaunchKernelGGL(s2_mm_gradx_kernel<2>, grid, dim3(256), 0, st, g2, y2, reinterpret_cast<float2*>(gx), nl, nbatch, f_in, f_out);
  else
    hipLaunchKernelGGL(s2_mm_gradx_kernel<1>, grid, dim3(256), 0, st, g2, y2, reinterpret_cast<float2*>(gx), nl, nbatch, f_in, f_out);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_s2_mm_grady(const float* gz, const float* x, float* gy, int nl, int nbatch, int f_in, int f_out, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(gz, x, gy, nl, nbatch, f_in, f_out)) return rc;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const float2 *g2 = reinterpret_cast<const float2*>(gz), *x2 = reinterpret_cast<const float2*>(x);
  if (f_out % 2 == 0 && s2cnn::aligned16(gz) && s2cnn::aligned16(gy)) {
    const dim3 grid(nl * nl, (f_out / 2 + 15) / 16, (f_in + KC - 1) / KC);
    hipLaunchKernelGGL((s2_mm_grady_kernel<2, 16>), grid, dim3(256), 0, st, g2, x2, reinterpret_cast<float2*>(gy), nl, nbatch, f_in, f_out);
  } else {
    const dim3 grid(nl * nl, (f_out + 31) / 32, (f_in + KC - 1) / KC);
    hipLaunchKernelGGL((s2_mm_grady_kernel<1, 32>), grid, dim3(256), 0, st, g2, x2, reinterpret_cast<float2*>(gy), nl, nbatch, f_in, f_out);
  }
  return s2cnn::launch_status();
}
