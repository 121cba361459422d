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

// ---- forward: grid.x = nl^2 (l,m), grid.y = quarter of the n range, grid.z = tile of 256 (i,j) outputs.
// A thread owns one (i, j): x[l,m,i,:] stays in registers while it walks n, so per n it reads one coalesced
// row of y and writes one coalesced row of z; consecutive n are consecutive blocks of z.
constexpr int NSPLIT = 4;

__global__ __launch_bounds__(256) void s2_mm_fwd_kernel(const float2* __restrict__ x, const float2* __restrict__ y,
                                                        float2* __restrict__ z, int nl, int nbatch, int fi, int fo) {
  const int lm = blockIdx.x;
  const int l = isqrt_floor(lm), m = lm - l * l - l;
  const int L = 2 * l + 1;
  const int n_lo = (int)((long)blockIdx.y * L / NSPLIT), n_hi = (int)((long)(blockIdx.y + 1) * L / NSPLIT);
  const int o = blockIdx.z * 256 + threadIdx.x;
  if (o >= nbatch * fo || n_lo >= n_hi) return;
  const int i = o / fo, j = o - i * fo;
  const float2* xs = x + ((size_t)lm * nbatch + i) * fi;
  const size_t zbase = (size_t)l * (4 * l * l - 1) / 3 + (size_t)(l + m) * L;
  for (int k0 = 0; k0 < fi; k0 += KC) {
    float2 xr[KC];
#pragma unroll
    for (int u = 0; u < KC; ++u) xr[u] = k0 + u < fi ? xs[k0 + u] : make_float2(0.f, 0.f);
    for (int nn = n_lo; nn < n_hi; ++nn) {
      const float2* ys = y + ((size_t)(l * l + nn) * fi + k0) * fo + j;
      float2* zp = z + (zbase + nn) * nbatch * fo + o;
      float re = 0.f, im = 0.f;
      if (k0 > 0) { const float2 p = *zp; re = p.x; im = p.y; }     // later feature passes accumulate
#pragma unroll
      for (int u = 0; u < KC; ++u) {
        if (k0 + u < fi) {
          const float2 b = ys[(size_t)u * fo];
          re += xr[u].x * b.x + xr[u].y * b.y;
          im += xr[u].y * b.x - xr[u].x * b.y;
        }
      }
      *zp = make_float2(re, im);
    }
  }
}

// ---- grad x: grid.x = nl^2 (l,m), grid.y = batch item i, grid.z = feature pass.  Lanes run along j, every wave takes
// the n = wave, wave + nwaves, ...; each lane accumulates KC features, then lanes and waves are reduced.
__global__ __launch_bounds__(256) void s2_mm_gradx_kernel(const float2* __restrict__ gz, const float2* __restrict__ y,
                                                          float2* __restrict__ gx, int nl, int nbatch, int fi, int fo) {
  __shared__ float2 part[4][KC];
  const int lm = blockIdx.x, i = blockIdx.y, k0 = blockIdx.z * KC;
  const int l = isqrt_floor(lm), m = lm - l * l - l;
  const int L = 2 * l + 1;
  const size_t base = (size_t)l * (4 * l * l - 1) / 3 + (size_t)(l + m) * L;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  float2 acc[KC];
#pragma unroll
  for (int u = 0; u < KC; ++u) acc[u] = make_float2(0.f, 0.f);
  for (int nn = wave; nn < L; nn += 4) {
    const float2* g = gz + ((base + nn) * nbatch + i) * fo;
    const float2* yy = y + (size_t)(l * l + nn) * fi * fo;
    for (int j = lane; j < fo; j += 64) {
      const float2 a = g[j];
#pragma unroll
      for (int u = 0; u < KC; ++u) {
        if (k0 + u < fi) {
          const float2 b = yy[(size_t)(k0 + u) * fo + j];
          acc[u].x += a.x * b.x - a.y * b.y;
          acc[u].y += a.x * b.y + a.y * b.x;
        }
      }
    }
  }
#pragma unroll
  for (int u = 0; u < KC; ++u) {
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
      acc[u].x += __shfl_down(acc[u].x, s, 64);
      acc[u].y += __shfl_down(acc[u].y, s, 64);
    }
    if (lane == 0) part[wave][u] = acc[u];
  }
  __syncthreads();
  if (threadIdx.x < KC && k0 + (int)threadIdx.x < fi) {
    const int u = threadIdx.x;
    const float2 a = part[0][u], b = part[1][u], c = part[2][u], d = part[3][u];
    gx[((size_t)lm * nbatch + i) * fi + k0 + u] = make_float2(a.x + b.x + c.x + d.x, a.y + b.y + c.y + d.y);
  }
}

// ---- grad y: grid.x = nl^2 (l,n), grid.y = tiles of 64 output features j, grid.z = feature pass.  Lane = j; the four
// waves split the (m, i) reduction; each lane accumulates KC input features (x is wave-uniform), then waves are reduced.
__global__ __launch_bounds__(256) void s2_mm_grady_kernel(const float2* __restrict__ gz, const float2* __restrict__ x,
                                                          float2* __restrict__ gy, int nl, int nbatch, int fi, int fo) {
  __shared__ float2 part[4][KC][64];
  const int ln = blockIdx.x, k0 = blockIdx.z * KC;
  const int l = isqrt_floor(ln), n = ln - l * l - l;
  const int L = 2 * l + 1;
  const size_t base = (size_t)l * (4 * l * l - 1) / 3 + (size_t)(l + n);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int j = blockIdx.y * 64 + lane;
  float2 acc[KC];
#pragma unroll
  for (int u = 0; u < KC; ++u) acc[u] = make_float2(0.f, 0.f);
  const int total = L * nbatch;                       // (m, i) pairs
  for (int r = wave; r < total; r += 4) {
    const int mm = r / nbatch, i = r - mm * nbatch;
    const float2 a = j < fo ? gz[((base + (size_t)mm * L) * nbatch + i) * fo + j] : make_float2(0.f, 0.f);
    const float2* xx = x + ((size_t)(l * l + mm) * nbatch + i) * fi + k0;
#pragma unroll
    for (int u = 0; u < KC; ++u) {
      if (k0 + u < fi) {
        const float2 b = xx[u];
        acc[u].x += a.x * b.x + a.y * b.y;            // conj(a) * b
        acc[u].y += a.x * b.y - a.y * b.x;
      }
    }
  }
#pragma unroll
  for (int u = 0; u < KC; ++u) part[wave][u][lane] = acc[u];
  __syncthreads();
  for (int o = threadIdx.x; o < KC * 64; o += 256) {
    const int u = o >> 6, jj = o & 63;
    const int jg = blockIdx.y * 64 + jj;
    if (k0 + u < fi && jg < fo) {
      const float2 a = part[0][u][jj], b = part[1][u][jj], c = part[2][u][jj], d = part[3][u][jj];
      gy[((size_t)ln * fi + k0 + u) * fo + jg] = make_float2(a.x + b.x + c.x + d.x, a.y + b.y + c.y + d.y);
    }
  }
}

int check(const void* a, const void* b, const void* c, int nl, int nbatch, int fi, int fo) {
  if (!a || !b || !c || nl < 1 || nl > 255 || nbatch < 1 || nbatch > 65535 || fi < 1 || fo < 1) return S2CNN_EINVAL;
  if ((long)nbatch * fo >= (1L << 31) || (long)nbatch * fi >= (1L << 31) || (long)fi * fo >= (1L << 31)) return S2CNN_EINVAL;
  if ((fi + KC - 1) / KC > 65535 || (fo + 63) / 64 > 65535 || ((long)nbatch * fo + 255) / 256 > 65535) return S2CNN_EINVAL;
  if (!s2cnn::aligned8(a) || !s2cnn::aligned8(b) || !s2cnn::aligned8(c)) return S2CNN_EALIGN;
  return S2CNN_OK;
}

}  // namespace

extern "C" int s2cnn_s2_mm_fwd(const float* x, const float* y, float* z, int nl, int nbatch, int f_in, int f_out, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(x, y, z, nl, nbatch, f_in, f_out)) return rc;
  hipLaunchKernelGGL(s2_mm_fwd_kernel, dim3(nl * nl, NSPLIT, (unsigned)(((long)nbatch * f_out + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream),
                     reinterpret_cast<const float2*>(x), reinterpret_cast<const float2*>(y), reinterpret_cast<float2*>(z),
                     nl, nbatch, f_in, f_out);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_s2_mm_gradx(const float* gz, const float* y, float* gx, int nl, int nbatch, int f_in, int f_out, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(gz, y, gx, nl, nbatch, f_in, f_out)) return rc;
  hipLaunchKernelGGL(s2_mm_gradx_kernel, dim3(nl * nl, nbatch, (f_in + KC - 1) / KC), dim3(256), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<const float2*>(gz), reinterpret_cast<const float2*>(y), reinterpret_cast<float2*>(gx),
                     nl, nbatch, f_in, f_out);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_s2_mm_grady(const float* gz, const float* x, float* gy, int nl, int nbatch, int f_in, int f_out, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(gz, x, gy, nl, nbatch, f_in, f_out)) return rc;
  hipLaunchKernelGGL(s2_mm_grady_kernel, dim3(nl * nl, (f_out + 63) / 64, (f_in + KC - 1) / KC), dim3(256), 0,
                     static_cast<hipStream_t>(stream), reinterpret_cast<const float2*>(gz), reinterpret_cast<const float2*>(x),
                     reinterpret_cast<float2*>(gy), nl, nbatch, f_in, f_out);
  return s2cnn::launch_status();
}
