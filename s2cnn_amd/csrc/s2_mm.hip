// S^2 x S^2 -> SO(3) spectral outer product and its two adjoints.
//
//   fwd   : z [l,m,n,i,j] = sum_k x[l,m,i,k] * conj(y[l,n,k,j])
//   gradx : gx[l,m,i,k]   = sum_{n,j} gz[l,m,n,i,j] * y[l,n,k,j]
//   grady : gy[l,n,k,j]   = sum_{m,i} conj(gz[l,m,n,i,j]) * x[l,m,i,k]
//
// The contraction of the forward product runs over input features only, so for the few input
// features of a first layer the product is bound by writing z; the kernels are plain FMA code
// whose lanes run along the fastest output index.
#include "common.h"

namespace {

__device__ inline void decode_lmn(int s, int nl, int& l, int& m, int& n) {
  l = 0;
  while (l + 1 < nl && (l + 1) * (4 * (l + 1) * (l + 1) - 1) / 3 <= s) ++l;
  const int r = s - l * (4 * l * l - 1) / 3;
  const int L = 2 * l + 1;
  m = r / L - l;
  n = r % L - l;
}

// grid.x = nspec_so3, threads over (i, j) with j fastest
__global__ __launch_bounds__(256) void s2_mm_fwd_kernel(const float2* __restrict__ x, const float2* __restrict__ y,
                                                        float2* __restrict__ z, int nl, int nbatch, int fi, int fo) {
  int l, m, n;
  decode_lmn(blockIdx.x, nl, l, m, n);
  const float2* xs = x + (size_t)(l * l + l + m) * nbatch * fi;
  const float2* ys = y + (size_t)(l * l + l + n) * fi * fo;
  float2* zs = z + (size_t)blockIdx.x * nbatch * fo;
  for (int o = threadIdx.x; o < nbatch * fo; o += blockDim.x) {
    const int i = o / fo, j = o - i * fo;
    float re = 0.f, im = 0.f;
    for (int k = 0; k < fi; ++k) {
      const float2 a = xs[i * fi + k];
      const float2 b = ys[k * fo + j];
      re += a.x * b.x + a.y * b.y;
      im += a.y * b.x - a.x * b.y;
    }
    zs[o] = make_float2(re, im);
  }
}

// grid.x = nl^2 (l,m), threads over (i, k); the reduction runs over n and j
__global__ __launch_bounds__(256) void s2_mm_gradx_kernel(const float2* __restrict__ gz, const float2* __restrict__ y,
                                                          float2* __restrict__ gx, int nl, int nbatch, int fi, int fo) {
  const int lm = blockIdx.x;
  int l = (int)sqrtf((float)lm);
  while (l * l > lm) --l;
  while ((l + 1) * (l + 1) <= lm) ++l;
  const int m = lm - l * l - l;
  const int L = 2 * l + 1;
  const size_t base = (size_t)l * (4 * l * l - 1) / 3 + (size_t)(l + m) * L;
  for (int o = threadIdx.x; o < nbatch * fi; o += blockDim.x) {
    const int i = o / fi, k = o - i * fi;
    float re = 0.f, im = 0.f;
    for (int nn = 0; nn < L; ++nn) {
      const float2* g = gz + ((base + nn) * nbatch + i) * fo;
      const float2* yy = y + ((size_t)(l * l + nn) * fi + k) * fo;
      for (int j = 0; j < fo; ++j) {
        const float2 a = g[j], b = yy[j];
        re += a.x * b.x - a.y * b.y;
        im += a.x * b.y + a.y * b.x;
      }
    }
    gx[(size_t)lm * nbatch * fi + o] = make_float2(re, im);
  }
}

// grid.x = nl^2 (l,n), threads over (k, j) with j fastest; the reduction runs over m and i
__global__ __launch_bounds__(256) void s2_mm_grady_kernel(const float2* __restrict__ gz, const float2* __restrict__ x,
                                                          float2* __restrict__ gy, int nl, int nbatch, int fi, int fo) {
  const int ln = blockIdx.x;
  int l = (int)sqrtf((float)ln);
  while (l * l > ln) --l;
  while ((l + 1) * (l + 1) <= ln) ++l;
  const int n = ln - l * l - l;
  const int L = 2 * l + 1;
  const size_t base = (size_t)l * (4 * l * l - 1) / 3 + (size_t)(l + n);
  for (int o = threadIdx.x; o < fi * fo; o += blockDim.x) {
    const int k = o / fo, j = o - k * fo;
    float re = 0.f, im = 0.f;
    for (int mm = 0; mm < L; ++mm) {
      const float2* g = gz + (base + (size_t)mm * L) * nbatch * fo + j;
      const float2* xx = x + (size_t)(l * l + mm) * nbatch * fi + k;
      for (int i = 0; i < nbatch; ++i) {
        const float2 a = g[(size_t)i * fo], b = xx[(size_t)i * fi];
        re += a.x * b.x + a.y * b.y;      // conj(a) * b
        im += a.x * b.y - a.y * b.x;
      }
    }
    gy[(size_t)ln * fi * fo + o] = make_float2(re, im);
  }
}

int check(const void* a, const void* b, const void* c, int nl, int nbatch, int fi, int fo) {
  if (!a || !b || !c || nl < 1 || nl > 812 || nbatch < 1 || fi < 1 || fo < 1) return S2CNN_EINVAL;
  if ((long)nbatch * fo >= (1L << 31) || (long)nbatch * fi >= (1L << 31) || (long)fi * fo >= (1L << 31)) return S2CNN_EINVAL;
  if (!s2cnn::aligned8(a) || !s2cnn::aligned8(b) || !s2cnn::aligned8(c)) return S2CNN_EALIGN;
  return S2CNN_OK;
}

}  // namespace

extern "C" int s2cnn_s2_mm_fwd(const float* x, const float* y, float* z, int nl, int nbatch, int f_in, int f_out, void* stream) {
  if (int rc = check(x, y, z, nl, nbatch, f_in, f_out)) return rc;
  hipLaunchKernelGGL(s2_mm_fwd_kernel, dim3((unsigned)s2cnn::so3_nspec(nl)), dim3(256), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<const float2*>(x), reinterpret_cast<const float2*>(y), reinterpret_cast<float2*>(z),
                     nl, nbatch, f_in, f_out);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_s2_mm_gradx(const float* gz, const float* y, float* gx, int nl, int nbatch, int f_in, int f_out, void* stream) {
  if (int rc = check(gz, y, gx, nl, nbatch, f_in, f_out)) return rc;
  hipLaunchKernelGGL(s2_mm_gradx_kernel, dim3(nl * nl), dim3(256), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<const float2*>(gz), reinterpret_cast<const float2*>(y), reinterpret_cast<float2*>(gx),
                     nl, nbatch, f_in, f_out);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_s2_mm_grady(const float* gz, const float* x, float* gy, int nl, int nbatch, int f_in, int f_out, void* stream) {
  if (int rc = check(gz, x, gy, nl, nbatch, f_in, f_out)) return rc;
  hipLaunchKernelGGL(s2_mm_grady_kernel, dim3(nl * nl), dim3(256), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<const float2*>(gz), reinterpret_cast<const float2*>(x), reinterpret_cast<float2*>(gy),
                     nl, nbatch, f_in, f_out);
  return s2cnn::launch_status();
}
