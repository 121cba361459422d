// Kernel spectrum of the SO(3) convolution layer for grids with few distinct beta values.
//
// The reference evaluates  y[l,m,n] = sum_a x_a conj(D^l_{mn}(alpha_a, beta_a, gamma_a))  as one dense product with a
// [len(grid), nspec] matrix (s2cnn/so3_ft.py:8-24).  For the points A_i that share beta_i,
//     conj D^l_{mn} = d^l_{mn}(beta_i) * exp(-i (m alpha_a + n gamma_a)),
// so  y[l,m,n] = sum_i d^l_{mn}(beta_i) G_i[m,n]  with the plane coefficients G_i[m,n] = sum_{a in A_i} x_a e^{-i(m alpha_a + n gamma_a)}
// (a small library GEMM on the host side).  The kernels here do the second step and its adjoint, directly in the
// real basis of so3_real_basis.hip; x is real, so G_i[-m,-n] = conj G_i[m,n] and only n >= 0 is stored:
//     G [nbeta][(m + b-1) * b + n][re, im][ncols],  m in -(b-1)..b-1,  n in 0..b-1
// With A = y[l,+a,n], C = y[l,-a,n] (a, n >= 0) and s = (-1)^a the real-basis entries are
//     R[+a,+n] = A.re + s C.re    R[+a,-n] = -A.im - s C.im    R[-a,+n] = A.im - s C.im    R[-a,-n] = A.re - s C.re
//     a = 0: sqrt2 A.re, -sqrt2 A.im     n = 0: (A.re + s C.re)/sqrt2, (A.im - s C.im)/sqrt2     a = n = 0: A.re
// The complex form of the same spectrum needs no combination at all: y[l,+a,n] = A, y[l,-a,n] = C and, x being real,
// y[l,-a,-n] = (-1)^(a+n) conj A, y[l,+a,-n] = (-1)^(a+n) conj C (template argument CPLX: y [nspec][ncols][re, im]).
// One thread owns one pair (a, n) and four columns and walks over the degrees: G stays in registers, the
// d-values are uniform (scalar loads), every access to y is a 16-byte piece of a contiguous row.
#include "common.h"

namespace {

constexpr float SQRT2 = 1.41421356237309504880f, RSQRT2 = 0.70710678118654752440f;
constexpr int NBMAX = 4;

__device__ __forceinline__ int lmn_index(int l, int m, int n) { return l * (4 * l * l - 1) / 3 + (l + m) * (2 * l + 1) + (l + n); }
__device__ __forceinline__ float4 fma4(float s, float4 v, float4 acc) {
  return make_float4(fmaf(s, v.x, acc.x), fmaf(s, v.y, acc.y), fmaf(s, v.z, acc.z), fmaf(s, v.w, acc.w));
}
__device__ __forceinline__ float4 lin4(float p, float4 u, float q, float4 v) {   // p u + q v
  return make_float4(p * u.x + q * v.x, p * u.y + q * v.y, p * u.z + q * v.z, p * u.w + q * v.w);
}

template <int NB, bool CPLX>
__global__ __launch_bounds__(256) void rft_expand_kernel(const float* __restrict__ G, const float* __restrict__ dtab,
                                                         float* __restrict__ y, int b, long ncols) {
  const int a = blockIdx.x / b, n = blockIdx.x - a * b;
  // the thread's four columns: c0 .. c0 + 3, or, for complex output, the pairs c0, c0 + 1 and c1, c1 + 1 half a tile apart,
  // so that the 16 bytes (two complex numbers) a lane stores lie next to its neighbours'
  const long c0 = CPLX ? (long)blockIdx.y * 1024 + 2 * threadIdx.x : ((long)blockIdx.y * 256 + threadIdx.x) * 4;
  const long c1 = c0 + 512;
  if (c0 >= ncols) return;
  const bool has1 = !CPLX || c1 < ncols;
  const long nspec = (long)b * (4L * b * b - 1) / 3;
  const size_t R = (size_t)(2 * b - 1) * b * 2;
  const bool stream = (size_t)nspec * (size_t)ncols * (CPLX ? 8 : 4) >= s2cnn::STREAM_BYTES;    // the spectrum is streamed: uniform
  const size_t rp = (size_t)((a + b - 1) * b + n) * 2, rm = (size_t)((-a + b - 1) * b + n) * 2;
  auto columns = [&](const float* row) {      // the thread's four columns of a row of G
    if constexpr (CPLX) {
      const float2 u = *reinterpret_cast<const float2*>(row + c0);
      const float2 v = has1 ? *reinterpret_cast<const float2*>(row + c1) : make_float2(0.f, 0.f);
      return make_float4(u.x, u.y, v.x, v.y);
    } else {
      return *reinterpret_cast<const float4*>(row + c0);
    }
  };
  float4 pr[NB], pi[NB], mr[NB], mi[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const float* g = G + (size_t)i * R * ncols;
    pr[i] = columns(g + rp * ncols);
    pi[i] = columns(g + (rp + 1) * ncols);
    mr[i] = columns(g + rm * ncols);
    mi[i] = columns(g + (rm + 1) * ncols);
  }
  const float s = (a & 1) ? -1.f : 1.f;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int l = a > n ? a : n; l < b; ++l) {
    const int ip = lmn_index(l, a, n), im = lmn_index(l, -a, n);
    float4 Ar = zero, Ai = zero, Cr = zero, Ci = zero;
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const float d1 = dtab[i * nspec + ip], d2 = dtab[i * nspec + im];
      Ar = fma4(d1, pr[i], Ar); Ai = fma4(d1, pi[i], Ai);
      Cr = fma4(d2, mr[i], Cr); Ci = fma4(d2, mi[i], Ci);
    }
    if constexpr (CPLX) {
      // the two column pairs of a row, (re, im) interleaved: 16 bytes each
      auto put = [&](int lmn, float4 re, float4 im, float sg) {
        float* d = y + (size_t)lmn * ncols * 2;
        s2cnn::store_policy(make_float4(sg * re.x, im.x, sg * re.y, im.y), reinterpret_cast<float4*>(d + c0 * 2), stream);
        if (has1) s2cnn::store_policy(make_float4(sg * re.z, im.z, sg * re.w, im.w), reinterpret_cast<float4*>(d + c1 * 2), stream);
      };
      const float sg = ((a + n) & 1) ? -1.f : 1.f;
      const float4 nAi = make_float4(-sg * Ai.x, -sg * Ai.y, -sg * Ai.z, -sg * Ai.w);      // sg conj: (sg re, -sg im)
      const float4 nCi = make_float4(-sg * Ci.x, -sg * Ci.y, -sg * Ci.z, -sg * Ci.w);
      put(ip, Ar, Ai, 1.f);
      if (a > 0) put(im, Cr, Ci, 1.f);
      if (n > 0) {
        put(lmn_index(l, -a, -n), Ar, nAi, sg);
        if (a > 0) put(lmn_index(l, a, -n), Cr, nCi, sg);
      }
      continue;
    }
    float* row = y + c0;
    if (a > 0 && n > 0) {
      s2cnn::store_policy(lin4(1.f, Ar, s, Cr), reinterpret_cast<float4*>(row + (size_t)ip * ncols), stream);
      s2cnn::store_policy(lin4(-1.f, Ai, -s, Ci), reinterpret_cast<float4*>(row + (size_t)lmn_index(l, a, -n) * ncols), stream);
      s2cnn::store_policy(lin4(1.f, Ai, -s, Ci), reinterpret_cast<float4*>(row + (size_t)im * ncols), stream);
      s2cnn::store_policy(lin4(1.f, Ar, -s, Cr), reinterpret_cast<float4*>(row + (size_t)lmn_index(l, -a, -n) * ncols), stream);
    } else if (a > 0) {
      s2cnn::store_policy(lin4(RSQRT2, Ar, s * RSQRT2, Cr), reinterpret_cast<float4*>(row + (size_t)ip * ncols), stream);
      s2cnn::store_policy(lin4(RSQRT2, Ai, -s * RSQRT2, Ci), reinterpret_cast<float4*>(row + (size_t)im * ncols), stream);
    } else if (n > 0) {
      s2cnn::store_policy(lin4(SQRT2, Ar, 0.f, zero), reinterpret_cast<float4*>(row + (size_t)ip * ncols), stream);
      s2cnn::store_policy(lin4(-SQRT2, Ai, 0.f, zero), reinterpret_cast<float4*>(row + (size_t)lmn_index(l, 0, -n) * ncols), stream);
    } else {
      *reinterpret_cast<float4*>(row + (size_t)ip * ncols) = Ar;
    }
  }
}

// adjoint: gG_i[+-a, n] = sum_l d^l_{+-a,n}(beta_i) * (gA, gC)(l), with (gA, gC) the adjoint of the formulas above
template <int NB>
__global__ __launch_bounds__(256) void rft_expand_grad_kernel(const float* __restrict__ gy, const float* __restrict__ dtab,
                                                              float* __restrict__ gG, int b, long ncols) {
  const int a = blockIdx.x / b, n = blockIdx.x - a * b;
  const long c0 = ((long)blockIdx.y * 256 + threadIdx.x) * 4;
  if (c0 >= ncols) return;
  const long nspec = (long)b * (4L * b * b - 1) / 3;
  const size_t R = (size_t)(2 * b - 1) * b * 2;
  const bool stream = (size_t)nspec * (size_t)ncols * 4 >= s2cnn::STREAM_BYTES;    // the spectrum is streamed: uniform
  const size_t rp = (size_t)((a + b - 1) * b + n) * 2, rm = (size_t)((-a + b - 1) * b + n) * 2;
  const float4 zero = make_float4(0.f, 0.f, 0.f, 0.f);
  float4 pr[NB], pi[NB], mr[NB], mi[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) pr[i] = pi[i] = mr[i] = mi[i] = zero;
  const float s = (a & 1) ? -1.f : 1.f;
  for (int l = a > n ? a : n; l < b; ++l) {
    const int ip = lmn_index(l, a, n), im = lmn_index(l, -a, n);
    const float* row = gy + c0;
    float4 gAr, gAi, gCr = zero, gCi = zero;
    if (a > 0 && n > 0) {
      const float4 gpp = s2cnn::load_policy(reinterpret_cast<const float4*>(row + (size_t)ip * ncols), stream);
      const float4 gpm = s2cnn::load_policy(reinterpret_cast<const float4*>(row + (size_t)lmn_index(l, a, -n) * ncols), stream);
      const float4 gmp = s2cnn::load_policy(reinterpret_cast<const float4*>(row + (size_t)im * ncols), stream);
      const float4 gmm = s2cnn::load_policy(reinterpret_cast<const float4*>(row + (size_t)lmn_index(l, -a, -n) * ncols), stream);
      gAr = lin4(1.f, gpp, 1.f, gmm); gAi = lin4(-1.f, gpm, 1.f, gmp);
      gCr = lin4(s, gpp, -s, gmm);    gCi = lin4(-s, gpm, -s, gmp);
    } else if (a > 0) {
      const float4 gpp = s2cnn::load_policy(reinterpret_cast<const float4*>(row + (size_t)ip * ncols), stream);
      const float4 gmp = s2cnn::load_policy(reinterpret_cast<const float4*>(row + (size_t)im * ncols), stream);
      gAr = lin4(RSQRT2, gpp, 0.f, zero);     gAi = lin4(RSQRT2, gmp, 0.f, zero);
      gCr = lin4(s * RSQRT2, gpp, 0.f, zero); gCi = lin4(-s * RSQRT2, gmp, 0.f, zero);
    } else if (n > 0) {
      const float4 gpp = s2cnn::load_policy(reinterpret_cast<const float4*>(row + (size_t)ip * ncols), stream);
      const float4 gpm = s2cnn::load_policy(reinterpret_cast<const float4*>(row + (size_t)lmn_index(l, 0, -n) * ncols), stream);
      gAr = lin4(SQRT2, gpp, 0.f, zero); gAi = lin4(-SQRT2, gpm, 0.f, zero);
    } else {
      gAr = s2cnn::load_policy(reinterpret_cast<const float4*>(row + (size_t)ip * ncols), stream); gAi = zero;
    }
#pragma unroll
    for (int i = 0; i < NB; ++i) {
      const float d1 = dtab[i * nspec + ip], d2 = dtab[i * nspec + im];
      pr[i] = fma4(d1, gAr, pr[i]); pi[i] = fma4(d1, gAi, pi[i]);
      mr[i] = fma4(d2, gCr, mr[i]); mi[i] = fma4(d2, gCi, mi[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    float* g = gG + (size_t)i * R * ncols + c0;
    *reinterpret_cast<float4*>(g + rp * ncols) = pr[i];
    *reinterpret_cast<float4*>(g + (rp + 1) * ncols) = pi[i];
    if (a > 0) {   // for a = 0 the (-a) row is the (+a) row
      *reinterpret_cast<float4*>(g + rm * ncols) = mr[i];
      *reinterpret_cast<float4*>(g + (rm + 1) * ncols) = mi[i];
    }
  }
}

int check(const void* p, const void* q, const void* r, int b, int nbeta, long ncols) {
  if (!p || !q || !r || b < 1 || b > 512 || nbeta < 1 || nbeta > NBMAX || ncols < 4 || ncols % 4 || ncols >= (1L << 31)) return S2CNN_EINVAL;
  if (!s2cnn::aligned16(p) || !s2cnn::aligned16(r)) return S2CNN_EALIGN;
  return S2CNN_OK;
}

}  // namespace

namespace {
template <bool CPLX>
int expand(const float* G, const float* dtab, float* y, int b, int nbeta, long ncols, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(G, dtab, y, b, nbeta, ncols)) return rc;
  const dim3 grid((unsigned)(b * b), (unsigned)((ncols / 4 + 255) / 256));
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (nbeta) {
    case 1: hipLaunchKernelGGL((rft_expand_kernel<1, CPLX>), grid, dim3(256), 0, st, G, dtab, y, b, ncols); break;
    case 2: hipLaunchKernelGGL((rft_expand_kernel<2, CPLX>), grid, dim3(256), 0, st, G, dtab, y, b, ncols); break;
    case 3: hipLaunchKernelGGL((rft_expand_kernel<3, CPLX>), grid, dim3(256), 0, st, G, dtab, y, b, ncols); break;
    default: hipLaunchKernelGGL((rft_expand_kernel<4, CPLX>), grid, dim3(256), 0, st, G, dtab, y, b, ncols); break;
  }
  return s2cnn::launch_status();
}
}  // namespace

extern "C" int s2cnn_so3_rft_expand_real(const float* G, const float* dtab, float* y, int b, int nbeta, long ncols, void* stream) {
  return expand<false>(G, dtab, y, b, nbeta, ncols, stream);
}

extern "C" int s2cnn_so3_rft_expand(const float* G, const float* dtab, float* y, int b, int nbeta, long ncols, void* stream) {
  return expand<true>(G, dtab, y, b, nbeta, ncols, stream);
}

extern "C" int s2cnn_so3_rft_expand_real_grad(const float* gy, const float* dtab, float* gG, int b, int nbeta, long ncols, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(gy, dtab, gG, b, nbeta, ncols)) return rc;
  const dim3 grid((unsigned)(b * b), (unsigned)((ncols / 4 + 255) / 256));
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (nbeta) {
    case 1: hipLaunchKernelGGL(rft_expand_grad_kernel<1>, grid, dim3(256), 0, st, gy, dtab, gG, b, ncols); break;
    case 2: hipLaunchKernelGGL(rft_expand_grad_kernel<2>, grid, dim3(256), 0, st, gy, dtab, gG, b, ncols); break;
    case 3: hipLaunchKernelGGL(rft_expand_grad_kernel<3>, grid, dim3(256), 0, st, gy, dtab, gG, b, ncols); break;
    default: hipLaunchKernelGGL(rft_expand_grad_kernel<4>, grid, dim3(256), 0, st, gy, dtab, gG, b, ncols); break;
  }
  return s2cnn::launch_status();
}
