// Change of basis between the complex SO(3) spectrum and the real one.
//
// The spectrum of a real signal obeys X[l,-m,-n] = (-1)^(m-n) conj(X[l,m,n]).  With the unitary U_l
//     U[0,0] = 1,   U[+m, m] = 1/sqrt2,   U[+m,-m] = (-1)^m / sqrt2,
//                   U[-m, m] = -i/sqrt2,  U[-m,-m] = i (-1)^m / sqrt2        (m = 1..l)
// (rows: real index r = -l..l, stored at l + r like m) the block U X U^H of such a spectrum is real, and
// products of spectra carry over:  U (X Y^H) U^H = (U X U^H)(U Y U^H)^T.
//
//   to_real    : R = Re(U X U^H)   for ANY complex X (the imaginary part vanishes for a real signal's spectrum)
//   to_complex : X = U^H R U       the inverse on real R, and the adjoint of to_real as a real-linear map
//
// Both move each element once: a workgroup owns one quadruple {(+-m, +-n)} of one degree and walks the
// columns (batch x feature) with coalesced accesses.
#include "common.h"

namespace {

constexpr float RSQRT2 = 0.70710678118654752440f;

struct Quad {
  size_t pp, pm, mp, mm;   // flat spectral indices of (m,n), (m,-n), (-m,n), (-m,-n)
  int m, n;
  float sm, sn;            // (-1)^m, (-1)^n
};

__device__ inline Quad decode_quad(int q, int nl) {
  int l = 0;
  for (; l < nl; ++l) {
    const int cnt = (l + 1) * (l + 1);
    if (q < cnt) break;
    q -= cnt;
  }
  Quad o;
  o.m = q / (l + 1);
  o.n = q - o.m * (l + 1);
  const int L = 2 * l + 1;
  const size_t base = (size_t)l * (4 * l * l - 1) / 3;
  o.pp = base + (size_t)(l + o.m) * L + (l + o.n);
  o.pm = base + (size_t)(l + o.m) * L + (l - o.n);
  o.mp = base + (size_t)(l - o.m) * L + (l + o.n);
  o.mm = base + (size_t)(l - o.m) * L + (l - o.n);
  o.sm = (o.m & 1) ? -1.f : 1.f;
  o.sn = (o.n & 1) ? -1.f : 1.f;
  return o;
}

__global__ __launch_bounds__(256) void to_real_kernel(const float2* __restrict__ x, float* __restrict__ r, int nl, long ncols) {
  const Quad q = decode_quad(blockIdx.x, nl);
  for (long c = (long)blockIdx.y * 256 + threadIdx.x; c < ncols; c += 256L * gridDim.y) {
    const float2 A = x[q.pp * ncols + c];
    if (q.m == 0 && q.n == 0) {
      r[q.pp * ncols + c] = A.x;
    } else if (q.m == 0) {          // row 0: columns cos_n (at +n) and sin_n (at -n)
      const float2 B = x[q.pm * ncols + c];
      r[q.pp * ncols + c] = RSQRT2 * (A.x + q.sn * B.x);
      r[q.pm * ncols + c] = RSQRT2 * (-A.y + q.sn * B.y);
    } else if (q.n == 0) {          // column 0: rows cos_m (at +m) and sin_m (at -m)
      const float2 C = x[q.mp * ncols + c];
      r[q.pp * ncols + c] = RSQRT2 * (A.x + q.sm * C.x);
      r[q.mp * ncols + c] = RSQRT2 * (A.y - q.sm * C.y);
    } else {
      const float2 B = x[q.pm * ncols + c], C = x[q.mp * ncols + c], D = x[q.mm * ncols + c];
      const float smn = q.sm * q.sn;
      r[q.pp * ncols + c] = 0.5f * (A.x + q.sn * B.x + q.sm * C.x + smn * D.x);    // cos cos
      r[q.pm * ncols + c] = 0.5f * (-A.y + q.sn * B.y - q.sm * C.y + smn * D.y);   // cos sin
      r[q.mp * ncols + c] = 0.5f * (A.y + q.sn * B.y - q.sm * C.y - smn * D.y);    // sin cos
      r[q.mm * ncols + c] = 0.5f * (A.x - q.sn * B.x - q.sm * C.x + smn * D.x);    // sin sin
    }
  }
}

__global__ __launch_bounds__(256) void to_complex_kernel(const float* __restrict__ r, float2* __restrict__ x, int nl, long ncols) {
  const Quad q = decode_quad(blockIdx.x, nl);
  for (long c = (long)blockIdx.y * 256 + threadIdx.x; c < ncols; c += 256L * gridDim.y) {
    const float cc = r[q.pp * ncols + c];
    if (q.m == 0 && q.n == 0) {
      x[q.pp * ncols + c] = make_float2(cc, 0.f);
    } else if (q.m == 0) {
      const float cs = r[q.pm * ncols + c];
      x[q.pp * ncols + c] = make_float2(RSQRT2 * cc, -RSQRT2 * cs);
      x[q.pm * ncols + c] = make_float2(q.sn * RSQRT2 * cc, q.sn * RSQRT2 * cs);
    } else if (q.n == 0) {
      const float sc = r[q.mp * ncols + c];
      x[q.pp * ncols + c] = make_float2(RSQRT2 * cc, RSQRT2 * sc);
      x[q.mp * ncols + c] = make_float2(q.sm * RSQRT2 * cc, -q.sm * RSQRT2 * sc);
    } else {
      const float cs = r[q.pm * ncols + c], sc = r[q.mp * ncols + c], ss = r[q.mm * ncols + c];
      const float smn = q.sm * q.sn;
      const float ar = 0.5f * (cc + ss), ai = 0.5f * (sc - cs);
      const float br = 0.5f * (cc - ss), bi = 0.5f * (cs + sc);
      x[q.pp * ncols + c] = make_float2(ar, ai);
      x[q.pm * ncols + c] = make_float2(q.sn * br, q.sn * bi);
      x[q.mp * ncols + c] = make_float2(q.sm * br, -q.sm * bi);
      x[q.mm * ncols + c] = make_float2(smn * ar, -smn * ai);
    }
  }
}

int check(const void* a, const void* b, int nl, long ncols) {
  if (!a || !b || nl < 1 || nl > 512 || ncols < 1 || ncols >= (1L << 31)) return S2CNN_EINVAL;
  return S2CNN_OK;
}

dim3 grid_for(int nl, long ncols) {
  const long quads = (long)nl * (nl + 1) * (2 * nl + 1) / 6;
  long gy = (ncols + 255) / 256;
  if (gy > 64) gy = 64;
  return dim3((unsigned)quads, (unsigned)gy);
}

}  // namespace

extern "C" int s2cnn_so3_spectrum_to_real(const float* x, float* r, int nl, long ncols, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(x, r, nl, ncols)) return rc;
  if (!s2cnn::aligned8(x)) return S2CNN_EALIGN;
  hipLaunchKernelGGL(to_real_kernel, grid_for(nl, ncols), dim3(256), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<const float2*>(x), r, nl, ncols);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_so3_spectrum_to_complex(const float* r, float* x, int nl, long ncols, void* stream) {
  s2cnn::clear_stale_error();
  if (int rc = check(r, x, nl, ncols)) return rc;
  if (!s2cnn::aligned8(x)) return S2CNN_EALIGN;
  hipLaunchKernelGGL(to_complex_kernel, grid_for(nl, ncols), dim3(256), 0, static_cast<hipStream_t>(stream),
                     r, reinterpret_cast<float2*>(x), nl, ncols);
  return s2cnn::launch_status();
}
