// SO(3) Fourier analysis and synthesis on the SOFT grid.
//
// Analysis   out[l,m,n,z]  = sum_beta T[beta,lmn] * X[z,beta,m,n],
//            X[z,beta,m,n] = sum_{alpha,gamma} x[z,beta,alpha,gamma] e^{-i(m alpha + n gamma)}
// Synthesis  y[z,beta,alpha,gamma] = sum_{m,n} e^{+i(m alpha + n gamma)} S[z,beta,m,n],
//            S[z,beta,m,n] = sum_l T[beta,lmn] * xhat[l,m,n,z]
//
// Only frequencies |m|,|n| < nb = min(b_in, b_out) are ever consumed, so the (alpha,gamma)
// transform is a DFT pruned to those bins, done per (z,beta) plane inside LDS, and the
// intermediate X / S lives in a workspace laid out [z][beta][m][n] (n fastest).
//
// Real signals use the half plane n >= 0:
//   analysis : the other half follows from X[-m,-n] = conj X[m,n] and
//              T[l,-m,-n] = (-1)^(m-n) T[l,m,n]  =>  out[l,-m,-n] = (-1)^(m-n) conj out[l,m,n];
//   synthesis: Re sum_{m,n} e^{i.}S[m,n] = sum_{m,n} e^{i.}G[m,n] with the Hermitian
//              G[m,n] = (S[m,n] + conj S[-m,-n])/2, and by the same table symmetry
//              G = sum_l T[l,m,n] (xhat[l,m,n] + (-1)^(m-n) conj xhat[l,-m,-n])/2,
//              so the spectrum is symmetrised on load and no symmetry of xhat is assumed.
#include "common.h"
#include "so3_plane_fft64.h"
#include "so3_wigner_tiled.h"
#include "so3_fused64.h"
#include "so3_fused4r.h"
#include "so3_plane_dft_real.h"
#include <mutex>

namespace {

__device__ inline float2 cmul(float2 a, float2 b) { return make_float2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x); }
__device__ inline float2 cmul_conj(float2 a, float2 b) { return make_float2(a.x * b.x + a.y * b.y, a.y * b.x - a.x * b.y); }  // a*conj(b)

__device__ inline int lmn_index(int l, int m, int n) { return l * (4 * l * l - 1) / 3 + (l + m) * (2 * l + 1) + (l + n); }

// w[k] = e^{-2 pi i k / n2}
__device__ inline void fill_twiddles(float2* w, int n2) {
  for (int k = threadIdx.x; k < n2; k += blockDim.x) {
    float s, c;
    sincospif(2.0f * (float)k / (float)n2, &s, &c);
    w[k] = make_float2(c, -s);
  }
}

// ---------------------------------------------------------------------------------------
// analysis stage 1: one workgroup per (z,beta) plane
//   x plane [n2][n2] (real or complex) -> X[mi][ni], mi = m + nb-1, ni = n (real) or n + nb-1
// LDS: twiddles n2 | plane n2*n2 (float or float2) | Y n2*NW
// ---------------------------------------------------------------------------------------
template <bool CPLX>
__global__ __launch_bounds__(256) void so3_plane_dft_fwd(const float* __restrict__ x, float2* __restrict__ X,
                                                         int n2, int nb, int ztile, const float* __restrict__ mask) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int MW = 2 * nb - 1;
  const int NW = CPLX ? MW : nb;
  float2* w = reinterpret_cast<float2*>(smem);
  float* plane = smem + 2 * n2;
  float2* Y = reinterpret_cast<float2*>(plane + (CPLX ? 2 : 1) * n2 * n2);
  const size_t pl = blockIdx.x;

  fill_twiddles(w, n2);
  const int nin = (CPLX ? 2 : 1) * n2 * n2;
  const float* src = x + pl * nin;
  if (mask) {     // samples where the mask is not positive count as zero
    const float* msk = mask + pl * nin;
    for (int i = threadIdx.x; i < nin; i += blockDim.x) plane[i] = s2cnn::relu_pass(src[i], msk[i]);
  } else {
    for (int i = threadIdx.x; i < nin; i += blockDim.x) plane[i] = src[i];
  }
  __syncthreads();

  // Y[alpha][ni] = sum_gamma x[alpha][gamma] w^(n gamma)
  for (int o = threadIdx.x; o < n2 * NW; o += blockDim.x) {
    const int a = o / NW, ni = o - a * NW;
    const int n = CPLX ? ni - (nb - 1) : ni;
    const int step = ((n % n2) + n2) % n2;
    int tw = 0;
    float2 acc = make_float2(0.f, 0.f);
    for (int g = 0; g < n2; ++g) {
      const float2 t = w[tw];
      if (CPLX) {
        const float2 v = reinterpret_cast<const float2*>(plane)[a * n2 + g];
        const float2 pr = cmul(v, t);
        acc.x += pr.x; acc.y += pr.y;
      } else {
        const float v = plane[a * n2 + g];
        acc.x += v * t.x; acc.y += v * t.y;
      }
      tw += step; if (tw >= n2) tw -= n2;
    }
    Y[o] = acc;
  }
  __syncthreads();

  // X[mi][ni] = sum_alpha Y[alpha][ni] w^(m alpha)
  // ztile = 0: X is [plane][mi][ni];  ztile = Z > 0: [z / Z][mi][beta][z % Z][ni] (plane = z * n2 + beta)
  float2* dst = X + pl * (size_t)(MW * NW);
  size_t mstride = NW;
  if (ztile > 0) {
    const size_t z = pl / n2, beta = pl % n2;
    dst = X + ((z / ztile) * MW * n2 + beta) * ztile * NW + (z % ztile) * NW;
    mstride = (size_t)n2 * ztile * NW;
  }
  for (int o = threadIdx.x; o < MW * NW; o += blockDim.x) {
    const int mi = o / NW, ni = o - mi * NW;
    const int m = mi - (nb - 1);
    const int step = ((m % n2) + n2) % n2;
    int tw = 0;
    float2 acc = make_float2(0.f, 0.f);
    for (int a = 0; a < n2; ++a) {
      const float2 pr = cmul(Y[a * NW + ni], w[tw]);
      acc.x += pr.x; acc.y += pr.y;
      tw += step; if (tw >= n2) tw -= n2;
    }
    dst[mi * mstride + ni] = acc;
  }
}

// ---------------------------------------------------------------------------------------
// analysis stage 2: contraction over beta with the Wigner table.
// block (16 ni, 16 z); grid (ceil(NW/16), MW, ceil(nbatch/16))
// ---------------------------------------------------------------------------------------
constexpr int LG = 8;  // degrees accumulated per pass over beta

template <bool CPLX>
__global__ __launch_bounds__(256) void so3_wigner_fwd(const float2* __restrict__ X, const float* __restrict__ T,
                                                      float2* __restrict__ out, int n2, int nb, int b_out,
                                                      long nbatch) {
  const int MW = 2 * nb - 1;
  const int NW = CPLX ? MW : nb;
  const int ni = blockIdx.x * 16 + threadIdx.x;
  const int mi = blockIdx.y;
  const long z = (long)blockIdx.z * 16 + threadIdx.y;
  if (ni >= NW || z >= nbatch) return;
  const int m = mi - (nb - 1);
  const int n = CPLX ? ni - (nb - 1) : ni;
  if (!CPLX && n == 0 && m < 0) return;  // written as the mirror of (-m, 0)
  const int lmin = max(abs(m), abs(n));
  const long nspec = (long)b_out * (4L * b_out * b_out - 1) / 3;
  const float2* xp = X + ((size_t)z * n2 * MW + mi) * NW + ni;  // + beta * MW*NW
  const size_t xstride = (size_t)MW * NW;
  const float sgn = ((m - n) & 1) ? -1.f : 1.f;

  for (int l0 = lmin; l0 < b_out; l0 += LG) {
    float2 acc[LG];
    int idx[LG];
#pragma unroll
    for (int u = 0; u < LG; ++u) {
      acc[u] = make_float2(0.f, 0.f);
      const int l = min(l0 + u, b_out - 1);
      idx[u] = lmn_index(l, m, n);
    }
    for (int bt = 0; bt < n2; ++bt) {
      const float2 v = xp[bt * xstride];
      const float* Tr = T + (size_t)bt * nspec;
#pragma unroll
      for (int u = 0; u < LG; ++u) {
        const float t = Tr[idx[u]];
        acc[u].x += t * v.x; acc[u].y += t * v.y;
      }
    }
#pragma unroll
    for (int u = 0; u < LG; ++u) {
      const int l = l0 + u;
      if (l < b_out) {
        out[(size_t)idx[u] * nbatch + z] = acc[u];
        if (!CPLX && (n > 0 || m > 0))
          out[(size_t)lmn_index(l, -m, -n) * nbatch + z] = make_float2(sgn * acc[u].x, -sgn * acc[u].y);
      }
    }
  }
}

__global__ void fill_zero(float* p, size_t n) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0.f;
}

// ---------------------------------------------------------------------------------------
// synthesis stage 1: S[z][beta][mi][ni] = sum_l T[beta,lmn] xs[lmn][z]
// block (16 ni, 16 z); grid (ceil(NW/16), MW, ceil(nbatch/16))
// ---------------------------------------------------------------------------------------
constexpr int BG = 8;  // betas accumulated per pass over l

template <bool CPLX>
__global__ __launch_bounds__(256) void so3_wigner_inv(const float2* __restrict__ xh, const float* __restrict__ T,
                                                      float2* __restrict__ S, int n2, int nb, int b_spec,
                                                      long nbatch) {
  const int MW = 2 * nb - 1;
  const int NW = CPLX ? MW : nb;
  const int ni = blockIdx.x * 16 + threadIdx.x;
  const int mi = blockIdx.y;
  const long z = (long)blockIdx.z * 16 + threadIdx.y;
  if (ni >= NW || z >= nbatch) return;
  const int m = mi - (nb - 1);
  const int n = CPLX ? ni - (nb - 1) : ni;
  const int lmin = max(abs(m), abs(n));
  const long nspec = (long)b_spec * (4L * b_spec * b_spec - 1) / 3;
  float2* sp = S + ((size_t)z * n2 * MW + mi) * NW + ni;
  const size_t sstride = (size_t)MW * NW;
  const float sgn = ((m - n) & 1) ? -0.5f : 0.5f;

  for (int b0 = 0; b0 < n2; b0 += BG) {
    float2 acc[BG];
#pragma unroll
    for (int u = 0; u < BG; ++u) acc[u] = make_float2(0.f, 0.f);
    for (int l = lmin; l < nb; ++l) {
      const int i1 = lmn_index(l, m, n);
      float2 v = xh[(size_t)i1 * nbatch + z];
      if (!CPLX) {
        const float2 u2 = xh[(size_t)lmn_index(l, -m, -n) * nbatch + z];
        v = make_float2(0.5f * v.x + sgn * u2.x, 0.5f * v.y - sgn * u2.y);
      }
#pragma unroll
      for (int u = 0; u < BG; ++u) {
        const int bt = min(b0 + u, n2 - 1);
        const float t = T[(size_t)bt * nspec + i1];
        acc[u].x += t * v.x; acc[u].y += t * v.y;
      }
    }
#pragma unroll
    for (int u = 0; u < BG; ++u)
      if (b0 + u < n2) sp[(size_t)(b0 + u) * sstride] = acc[u];
  }
}

// ---------------------------------------------------------------------------------------
// synthesis stage 2: one workgroup per (z,beta) plane, S[mi][ni] -> y[alpha][gamma]
// LDS: twiddles n2 | S MW*NW | U n2*NW
// ---------------------------------------------------------------------------------------
template <bool CPLX>
__global__ __launch_bounds__(256) void so3_plane_dft_inv(const float2* __restrict__ S, float* __restrict__ y,
                                                         int n2, int nb) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int MW = 2 * nb - 1;
  const int NW = CPLX ? MW : nb;
  float2* w = reinterpret_cast<float2*>(smem);
  float2* Sp = w + n2;
  float2* U = Sp + MW * NW;
  const size_t pl = blockIdx.x;

  fill_twiddles(w, n2);
  const float2* src = S + pl * (size_t)(MW * NW);
  for (int i = threadIdx.x; i < MW * NW; i += blockDim.x) Sp[i] = src[i];
  __syncthreads();

  // U[alpha][ni] = sum_mi S[mi][ni] conj(w)^(m alpha)
  for (int o = threadIdx.x; o < n2 * NW; o += blockDim.x) {
    const int a = o / NW, ni = o - a * NW;
    const int step = a;                                  // m -> m+1 advances the phase by alpha
    int tw = (int)(((long)(-(nb - 1)) * a) % n2); if (tw < 0) tw += n2;
    float2 acc = make_float2(0.f, 0.f);
    for (int mi = 0; mi < MW; ++mi) {
      const float2 pr = cmul_conj(Sp[mi * NW + ni], w[tw]);
      acc.x += pr.x; acc.y += pr.y;
      tw += step; if (tw >= n2) tw -= n2;
    }
    U[o] = acc;
  }
  __syncthreads();

  if (CPLX) {
    float2* dst = reinterpret_cast<float2*>(y) + pl * (size_t)(n2 * n2);
    for (int o = threadIdx.x; o < n2 * n2; o += blockDim.x) {
      const int a = o / n2, g = o - a * n2;
      int tw = (int)(((long)(-(nb - 1)) * g) % n2); if (tw < 0) tw += n2;
      float2 acc = make_float2(0.f, 0.f);
      for (int ni = 0; ni < NW; ++ni) {
        const float2 pr = cmul_conj(U[a * NW + ni], w[tw]);
        acc.x += pr.x; acc.y += pr.y;
        tw += g; if (tw >= n2) tw -= n2;
      }
      dst[o] = acc;
    }
  } else {
    float* dst = y + pl * (size_t)(n2 * n2);
    for (int o = threadIdx.x; o < n2 * n2; o += blockDim.x) {
      const int a = o / n2, g = o - a * n2;
      float acc = U[a * NW].x;
      int tw = g;
      float part = 0.f;
      for (int ni = 1; ni < NW; ++ni) {
        const float2 u = U[a * NW + ni];
        const float2 t = w[tw];                          // conj(t) = e^{+i n gamma}
        part += u.x * t.x + u.y * t.y;                  // Re(u * conj(t))
        tw += g; if (tw >= n2) tw -= n2;
      }
      dst[o] = acc + 2.f * part;
    }
  }
}

// y[z, :] += bias[z % nfeature] for volumes of `vol` samples (bias may be NULL), then max(y, 0) if relu; only behind
// the plane kernels that have no epilogue of their own
__global__ void add_bias_kernel(float* __restrict__ y, const float* __restrict__ bias, size_t vol, int nfeature, size_t total, int relu) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    const float v = y[i] + (bias ? bias[(i / vol) % nfeature] : 0.f);
    y[i] = relu ? s2cnn::relu_f(v) : v;
  }
}

// Real signals on the 64^3, 44^3, 32^3 and 20^3 grids go through the per-volume kernels of so3_fused64.h / so3_fused4r.h
// (the planes never leave the CU).
using fused4r::Grid20;
using fused4r::Grid32;
using fused4r::Grid44;
enum FusedKind { FUSED_NONE = 0, FUSED_64, FUSED_44, FUSED_32, FUSED_20 };
int fused_bandwidth(FusedKind k) { return k == FUSED_64 ? 32 : k == FUSED_44 ? 22 : k == FUSED_32 ? 16 : 10; }
FusedKind fused_kind(int b_grid, int b_spec, int cplx, bool synthesis) {
  if (cplx) return FUSED_NONE;
  const FusedKind k = b_grid == 32 ? FUSED_64 : b_grid == 22 ? FUSED_44 : b_grid == 16 ? FUSED_32 : b_grid == 10 ? FUSED_20 : FUSED_NONE;
  return synthesis || b_spec <= b_grid ? k : FUSED_NONE;
}
bool fused_path(int b_grid, int b_spec, int cplx, bool synthesis) { return fused_kind(b_grid, b_spec, cplx, synthesis) != FUSED_NONE; }
// f.template operator()<G>() for the grid G of a kind other than FUSED_64
template <class F>
auto with_grid(FusedKind k, F f) {
  if (k == FUSED_44) return f(Grid44{});
  if (k == FUSED_32) return f(Grid32{});
  return f(Grid20{});
}
size_t fused_scratch_bytes(FusedKind k, long nbatch) {
  if (k == FUSED_64) return fused64::scratch_bytes(nbatch);
  return with_grid(k, [&](auto g) { return decltype(g)::scratch_bytes(nbatch); });
}
size_t fused_packed_floats(FusedKind k) {
  if (k == FUSED_64) return fused64::PACKED_FLOATS;
  return with_grid(k, [](auto g) { return (size_t) decltype(g)::PACKED_FLOATS; });
}
// table [2 b_grid][nspec(b_spec)] -> the packed table of the per-volume kernels, degrees below nl
void fused_pack_table(FusedKind k, hipStream_t st, const float* table, float* packed, int b_spec, int nl) {
  const long stride = s2cnn::so3_nspec(b_spec);
  if (k == FUSED_64) { hipLaunchKernelGGL(fused64::pack_table, dim3(1024), dim3(256), 0, st, table, packed, stride, nl); return; }
  with_grid(k, [&](auto g) {
    using G = decltype(g);
    hipLaunchKernelGGL(fused4r::pack_table<G>, dim3((unsigned)((G::PACKED_FLOATS + 1023) / 1024)), dim3(256), 0, st, table, packed, stride, nl);
    return 0;
  });
}
// per-volume kernel + the pass between its records and the spectral rows, for the grids of so3_fused4r.h
template <class G>
void fused4r_analysis(const s2cnn::Input& in, const float* Tf, float4* rec, float* out, int b_out, long nbatch, bool real_basis, hipStream_t st) {
  const unsigned tiles_r = (unsigned)((nbatch + fused64::ZR - 1) / fused64::ZR), tiles_c = (unsigned)((nbatch + fused64::ZT - 1) / fused64::ZT);
  const int rounds = G::active_rounds(b_out), nparts = G::parts(nbatch);
  fused4r::launch_analysis<G>(b_out, st, in, Tf, rec, nbatch, nparts);
  if (real_basis)
    hipLaunchKernelGGL(fused64::spectrum_scatter_real<G>, dim3(tiles_r, rounds * (G::THREADS / fused64::IT_TILE_R)), dim3(256), 0, st, rec, out, b_out, nbatch, nparts);
  else
    hipLaunchKernelGGL(fused64::spectrum_scatter<G>, dim3(tiles_c, rounds * (G::THREADS / fused64::IT_TILE)), dim3(256), 0, st, rec,
                       reinterpret_cast<float2*>(out), b_out, nbatch, nparts);
}
template <class G>
void fused4r_synthesis(const float* xhat, const float* Tf, float4* rec, float* out, int nl, long nbatch, bool real_basis, const float* bias,
                       int nfeature, int relu, hipStream_t st, float2* mom, const float* yref, const float* params) {
  const unsigned tiles_r = (unsigned)((nbatch + fused64::ZR - 1) / fused64::ZR), tiles_c = (unsigned)((nbatch + fused64::ZT - 1) / fused64::ZT);
  const int rounds = G::active_rounds(nl);
  if (real_basis)
    hipLaunchKernelGGL(fused64::spectrum_gather_real<G>, dim3(tiles_r, rounds * (G::THREADS / fused64::IT_TILE_R)), dim3(256), 0, st, xhat, rec, nl, nbatch);
  else
    hipLaunchKernelGGL(fused64::spectrum_gather<G>, dim3(tiles_c, rounds * (G::THREADS / fused64::IT_TILE)), dim3(256), 0, st,
                       reinterpret_cast<const float2*>(xhat), rec, nl, nbatch);
  fused4r::launch_synthesis<G>(nl, st, rec, Tf, out, nbatch, bias, nfeature, relu, G::parts(nbatch), mom, yref, params);
}

// Bytes of the intermediate; batch items padded to the z tile of the tiled Wigner kernels.
size_t ws_bytes(int b_grid, int b_spec, long nbatch, int cplx, bool synthesis) {
  if (b_grid < 1 || b_spec < 1 || nbatch < 1) return 0;
  if (const FusedKind k = fused_kind(b_grid, b_spec, cplx, synthesis)) return fused_scratch_bytes(k, nbatch);
  const long nb = b_grid < b_spec ? b_grid : b_spec;
  const long MW = 2 * nb - 1, NW = cplx ? MW : nb;
  const long zpad = (nbatch + wigner_tiled::ZT - 1) / wigner_tiled::ZT * wigner_tiled::ZT;
  return (size_t)zpad * (2 * b_grid) * MW * NW * sizeof(float2);
}

bool sizes_ok(int b_grid, int b_spec, long nbatch) {
  return b_grid >= 1 && b_spec >= 1 && nbatch >= 1 && b_grid <= 512 && b_spec <= 512 &&
         nbatch * 2L * b_grid < (1L << 31) && (nbatch + 15) / 16 <= 65535;
}

// Bytes of the packed table of the tiled fast path; 0 when that path does not apply.
size_t packed_bytes(int b_grid, int b_spec, int cplx, bool synthesis) {
  if (const FusedKind k = fused_kind(b_grid, b_spec, cplx, synthesis)) return fused_packed_floats(k) * sizeof(float);
  const int nb = b_grid < b_spec ? b_grid : b_spec;
  if (cplx || nb > 64) return 0;
  if (synthesis) return 2 * b_grid <= 128 ? wigner_tiled::packed_floats_synthesis(2 * b_grid, nb) * sizeof(float) : 0;
  return b_spec <= 64 ? wigner_tiled::packed_floats_analysis(2 * b_grid, nb, b_spec) * sizeof(float) : 0;
}

size_t round256(size_t n) { return (n + 255) & ~(size_t)255; }

// A synthesis of real signals that reads its spectrum in the real basis: the per-volume kernels of the 64^3 grid and the
// tiled Wigner stage of the other grids.
bool real_basis_synthesis(int b_in, int b_out) {
  return b_in >= 1 && b_out >= 1 && (fused_path(b_out, b_in, 0, true) || packed_bytes(b_out, b_in, 0, true) != 0);
}
// The same for an analysis that writes the real basis: the tiled Wigner stage does where one part covers the spectrum.
bool real_basis_analysis(int b_in, int b_out) {
  return b_in >= 1 && b_out >= 1 && (fused_path(b_in, b_out, 0, false) || (packed_bytes(b_in, b_out, 0, false) != 0 && b_out <= 32));
}

// Real signals on the 64^3 or 32^3 grid: per-volume kernel + the pass between its records and the spectral rows.
// real_basis: the spectrum is stored in the real basis (one float per entry) instead of complex pairs.
int fused_analysis(FusedKind kind, const s2cnn::Input& in, const float* table, const float* packed_table, float* out,
                   void* workspace, size_t workspace_bytes, int b_out, long nbatch, bool real_basis, hipStream_t st) {
  if (kind == FUSED_64 && (!s2cnn::aligned16(in.x) || !s2cnn::aligned16(in.w))) return S2CNN_EALIGN;     // the other grids: any float pointer
  const size_t need = round256(fused_scratch_bytes(kind, nbatch)) + fused_packed_floats(kind) * sizeof(float);
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return S2CNN_EWORKSPACE;
  float4* rec = static_cast<float4*>(workspace);
  const float* Tf = packed_table;
  if (!Tf) {  // pack behind the records on every call
    float* dst = reinterpret_cast<float*>(static_cast<char*>(workspace) + round256(fused_scratch_bytes(kind, nbatch)));
    fused_pack_table(kind, st, table, dst, b_out, b_out);
    Tf = dst;
  }
  const unsigned tiles_r = (unsigned)((nbatch + fused64::ZR - 1) / fused64::ZR), tiles_c = (unsigned)((nbatch + fused64::ZT - 1) / fused64::ZT);
  float2* outc = reinterpret_cast<float2*>(out);
  if (kind == FUSED_64) {
    const int rounds = fused64::active_rounds(b_out), nparts = fused64::parts(nbatch);
    fused64::launch_analysis(b_out, st, in, Tf, rec, nbatch, nparts);
    if (real_basis) hipLaunchKernelGGL(fused64::spectrum_scatter_real<>, dim3(tiles_r, rounds * (fused64::THREADS / fused64::IT_TILE_R)), dim3(256), 0, st, rec, out, b_out, nbatch, nparts);
    else hipLaunchKernelGGL(fused64::spectrum_scatter<>, dim3(tiles_c, rounds * (fused64::THREADS / fused64::IT_TILE)), dim3(256), 0, st, rec, outc, b_out, nbatch, nparts);
  } else {
    with_grid(kind, [&](auto g) { fused4r_analysis<decltype(g)>(in, Tf, rec, out, b_out, nbatch, real_basis, st); return 0; });
  }
  return s2cnn::launch_status();
}

int fused_synthesis(FusedKind kind, const float* xhat, const float* table, const float* packed_table, float* out, void* workspace,
                    size_t workspace_bytes, int b_in, long nbatch, bool real_basis, const float* bias, int nfeature, int relu,
                    unsigned long long* bits, hipStream_t st, float* moments = nullptr, const float* yref = nullptr,
                    const float* params = nullptr) {
  if (kind == FUSED_64 && (!s2cnn::aligned16(out) || !s2cnn::aligned16(bits) || !s2cnn::aligned16(yref))) return S2CNN_EALIGN;
  if (!s2cnn::aligned8(moments)) return S2CNN_EALIGN;
  if (bits && kind != FUSED_64) return S2CNN_EINVAL;
  const int b_grid = fused_bandwidth(kind);
  const int nl = b_in < b_grid ? b_in : b_grid;
  const size_t need = round256(fused_scratch_bytes(kind, nbatch)) + fused_packed_floats(kind) * sizeof(float);
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return S2CNN_EWORKSPACE;
  float4* rec = static_cast<float4*>(workspace);
  const float* Tf = packed_table;
  if (!Tf) {
    float* dst = reinterpret_cast<float*>(static_cast<char*>(workspace) + round256(fused_scratch_bytes(kind, nbatch)));
    fused_pack_table(kind, st, table, dst, b_in, nl);
    Tf = dst;
  }
  const unsigned tiles_r = (unsigned)((nbatch + fused64::ZR - 1) / fused64::ZR), tiles_c = (unsigned)((nbatch + fused64::ZT - 1) / fused64::ZT);
  const float2* xc = reinterpret_cast<const float2*>(xhat);
  float2* mom = reinterpret_cast<float2*>(moments);
  if (kind == FUSED_64) {
    const int rounds = fused64::active_rounds(nl);
    if (real_basis) hipLaunchKernelGGL(fused64::spectrum_gather_real<>, dim3(tiles_r, rounds * (fused64::THREADS / fused64::IT_TILE_R)), dim3(256), 0, st, xhat, rec, nl, nbatch);
    else hipLaunchKernelGGL(fused64::spectrum_gather<>, dim3(tiles_c, rounds * (fused64::THREADS / fused64::IT_TILE)), dim3(256), 0, st, xc, rec, nl, nbatch);
    fused64::launch_synthesis(nl, st, rec, Tf, out, nbatch, bias, nfeature, relu, bits, mom, yref, params, fused64::parts(nbatch));
  } else {
    with_grid(kind, [&](auto g) {
      fused4r_synthesis<decltype(g)>(xhat, Tf, rec, out, nl, nbatch, real_basis, bias, nfeature, relu, st, mom, yref, params);
      return 0;
    });
  }
  return s2cnn::launch_status();
}

}  // namespace

extern "C" int s2cnn_so3_real_basis_transform_available(int b_in, int b_out, int synthesis) {
  if (b_in < 1 || b_out < 1) return 0;
  return synthesis ? real_basis_synthesis(b_in, b_out) : real_basis_analysis(b_in, b_out);
}

extern "C" size_t s2cnn_so3_packed_table_bytes(int b_in, int b_out, int synthesis) {
  if (b_in < 1 || b_out < 1) return 0;
  return synthesis ? packed_bytes(b_out, b_in, 0, true) : packed_bytes(b_in, b_out, 0, false);
}

extern "C" int s2cnn_so3_pack_table(const float* table, float* packed, int b_in, int b_out, int synthesis, void* stream) {
  s2cnn::clear_stale_error();
  if (!table || !packed || b_in < 1 || b_out < 1 || b_in > 512 || b_out > 512) return S2CNN_EINVAL;
  if (s2cnn_so3_packed_table_bytes(b_in, b_out, synthesis) == 0) return S2CNN_EINVAL;
  if (!s2cnn::aligned16(packed)) return S2CNN_EALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int nb = b_in < b_out ? b_in : b_out;
  if (const FusedKind k = fused_kind(synthesis ? b_out : b_in, synthesis ? b_in : b_out, 0, synthesis != 0)) {
    const int b_spec = synthesis ? b_in : b_out, b_grid = synthesis ? b_out : b_in;
    fused_pack_table(k, st, table, packed, b_spec, b_spec < b_grid ? b_spec : b_grid);
  } else if (synthesis) {
    hipLaunchKernelGGL(wigner_tiled::pack_table_synthesis, dim3(2048), dim3(256), 0, st, table, packed, 2 * b_out, nb, b_in);
  } else {
    hipLaunchKernelGGL(wigner_tiled::pack_table_analysis, dim3(2048), dim3(256), 0, st, table, packed, 2 * b_in, nb, b_out);
  }
  return s2cnn::launch_status();
}

extern "C" size_t s2cnn_so3_analysis_workspace(int b_in, int b_out, long nbatch, int complex_in) {
  if (!sizes_ok(b_in, b_out, nbatch)) return 0;
  return round256(ws_bytes(b_in, b_out, nbatch, complex_in, false)) + packed_bytes(b_in, b_out, complex_in, false);
}

extern "C" size_t s2cnn_so3_synthesis_workspace(int b_in, int b_out, long nbatch, int complex_out) {
  if (!sizes_ok(b_out, b_in, nbatch)) return 0;
  return round256(ws_bytes(b_out, b_in, nbatch, complex_out, true)) + packed_bytes(b_out, b_in, complex_out, true);
}

namespace {
// Where the loads of an analysis can do more than select samples (s2cnn::PRO_AFFINE_RELU, PRO_BN_RELU_GRAD): the per-volume
// kernels of the 64^3 grid and the folded plane kernel of the other grids that fit the LDS.
bool prologue_path(int b_in, int b_out) {
  if (!sizes_ok(b_in, b_out, 1)) return false;
  if (fused_path(b_in, b_out, 0, false)) return true;
  return 2 * b_in != 64 && plane_real::plan_fwd(2 * b_in, b_in < b_out ? b_in : b_out, 2 * b_in).pl > 0;
}

// in: the signal and what its loads do to it (real signals only for anything but PRO_NONE)
int analysis_impl(const s2cnn::Input& in, const float* table, const float* packed_table, float* out,
                  void* workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch, int complex_in, void* stream,
                  bool real_basis = false) {
  const float* x = in.x;
  if (real_basis && (complex_in || !real_basis_analysis(b_in, b_out))) return S2CNN_EINVAL;
  const float* mask = in.second_tensor() ? in.w : nullptr;
  if (!x || !table || !out || !sizes_ok(b_in, b_out, nbatch) || (in.kind != s2cnn::PRO_NONE && complex_in)) return S2CNN_EINVAL;
  if (in.kind != s2cnn::PRO_NONE && in.kind != s2cnn::PRO_AFFINE_RELU && !in.w) return S2CNN_EINVAL;
  if (in.kind == s2cnn::PRO_BITS && fused_kind(b_in, b_out, complex_in, false) != FUSED_64) return S2CNN_EINVAL;
  if (in.kind >= s2cnn::PRO_AFFINE_RELU && (!in.params || in.nfeature < 1 || nbatch % in.nfeature != 0 || !prologue_path(b_in, b_out)))
    return S2CNN_EINVAL;
  if ((!real_basis && !s2cnn::aligned8(out)) || (complex_in && !s2cnn::aligned8(x))) return S2CNN_EALIGN;
  if (packed_table && !s2cnn::aligned16(packed_table)) return S2CNN_EALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (const FusedKind k = fused_kind(b_in, b_out, complex_in, false))
    return fused_analysis(k, in, table, packed_table, out, workspace, workspace_bytes, b_out, nbatch, real_basis, st);
  const size_t need = s2cnn_so3_analysis_workspace(b_in, b_out, nbatch, complex_in);
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return S2CNN_EWORKSPACE;
  const int n2 = 2 * b_in, nb = b_in < b_out ? b_in : b_out;
  const int MW = 2 * nb - 1, NW = complex_in ? MW : nb;
  float2* X = static_cast<float2*>(workspace);
  const size_t lds = sizeof(float) * (2 * n2 + (complex_in ? 2 : 1) * n2 * n2 + 2 * n2 * NW);
  const unsigned planes = (unsigned)(nbatch * n2);
  const bool tiled = packed_bytes(b_in, b_out, complex_in, false) != 0;
  const int ztile = !tiled ? 0 : real_basis ? wigner_tiled::ZH : wigner_tiled::ZT;   // batch items per tile of the intermediate
  const bool x16 = s2cnn::aligned16(x) && s2cnn::aligned16(mask);
  const plane_real::Plan plan = complex_in ? plane_real::Plan{0, 0, 0, 0} : plane_real::plan_fwd(n2, nb, planes);
  if (lds > 160 * 1024 && plan.pl == 0) return S2CNN_EINVAL;
  if (complex_in) {
    if (lds > 48 * 1024) (void)hipFuncSetAttribute((const void*)so3_plane_dft_fwd<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(so3_plane_dft_fwd<true>, dim3(planes), dim3(256), lds, st, x, X, n2, nb, 0, nullptr);
  } else if (n2 == 64 && x16) {
    const long npairs = nbatch * 32;
    hipLaunchKernelGGL(fft64::plane_fft64_fwd, dim3((unsigned)(npairs < 2048 ? npairs : 2048)), dim3(fft64::THREADS), 0, st, x, X, npairs, nb,
                       ztile, mask);
  } else if (plan.pl > 0) {
    if (plan.lds > 48 * 1024) (void)hipFuncSetAttribute((const void*)plane_real::plane_dft_fwd, hipFuncAttributeMaxDynamicSharedMemorySize, (int)plan.lds);
    hipLaunchKernelGGL(plane_real::plane_dft_fwd, dim3((planes + plan.pl - 1) / plan.pl), dim3(plan.nt), plan.lds, st, x, X, n2, nb,
                       ztile, (long)planes, plan.pl, plan.alias, mask, in.kind, in.params, in.nfeature);
  } else {
    if (lds > 48 * 1024) (void)hipFuncSetAttribute((const void*)so3_plane_dft_fwd<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(so3_plane_dft_fwd<false>, dim3(planes), dim3(256), lds, st, x, X, n2, nb, ztile, mask);
  }
  int rc = s2cnn::launch_status();
  if (rc) return rc;
  if (b_out > b_in) {  // entries with |m| or |n| >= b_in are never touched by stage 2
    const size_t nfl = (size_t)s2cnn::so3_nspec(b_out) * nbatch * (real_basis ? 1 : 2);
    hipLaunchKernelGGL(fill_zero, dim3(1024), dim3(256), 0, st, out, nfl);
  }
  if (tiled) {
    const float* Tp = packed_table;
    if (!Tp) {  // pack on the fly behind the intermediate
      float* dst = reinterpret_cast<float*>(static_cast<char*>(workspace) + round256(ws_bytes(b_in, b_out, nbatch, complex_in, false)));
      hipLaunchKernelGGL(wigner_tiled::pack_table_analysis, dim3(2048), dim3(256), 0, st, table, dst, n2, nb, b_out);
      Tp = dst;
    }
    const int parts = wigner_tiled::parts_analysis(nb, b_out);
    if (real_basis) {
      const dim3 gh(wigner_tiled::grid_size_half(nb, nbatch), nb > wigner_tiled::NC ? 2 : 1);
      if (wigner_tiled::small_analysis(nb, b_out))
        hipLaunchKernelGGL((wigner_tiled::wigner_fwd_tiled_real<16>), gh, dim3(256), 0, st, X, Tp, out, n2, nb, b_out, nbatch);
      else
        hipLaunchKernelGGL((wigner_tiled::wigner_fwd_tiled_real<32>), gh, dim3(256), 0, st, X, Tp, out, n2, nb, b_out, nbatch);
    } else if (wigner_tiled::small_analysis(nb, b_out))
      hipLaunchKernelGGL((wigner_tiled::wigner_fwd_tiled<false, 16>), dim3(wigner_tiled::grid_size(MW, nbatch)), dim3(256), 0, st, X, Tp,
                         reinterpret_cast<float2*>(out), n2, nb, b_out, nbatch);
    else if (parts == 1)
      hipLaunchKernelGGL(wigner_tiled::wigner_fwd_tiled<false>, dim3(wigner_tiled::grid_size(MW, nbatch)), dim3(256), 0, st, X, Tp,
                         reinterpret_cast<float2*>(out), n2, nb, b_out, nbatch);
    else
      hipLaunchKernelGGL(wigner_tiled::wigner_fwd_tiled<true>, dim3(wigner_tiled::grid_size(MW, nbatch), parts), dim3(256), 0, st, X, Tp,
                         reinterpret_cast<float2*>(out), n2, nb, b_out, nbatch);
    return s2cnn::launch_status();
  }
  dim3 grid(s2cnn::ceil_div(NW, 16), MW, (unsigned)((nbatch + 15) / 16));
  if (complex_in)
    hipLaunchKernelGGL(so3_wigner_fwd<true>, grid, dim3(16, 16), 0, st, X, table, reinterpret_cast<float2*>(out), n2, nb, b_out, nbatch);
  else
    hipLaunchKernelGGL(so3_wigner_fwd<false>, grid, dim3(16, 16), 0, st, X, table, reinterpret_cast<float2*>(out), n2, nb, b_out, nbatch);
  return s2cnn::launch_status();
}

// Sums over the planes of the output that the synthesis can form where it stages whole planes in LDS (the folded plane
// kernel in its one-round mode): see plane_real::plane_dft_inv.
struct PlaneMoments {
  float* out = nullptr;            // [nbatch * 2 b_out][2]
  const float* yref = nullptr;
  const float* params = nullptr;   // [2][nfeature]
};

// Pairs of sums per volume where the real synthesis b_in -> b_out of a complex spectrum can form them: 2 b_out (one per plane)
// on the two-stage path, 1 from the per-volume kernels of the 32^3 grid, else 0
int moment_parts(int b_in, int b_out) {
  if (!sizes_ok(b_out, b_in, 1)) return 0;
  const FusedKind k = fused_kind(b_out, b_in, 0, true);
  if (k != FUSED_NONE && k != FUSED_64) return 1;
  if (k != FUSED_NONE || 2 * b_out == 64) return 0;
  const plane_real::Plan plan = plane_real::plan_inv(2 * b_out, b_in < b_out ? b_in : b_out, 2 * b_out);
  return plan.pl > 0 && plan.alias ? 2 * b_out : 0;
}

int synthesis_impl(const float* xhat, const float* table, const float* packed_table, float* out, void* workspace,
                   size_t workspace_bytes, int b_in, int b_out, long nbatch, int complex_out, const float* bias, int nfeature,
                   int relu, unsigned long long* bits, void* stream, const PlaneMoments& mom = PlaneMoments(), bool real_basis = false) {
  if (!xhat || !table || !out || !sizes_ok(b_out, b_in, nbatch)) return S2CNN_EINVAL;
  if (real_basis && !real_basis_synthesis(b_in, b_out)) return S2CNN_EINVAL;
  if (real_basis && fused_path(b_out, b_in, 0, true) && mom.out) return S2CNN_EINVAL;     // per volume: fused_synthesis, by its callers
  if (mom.out && (complex_out || moment_parts(b_in, b_out) == 0 || !s2cnn::aligned8(mom.out))) return S2CNN_EINVAL;
  if (mom.yref && (!mom.params || nfeature < 1 || nbatch % nfeature != 0)) return S2CNN_EINVAL;
  if (bits && fused_kind(b_out, b_in, complex_out, true) != FUSED_64) return S2CNN_EINVAL;
  if (bias && (complex_out || nfeature < 1 || nbatch % nfeature != 0)) return S2CNN_EINVAL;
  if (relu && complex_out) return S2CNN_EINVAL;
  if ((!real_basis && !s2cnn::aligned8(xhat)) || (complex_out && !s2cnn::aligned8(out))) return S2CNN_EALIGN;
  if (packed_table && !s2cnn::aligned16(packed_table)) return S2CNN_EALIGN;
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (const FusedKind k = fused_kind(b_out, b_in, complex_out, true)) {
    if (mom.yref && bias) return S2CNN_EINVAL;
    return fused_synthesis(k, xhat, table, packed_table, out, workspace, workspace_bytes, b_in, nbatch, real_basis, bias,
                           (bias || mom.yref) ? nfeature : 1, relu, bits, st, mom.out, mom.yref, mom.params);
  }
  const size_t need = s2cnn_so3_synthesis_workspace(b_in, b_out, nbatch, complex_out);
  if (!workspace || workspace_bytes < need || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return S2CNN_EWORKSPACE;
  const int n2 = 2 * b_out, nb = b_in < b_out ? b_in : b_out;
  const int MW = 2 * nb - 1, NW = complex_out ? MW : nb;
  float2* S = static_cast<float2*>(workspace);
  const size_t lds = sizeof(float2) * (n2 + MW * NW + n2 * NW);
  const plane_real::Plan plan = complex_out ? plane_real::Plan{0, 0, 0, 0} : plane_real::plan_inv(n2, nb, nbatch * n2);
  if (lds > 160 * 1024 && plan.pl == 0) return S2CNN_EINVAL;
  dim3 grid(s2cnn::ceil_div(NW, 16), MW, (unsigned)((nbatch + 15) / 16));
  const float2* xh = reinterpret_cast<const float2*>(xhat);
  const bool tiled = packed_bytes(b_out, b_in, complex_out, true) != 0;
  if (tiled) {
    const float* Tq = packed_table;
    if (!Tq) {
      float* dst = reinterpret_cast<float*>(static_cast<char*>(workspace) + round256(ws_bytes(b_out, b_in, nbatch, complex_out, true)));
      hipLaunchKernelGGL(wigner_tiled::pack_table_synthesis, dim3(2048), dim3(256), 0, st, table, dst, n2, nb, b_in);
      Tq = dst;
    }
    const dim3 gs(wigner_tiled::grid_size_by_weight(MW, nbatch)), gl(wigner_tiled::grid_size_by_weight(MW, nbatch), wigner_tiled::parts_synthesis(n2, nb));
    const void* spectrum = xhat;
    if (wigner_tiled::small_synthesis(n2, nb)) {
      if (real_basis) hipLaunchKernelGGL((wigner_tiled::wigner_inv_tiled<16, 32, true>), gs, dim3(512), 0, st, spectrum, Tq, S, n2, nb, b_in, nbatch);
      else hipLaunchKernelGGL((wigner_tiled::wigner_inv_tiled<16, 32>), gs, dim3(512), 0, st, spectrum, Tq, S, n2, nb, b_in, nbatch);
    } else {
      if (real_basis) hipLaunchKernelGGL((wigner_tiled::wigner_inv_tiled<32, 64, true>), gl, dim3(512), 0, st, spectrum, Tq, S, n2, nb, b_in, nbatch);
      else hipLaunchKernelGGL((wigner_tiled::wigner_inv_tiled<32, 64>), gl, dim3(512), 0, st, spectrum, Tq, S, n2, nb, b_in, nbatch);
    }
  } else if (complex_out) {
    hipLaunchKernelGGL(so3_wigner_inv<true>, grid, dim3(16, 16), 0, st, xh, table, S, n2, nb, b_in, nbatch);
  } else {
    hipLaunchKernelGGL(so3_wigner_inv<false>, grid, dim3(16, 16), 0, st, xh, table, S, n2, nb, b_in, nbatch);
  }
  int rc = s2cnn::launch_status();
  if (rc) return rc;
  const unsigned planes = (unsigned)(nbatch * n2);
  if (complex_out) {
    if (lds > 48 * 1024) (void)hipFuncSetAttribute((const void*)so3_plane_dft_inv<true>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(so3_plane_dft_inv<true>, dim3(planes), dim3(256), lds, st, S, out, n2, nb);
  } else if (n2 == 64 && s2cnn::aligned16(out)) {
    const long npairs = nbatch * 32;
    hipLaunchKernelGGL(fft64::plane_fft64_inv, dim3((unsigned)(npairs < 2048 ? npairs : 2048)), dim3(fft64::THREADS), 0, st, S, out, npairs, nb);
  } else if (plan.pl > 0) {
    if (plan.lds > 48 * 1024) (void)hipFuncSetAttribute((const void*)plane_real::plane_dft_inv, hipFuncAttributeMaxDynamicSharedMemorySize, (int)plan.lds);
    hipLaunchKernelGGL(plane_real::plane_dft_inv, dim3((planes + plan.pl - 1) / plan.pl), dim3(plan.nt), plan.lds, st, S, out, n2, nb,
                       (long)planes, plan.pl, plan.alias, relu, bias, (bias || mom.yref) ? nfeature : 1,
                       reinterpret_cast<float2*>(mom.out), mom.yref, mom.params);
    return s2cnn::launch_status();
  } else {
    if (lds > 48 * 1024) (void)hipFuncSetAttribute((const void*)so3_plane_dft_inv<false>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    hipLaunchKernelGGL(so3_plane_dft_inv<false>, dim3(planes), dim3(256), lds, st, S, out, n2, nb);
  }
  if (bias || relu) {
    const size_t vol = (size_t)n2 * n2 * n2;
    hipLaunchKernelGGL(add_bias_kernel, dim3(2048), dim3(256), 0, st, out, bias, vol, bias ? nfeature : 1, vol * nbatch, relu);
  }
  return s2cnn::launch_status();
}
}  // namespace

extern "C" int s2cnn_so3_analysis(const float* x, const float* table, const float* packed_table, float* out,
                                  void* workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch,
                                  int complex_in, void* stream) {
  s2cnn::clear_stale_error();
  return analysis_impl(s2cnn::Input{x}, table, packed_table, out, workspace, workspace_bytes, b_in, b_out, nbatch, complex_in, stream);
}

extern "C" int s2cnn_so3_synthesis(const float* xhat, const float* table, const float* packed_table, float* out,
                                   void* workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch,
                                   int complex_out, void* stream) {
  s2cnn::clear_stale_error();
  return synthesis_impl(xhat, table, packed_table, out, workspace, workspace_bytes, b_in, b_out, nbatch, complex_out, nullptr, 1, 0, nullptr, stream);
}

extern "C" int s2cnn_so3_synthesis_real_bias(const float* xhat, const float* table, const float* packed_table, float* out,
                                             void* workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch,
                                             const float* bias, int nfeature, void* stream) {
  s2cnn::clear_stale_error();
  return synthesis_impl(xhat, table, packed_table, out, workspace, workspace_bytes, b_in, b_out, nbatch, 0, bias, nfeature, 0, nullptr, stream);
}

namespace {
int synthesis_relu_impl(const float* xhat, const float* table, const float* packed_table, float* out, unsigned long long* bits,
                        void* workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch, const float* bias, int nfeature,
                        int real_basis, void* stream) {
  return synthesis_impl(xhat, table, packed_table, out, workspace, workspace_bytes, b_in, b_out, nbatch, 0, bias, nfeature, 1, bits, stream,
                        PlaneMoments(), real_basis != 0);
}

int analysis_prologue_impl(const s2cnn::Input& in, const float* table, const float* packed_table, float* out,
                           void* workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch, int real_basis, void* stream) {
  if (in.kind == s2cnn::PRO_NONE) return S2CNN_EINVAL;
  return analysis_impl(in, table, packed_table, out, workspace, workspace_bytes, b_in, b_out, nbatch, 0, stream, real_basis != 0);
}
}  // namespace

extern "C" int s2cnn_so3_synthesis_real_relu(const float* xhat, const float* table, const float* packed_table, float* out,
                                             void* workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch,
                                             const float* bias, int nfeature, int real_basis, void* stream) {
  s2cnn::clear_stale_error();
  return synthesis_relu_impl(xhat, table, packed_table, out, nullptr, workspace, workspace_bytes, b_in, b_out, nbatch, bias, nfeature, real_basis, stream);
}

extern "C" size_t s2cnn_so3_relu_bits_bytes(int b_grid, long nbatch) {
  if (nbatch < 1 || fused_kind(b_grid, b_grid, 0, true) != FUSED_64) return 0;      // the kernels of the 64^3 grid write them
  return (size_t)nbatch * fused64::BITS_WORDS * sizeof(unsigned long long);
}

extern "C" int s2cnn_so3_synthesis_real_relu_bits(const float* xhat, const float* table, const float* packed_table, float* out,
                                                  void* bits, void* workspace, size_t workspace_bytes, int b_in, int b_out,
                                                  long nbatch, const float* bias, int nfeature, int real_basis, void* stream) {
  s2cnn::clear_stale_error();
  if (!bits || s2cnn_so3_relu_bits_bytes(b_out, nbatch) == 0) return S2CNN_EINVAL;
  return synthesis_relu_impl(xhat, table, packed_table, out, static_cast<unsigned long long*>(bits), workspace, workspace_bytes, b_in, b_out,
                             nbatch, bias, nfeature, real_basis, stream);
}

extern "C" int s2cnn_so3_analysis_real_masked(const float* x, const float* mask, const float* table, const float* packed_table,
                                              float* out, void* workspace, size_t workspace_bytes, int b_in, int b_out,
                                              long nbatch, int real_basis, void* stream) {
  s2cnn::clear_stale_error();
  return analysis_prologue_impl(s2cnn::Input{x, mask, s2cnn::PRO_MASK}, table, packed_table, out, workspace, workspace_bytes, b_in, b_out, nbatch,
                                real_basis, stream);
}

extern "C" int s2cnn_so3_analysis_real_masked_bits(const float* x, const void* bits, const float* table, const float* packed_table,
                                                   float* out, void* workspace, size_t workspace_bytes, int b_in, int b_out,
                                                   long nbatch, int real_basis, void* stream) {
  s2cnn::clear_stale_error();
  if (s2cnn_so3_relu_bits_bytes(b_in, nbatch) == 0) return S2CNN_EINVAL;
  return analysis_prologue_impl(s2cnn::Input{x, static_cast<const float*>(bits), s2cnn::PRO_BITS}, table, packed_table, out, workspace,
                                workspace_bytes, b_in, b_out, nbatch, real_basis, stream);
}

extern "C" int s2cnn_so3_synthesis_moment_parts(int b_in, int b_out) { return moment_parts(b_in, b_out); }

extern "C" int s2cnn_so3_synthesis_real_moments(const float* xhat, const float* table, const float* packed_table, float* out,
                                                void* workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch,
                                                const float* bias, int nfeature, float* moments, const float* yref,
                                                const float* params, void* stream) {
  s2cnn::clear_stale_error();
  if (!moments) return S2CNN_EINVAL;
  PlaneMoments mom;
  mom.out = moments; mom.yref = yref; mom.params = params;
  return synthesis_impl(xhat, table, packed_table, out, workspace, workspace_bytes, b_in, b_out, nbatch, 0, bias, nfeature, 0, nullptr, stream, mom);
}

extern "C" int s2cnn_so3_analysis_real_basis(const float* x, const float* table, const float* packed_table, float* out,
                                             void* workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch, void* stream) {
  s2cnn::clear_stale_error();
  return analysis_impl(s2cnn::Input{x}, table, packed_table, out, workspace, workspace_bytes, b_in, b_out, nbatch, 0, stream, true);
}

extern "C" int s2cnn_so3_synthesis_real_basis(const float* r, const float* table, const float* packed_table, float* out,
                                              void* workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch,
                                              const float* bias, int nfeature, void* stream) {
  s2cnn::clear_stale_error();
  return synthesis_impl(r, table, packed_table, out, workspace, workspace_bytes, b_in, b_out, nbatch, 0, bias, nfeature, 0, nullptr, stream,
                        PlaneMoments(), true);
}

extern "C" int s2cnn_so3_synthesis_real_basis_moment_parts(int b_in, int b_out, int grad) {
  if (!sizes_ok(b_out, b_in, 1) || !real_basis_synthesis(b_in, b_out)) return 0;
  const FusedKind k = fused_kind(b_out, b_in, 0, true);
  if (k == FUSED_NONE) return moment_parts(b_in, b_out);
  return !grad || k != FUSED_64 || b_in <= fused64::GRAD_MOMENTS_MAX_NL ? 1 : 0;
}

extern "C" int s2cnn_so3_synthesis_real_basis_moments(const float* r, const float* table, const float* packed_table, float* out,
                                                      void* workspace, size_t workspace_bytes, int b_in, int b_out, long nbatch,
                                                      const float* bias, int nfeature, float* moments, const float* yref,
                                                      const float* params, void* stream) {
  s2cnn::clear_stale_error();
  if (!r || !table || !out || !moments || !sizes_ok(b_out, b_in, nbatch)) return S2CNN_EINVAL;
  if ((bias || yref) && (nfeature < 1 || nbatch % nfeature != 0)) return S2CNN_EINVAL;
  if (yref && !params) return S2CNN_EINVAL;
  if (s2cnn_so3_synthesis_real_basis_moment_parts(b_in, b_out, yref != nullptr) == 0) return S2CNN_EINVAL;
  if (packed_table && !s2cnn::aligned16(packed_table)) return S2CNN_EALIGN;
  if (const FusedKind k = fused_kind(b_out, b_in, 0, true)) {
    if (yref && bias) return S2CNN_EINVAL;
    return fused_synthesis(k, r, table, packed_table, out, workspace, workspace_bytes, b_in, nbatch, true, bias, bias || yref ? nfeature : 1, 0,
                           nullptr, static_cast<hipStream_t>(stream), moments, yref, params);
  }
  PlaneMoments mom;
  mom.out = moments; mom.yref = yref; mom.params = params;
  return synthesis_impl(r, table, packed_table, out, workspace, workspace_bytes, b_in, b_out, nbatch, 0, bias, nfeature, 0, nullptr, stream, mom, true);
}

extern "C" int s2cnn_so3_analysis_prologue_available(int b_in, int b_out) { return prologue_path(b_in, b_out) ? 1 : 0; }

extern "C" int s2cnn_so3_analysis_real_affine_relu(const float* x, const float* params, int nfeature, const float* table,
                                                   const float* packed_table, float* out, void* workspace, size_t workspace_bytes,
                                                   int b_in, int b_out, long nbatch, int real_basis, void* stream) {
  s2cnn::clear_stale_error();
  return analysis_prologue_impl(s2cnn::Input{x, nullptr, s2cnn::PRO_AFFINE_RELU, params, nfeature}, table, packed_table, out, workspace,
                                workspace_bytes, b_in, b_out, nbatch, real_basis, stream);
}

extern "C" int s2cnn_so3_analysis_real_bn_relu_grad(const float* g, const float* y, const float* params, int nfeature, const float* table,
                                                    const float* packed_table, float* out, void* workspace, size_t workspace_bytes,
                                                    int b_in, int b_out, long nbatch, int real_basis, void* stream) {
  s2cnn::clear_stale_error();
  return analysis_prologue_impl(s2cnn::Input{g, y, s2cnn::PRO_BN_RELU_GRAD, params, nfeature}, table, packed_table, out, workspace,
                                workspace_bytes, b_in, b_out, nbatch, real_basis, stream);
}

// ---------------------------------------------------------------------------------------------
// s2cnn_so3_analysis for callers that cannot allocate: the scratch is a buffer of the library's own.
// `scratch` below is the host-side stand-in of the device array, not a device address: host code uses the
// address that hipGetSymbolAddress returns for the current device (every GPU holds its own copy).
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[S2CNN_STATIC_SCRATCH_BYTES];

namespace {
constexpr int MAX_DEVICES = 64;
void* scratch_ptr[MAX_DEVICES];     // device address of `scratch` per GPU, resolved on the first call with that GPU current
std::mutex scratch_mutex;

int static_scratch(void** p) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return static_cast<int>(e);
  if (dev < 0 || dev >= MAX_DEVICES) return S2CNN_EINVAL;
  std::lock_guard<std::mutex> lock(scratch_mutex);
  if (!scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return static_cast<int>(e);
    if (!ptr) return S2CNN_EINVAL;
    scratch_ptr[dev] = ptr;
  }
  *p = scratch_ptr[dev];
  return S2CNN_OK;
}
}  // namespace

extern "C" int s2cnn_so3_analysis_static(const float* x, const float* table, const float* packed_table, float* out,
                                         int b_in, int b_out, long nbatch, int complex_in, void* stream) {
  s2cnn::clear_stale_error();
  if (!x || !table || !out || !sizes_ok(b_in, b_out, nbatch)) return S2CNN_EINVAL;
  const size_t need = s2cnn_so3_analysis_workspace(b_in, b_out, nbatch, complex_in);
  if (need == 0) return S2CNN_EINVAL;
  if (need > (size_t)S2CNN_STATIC_SCRATCH_BYTES) return S2CNN_ETOOBIG;
  void* ws = nullptr;
  const int rc = static_scratch(&ws);
  if (rc) return rc;
  return analysis_impl(s2cnn::Input{x}, table, packed_table, out, ws, (size_t)S2CNN_STATIC_SCRATCH_BYTES, b_in, b_out, nbatch, complex_in, stream);
}
