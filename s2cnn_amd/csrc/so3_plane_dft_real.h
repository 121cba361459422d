// (alpha, gamma) transform of the planes of REAL signals for any grid size: a DFT pruned to the
// frequencies |m|, n < nb, folded over both mirror symmetries of the trigonometric matrix and
// register-blocked so that the inner loops are fused multiply-adds fed by 16-byte LDS reads.
//
// With h = n2/2, c[jk] = cos(2 pi j k / n2) and s[jk] = sin(2 pi j k / n2):
//
//   analysis   X[m][n] = sum_{a,g} x[a][g] e^{-i(m a + n g) 2 pi / n2}
//     gamma:   E[a][g] = x[a][g] + x[a][n2-g],  O[a][g] = x[a][g] - x[a][n2-g]   (g = 0 and g = h stand alone)
//              Y[a][n] = sum_{g<=h} E[a][g] c[gn]  -  i sum_{g<=h} O[a][g] s[gn]
//     alpha:   Ye[a] = Y[a] + Y[n2-a],  Yo[a] = Y[a] - Y[n2-a]                      (a = 0 and a = h stand alone)
//              P[m][n] = sum_{a<=h} Ye[a][n] c[am],   Q[m][n] = sum_{a<=h} Yo[a][n] s[am]
//              X[+m] = P - iQ,  X[-m] = P + iQ
//
//   synthesis  y[a][g] = sum_n w_n Re( U[a][n] e^{+i n g 2 pi / n2} ),  U[a][n] = sum_m S[m][n] e^{+i m a 2 pi / n2},
//              w_0 = 1, w_n = 2 (the half plane n >= 0 of a Hermitian spectrum)
//     alpha:   A[m] = S[m] + S[-m],  B[m] = i (S[m] - S[-m])  (A[0] = S[0], B[0] = 0)
//              Uc[a][n] = sum_m A[m][n] c[ma],  Us[a][n] = sum_m B[m][n] s[ma];   U[a] = Uc + Us,  U[n2-a] = Uc - Us
//     gamma:   for the row pair (a, n2-a) and g <= h four sums over n,
//              CC = w Re Uc c[ng], SC = w Re Us c[ng], CS = w Im Uc s[ng], SS = w Im Us s[ng], give
//              y[a][g] = (CC+SC) - (CS+SS),        y[a][n2-g] = (CC+SC) + (CS+SS),
//              y[n2-a][g] = (CC-SC) - (CS-SS),     y[n2-a][n2-g] = (CC-SC) + (CS-SS).
//
// A workgroup takes PL planes at once (small planes have too few 4x4 register blocks to fill it otherwise);
// every thread owns 32 accumulators and reads four 16-byte LDS words per 32 FMAs.  When one round of the
// workgroup covers all blocks of its planes, the output of each pass overwrites its input (after a barrier,
// out of the accumulators): half the LDS per plane and twice the workgroups per CU, and the planes of the
// synthesis leave the LDS as one contiguous run of 16-byte stores instead of four-byte scatters.
#pragma once
#include <hip/hip_runtime.h>
#include <type_traits>
#include "common.h"
#include "dft_common.h"

namespace plane_real {

using dft_common::pad;
using dft_common::cs_entry;

constexpr int NT_MAX = 1024;
constexpr int PL_MAX = 64;                  // planes per workgroup
constexpr unsigned LDS_SOFT = 32 * 1024;    // five workgroups per CU when the planes allow it
constexpr unsigned LDS_HARD = 160 * 1024;


struct Plan {
  int pl;         // planes per workgroup; 0: the plane does not fit the LDS
  int nt;         // threads per workgroup
  int alias;      // the first pass writes over its input
  unsigned lds;   // bytes of dynamic LDS
};

// analysis: table [h+1][nbp] float2 | per plane: EO [h+1][ns] float2, Yf [h+1][nbp] float4
// synthesis: table [nb][hp] float2  | per plane: AB [nb][nb2] float4, UU [nb][npp] float4
inline Plan make_plan(unsigned table_bytes, unsigned in_bytes, unsigned mid_bytes, unsigned out_bytes, int items1, int items2,
                      long nplanes) {
  Plan p{0, 0, 0, 0};
  const int items = items1 > items2 ? items1 : items2;
  p.nt = items <= 256 ? 256 : items <= 512 ? 512 : NT_MAX;
  p.alias = items <= p.nt;     // one round per pass: folded input, intermediate and staged output share one region
  unsigned plane_bytes = in_bytes + mid_bytes;
  if (p.alias) {
    plane_bytes = in_bytes > mid_bytes ? in_bytes : mid_bytes;
    if (out_bytes > plane_bytes) plane_bytes = out_bytes;
    plane_bytes = (plane_bytes + 15u) & ~15u;
  }
  if (table_bytes + plane_bytes > LDS_HARD) return p;
  int pl = p.nt / (items > 0 ? items : 1);
  if (pl < 1) pl = 1;
  if (table_bytes + plane_bytes > LDS_SOFT) pl = 1;
  else if (table_bytes + (unsigned long)pl * plane_bytes > LDS_SOFT) pl = (int)((LDS_SOFT - table_bytes) / plane_bytes);
  if (pl > nplanes) pl = (int)nplanes;
  if (pl > PL_MAX) pl = PL_MAX;
  // among the counts that fit, the one that fills its wavefronts best (the larger on a tie)
  int best = 1;
  float best_fill = 0.f;
  for (int c = 1; c <= pl; ++c) {
    const float fill = (float)(c * items) / (float)(64 * ((c * items + 63) / 64));
    if (fill >= best_fill) { best_fill = fill; best = c; }
  }
  pl = best;
  p.pl = pl;
  p.lds = table_bytes + (unsigned)pl * plane_bytes;
  return p;
}

inline Plan plan_fwd(int n2, int nb, long nplanes) {
  const int hg = n2 / 2 + 1, ns = pad(n2, 4), nbp = pad(nb, 4);
  return make_plan(hg * nbp * 8, hg * ns * 8, hg * nbp * 16, 0, ns / 4 * (nbp / 4), nbp / 4 * (nbp / 2), nplanes);
}

inline Plan plan_inv(int n2, int nb, long nplanes) {
  const int hp = pad(n2 / 2 + 1, 4), npp = pad(n2 / 2 + 1, 2), nb2 = pad(nb, 2);
  return make_plan(nb * hp * 8, nb * nb2 * 16, nb * npp * 16, n2 * n2 * 4, hp / 4 * (nb2 / 2), npp / 2 * (hp / 4), nplanes);
}

struct F2x4 { float2 v[4]; };

__device__ __forceinline__ F2x4 lds_read_f2x4(const float2* p) {
  const float4 lo = reinterpret_cast<const float4*>(p)[0], hi = reinterpret_cast<const float4*>(p)[1];
  F2x4 r;
  r.v[0] = make_float2(lo.x, lo.y); r.v[1] = make_float2(lo.z, lo.w);
  r.v[2] = make_float2(hi.x, hi.y); r.v[3] = make_float2(hi.z, hi.w);
  return r;
}


constexpr int LOADS = 8;   // global loads a thread has in flight while it stages planes

// ---------------------------------------------------------------------------------------------------
// analysis: x [nplanes][n2][n2] -> X, laid out [plane][mi][ni] (ztile = 0) or
// [z / Z][mi][beta][z % Z][ni] (ztile = Z, plane = z n2 + beta); mi = m + nb-1, ni = n.
// ---------------------------------------------------------------------------------------------------
// kind, mask, params, nfeature: what is done to x as it is loaded (s2cnn::Prologue; mask = the second tensor, if any;
// kind 2, bit masks, is not supported here)
__global__ __launch_bounds__(NT_MAX) void plane_dft_fwd(const float* __restrict__ x, float2* __restrict__ X, int n2, int nb,
                                                        int ztile, long nplanes, int PL, int alias, const float* __restrict__ mask,
                                                        int kind, const float* __restrict__ params, int nfeature) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  __shared__ float4 par[PL_MAX];                                      // (a, b, p, q) of the feature of each plane of the workgroup
  const int h = n2 / 2, nbp = pad(nb, 4), ns = pad(n2, 4);
  float2* tab = reinterpret_cast<float2*>(smem);                      // [h+1][nbp]
  float2* EO = tab + (h + 1) * nbp;                                   // [PL][h+1][ns]
  float4* Yf = reinterpret_cast<float4*>(alias ? EO : EO + (size_t)PL * (h + 1) * ns);   // [PL][h+1][nbp]
  const long plane0 = (long)blockIdx.x * PL;
  const int t = threadIdx.x, NT = blockDim.x;
  // volume and beta of the workgroup's first plane, once (plane counts fit 32 bits: the host refuses more than 2^31 planes)
  const unsigned vol0 = (unsigned)plane0 / (unsigned)n2, beta0 = (unsigned)plane0 - vol0 * n2;
  const float inv_n2f = 1.0f / (float)n2;

  for (int i = t; i < (h + 1) * nbp; i += NT) {
    const int j = i / nbp, k = i - j * nbp;
    tab[i] = k < nb ? cs_entry(j, k, n2) : make_float2(0.f, 0.f);
  }
  if (kind >= 3 && t < PL) {
    const int c = (int)(((plane0 + t) / n2) % nfeature);
    par[t] = make_float4(params[c], params[nfeature + c], kind == 4 ? params[2 * nfeature + c] : 0.f, kind == 4 ? params[3 * nfeature + c] : 0.f);
  }
  if (kind >= 3) __syncthreads();
  // fold gamma; rows go to slots so that the pair (a, n2-a) is adjacent: 0 -> 0, h -> 1, a -> 2a, n2-a -> 2a+1.
  // The planes of a workgroup are one contiguous run of rows; LOADS of them are issued before the first is used.
  {
    const int hg = h + 1;
    const long rows_valid = (nplanes - plane0) * n2;
    const float* src = x + (size_t)plane0 * n2 * n2;
    const float* msk = mask ? mask + (size_t)plane0 * n2 * n2 : nullptr;
    const float inv_n2 = 1.0f / (float)n2;
    // one copy of the loop per case, so that the batched loads of the plain case stay one run of loads.
    // A thread keeps one column g (and its mirror n2 - g) and walks down the rows of the workgroup's planes in steps of
    // RS = NT / hg rows: the loads of a wave are runs of hg consecutive floats of consecutive rows, and per element there
    // is no more index arithmetic than the plane and the slot of its row.
    auto fold_rows = [&](auto kind_c) {
      constexpr int KIND = decltype(kind_c)::value;
      constexpr bool SECOND = KIND == 1 || KIND == 4;
      const int RS = NT / hg;
      const int g = t % hg, r0 = t / hg;
      const bool lane_on = r0 < RS;
      const bool paired = g > 0 && g < h;
      const int g2 = paired ? n2 - g : g;
      const int nrows = PL * n2;
      for (int Rb = r0; Rb - r0 < nrows; Rb += LOADS * RS) {      // the same number of rounds for every thread
        float v1[LOADS], v2[LOADS], m1[LOADS], m2[LOADS];
#pragma unroll
        for (int u = 0; u < LOADS; ++u) {
          const int R = Rb + u * RS;
          const bool valid = lane_on && R < nrows && R < rows_valid;
          const int o = valid ? R * n2 : 0;
          v1[u] = src[o + g];
          v2[u] = src[o + g2];
          if constexpr (SECOND) { m1[u] = msk[o + g]; m2[u] = msk[o + g2]; }
        }
#pragma unroll
        for (int u = 0; u < LOADS; ++u) {
          const int R = Rb + u * RS;
          if (!(lane_on && R < nrows)) continue;
          const int q = (int)(((float)R + 0.5f) * inv_n2), a = R - q * n2;     // plane of the workgroup, row of the plane
          float va = v1[u], vb = v2[u];
          if constexpr (KIND == 1) { va = s2cnn::relu_pass(va, m1[u]); vb = s2cnn::relu_pass(vb, m2[u]); }
          if constexpr (KIND == 3) {
            const float4 c = par[q];
            va = s2cnn::affine_relu(va, c.x, c.y); vb = s2cnn::affine_relu(vb, c.x, c.y);
          }
          if constexpr (KIND == 4) {
            const float4 c = par[q];
            va = s2cnn::bn_relu_grad(va, m1[u], c.x, c.y, c.z, c.w); vb = s2cnn::bn_relu_grad(vb, m2[u], c.x, c.y, c.z, c.w);
          }
          if (R >= rows_valid) va = vb = 0.f;
          int slot = a < h ? 2 * a : 2 * (n2 - a) + 1;
          slot = a == 0 ? 0 : a == h ? 1 : slot;
          EO[(q * hg + g) * ns + slot] = make_float2(paired ? va + vb : va, paired ? va - vb : 0.f);
        }
      }
    };
    // The same for four columns g0 .. g0 + 3 per thread and step (n2 >= 8): two 16-byte loads per tensor, the row's
    // plane and slot worked out once for four numbers.  The mirror columns n2 - g0 - j come as the run
    // [n2 - g0 - 3, n2 - g0]; for g0 = 0, whose column 0 has no mirror, as [n2 - 4, n2 - 1] (the run never leaves the row).
    auto fold_quads = [&](auto kind_c) {
      constexpr int KIND = decltype(kind_c)::value;
      constexpr bool SECOND = KIND == 1 || KIND == 4;
      constexpr int QL = SECOND ? LOADS / 4 : LOADS / 2;      // 16-byte loads per tensor in flight: the registers of LOADS numbers
      const int GQ = (hg + 3) / 4;
      const int RS = NT / GQ;
      const int g0 = 4 * (t % GQ), r0 = t / GQ;
      const bool lane_on = r0 < RS;
      const int gm = g0 == 0 ? n2 - 4 : n2 - g0 - 3;       // where the run of mirror columns starts
      const int nrows = PL * n2;
      auto ld4 = [](const float* p) { return make_float4(p[0], p[1], p[2], p[3]); };
      for (int Rb = r0; Rb - r0 < nrows; Rb += QL * RS) {      // the same number of rounds for every thread
        float4 v1[QL], v2[QL], m1[QL], m2[QL];
#pragma unroll
        for (int u = 0; u < QL; ++u) {
          const int R = Rb + u * RS;
          const bool valid = lane_on && R < nrows && R < rows_valid;
          const int o = valid ? R * n2 : 0;
          v1[u] = ld4(src + o + g0);
          v2[u] = ld4(src + o + gm);
          if constexpr (SECOND) { m1[u] = ld4(msk + o + g0); m2[u] = ld4(msk + o + gm); }
        }
#pragma unroll
        for (int u = 0; u < QL; ++u) {
          const int R = Rb + u * RS;
          if (!(lane_on && R < nrows)) continue;
          const int q = (int)(((float)R + 0.5f) * inv_n2), a = R - q * n2;     // plane of the workgroup, row of the plane
          int slot = a < h ? 2 * a : 2 * (n2 - a) + 1;
          slot = a == 0 ? 0 : a == h ? 1 : slot;
          const bool zero = R >= rows_valid;
          [[maybe_unused]] float4 c = make_float4(0.f, 0.f, 0.f, 0.f);
          if constexpr (KIND >= 3) c = par[q];
          const float xa[4] = {v1[u].x, v1[u].y, v1[u].z, v1[u].w}, ma[4] = {m1[u].x, m1[u].y, m1[u].z, m1[u].w};
          // mirror of column g0 + j: element 3 - j of the run, or 4 - j of the run that starts one later (g0 = 0, j >= 1)
          const float xr[4] = {v2[u].x, v2[u].y, v2[u].z, v2[u].w}, mr[4] = {m2[u].x, m2[u].y, m2[u].z, m2[u].w};
          float2* dst = EO + (q * hg + g0) * ns + slot;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const int g = g0 + j;
            if (g > h) continue;
            const bool paired = g > 0 && g < h;
            float va = xa[j], vb = g0 == 0 ? xr[(4 - j) & 3] : xr[3 - j];
            [[maybe_unused]] const float wa = ma[j], wb = g0 == 0 ? mr[(4 - j) & 3] : mr[3 - j];
            if constexpr (KIND == 1) { va = s2cnn::relu_pass(va, wa); vb = s2cnn::relu_pass(vb, wb); }
            if constexpr (KIND == 3) { va = s2cnn::affine_relu(va, c.x, c.y); vb = s2cnn::affine_relu(vb, c.x, c.y); }
            if constexpr (KIND == 4) { va = s2cnn::bn_relu_grad(va, wa, c.x, c.y, c.z, c.w); vb = s2cnn::bn_relu_grad(vb, wb, c.x, c.y, c.z, c.w); }
            if (zero) va = vb = 0.f;
            dst[j * ns] = make_float2(paired ? va + vb : va, paired ? va - vb : 0.f);
          }
        }
      }
    };
    if (n2 >= 8) {
      if (kind == 1) fold_quads(std::integral_constant<int, 1>{});
      else if (kind == 3) fold_quads(std::integral_constant<int, 3>{});
      else if (kind == 4) fold_quads(std::integral_constant<int, 4>{});
      else fold_quads(std::integral_constant<int, 0>{});
    } else {
      if (kind == 1) fold_rows(std::integral_constant<int, 1>{});
      else if (kind == 3) fold_rows(std::integral_constant<int, 3>{});
      else if (kind == 4) fold_rows(std::integral_constant<int, 4>{});
      else fold_rows(std::integral_constant<int, 0>{});
    }
    if (ns > n2)   // n2 = 2 mod 4: two empty slots
      for (int i = t; i < PL * hg * (ns - n2); i += NT) EO[(i / (ns - n2)) * ns + n2 + i % (ns - n2)] = make_float2(0.f, 0.f);
  }
  __syncthreads();

  // gamma pass: 4 row slots x 4 frequencies per thread
  const int nkb = nbp / 4, i1 = ns / 4 * nkb;
  for (int it = t; it - t < PL * i1; it += NT) {      // the same number of rounds for every thread
    const bool active = it < PL * i1;
    const int q = it / i1, r = it - q * i1;
    const int sb = r / nkb, kb = r - sb * nkb;
    const float2* eo = EO + (size_t)q * (h + 1) * ns + 4 * sb;
    const float2* tb = tab + 4 * kb;
    float yr[4][4], yi[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int k = 0; k < 4; ++k) yr[i][k] = yi[i][k] = 0.f;
    if (active)
      for (int g = 0; g <= h; ++g) {
        const F2x4 e = lds_read_f2x4(eo + g * ns), w = lds_read_f2x4(tb + g * nbp);
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            yr[i][k] = fmaf(e.v[i].x, w.v[k].x, yr[i][k]);
            yi[i][k] = fmaf(e.v[i].y, w.v[k].y, yi[i][k]);
          }
      }
    if (alias) __syncthreads();                        // one round only: every read of EO is done
    float4* yf = Yf + (size_t)q * (h + 1) * nbp + 4 * kb;
#pragma unroll
    for (int pi = 0; pi < 2; ++pi) {
      const int p = 2 * sb + pi;
      if (p >= h || !active) continue;
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        const float r1 = yr[2 * pi][k], m1 = -yi[2 * pi][k], r2 = yr[2 * pi + 1][k], m2 = -yi[2 * pi + 1][k];
        if (p == 0) {
          yf[k] = make_float4(r1, m1, 0.f, 0.f);
          yf[h * nbp + k] = make_float4(r2, m2, 0.f, 0.f);
        } else {
          yf[p * nbp + k] = make_float4(r1 + r2, m1 + m2, r1 - r2, m1 - m2);
        }
      }
    }
  }
  __syncthreads();

  // alpha pass: 4 frequencies m >= 0 x 2 frequencies n per thread
  const int nnb = nbp / 2, i2 = nkb * nnb;
  // X leaves straight from the accumulators: its rows lie far apart in the tiled layout, staging them does not pay
  for (int it = t; it < PL * i2; it += NT) {
    const int q = it / i2, r = it - q * i2;
    const int mb = r / nnb, nk = r - mb * nnb;
    const long pl = plane0 + q;
    const float4* yf = Yf + (size_t)q * (h + 1) * nbp + 2 * nk;
    const float2* tb = tab + 4 * mb;
    float pr[4][2], pi_[4][2], qr[4][2], qi[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int k = 0; k < 2; ++k) pr[i][k] = pi_[i][k] = qr[i][k] = qi[i][k] = 0.f;
    for (int a = 0; a <= h; ++a) {
      const float4 y0 = yf[a * nbp], y1 = yf[a * nbp + 1];
      const F2x4 w = lds_read_f2x4(tb + a * nbp);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        pr[i][0] = fmaf(y0.x, w.v[i].x, pr[i][0]); pi_[i][0] = fmaf(y0.y, w.v[i].x, pi_[i][0]);
        qr[i][0] = fmaf(y0.z, w.v[i].y, qr[i][0]); qi[i][0] = fmaf(y0.w, w.v[i].y, qi[i][0]);
        pr[i][1] = fmaf(y1.x, w.v[i].x, pr[i][1]); pi_[i][1] = fmaf(y1.y, w.v[i].x, pi_[i][1]);
        qr[i][1] = fmaf(y1.z, w.v[i].y, qr[i][1]); qi[i][1] = fmaf(y1.w, w.v[i].y, qi[i][1]);
      }
    }
    if (pl >= nplanes) continue;
    float2* dst = X + (size_t)pl * ((2 * nb - 1) * nb);
    size_t mstride = nb;
    if (ztile > 0) {              // volume and beta of the plane, tile and place in the tile of the volume: 32-bit arithmetic
      const unsigned bq = beta0 + q, dz = (unsigned)(((float)bq + 0.5f) * inv_n2f);
      const unsigned beta = bq - dz * n2, z = vol0 + dz;
      const unsigned zt = z / (unsigned)ztile, zr = z - zt * ztile;
      dst = X + ((size_t)zt * (2 * nb - 1) * n2 + beta) * ztile * nb + zr * nb;
      mstride = (size_t)n2 * ztile * nb;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int m = 4 * mb + i;
      if (m >= nb) continue;
#pragma unroll
      for (int k = 0; k < 2; ++k) {
        const int n = 2 * nk + k;
        if (n >= nb) continue;
        dst[(size_t)(nb - 1 + m) * mstride + n] = make_float2(pr[i][k] + qi[i][k], pi_[i][k] - qr[i][k]);
        if (m > 0) dst[(size_t)(nb - 1 - m) * mstride + n] = make_float2(pr[i][k] - qi[i][k], pi_[i][k] + qr[i][k]);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------------
// synthesis: S [nplanes][2nb-1][nb] -> y [nplanes][n2][n2]
// ---------------------------------------------------------------------------------------------------
// bias: NULL, or nfeature values; bias[z % nfeature] is added to every sample of volume z = plane / n2
// relu: nonzero = negative samples (after the bias) are stored as zero
// moments (alias mode only): NULL, or [nplanes] pairs of sums over each plane of the output v, formed from the staged
// planes in a fixed order: yref == NULL: (sum v, sum (v - mean of the plane)^2), the squares summed around a pivot so that
// a large mean costs no digits; else, with m = (a yref + b > 0), a = params[f],
// b = params[nfeature + f] of the plane's feature f: (sum v m, sum v m yref): what a batch normalisation over the
// volumes of a feature needs of its input, or (v being the gradient with respect to its activated output) of its gradient.
__global__ __launch_bounds__(NT_MAX) void plane_dft_inv(const float2* __restrict__ S, float* __restrict__ y, int n2, int nb,
                                                        long nplanes, int PL, int alias, int relu, const float* __restrict__ bias,
                                                        int nfeature, float2* __restrict__ moments, const float* __restrict__ yref,
                                                        const float* __restrict__ params) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int h = n2 / 2, hp = pad(h + 1, 4), nb2 = pad(nb, 2), npp = pad(h + 1, 2);
  float2* tab = reinterpret_cast<float2*>(smem);                          // [nb][hp]
  float4* AB = reinterpret_cast<float4*>(tab + nb * hp);                  // [PL][nb][nb2]
  float4* UU = alias ? AB : AB + (size_t)PL * nb * nb2;                   // [PL][nb][npp]
  const long plane0 = (long)blockIdx.x * PL;
  const int t = threadIdx.x, NT = blockDim.x;
  // volume and beta of the workgroup's first plane, once (plane counts fit 32 bits: the host refuses more than 2^31 planes)
  const unsigned vol0 = (unsigned)plane0 / (unsigned)n2, beta0 = (unsigned)plane0 - vol0 * n2;
  const unsigned feat0 = nfeature > 1 ? vol0 % (unsigned)nfeature : 0u;     // feature of that volume
  const float inv_n2f = 1.0f / (float)n2;

  for (int i = t; i < nb * hp; i += NT) {
    const int k = i / hp, j = i - k * hp;
    tab[i] = j <= h ? cs_entry(j, k, n2) : make_float2(0.f, 0.f);
  }
  // A, B from the rows +m and -m of S; LOADS pairs of rows are in flight per thread.  A thread keeps one column n (two
  // adjacent ones where nb is even: 16-byte loads and LDS stores) and walks down the rows R = q nb + m of the workgroup's
  // planes in steps of RS rows: per element nothing but the plane and the frequency of its row is worked out.
  {
    const int srow = (2 * nb - 1) * nb, nrows = PL * nb;
    const float2* src = S + (size_t)plane0 * srow;
    const long planes_valid = nplanes - plane0;
    const float inv_nb = 1.0f / (float)nb;
    auto combine = [](float2 p, float2 m, bool both) {
      return both ? make_float4(p.x + m.x, p.y + m.y, m.y - p.y, p.x - m.x) : make_float4(p.x, p.y, 0.f, 0.f);
    };
    if ((nb & 1) == 0) {
      const int CP = nb / 2, RS = NT / CP;
      const int n = 2 * (t % CP), r0 = t / CP;
      const bool lane_on = r0 < RS;
      constexpr int QL = LOADS / 2;
      for (int Rb = r0; Rb - r0 < nrows; Rb += QL * RS) {
        float4 sp[QL], sm[QL];
#pragma unroll
        for (int u = 0; u < QL; ++u) {
          const int R = Rb + u * RS;
          const int q = (int)(((float)R + 0.5f) * inv_nb), m = R - q * nb;
          const bool valid = lane_on && R < nrows && q < planes_valid;
          sp[u] = *reinterpret_cast<const float4*>(src + (valid ? q * srow + (nb - 1 + m) * nb + n : 0));
          sm[u] = *reinterpret_cast<const float4*>(src + (valid ? q * srow + (nb - 1 - m) * nb + n : 0));
        }
#pragma unroll
        for (int u = 0; u < QL; ++u) {
          const int R = Rb + u * RS;
          if (!(lane_on && R < nrows)) continue;
          const int q = (int)(((float)R + 0.5f) * inv_nb), m = R - q * nb;
          float4 a0 = make_float4(0.f, 0.f, 0.f, 0.f), a1 = a0;
          if (q < planes_valid) {
            a0 = combine(make_float2(sp[u].x, sp[u].y), make_float2(sm[u].x, sm[u].y), m > 0);
            a1 = combine(make_float2(sp[u].z, sp[u].w), make_float2(sm[u].z, sm[u].w), m > 0);
          }
          AB[R * nb2 + n] = a0;
          AB[R * nb2 + n + 1] = a1;
        }
      }
    } else {
      const int RS = NT / nb2;
      const int n = t % nb2, r0 = t / nb2;
      const bool lane_on = r0 < RS;
      for (int Rb = r0; Rb - r0 < nrows; Rb += LOADS * RS) {
        float2 sp[LOADS], sm[LOADS];
#pragma unroll
        for (int u = 0; u < LOADS; ++u) {
          const int R = Rb + u * RS;
          const int q = (int)(((float)R + 0.5f) * inv_nb), m = R - q * nb;
          const bool valid = lane_on && R < nrows && n < nb && q < planes_valid;
          sp[u] = src[valid ? q * srow + (nb - 1 + m) * nb + n : 0];
          sm[u] = src[valid ? q * srow + (nb - 1 - m) * nb + n : 0];
        }
#pragma unroll
        for (int u = 0; u < LOADS; ++u) {
          const int R = Rb + u * RS;
          if (!(lane_on && R < nrows)) continue;
          const int q = (int)(((float)R + 0.5f) * inv_nb), m = R - q * nb;
          AB[R * nb2 + n] = n < nb && q < planes_valid ? combine(sp[u], sm[u], m > 0) : make_float4(0.f, 0.f, 0.f, 0.f);
        }
      }
    }
  }
  __syncthreads();

  // alpha pass: 4 angles a <= h x 2 frequencies n per thread
  const int njb = hp / 4, nnb = nb2 / 2, i1 = njb * nnb;
  for (int it = t; it - t < PL * i1; it += NT) {      // the same number of rounds for every thread
    const bool active = it < PL * i1;
    const int q = it / i1, r = it - q * i1;
    const int jb = r / nnb, nk = r - jb * nnb;
    const float4* ab = AB + (size_t)q * nb * nb2 + 2 * nk;
    const float2* tb = tab + 4 * jb;
    float cr[4][2], ci[4][2], sr[4][2], si[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int k = 0; k < 2; ++k) cr[i][k] = ci[i][k] = sr[i][k] = si[i][k] = 0.f;
    for (int m = 0; m < (active ? nb : 0); ++m) {
      const float4 a0 = ab[m * nb2], a1 = ab[m * nb2 + 1];
      const F2x4 w = lds_read_f2x4(tb + m * hp);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        cr[i][0] = fmaf(a0.x, w.v[i].x, cr[i][0]); ci[i][0] = fmaf(a0.y, w.v[i].x, ci[i][0]);
        sr[i][0] = fmaf(a0.z, w.v[i].y, sr[i][0]); si[i][0] = fmaf(a0.w, w.v[i].y, si[i][0]);
        cr[i][1] = fmaf(a1.x, w.v[i].x, cr[i][1]); ci[i][1] = fmaf(a1.y, w.v[i].x, ci[i][1]);
        sr[i][1] = fmaf(a1.z, w.v[i].y, sr[i][1]); si[i][1] = fmaf(a1.w, w.v[i].y, si[i][1]);
      }
    }
    if (alias) __syncthreads();                        // one round only: every read of AB is done
    float4* uu = UU + (size_t)q * nb * npp;
#pragma unroll
    for (int k = 0; k < 2; ++k) {
      const int n = 2 * nk + k;
      if (n >= nb || !active) continue;
      const float wn = n == 0 ? 1.f : 2.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int a = 4 * jb + i;
        if (a < npp) uu[n * npp + a] = make_float4(wn * cr[i][k], wn * ci[i][k], wn * sr[i][k], wn * si[i][k]);
      }
    }
  }
  __syncthreads();

  // gamma pass: 2 row pairs (a, n2-a) x 4 angles g <= h per thread
  const int npb = npp / 2, i2 = npb * njb;
  float* Ys = reinterpret_cast<float*>(AB);            // staged mode: the planes of y
  for (int it = t; it - t < PL * i2; it += NT) {
    const bool active = it < PL * i2;
    const int q = it / i2, r = it - q * i2;
    const int pb = r / njb, gb = r - pb * njb;
    const long pl = plane0 + q;
    const float4* uu = UU + (size_t)q * nb * npp + 2 * pb;
    const float2* tb = tab + 4 * gb;
    float cc[2][4], sc[2][4], cs[2][4], ss[2][4];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int k = 0; k < 4; ++k) cc[i][k] = sc[i][k] = cs[i][k] = ss[i][k] = 0.f;
    for (int n = 0; n < (active ? nb : 0); ++n) {
      const float4 u0 = uu[n * npp], u1 = uu[n * npp + 1];
      const F2x4 w = lds_read_f2x4(tb + n * hp);
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        cc[0][k] = fmaf(u0.x, w.v[k].x, cc[0][k]); cs[0][k] = fmaf(u0.y, w.v[k].y, cs[0][k]);
        sc[0][k] = fmaf(u0.z, w.v[k].x, sc[0][k]); ss[0][k] = fmaf(u0.w, w.v[k].y, ss[0][k]);
        cc[1][k] = fmaf(u1.x, w.v[k].x, cc[1][k]); cs[1][k] = fmaf(u1.y, w.v[k].y, cs[1][k]);
        sc[1][k] = fmaf(u1.z, w.v[k].x, sc[1][k]); ss[1][k] = fmaf(u1.w, w.v[k].y, ss[1][k]);
      }
    }
    // staged mode (one round): y goes to LDS over the consumed spectra and leaves as one contiguous run below
    if (alias) __syncthreads();
    if (!active || pl >= nplanes) continue;
    float bz = 0.f;
    if (bias) {                   // the feature of the plane's volume, without a division per item
      unsigned f = feat0 + (unsigned)(((float)(beta0 + q) + 0.5f) * inv_n2f);
      while (f >= (unsigned)nfeature) f -= nfeature;
      bz = bias[f];
    }
    const float lo = relu ? 0.f : -INFINITY;             // v < lo ? lo : v  is max(v, 0) that keeps a NaN, or v
    // one copy per address space, so that the staged mode writes LDS with immediate offsets
    auto emit = [&](float* dst) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int a = 2 * pb + i;
        if (a > h) continue;
        const bool mirror_a = a > 0 && a < h;
        float* r0 = dst + a * n2 + 4 * gb;               // columns g = 4 gb + k
        float* r1 = dst + a * n2 + n2 - 4 * gb;          // columns n2 - g
        float* r2 = dst + (n2 - a) * n2 + 4 * gb;
        float* r3 = dst + (n2 - a) * n2 + n2 - 4 * gb;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
          const int g = 4 * gb + k;
          if (g > h) continue;
          const bool mirror_g = g > 0 && g < h;
          const float c0 = cc[i][k] + bz;
          const float yc = c0 + sc[i][k], ys = cs[i][k] + ss[i][k];
          float v = yc - ys;
          r0[k] = v < lo ? lo : v;
          if (mirror_g) { v = yc + ys; r1[-k] = v < lo ? lo : v; }
          if (mirror_a) {
            const float zc = c0 - sc[i][k], zs = cs[i][k] - ss[i][k];
            v = zc - zs;
            r2[k] = v < lo ? lo : v;
            if (mirror_g) { v = zc + zs; r3[-k] = v < lo ? lo : v; }
          }
        }
      }
    };
    if (alias) emit(Ys + (size_t)q * n2 * n2);
    else emit(y + (size_t)pl * n2 * n2);
  }
  if (!alias) return;
  __syncthreads();
  {
    long pv = nplanes - plane0;
    if (pv > PL) pv = PL;
    const int total = (int)pv * n2 * n2;                 // a multiple of 4
    float* dst = y + (size_t)plane0 * n2 * n2;
    if (moments) {                                       // one wave per plane at a time, lanes stride over its samples
      const int lane = t & 63, wave = t >> 6, nwave = NT >> 6, psize = n2 * n2;
      for (int q = wave; q < (int)pv; q += nwave) {
        const float* v = Ys + (size_t)q * psize;
        float s1 = 0.f, s2 = 0.f;
        if (yref) {
          const int f = (int)(((plane0 + q) / n2) % nfeature);
          const float a = params[f], b = params[nfeature + f];
          const float* yr = yref + (size_t)(plane0 + q) * psize;
          if ((reinterpret_cast<uintptr_t>(yr) & 15u) == 0) {       // four samples per load, four loads in flight (n2 is even)
            const float4* yr4 = reinterpret_cast<const float4*>(yr);
            const float4* v4 = reinterpret_cast<const float4*>(v);
#pragma unroll 4
            for (int i = lane; i < psize / 4; i += 64) {
              const float4 yv = yr4[i], g = v4[i];
              const float g0 = s2cnn::relu_pass(g.x, fmaf(a, yv.x, b)), g1 = s2cnn::relu_pass(g.y, fmaf(a, yv.y, b));
              const float g2 = s2cnn::relu_pass(g.z, fmaf(a, yv.z, b)), g3 = s2cnn::relu_pass(g.w, fmaf(a, yv.w, b));
              s1 += (g0 + g1) + (g2 + g3);
              s2 = fmaf(g0, yv.x, fmaf(g1, yv.y, fmaf(g2, yv.z, fmaf(g3, yv.w, s2))));
            }
          } else {
            for (int i = lane; i < psize; i += 64) {
              const float yv = yr[i], gm = s2cnn::relu_pass(v[i], fmaf(a, yv, b));
              s1 += gm; s2 = fmaf(gm, yv, s2);
            }
          }
        } else {                                         // squares around a pivot (the plane's first sample), moved to the plane's mean below
          const float4* v4 = reinterpret_cast<const float4*>(v);
          const float pivot = v[0];
#pragma unroll 4
          for (int i = lane; i < psize / 4; i += 64) {
            const float4 x = v4[i];
            const float d0 = x.x - pivot, d1 = x.y - pivot, d2 = x.z - pivot, d3 = x.w - pivot;
            s1 += (d0 + d1) + (d2 + d3);
            s2 = fmaf(d0, d0, fmaf(d1, d1, fmaf(d2, d2, fmaf(d3, d3, s2))));
          }
#pragma unroll
          for (int o = 32; o > 0; o >>= 1) { s1 += __shfl_xor(s1, o); s2 += __shfl_xor(s2, o); }
          if (lane == 0) moments[plane0 + q] = make_float2(fmaf((float)psize, pivot, s1), s2 - s1 * s1 / (float)psize);   // (sum v, sum (v - mean)^2)
          continue;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) { s1 += __shfl_xor(s1, o); s2 += __shfl_xor(s2, o); }
        if (lane == 0) moments[plane0 + q] = make_float2(s1, s2);
      }
    }
    if ((reinterpret_cast<uintptr_t>(y) & 15u) == 0) {
      for (int i = t; i < total / 4; i += NT) reinterpret_cast<float4*>(dst)[i] = reinterpret_cast<const float4*>(Ys)[i];
    } else {
      for (int i = t; i < total; i += NT) dst[i] = Ys[i];
    }
  }
}

}  // namespace plane_real
