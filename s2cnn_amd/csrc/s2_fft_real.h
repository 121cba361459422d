// S^2 Fourier analysis and synthesis of REAL signals with b_spec <= 32 (the bandwidth an S^2 convolution keeps):
// one workgroup per signal, both stages in one kernel, the intermediate [beta][m] never leaves the LDS.
//
//   analysis   out[l,m,z] = sum_beta T[beta,lm] X[beta,m],   X[beta,m] = sum_alpha x[z,beta,alpha] e^{-i m alpha}
//     The rows are folded, E/O[alpha] = x[alpha] +- x[n2-alpha] (alpha = 0 and n2/2 stand alone), so that
//     Re X[m] = sum_{alpha<=h} E c[alpha m], Im X[m] = -sum_{alpha<=h} O s[alpha m], only m >= 0 is transformed
//     (X[-m] = conj X[m]) and a thread owns 2 rows x 2 frequencies: two 16-byte LDS reads per 8 FMAs.  The table
//     contraction takes the b^2 entries (l,m) in their memory order, two per thread: the table is read in whole rows.
//
//   synthesis  y[z,beta,alpha] = Re sum_m e^{+i m alpha} S[beta,m],   S[beta,m] = sum_{l>=|m|} T[beta,lm] xhat[l,m,z]
//     With A[m] = Re S[m] + Re S[-m], B[m] = Im S[m] - Im S[-m] (A[0] = Re S[0], B[0] = 0):
//     Yc[alpha] = sum_m A[m] c[m alpha], Ys[alpha] = sum_m B[m] s[m alpha], y[alpha] = Yc - Ys, y[n2-alpha] = Yc + Ys.
//
// The signal is processed in chunks of RB rows (betas); the next chunk's loads are in flight while one is transformed.
// A batch too small to fill the chip with one workgroup per signal is split along beta (grid.y = split): the synthesis
// needs nothing more, the analysis writes one partial spectrum per split and reduce_splits adds them in a fixed order.
#pragma once
#include <hip/hip_runtime.h>
#include "dft_common.h"

namespace s2_real {

using dft_common::Walk2;
using dft_common::pad;

constexpr int NT = 512;
constexpr int PF = 20;          // prefetched (alpha, row) elements per thread and chunk
constexpr int NB_MAX = 32;
constexpr unsigned LDS_MAX = 150 * 1024;

struct Plan {
  int rb;         // rows per chunk; 0: this path does not apply
  unsigned lds;
};

// analysis: tab [h+1][nbp] float2 | EO [h+1][rb] float2 | X [rb][nbp] float2
inline Plan plan_fwd(int n2, int nb) {
  Plan p{0, 0};
  if (nb > NB_MAX || (n2 & 1)) return p;
  const int hg = n2 / 2 + 1, nbp = pad(nb, 2);
  for (int rb = 64; rb >= 2; rb >>= 1) {
    const unsigned lds = (unsigned)(hg * nbp * 8 + hg * rb * 8 + rb * nbp * 8);
    if (rb * hg <= PF * NT && lds <= LDS_MAX) { p.rb = rb; p.lds = lds; return p; }
  }
  return p;
}

// synthesis: tab [nb][hp] float2 | xh [nb^2] float2 | AB [nb][rb] float2
inline Plan plan_inv(int n2, int nb) {
  Plan p{0, 0};
  if (nb > NB_MAX || (n2 & 1)) return p;
  const int hp = pad(n2 / 2 + 1, 2);
  const unsigned lds = (unsigned)(nb * hp * 8 + pad(nb * nb, 2) * 8 + nb * 64 * 8);
  if (lds > LDS_MAX) return p;
  p.rb = 64; p.lds = lds;
  return p;
}

__device__ __forceinline__ int isqrt_floor(int v) {
  int l = (int)sqrtf((float)v);
  while (l * l > v) --l;
  while ((l + 1) * (l + 1) <= v) ++l;
  return l;
}

// chunks of RB rows per split, for `nsplit` splits of n2 rows
__host__ __device__ inline int rows_per_split(int n2, int RB, int nsplit) {
  const int nchunk = (n2 + RB - 1) / RB;
  return RB * ((nchunk + nsplit - 1) / nsplit);
}

// How many splits along beta a batch of nbatch signals gets: enough workgroups for four per CU (the kernels are bound by
// what one CU issues, so the work has to spread evenly over all of them), whole chunks per split.
inline int splits_for(int n2, int RB, long nbatch) {
  const int nchunk = (n2 + RB - 1) / RB;
  long want = (1024 + nbatch - 1) / nbatch;
  if (want > nchunk) want = nchunk;
  if (want > 8) want = 8;
  return want < 1 ? 1 : (int)want;
}

// out[e][z] = sum over the splits of partial[s][e][z], in the order of s
__global__ void reduce_splits(const float2* __restrict__ partial, float2* __restrict__ out, long n, int nsplit) {
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    float2 v = partial[i];
    for (int s = 1; s < nsplit; ++s) { const float2 p = partial[(size_t)s * n + i]; v.x += p.x; v.y += p.y; }
    out[i] = v;
  }
}

// x [nbatch][n2][n2] -> out [nb^2][nbatch] complex;  T [n2][nb^2]
// grid.y > 1: split blockIdx.y takes its share of the rows and writes out + blockIdx.y * nb^2 * nbatch (partial spectra)
__global__ __launch_bounds__(NT) void analysis_kernel(const float* __restrict__ x, const float* __restrict__ T,
                                                      float2* __restrict__ out, int n2, int nb, long nbatch, int RB) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  const int h = n2 / 2, hg = h + 1, nbp = pad(nb, 2), nspec = nb * nb;
  float2* tab = reinterpret_cast<float2*>(smem);      // [hg][nbp]
  float2* EO = tab + hg * nbp;                        // [hg][RB]
  float2* X = EO + hg * RB;                           // [RB][nbp]
  const long z = blockIdx.x;
  const int t = threadIdx.x;
  const float* xs = x + (size_t)z * n2 * n2;
  const int rps = rows_per_split(n2, RB, gridDim.y);
  const int rbeg = blockIdx.y * rps, rend = rbeg + rps < n2 ? rbeg + rps : n2;       // this workgroup's rows
  out += (size_t)blockIdx.y * nspec * nbatch;

  for (int i = t; i < hg * nbp; i += NT) {
    const int j = i / nbp, k = i - j * nbp;
    tab[i] = k < nb ? dft_common::cs_entry(j, k, n2) : make_float2(0.f, 0.f);
  }
  // the two table entries of this thread: e0 = t, e1 = t + NT (b^2 <= 1024)
  int em[2], eok[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) {
    const int e = t + q * NT;
    eok[q] = e < nspec;
    const int l = isqrt_floor(eok[q] ? e : 0);
    em[q] = (eok[q] ? e : 0) - l * l - l;
  }
  float2 acc[2] = {make_float2(0.f, 0.f), make_float2(0.f, 0.f)};

  float v1[PF], v2[PF];
  const int per_chunk = RB * hg;
  auto prefetch = [&](int row0) {
    Walk2 wk;
    wk.init(t, NT, hg);
#pragma unroll
    for (int u = 0; u < PF; ++u) {
      const int r = row0 + wk.row, a = wk.col;
      const bool ok = t + u * NT < per_chunk && r < rend;
      const bool paired = a > 0 && a < h;
      const int o = ok ? r * n2 + a : 0;
      v1[u] = xs[o];
      v2[u] = xs[ok && paired ? r * n2 + n2 - a : o];      // unpaired: not used below
      if (!ok) v1[u] = v2[u] = 0.f;
      wk.step();
    }
  };
  prefetch(rbeg);
  for (int row0 = rbeg; row0 < rend; row0 += RB) {
    {   // registers -> folded rows in LDS
      Walk2 wk;
      wk.init(t, NT, hg);
#pragma unroll
      for (int u = 0; u < PF; ++u) {
        if (t + u * NT < per_chunk) {
          const int a = wk.col;
          const bool paired = a > 0 && a < h;
          EO[a * RB + wk.row] = paired ? make_float2(v1[u] + v2[u], v1[u] - v2[u]) : make_float2(v1[u], 0.f);
        }
        wk.step();
      }
    }
    __syncthreads();
    if (row0 + RB < rend) prefetch(row0 + RB);
    // row transform: 2 rows x 2 frequencies per thread
    const int nmp = nbp / 2, items = RB / 2 * nmp;
    for (int it = t; it < items; it += NT) {
      const int rp = it / nmp, mp = it - rp * nmp;
      const float4* eo = reinterpret_cast<const float4*>(EO + 2 * rp);
      const float4* tb = reinterpret_cast<const float4*>(tab + 2 * mp);
      float re[2][2] = {{0.f, 0.f}, {0.f, 0.f}}, im[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
      for (int a = 0; a <= h; ++a) {
        const float4 e = eo[a * (RB / 2)], w = tb[a * nmp];     // e: (E0, O0, E1, O1); w: (c0, s0, c1, s1)
        re[0][0] = fmaf(e.x, w.x, re[0][0]); im[0][0] = fmaf(e.y, w.y, im[0][0]);
        re[0][1] = fmaf(e.x, w.z, re[0][1]); im[0][1] = fmaf(e.y, w.w, im[0][1]);
        re[1][0] = fmaf(e.z, w.x, re[1][0]); im[1][0] = fmaf(e.w, w.y, im[1][0]);
        re[1][1] = fmaf(e.z, w.z, re[1][1]); im[1][1] = fmaf(e.w, w.w, im[1][1]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i)
        *reinterpret_cast<float4*>(X + (2 * rp + i) * nbp + 2 * mp) = make_float4(re[i][0], -im[i][0], re[i][1], -im[i][1]);
    }
    __syncthreads();
    // table contraction over the rows of this chunk
    const int nrow = rend - row0 < RB ? rend - row0 : RB;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      if (!eok[q]) continue;
      const int m = em[q], am = m < 0 ? -m : m;
      const float* tp = T + (size_t)row0 * nspec + t + q * NT;
      float ar = 0.f, ai = 0.f;
#pragma unroll 8
      for (int r = 0; r < nrow; ++r) {
        const float tv = tp[(size_t)r * nspec];
        const float2 xv = X[r * nbp + am];
        ar = fmaf(tv, xv.x, ar); ai = fmaf(tv, xv.y, ai);
      }
      acc[q].x += ar; acc[q].y += m < 0 ? -ai : ai;            // X[-m] = conj X[m]
    }
    // no barrier here: the next chunk first overwrites EO (its readers passed the barrier above) and writes X only
    // behind its own first barrier
  }
#pragma unroll
  for (int q = 0; q < 2; ++q)
    if (eok[q]) out[(size_t)(t + q * NT) * nbatch + z] = acc[q];
}

// xhat [nb^2][nbatch] complex -> y [nbatch][n2][n2];  T [n2][nb^2]; grid.y splits the rows
__global__ __launch_bounds__(NT) void synthesis_kernel(const float2* __restrict__ xhat, const float* __restrict__ T,
                                                       float* __restrict__ y, int n2, int nb, long nbatch) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  constexpr int RB = 64;
  const int h = n2 / 2, hp = pad(h + 1, 2), nspec = nb * nb;
  float2* tab = reinterpret_cast<float2*>(smem);      // [nb][hp]
  float2* xh = tab + nb * hp;                         // [nb^2]
  float2* AB = xh + pad(nspec, 2);                    // [nb][RB]
  const long z = blockIdx.x;
  const int t = threadIdx.x;
  float* ys = y + (size_t)z * n2 * n2;

  for (int i = t; i < nb * hp; i += NT) {
    const int k = i / hp, j = i - k * hp;
    tab[i] = j <= h ? dft_common::cs_entry(j, k, n2) : make_float2(0.f, 0.f);
  }
  for (int e = t; e < nspec; e += NT) xh[e] = xhat[(size_t)e * nbatch + z];
  __syncthreads();
  const int rps = rows_per_split(n2, RB, gridDim.y);
  const int rbeg = blockIdx.y * rps, rend = rbeg + rps < n2 ? rbeg + rps : n2;

  for (int row0 = rbeg; row0 < rend; row0 += RB) {
    // A, B of the rows of this chunk: thread = (row, m >= 0), sum over l >= m
    for (int it = t; it < RB * nb; it += NT) {
      const int r = it / nb, m = it - r * nb;
      float a = 0.f, b = 0.f;
      // every lane walks all degrees (entries with l < m are read at a clamped index and dropped): the trip count is
      // uniform and the table loads of several degrees are in flight together
      const float* tp = T + (size_t)(row0 + r < n2 ? row0 + r : 0) * nspec;
#pragma unroll 8
      for (int l = 0; l < nb; ++l) {
        const int c = l * l + l;
        const bool in = l >= m;
        const int ep = in ? c + m : c, en = in ? c - m : c;
        const float tpv = in ? tp[ep] : 0.f, tmv = in && m > 0 ? tp[en] : 0.f;
        const float2 xp = xh[ep], xm = xh[en];
        a = fmaf(tpv, xp.x, a); b = fmaf(tpv, xp.y, b);
        a = fmaf(tmv, xm.x, a); b = fmaf(-tmv, xm.y, b);
      }
      if (row0 + r >= n2) a = b = 0.f;
      AB[m * RB + r] = make_float2(a, b);
    }
    __syncthreads();
    // rows: 2 rows x 2 angles alpha <= h per thread
    const int nap = hp / 2, items = RB / 2 * nap;
    for (int it = t; it < items; it += NT) {
      const int rp = it / nap, ap = it - rp * nap;
      const float4* ab = reinterpret_cast<const float4*>(AB + 2 * rp);
      const float4* tb = reinterpret_cast<const float4*>(tab + 2 * ap);
      float yc[2][2] = {{0.f, 0.f}, {0.f, 0.f}}, yv[2][2] = {{0.f, 0.f}, {0.f, 0.f}};
      for (int m = 0; m < nb; ++m) {
        const float4 s = ab[m * (RB / 2)], w = tb[m * nap];     // s: (A0, B0, A1, B1); w: (c0, s0, c1, s1)
        yc[0][0] = fmaf(s.x, w.x, yc[0][0]); yv[0][0] = fmaf(s.y, w.y, yv[0][0]);
        yc[0][1] = fmaf(s.x, w.z, yc[0][1]); yv[0][1] = fmaf(s.y, w.w, yv[0][1]);
        yc[1][0] = fmaf(s.z, w.x, yc[1][0]); yv[1][0] = fmaf(s.w, w.y, yv[1][0]);
        yc[1][1] = fmaf(s.z, w.z, yc[1][1]); yv[1][1] = fmaf(s.w, w.w, yv[1][1]);
      }
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int r = row0 + 2 * rp + i;
        if (r >= n2) continue;
#pragma unroll
        for (int k = 0; k < 2; ++k) {
          const int a = 2 * ap + k;
          if (a > h) continue;
          ys[r * n2 + a] = yc[i][k] - yv[i][k];
          if (a > 0 && a < h) ys[r * n2 + n2 - a] = yc[i][k] + yv[i][k];
        }
      }
    }
    __syncthreads();
  }
}

}  // namespace s2_real
