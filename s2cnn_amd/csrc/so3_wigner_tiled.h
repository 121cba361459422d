// Contraction with the Wigner table for real signals, tiled through LDS (FMA bound work that must
// not re-read HBM): a workgroup owns one frequency m, all n >= 0, a tile of 16 batch items and
// streams the reduction index (beta for analysis, l for synthesis) in chunks.
//
//   analysis : out[l,m,n,z] = sum_beta T[beta, lmn] X[z,beta,m,n]          (accumulators over l)
//   synthesis: S[z,beta,m,n] = sum_l   T[beta, lmn] xs[l,m,n,z]            (accumulators over beta)
//              xs = (xhat[l,m,n] + (-1)^(m-n) conj xhat[l,-m,-n]) / 2
//
// The table is consumed in a packed, zero-padded order that makes every chunk one contiguous block:
//   analysis : Tp[part][mi][beta][n (32)][l (32)]        (pack_table_analysis; [n (16)][l (16)] for small problems)
//   synthesis: Tq[part][mi][l (nb)][n (32)][beta (64)]   (pack_table_synthesis; [n (16)][beta (32)] for small grids)
// with zeros outside max(|m|, n) <= l < number of degrees, n < nb, beta < 2 b_grid.
// A workgroup covers 32 values of n and 32 degrees (analysis) or 64 betas (synthesis); larger problems are cut
// into parts, one more grid dimension: analysis (l0, n0) = (0,0), (32,0), (32,32) (n <= l), synthesis
// (n0, beta0) in {0, 32} x {0, 64}.
// Requirements: nb = min(b_grid, b_spec) <= 64, degrees <= 64 (analysis), 2 b_grid <= 128 (synthesis).
#pragma once
#include <hip/hip_runtime.h>

namespace wigner_tiled {

constexpr int ZT = 16;        // batch items per workgroup
constexpr int KB = 8;         // analysis: betas per chunk
constexpr int SLD = 33;       // synthesis: z stride (complex) of the spectrum chunk
constexpr int QLD = 68;       // synthesis: n stride (floats) of the T chunk, 64 betas + pad
constexpr int LC = 4;         // synthesis: degrees per chunk (LDS stays under 64 KB)

__device__ __forceinline__ int lmn_index(int l, int m, int n) { return l * (4 * l * l - 1) / 3 + (l + m) * (2 * l + 1) + (l + n); }

// Workgroup -> item (o, zi) of no x nz.  Consecutive workgroups go round-robin over the 8 XCDs; the items, o-major,
// are cut into 8 contiguous ranges of equal length, one per XCD: every XCD gets the same number of workgroups whatever
// no is, and those of one XCD that run together share o (and so the table slab in that XCD's L2).  Returns false for
// padding workgroups.
__device__ __forceinline__ bool decode_item(int no, int nz, int& o, int& zi) {
  const int wid = blockIdx.x;
  const int xcd = wid & 7, slot = wid >> 3;
  const int total = no * nz, per = (total + 7) >> 3;
  const int item = xcd * per + slot;
  if (item >= total) return false;
  o = item / nz;
  zi = item - o * nz;
  return true;
}
inline int grid_items(int no, long nz) { return (int)(8L * ((no * nz + 7) / 8)); }

// Workgroup -> (m, z tile); o = 0, 1, 2, ... is m = 0, 1, -1, 2, -2, ...
__device__ __forceinline__ bool decode_block(int MW, int nb, int nzt, int& m, int& zt) {
  int o;
  if (!decode_item(MW, nzt, o, zt)) return false;
  m = (o & 1) ? (o + 1) / 2 : -(o / 2);
  return true;
}

inline int grid_size(int MW, long nbatch) { return grid_items(MW, (nbatch + ZT - 1) / ZT); }

// The same for the synthesis, whose work per workgroup falls with |m| (no degree below |m| contributes): equal counts
// of consecutive o would give the first XCD all the long ones.  Whole frequencies are dealt to the XCDs instead, in the
// order o = 0, 1, 2, ... of falling work, back and forth (XCD 0 .. 7, then 7 .. 0, ...): every XCD gets long and short
// ones, and an uneven last sweep holds the shortest.
__device__ __forceinline__ bool decode_block_by_weight(int MW, int nzt, int& m, int& zt) {
  const int wid = blockIdx.x;
  const int xcd = wid & 7, slot = wid >> 3;
  const int sweep = slot / nzt;
  zt = slot - sweep * nzt;
  const int o = 8 * sweep + ((sweep & 1) ? 7 - xcd : xcd);
  if (o >= MW) return false;
  m = (o & 1) ? (o + 1) / 2 : -(o / 2);
  return true;
}
inline int grid_size_by_weight(int MW, long nbatch) { return (int)(8L * ((MW + 7) / 8) * ((nbatch + ZT - 1) / ZT)); }

// parts of the analysis: degrees [l0, l0 + 32) x frequencies n in [n0, n0 + 32)
__host__ __device__ inline int parts_analysis(int nb, int nl) { return nl <= 32 ? 1 : nb <= 32 ? 2 : 3; }
__host__ __device__ inline void part_analysis(int part, int& l0, int& n0) { l0 = part >= 1 ? 32 : 0; n0 = part == 2 ? 32 : 0; }
// The synthesis tile: 32 frequencies x 64 betas, or 16 x 32 where the whole problem fits that (b <= 16 on either side:
// the grids of the reference's own models), so that lanes and accumulators are not spent on padding.
__host__ __device__ inline bool small_synthesis(int n2, int nb) { return nb <= 16 && n2 <= 32; }
// parts of the synthesis: n in [n0, n0 + 32) x betas [beta0, beta0 + 64)
__host__ __device__ inline int parts_synthesis(int n2, int nb) { return (nb > 32 ? 2 : 1) * (n2 > 64 ? 2 : 1); }
__host__ __device__ inline void part_synthesis(int part, int nb, int& n0, int& beta0) {
  const int pn = nb > 32 ? 2 : 1;
  n0 = 32 * (part % pn); beta0 = 64 * (part / pn);
}

__host__ __device__ inline size_t packed_floats_analysis_part(int n2, int nb) { return (size_t)(2 * nb - 1) * n2 * 1024; }
// The analysis table tile: 32 frequencies x 32 degrees per beta, or 16 x 16 where the whole problem fits that (the padding
// of the larger tile would be three quarters of all the table bytes a workgroup reads).
__host__ __device__ inline bool small_analysis(int nb, int nl) { return nb <= 16 && nl <= 16; }
__host__ __device__ inline size_t packed_floats_analysis_small(int n2, int nb) { return (size_t)(2 * nb - 1) * n2 * 256; }
__host__ __device__ inline size_t packed_floats_synthesis_part(int nb) { return (size_t)(2 * nb - 1) * nb * 32 * 64; }
__host__ __device__ inline size_t packed_floats_synthesis_small(int nb) { return (size_t)(2 * nb - 1) * nb * 16 * 32; }
__host__ __device__ inline size_t packed_floats_analysis(int n2, int nb, int nl) {
  return small_analysis(nb, nl) ? packed_floats_analysis_small(n2, nb) : parts_analysis(nb, nl) * packed_floats_analysis_part(n2, nb);
}
__host__ __device__ inline size_t packed_floats_synthesis(int n2, int nb) {
  return small_synthesis(n2, nb) ? packed_floats_synthesis_small(nb) : parts_synthesis(n2, nb) * packed_floats_synthesis_part(nb);
}

// one thread per packed element
__global__ void pack_table_analysis(const float* __restrict__ T, float* __restrict__ Tp, int n2, int nb, int nl) {
  const bool small = small_analysis(nb, nl);
  const size_t per_part = small ? packed_floats_analysis_small(n2, nb) : packed_floats_analysis_part(n2, nb), total = packed_floats_analysis(n2, nb, nl);
  const long nspec = (long)nl * (4L * nl * nl - 1) / 3;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    int l0 = 0, n0 = 0;
    if (!small) part_analysis((int)(i / per_part), l0, n0);
    const size_t ip = i % per_part;
    const int l = l0 + (int)(small ? ip & 15 : ip & 31), n = n0 + (int)(small ? (ip >> 4) & 15 : (ip >> 5) & 31);
    const size_t r = small ? ip >> 8 : ip >> 10;
    const int bt = (int)(r % n2), m = (int)(r / n2) - (nb - 1);
    const int am = m < 0 ? -m : m;
    float v = 0.f;
    if (n < nb && l < nl && l >= am && l >= n) v = T[(size_t)bt * nspec + lmn_index(l, m, n)];
    Tp[i] = v;
  }
}

__global__ void pack_table_synthesis(const float* __restrict__ T, float* __restrict__ Tq, int n2, int nb, int b_spec) {
  const bool small = small_synthesis(n2, nb);
  const size_t per_part = small ? packed_floats_synthesis_small(nb) : packed_floats_synthesis_part(nb), total = packed_floats_synthesis(n2, nb);
  const long nspec = (long)b_spec * (4L * b_spec * b_spec - 1) / 3;
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < total; i += (size_t)gridDim.x * blockDim.x) {
    int n0 = 0, beta0 = 0;
    if (!small) part_synthesis((int)(i / per_part), nb, n0, beta0);
    const size_t ip = i % per_part;
    const int bt = beta0 + (int)(small ? ip & 31 : ip & 63), n = n0 + (int)(small ? (ip >> 5) & 15 : (ip >> 6) & 31);
    const size_t r = small ? ip >> 9 : ip >> 11;
    const int l = (int)(r % nb), m = (int)(r / nb) - (nb - 1);
    const int am = m < 0 ? -m : m;
    float v = 0.f;
    if (n < nb && bt < n2 && l >= am && l >= n) v = T[(size_t)bt * nspec + lmn_index(l, m, n)];
    Tq[i] = v;
  }
}

// ---------------------------------------------------------------------------------------------
// analysis: 256 threads = 4 waves; wave w owns n = w, w + 4, w + 8, ... (so that a part with fewer than 32
// frequencies still occupies all four waves, and no wave spends matrix-core time on columns beyond the part).
// For each n the contraction
//   D_n[l, (z,c)] += sum_beta T[beta, n, l] * X[beta, z, n].c        (32 degrees x 16 z x (re,im))
// is a 32x32 matrix-core tile with K = beta: v_mfma_f32_32x32x2_f32 takes two betas per instruction,
// A = T (lane = l, half-wave = beta parity), B = X (lane = 2 z + c).  T is zero outside the valid
// (l, n) range, so the padded rows cost matrix-core time but no correctness.
// ---------------------------------------------------------------------------------------------
typedef float v16f __attribute__((ext_vector_type(16)));

// PARTS = false: one part (nb, nl <= 32), the chunk of X is one contiguous run; true: the parts above, the chunk is
// KB*16 row pieces.  TS: the packed table holds TS x TS values per beta (32, or 16 for small_analysis: half the columns, so
// half the accumulators and a third of the LDS, twice the waves per SIMD; the matrix-core tile stays 32 x 32, its rows of
// degrees >= 16 read whatever follows in LDS and are never written out).
template <bool PARTS, int TS = 32>
__global__ __launch_bounds__(256, TS == 16 ? 4 : 2) void wigner_fwd_tiled(const float2* __restrict__ X, const float* __restrict__ Tp,
                                                                          float2* __restrict__ out, int n2, int nb, int nl, long nbatch) {
  constexpr int NJ = TS / 4;                    // columns n per wave
  constexpr int XLD_M = TS + 1;                 // z stride (complex) of the X chunk: (z, c) lanes hit 32 distinct banks
  constexpr int TLD = TS + 4;                   // n stride (floats) of the T chunk, 16-byte aligned rows of TS degrees
  __shared__ __attribute__((aligned(16))) float2 Xs[KB * ZT * XLD_M];
  __shared__ __attribute__((aligned(16))) float Ts[KB * TS * TLD + 32];
  const int MW = 2 * nb - 1, NW = nb;
  const int nzt = (int)((nbatch + ZT - 1) / ZT);
  int m, zt;
  if (!decode_block(MW, nb, nzt, m, zt)) return;
  const int mi = m + nb - 1;
  const long z0 = (long)zt * ZT;
  const int am = abs(m);
  int l0 = 0, n0 = 0;                           // this workgroup's part: degrees l0 .. l0+31, frequencies n0 .. n0+31
  if constexpr (PARTS) part_analysis(blockIdx.y, l0, n0);
  if (am >= l0 + 32) return;                    // no degree of the part reaches |m|
  const int CW = NW - n0 < 32 ? NW - n0 : 32;   // columns of the part

  const int t = threadIdx.x;
  const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l32 = lane & 31, h = lane >> 5;
  v16f acc[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

  // Loads are unconditional (clamped addresses, values zeroed by select) so that all of a chunk's
  // loads are in flight together, and the next chunk is fetched while the current one is consumed.
  static_assert(TS == 32 || (TS == 16 && !PARTS), "table tile");
  constexpr int BW = TS * TS / 4;               // 16-byte words of one beta of the packed table
  constexpr int TPT = KB * BW / 256;            // words of a chunk per thread
  constexpr int XPT = KB * ZT * TS / 256;     // numbers of a chunk of X per thread (NW <= TS)
  float2 xr[XPT];
  float4 tr_[TPT];
  // packed table: the chunk of KB betas is KB * TS * TS contiguous floats; word e = t + 256 i of it is
  // beta_local = e / BW, n = (e % BW) / (TS / 4), l = 4 (e % (TS / 4))
  const float4* tbase = reinterpret_cast<const float4*>(Tp + (PARTS ? blockIdx.y * packed_floats_analysis_part(n2, nb) : 0) + (size_t)mi * n2 * (TS * TS));
  // X is laid out [z tile][mi][beta][z % 16][n]: a chunk (KB betas) is KB*16 rows of NW complex numbers.
  // One part: the chunk is KB*16*NW contiguous numbers; thread slot i covers element e = t + 256 i of it.
  // Several parts: the part takes the CW columns from n0 of every row; a thread keeps one column (lc) and takes rows
  // lr, lr + 8, ...: offsets that advance by constants, nothing per slot to keep in registers.
  const int lc = t & 31, lr = t >> 5;
  const bool colok = lc < CW;
  const float2* xbase = X + ((size_t)zt * MW + mi) * n2 * ZT * NW + (PARTS ? n0 + (colok ? lc : 0) : 0);
  const int nrows = n2 * ZT;
  const int chunk_elems = KB * ZT * NW, n2elems = n2 * ZT * NW;
  const float inv_nw = 1.0f / (float)NW;         // e / NW for e < 4096, NW <= 32: (e + 0.5) * inv_nw truncates exactly
  // LDS that no load fills (columns n >= CW of the X chunk, the rows of degrees >= TS of the T chunk) only reaches rows and
  // columns of the tile that are skipped or never written out: it needs no clearing.

  auto load_chunk = [&](int b0) {
#pragma unroll
    for (int i = 0; i < XPT; ++i) {
      if constexpr (PARTS) {
        const int row = b0 * ZT + lr + 8 * i;                  // beta * 16 + z
        const bool ok = colok && row < nrows;
        const float2 v = xbase[ok ? row * NW : 0];
        xr[i] = ok ? v : make_float2(0.f, 0.f);
      } else {
        const int e = b0 * ZT * NW + t + 256 * i;
        const float2 v = xbase[e < n2elems ? e : 0];
        xr[i] = e < n2elems ? v : make_float2(0.f, 0.f);
      }
    }
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int e = t + 256 * i, bt = e / BW;
      const int bc = b0 + bt < n2 ? b0 + bt : n2 - 1;
      const float4 v = tbase[(size_t)bc * BW + e % BW];
      tr_[i] = b0 + bt < n2 ? v : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };

  // operand addresses of this lane: A = Ts[(beta_local * 32 + n) * TLD + l], B = Xs[(beta_local * 16 + z) * XLD_M + n].c
  const float* Xf = reinterpret_cast<const float*>(Xs);
  const int a_off = (h * TS + wave) * TLD + l32;
  const int b_off = ((h * ZT + (l32 >> 1)) * XLD_M + wave) * 2 + (l32 & 1);

  load_chunk(0);
  for (int b0 = 0; b0 < n2; b0 += KB) {
    __syncthreads();
    if constexpr (PARTS) {
      if (colok) {
#pragma unroll
        for (int i = 0; i < XPT; ++i) Xs[(lr + 8 * i) * XLD_M + lc] = xr[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < XPT; ++i) {
        const int e = t + 256 * i;
        const int row = (int)(((float)e + 0.5f) * inv_nw);     // beta_local * 16 + z
        if (e < chunk_elems) Xs[row * XLD_M + (e - row * NW)] = xr[i];
      }
    }
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int e = t + 256 * i, r = e % BW;
      *reinterpret_cast<float4*>(Ts + ((e / BW) * TS + r / (TS / 4)) * TLD + 4 * (r % (TS / 4))) = tr_[i];
    }
    __syncthreads();
    if (b0 + KB < n2) load_chunk(b0 + KB);
#pragma unroll
    for (int q = 0; q < KB / 2; ++q) {          // beta pair (2q, 2q+1) of the chunk
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if (4 * j + wave >= CW) continue;         // the same for the whole wave
        const float a = Ts[a_off + (2 * q * TS + 4 * j) * TLD];
        const float b = Xf[b_off + (2 * q * ZT * XLD_M + 4 * j) * 2];
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[j], 0, 0, 0);
      }
    }
  }

  // ---- write out[lmn][z].c and its mirror (-m,-n); (m < 0, n = 0) is written by the workgroup of -m.
  // Accumulator register v of lane (l32 = 2 z + c, h) holds degree l = l0 + 8 (v / 4) + 4 h + v % 4.
  const long z = z0 + (l32 >> 1);
  if (z >= nbatch) return;
  const int c = l32 & 1;
  float* outf = reinterpret_cast<float*>(out) + z * 2 + c;
  const size_t rowf = (size_t)nbatch * 2;        // floats per spectral row
  // lmn(l, m, n) = lbase + m (2l+1) + n with lbase = l(4l^2-1)/3 + l(2l+1) + l; the mirror is lbase - m(2l+1) - n
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int l = l0 + 8 * (v / 4) + 4 * h + (v % 4);
    if (l >= nl || l < am) continue;
    const int lcoef = 2 * l + 1;
    const int lbase = l * (4 * l * l - 1) / 3 + l * lcoef + l;
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int n = n0 + 4 * j + wave;
      if (n >= NW || n > l || (n == 0 && m < 0)) continue;
      const float sg = (((m - n) & 1) ? -1.f : 1.f) * (c ? -1.f : 1.f);
      const int d = m * lcoef + n;
      outf[(size_t)(lbase + d) * rowf] = acc[j][v];
      if (n > 0 || m > 0) outf[(size_t)(lbase - d) * rowf] = sg * acc[j][v];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// analysis with the spectrum written in the real basis (float rows [lmn][nbatch]; the entries (+-m, +-n) of a degree hold
// the cos cos, cos sin, sin cos and sin sin coefficients, as s2cnn_so3_spectrum_to_real lays them out).  One part only
// (nb, nl <= 32).  Those four coefficients mix the complex ones of +m and -m at the same n >= 0:
//   cc = A.x + sm C.x,  ss = A.x - sm C.x,  cs = -A.y - sm C.y,  sc = A.y - sm C.y,    A at (m, n), C at (-m, n), sm = (-1)^m
// and the table of -m is that of +m read backwards in beta: T[2b-1-k; l,m,n] = (-1)^(l-n) T[k; l,-m,n].  So a workgroup owns
// |m| and, instead of 16 batch items x (re, im), 8 batch items (X comes in tiles of 8) x four combinations of the two input rows,
//   U1 = P.x + s0 Q.x, U2 = P.x - s0 Q.x, V1 = P.y + s0 Q.y, V2 = P.y - s0 Q.y,   P = X[k, m, n], Q = X[2b-1-k, -m, n],
//   s0 = sm (-1)^n,
// as 32 rows (combination x batch item) of a matrix-core tile whose 32 columns are the degrees, with the table of +m: an
// even degree gets (cc, ss, -cs, sc) = T (U1, U2, V1, V2), an odd one (ss, cc, sc, -cs).  A lane then holds, for its degree,
// four consecutive batch items of each combination: one 16-byte store per coefficient row.  Same matrix-core work as the complex kernel, no conversion pass, half
// the bytes written.  Rows with m = 0 or n = 0 hold two coefficients (scaled by 1/sqrt 2, or 1/2 for the single one at
// m = n = 0); the other columns are not written.
// ---------------------------------------------------------------------------------------------
constexpr int ZH = 8;         // batch items per workgroup of the real-basis analysis

inline int grid_size_half(int nb, long nbatch) { return grid_items(nb, (nbatch + ZH - 1) / ZH); }

// A workgroup takes 16 of the columns n (blockIdx.y picks the half when the table tile holds 32): four accumulator tiles per
// wave and 28 to 36 KB of LDS leave room for three or four waves per SIMD.  TS: the packed table holds TS x TS values per beta; with
// TS = 16 the rows of degrees >= 16 of the 32 x 32 matrix-core tile read whatever follows in LDS and are never written out.
constexpr int NC = 16;        // columns n per workgroup of the real-basis analysis

template <int TS = 32>
__global__ __launch_bounds__(256, TS == 16 ? 4 : 3) void wigner_fwd_tiled_real(const float2* __restrict__ X, const float* __restrict__ Tp,
                                                                float* __restrict__ out, int n2, int nb, int nl, long nbatch) {
  constexpr int NJ = NC / 4;                    // columns n per wave
  constexpr int XL = NC + 1;                    // n stride of the X chunk (float4): z stride = 4 banks, the 32 lanes of a beta read 32 banks
  constexpr int TL = TS + 4;                    // n stride (floats) of the T chunk, 16-byte aligned rows of TS degrees
  __shared__ __attribute__((aligned(16))) float4 Xs[KB * ZH * XL];       // [beta_local][z][n] of (U1, U2, V1, V2)
  __shared__ __attribute__((aligned(16))) float Ts[KB * NC * TL + 32];   // [beta_local][n][l]
  const int MW = 2 * nb - 1, NW = nb;
  const int nzh = (int)((nbatch + ZH - 1) / ZH);
  int am, zh;
  if (!decode_item(nb, nzh, am, zh)) return;
  const long z0 = (long)zh * ZH;
  const int n0 = NC * blockIdx.y;               // this workgroup's columns: n0 .. n0 + 15
  if (n0 >= NW) return;
  const int CW = NW - n0 < NC ? NW - n0 : NC;

  const int t = threadIdx.x;
  const int lane = t & 63, wave = __builtin_amdgcn_readfirstlane(t >> 6);
  const int l32 = lane & 31, h = lane >> 5;
  v16f acc[NJ];
#pragma unroll
  for (int j = 0; j < NJ; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

  static_assert(TS == 32 || TS == 16, "table tile");
  constexpr int BW = TS * TS / 4;               // 16-byte words of one beta of the packed table
  constexpr int CWD = NC * TS / 4;              // of which this workgroup's columns are CWD contiguous ones
  constexpr int TPT = KB * CWD / 256;           // words of a chunk per thread
  constexpr int XPT = KB * ZH * NC / 256;       // numbers of a chunk of one input row per thread
  float2 xp[XPT], xq[XPT];
  float4 tr_[TPT];
  const float4* tbase = reinterpret_cast<const float4*>(Tp + (size_t)(am + nb - 1) * n2 * (TS * TS)) + n0 * (TS / 4);
  // LDS that no load fills (columns n >= CW, the rows of degrees >= TS) only reaches rows and columns of the tile that are
  // never written out: it needs no clearing.
  // X is laid out [z / 8][mi][beta][z % 8][n]: the two input rows of this workgroup are contiguous, 8 NW numbers per beta.
  // A thread keeps one column (lc) and takes the rows (beta_local, z) = lr, lr + 16, ... of the chunk's KB * 8 (two betas
  // per slot): offsets that advance by constants, nothing per slot to keep in registers.
  const int lc = t & (NC - 1), lr = t / NC;
  const bool colok = lc < CW;
  const int lb = lr >> 3, lz = lr & 7;          // beta_local (of slot 0) and z of this thread's rows
  const int bstep = ZH * NW;                    // numbers between two betas of X
  const float2* xpb = X + (((size_t)zh * MW + (nb - 1 + am)) * n2 * ZH + lz) * NW + n0 + (colok ? lc : 0);
  const float2* xqb = X + (((size_t)zh * MW + (nb - 1 - am)) * n2 * ZH + lz) * NW + n0 + (colok ? lc : 0);

  auto load_chunk = [&](int b0) {
#pragma unroll
    for (int i = 0; i < XPT; ++i) {
      const int bt = b0 + lb + 2 * i;
      const bool ok = colok && bt < n2;
      const float2 p = xpb[ok ? bt * bstep : 0];
      const float2 q = xqb[ok ? (n2 - 1 - bt) * bstep : 0];
      xp[i] = ok ? p : make_float2(0.f, 0.f);
      xq[i] = ok ? q : make_float2(0.f, 0.f);
    }
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int e = t + 256 * i, bt = e / CWD;
      const int bc = b0 + bt < n2 ? b0 + bt : n2 - 1;
      const float4 v = tbase[(size_t)bc * BW + e % CWD];
      tr_[i] = b0 + bt < n2 ? v : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };

  // operand addresses of this lane: A (row l32 = 8 combination + z) = Xs[(beta_local * 8 + z) * XL + n][combination],
  // B (column l32 = degree) = Ts[(beta_local * 16 + n) * TL + l]
  const float* Xf = reinterpret_cast<const float*>(Xs);
  const int a_off = ((h * ZH + (l32 & 7)) * XL + wave) * 4 + (l32 >> 3);
  const int b_off = (h * NC + wave) * TL + l32;
  const float s0 = ((am + lc) & 1) ? -1.f : 1.f;     // (-1)^(m + n) of this thread's column (n0 is even)

  load_chunk(0);
  for (int b0 = 0; b0 < n2; b0 += KB) {
    __syncthreads();
    if (colok) {
#pragma unroll
      for (int i = 0; i < XPT; ++i)
        Xs[(lr + 16 * i) * XL + lc] = make_float4(fmaf(s0, xq[i].x, xp[i].x), fmaf(-s0, xq[i].x, xp[i].x), fmaf(s0, xq[i].y, xp[i].y), fmaf(-s0, xq[i].y, xp[i].y));
    }
#pragma unroll
    for (int i = 0; i < TPT; ++i) {
      const int e = t + 256 * i, r = e % CWD;
      *reinterpret_cast<float4*>(Ts + ((e / CWD) * NC + r / (TS / 4)) * TL + 4 * (r % (TS / 4))) = tr_[i];
    }
    __syncthreads();
    if (b0 + KB < n2) load_chunk(b0 + KB);
#pragma unroll
    for (int q = 0; q < KB / 2; ++q) {          // beta pair (2q, 2q+1) of the chunk
#pragma unroll
      for (int j = 0; j < NJ; ++j) {
        if (4 * j + wave >= CW) continue;         // the same for the whole wave
        const float a = Xf[a_off + (2 * q * ZH * XL + 4 * j) * 4];
        const float b = Ts[b_off + (2 * q * NC + 4 * j) * TL];
        acc[j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a, b, acc[j], 0, 0, 0);
      }
    }
  }

  // Accumulator register v of lane (l32 = degree l, h) holds combination v / 4 of batch item z0 + 4 h + v % 4.  A
  // combination is one coefficient for even degrees and another for odd ones: 0 cc (+m,+n), 1 ss (-m,-n), 2 cs (+m,-n),
  // 3 sc (-m,+n); even degrees: the combination's number, odd ones: that number with its last bit flipped.
  const int l = l32;
  if (l >= nl || l < am) return;
  const long zq = z0 + 4 * h;
  if (zq >= nbatch) return;
  const bool vec = (nbatch & 3) == 0 && (reinterpret_cast<uintptr_t>(out) & 15u) == 0;   // then the four items exist and are aligned
  const float f0 = am > 0 ? 0.70710678118654752f : 0.5f, f1 = am > 0 ? 1.f : 0.70710678118654752f;   // scale at n = 0, n > 0
  const int lcoef = 2 * l + 1;
  const int lbase = l * (4 * l * l - 1) / 3 + l * lcoef + l;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int kind = k ^ (l & 1);
    const int row0 = lbase + ((kind == 0 || kind == 2) ? am : -am) * lcoef;      // column 0 of row +-m of degree l
    const int nsg = (kind == 0 || kind == 3) ? 1 : -1;
    const float sg = kind == 2 ? -1.f : 1.f;
    const bool w0 = kind == 0 || (kind == 3 && am > 0), w1 = kind == 0 || kind == 2 || am > 0;   // the coefficient exists at n = 0, n > 0
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const int n = n0 + 4 * j + wave;            // the same for the whole wave
      if (n >= NW) continue;
      if (!(n <= l && (n > 0 ? w1 : w0))) continue;
      const float g = sg * (n > 0 ? f1 : f0);
      float* dst = out + (long)(row0 + nsg * n) * nbatch + zq;
      if (vec) {
        *reinterpret_cast<float4*>(dst) = make_float4(g * acc[j][4 * k], g * acc[j][4 * k + 1], g * acc[j][4 * k + 2], g * acc[j][4 * k + 3]);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (zq + i < nbatch) dst[i] = g * acc[j][4 * k + i];
      }
    }
  }
}

// ---------------------------------------------------------------------------------------------
// synthesis: 512 threads, thread = (n = t % NP, zq = (t / NP) % 8, beta group = t / (8 NP)); the tile is NP
// frequencies x BP betas x 16 batch items: (32, 64), or (16, 32) for small grids (small_synthesis).  A thread keeps
// BP / (512 / (8 NP)) betas of two batch items.
// REAL: the spectrum comes in the real basis (float rows [lmn][nbatch]; the four entries (+-m, +-n) of a degree hold the
// cos cos, cos sin, sin cos and sin sin coefficients, as s2cnn_so3_spectrum_to_real lays them out), and xs is the complex
// coefficient at (m, n) that they stand for; else complex rows, symmetrised as above.
// ---------------------------------------------------------------------------------------------
template <int NP, int BP, bool REAL = false>
__global__ __launch_bounds__(512) void wigner_inv_tiled(const void* __restrict__ spectrum, const float* __restrict__ Tq_g,
                                                        float2* __restrict__ S, int n2, int nb, int b_spec, long nbatch) {
  const float2* __restrict__ xh = static_cast<const float2*>(spectrum);
  const float* __restrict__ xr = static_cast<const float*>(spectrum);
  constexpr int BH = 512 / (8 * NP);            // beta groups
  constexpr int BPT = BP / BH;                  // betas per thread
  constexpr int QL = BP + 4;                    // n stride (floats) of the T chunk
  constexpr int DEG4 = NP * BP / 4;             // 16-byte words of one degree of the packed table
  constexpr int TPT = LC * DEG4 / 512;          // words of a chunk per thread
  static_assert(LC * DEG4 % 512 == 0 && BPT % 4 == 0, "tile shape");
  __shared__ __attribute__((aligned(16))) float2 xs[LC * ZT * SLD];
  __shared__ __attribute__((aligned(16))) float Tq[LC * NP * QL];
  const int MW = 2 * nb - 1, NW = nb;
  const int nzt = (int)((nbatch + ZT - 1) / ZT);
  int m, zt;
  if (!decode_block_by_weight(MW, nzt, m, zt)) return;
  const int mi = m + nb - 1;
  const long z0 = (long)zt * ZT;
  const int am = abs(m);
  int n0 = 0, beta0 = 0;                        // this workgroup's part: frequencies n0 .. n0+NP-1, betas beta0 .. beta0+BP-1
  if constexpr (NP == 32) part_synthesis(blockIdx.y, nb, n0, beta0);

  const int t = threadIdx.x;
  const int n = t & (NP - 1), zq = (t / NP) & 7, bh = t / (8 * NP);
  float2 acc[BPT][2];
#pragma unroll
  for (int j = 0; j < BPT; ++j) { acc[j][0] = make_float2(0.f, 0.f); acc[j][1] = make_float2(0.f, 0.f); }

  const int xz = t & 15, xn = n0 + (t >> 4);    // spectrum loader: z fastest (contiguous in memory), t / 16 < NP values of n
  const bool xload = (t >> 4) < NP;
  const float hs = ((m & 1) ? -0.5f : 0.5f);    // (-1)^(m-n)/2 = hs * (-1)^n

  // Unconditional (clamped) loads, next chunk fetched while the current one is consumed.
  float2 xa[LC], xb[LC];
  float4 tq[TPT];
  // packed table: degree l of this m is NP*BP contiguous floats; a chunk of LC degrees is LC*DEG4 16-byte words, word
  // e = t + 512 k of it is degree l0 + e / DEG4, n = (e % DEG4) / (BP / 4), beta = 4 (e % (BP / 4))
  const size_t part_floats = NP == 32 ? packed_floats_synthesis_part(nb) : 0;
  const float4* tbase = reinterpret_cast<const float4*>(Tq_g + blockIdx.y * part_floats + (size_t)mi * nb * (NP * BP));
  const long zc = z0 + xz < nbatch ? z0 + xz : nbatch - 1;

  auto load_chunk = [&](int l0) {
#pragma unroll
    for (int i = 0; i < LC; ++i) {
      const int l = l0 + i;
      const bool okx = (xload && l < nb && l >= am && l >= xn && xn < NW);
      if constexpr (REAL) {                       // xa = (r[+|m|, +n], r[-|m|, -n]), xb = (r[-|m|, +n], r[+|m|, -n])
        const int rp = lmn_index(l, am, 0), rm = rp - 2 * am * (2 * l + 1);      // column 0 of the rows +|m| and -|m|
        const int ipp = okx ? rp + xn : 0, imm = okx ? rm - xn : 0, imp = okx ? rm + xn : 0, ipm = okx ? rp - xn : 0;
        xa[i] = make_float2(xr[(size_t)ipp * nbatch + zc], xr[(size_t)imm * nbatch + zc]);
        xb[i] = make_float2(xr[(size_t)imp * nbatch + zc], xr[(size_t)ipm * nbatch + zc]);
      } else {
        const int ia = okx ? lmn_index(l, m, xn) : 0, ib = okx ? lmn_index(l, -m, -xn) : 0;
        xa[i] = xh[(size_t)ia * nbatch + zc];
        xb[i] = xh[(size_t)ib * nbatch + zc];
      }
    }
#pragma unroll
    for (int k = 0; k < TPT; ++k) {
      const int e = t + 512 * k, l = l0 + e / DEG4;
      const float4 v = tbase[(size_t)(l < nb ? l : nb - 1) * DEG4 + e % DEG4];
      tq[k] = l < nb ? v : make_float4(0.f, 0.f, 0.f, 0.f);
    }
  };

  const int lstart = ((am > n0 ? am : n0) / LC) * LC;   // no degree below max(|m|, n0) contributes
  load_chunk(lstart);
  for (int l0 = lstart; l0 < nb; l0 += LC) {
    __syncthreads();
#pragma unroll
    for (int i = 0; i < LC; ++i) {
      const int l = l0 + i;
      const bool okx = (l < nb && l >= am && l >= xn && xn < NW && z0 + xz < nbatch);
      const float sg = (xn & 1) ? -hs : hs;
      const float2 a = xa[i], b = xb[i];
      float2 v;
      if constexpr (REAL) {
        const float pp = a.x, mm = a.y, mp = b.x, pm = b.y;
        const float sm = (m & 1) ? -1.f : 1.f, r2 = 0.70710678118654752f;
        if (am > 0 && xn > 0) v = m > 0 ? make_float2(0.5f * (pp + mm), 0.5f * (mp - pm)) : make_float2(sm * 0.5f * (pp - mm), -sm * 0.5f * (pm + mp));
        else if (xn > 0) v = make_float2(r2 * pp, -r2 * pm);
        else if (am > 0) v = m > 0 ? make_float2(r2 * pp, r2 * mp) : make_float2(sm * r2 * pp, -sm * r2 * mp);
        else v = make_float2(pp, 0.f);
      } else {
        v = make_float2(0.5f * a.x + sg * b.x, 0.5f * a.y - sg * b.y);
      }
      if (xload) xs[(i * ZT + xz) * SLD + (t >> 4)] = okx ? v : make_float2(0.f, 0.f);
    }
#pragma unroll
    for (int k = 0; k < TPT; ++k) {
      const int e = t + 512 * k, r = e % DEG4;
      *reinterpret_cast<float4*>(Tq + ((e / DEG4) * NP + r / (BP / 4)) * QL + 4 * (r % (BP / 4))) = tq[k];
    }
    __syncthreads();
    if (l0 + LC < nb) load_chunk(l0 + LC);
#pragma unroll 2
    for (int i = 0; i < LC; ++i) {
      if (l0 + i < am || l0 + i >= nb) continue;
      const float2 x0 = xs[(i * ZT + 2 * zq) * SLD + n];
      const float2 x1 = xs[(i * ZT + 2 * zq + 1) * SLD + n];
      const float4* tr = reinterpret_cast<const float4*>(Tq + (i * NP + n) * QL + BPT * bh);
#pragma unroll
      for (int b4 = 0; b4 < BPT / 4; ++b4) {
        const float4 tv = tr[b4];
        const float tt[4] = {tv.x, tv.y, tv.z, tv.w};
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          acc[4 * b4 + u][0].x += tt[u] * x0.x; acc[4 * b4 + u][0].y += tt[u] * x0.y;
          acc[4 * b4 + u][1].x += tt[u] * x1.x; acc[4 * b4 + u][1].y += tt[u] * x1.y;
        }
      }
    }
  }

  if (n0 + n >= NW) return;
  const size_t plane = (size_t)MW * NW;
#pragma unroll
  for (int zz = 0; zz < 2; ++zz) {
    const long z = z0 + 2 * zq + zz;
    if (z >= nbatch) continue;
    float2* p = S + ((size_t)z * n2 * MW + mi) * NW + n0 + n;
#pragma unroll
    for (int j = 0; j < BPT; ++j) {
      const int bt = beta0 + BPT * bh + j;
      if (bt < n2) p[(size_t)bt * plane] = acc[j][zz];
    }
  }
}

}  // namespace wigner_tiled
