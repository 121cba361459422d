// SO(3) analysis and synthesis of real signals on the 32^3 grid (bandwidth 16) as ONE kernel each, in the form of the
// 64^3 kernels of so3_fused64.h: a workgroup owns one volume, keeps its half spectrum in registers and walks over beta, so
// the transformed planes never leave the compute unit.  What is the same (the beta fold, the sign rules, the ITEMS, the
// quad layout, the per-volume records and the passes between records and spectral rows) is described there; this file
// says what differs.
//
// A volume of this grid is 1/8 of the work, so a workgroup is 256 threads (4 waves) and SEVERAL volumes are resident on a
// compute unit at once, each in another phase of its step: what the 64^3 kernels arrange inside one workgroup (two halves
// of the waves in different phases, two quad buffers) the hardware scheduler does here between workgroups, and a step is a
// plain sequence: transform a plane pair, barrier, contract it.
//
// A 32-point line is 4 x 8: with j = 8 j1 + j2 in, k = k1 + 4 k2 out,
//   X[k1 + 4 k2] = sum_{j2} w8^{j2 k2} ( w32^{j2 k1} sum_{j1} x[8 j1 + j2] w4^{j1 k1} ):
// pass A (256 threads = (line, j2)) does the 4-point sums and the twiddle in place (slots 8 j1 + j2 -> 8 k1 + j2), pass B
// (128 threads = (line, k1)) the 8-point sums in place (slots 8 k1 + j2 -> 8 k1 + k2): bin k sits at slot
// 8 (k % 4) + k / 4.  The B passes of the two axes are given to different halves of the workgroup, so each SIMD gets one.
//
// ITEMS (c, a, n), c < 4: 480 for 2 x 256 places.  Round 1 holds the 256 items with c = 3 (degrees 12..15: thread t has
// the column a = t / 16, n = t % 16), round 0 the 224 items with c <= 2, so a spectrum below degree 12 skips round 1.
// The assignment is a formula (decode_item), not a table.
#pragma once
#include <hip/hip_runtime.h>
#include "so3_fused64.h"

namespace fused32 {

using fft64::fft4;
using fft64::fft8;
using fused64::buf_load_f32;
using fused64::buf_load_f32x4;
using fused64::buf_store_f32;
using fused64::buf_store_f32x4;
using fused64::flip;
using fused64::lmn_index;
using fused64::make_rsrc;
using fused64::volume_of_block;
using fused64::grid_size;

constexpr int N = 32;
constexpr int PITCH = 33;                  // row pitch of the plane in complex elements (odd: conflict-free rows and columns)
constexpr int LDS_ELEMS = N * PITCH;
constexpr int THREADS = 256;
constexpr int NIT = 2;                     // item rounds
constexpr int NITEMS = 480;                // sum_{c<4} (4c+4)^2
constexpr int NJ = 16;                     // beta pairs
constexpr int NR = 16;                     // frequencies 0 <= a, n < NR
constexpr size_t PACKED_FLOATS = (size_t)NJ * NIT * 2 * THREADS * 4;
constexpr int REC_F4 = NIT * 4 * THREADS;
constexpr size_t REC_BYTES = (size_t)REC_F4 * 16;          // 32768
inline size_t scratch_bytes(long nbatch) { return (size_t)nbatch * REC_BYTES; }
constexpr int WAVES_PER_SIMD = 4;          // four workgroups per compute unit (five or six cost registers and time)

__host__ __device__ constexpr int slot_of(int k) { return 8 * (k & 3) + (k >> 2); }    // where bin (or sample) k of a line sits
__host__ __device__ constexpr int index_of(int s) { return (s >> 3) + 4 * (s & 7); }   // which bin (or sample) slot s holds

// place i = round * THREADS + thread -> its item (c, a, n); false for a place without an item
__host__ __device__ inline bool decode_item(int i, int& c, int& a, int& n) {
  const int it = i >> 8, t = i & 255;
  a = t >> 4; n = t & 15;
  if (it == 1) { c = 3; return true; }
  if (a < 12 && n < 12) { c = 2; return true; }
  const int k = a < 12 ? 4 * a + (n - 12) : 48 + 16 * (a - 12) + n;     // the 112 other threads in order
  if (k < 64) { c = 1; a = k >> 3; n = k & 7; return true; }
  if (k < 80) { c = 0; a = (k - 64) >> 2; n = (k - 64) & 3; return true; }
  c = 0; a = 0; n = 0;
  return false;
}

// what the record passes of so3_fused64.h need to know of this grid
struct Geometry {
  static constexpr int THREADS = fused32::THREADS;
  static constexpr int REC_F4 = fused32::REC_F4;
  static __device__ __forceinline__ bool decode(int i, int& c, int& a, int& n) { return decode_item(i, c, a, n); }
};

// item rounds that carry degrees below nl
inline int active_rounds(int nl) { return nl <= 12 ? 1 : NIT; }

// Packed table, as fused64::pack_table: float index ((((j*NIT + it)*2 + h)*THREADS + t)*4 + u) holds
// 0.5 * T[j, l = 4c+u, m = (h ? -a : +a), n] for the item of place it*THREADS + t.  T is [32][nspec_stride].
__global__ void pack_table(const float* __restrict__ T, float* __restrict__ Tf, long nspec_stride, int nl) {
  for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < PACKED_FLOATS; e += (size_t)gridDim.x * blockDim.x) {
    const int u = (int)(e & 3);
    const int t = (int)((e >> 2) & (THREADS - 1));
    const int h = (int)((e >> 10) & 1);
    const int r = (int)(e >> 11);
    const int it = r % NIT, j = r / NIT;
    int c, a, n;
    float v = 0.f;
    if (decode_item(it * THREADS + t, c, a, n)) {
      const int l = 4 * c + u;
      if (l >= a && l >= n && l < nl) v = 0.5f * T[(size_t)j * nspec_stride + lmn_index(l, h ? -a : a, n)];
    }
    Tf[e] = v;
  }
}

// w32^(d k), k = 1..3, for this thread's d = threadIdx.x / 32 (conjugated for the inverse)
struct Twiddles { float c[3], s[3]; };
template <bool INV>
__device__ __forceinline__ void make_twiddles(Twiddles& tw) {
  const int d = threadIdx.x >> 5;
#pragma unroll
  for (int k = 1; k < 4; ++k) {
    float s, c;
    sincospif((float)(d * k) / 16.0f, &s, &c);     // angle 2 pi d k / 32
    tw.c[k - 1] = c;
    tw.s[k - 1] = INV ? s : -s;
  }
}
__device__ __forceinline__ float2 twmul(float2 v, const Twiddles& tw, int k) {
  return make_float2(v.x * tw.c[k - 1] - v.y * tw.s[k - 1], v.x * tw.s[k - 1] + v.y * tw.c[k - 1]);
}

// pass A of an axis in place, all 256 threads: ROWS: line = row lo, elements along the row; else line = column lo
template <bool INV, bool ROWS>
__device__ __forceinline__ void pass_a(float2* buf, const Twiddles& tw) {
  const int lo = threadIdx.x & 31, d = threadIdx.x >> 5;
  float2* line = ROWS ? buf + lo * PITCH + d : buf + lo + d * PITCH;
  constexpr int stride = ROWS ? 8 : 8 * PITCH;
  float2 v0 = line[0], v1 = line[stride], v2 = line[2 * stride], v3 = line[3 * stride];
  fft4<INV>(v0, v1, v2, v3);
  line[0] = v0; line[stride] = twmul(v1, tw, 1); line[2 * stride] = twmul(v2, tw, 2); line[3 * stride] = twmul(v3, tw, 3);
}
// pass B of the row axis in place, by the 128 threads u = (line, k1)
template <bool INV>
__device__ __forceinline__ void pass_b_rows(float2* buf, int u) {
  float2* line = buf + (u & 31) * PITCH + 8 * (u >> 5);
  float2 v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = line[j];
  fft8<INV>(v);
#pragma unroll
  for (int j = 0; j < 8; ++j) line[j] = v[j];
}
template <bool INV>
__device__ __forceinline__ void pass_b_cols(float2* buf, int u) {
  float2* line = buf + (u & 31) + 8 * (u >> 5) * PITCH;
  float2 v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = line[j * PITCH];
  fft8<INV>(v);
#pragma unroll
  for (int j = 0; j < 8; ++j) line[j * PITCH] = v[j];
}

// quad layout as in so3_fused64.h: quad[a][n] = { Z[+a,n], Z[-a,-n], Z[-a,n], Z[+a,-n] }, rows a <= NR (row NR takes the
// bins of m = 16, which nobody reads), NR + 1 quads per row (the last takes n' = 16)
constexpr int QUAD_PITCH = NR * 4 + 14;
constexpr int QUAD_ELEMS = (NR + 1) * QUAD_PITCH;
__host__ __device__ constexpr int quad_row(int a) { return a * QUAD_PITCH + 2 * (a >> 3); }

// ---------------------------------------------------------------------------------------------
// analysis: x [nbatch][32][32][32] real -> records of the half spectrum n >= 0
// NA: item rounds with degrees below the output bandwidth; MASK: s2cnn::Prologue (bit masks, 2, are not supported)
// ---------------------------------------------------------------------------------------------
template <int NA, int MASK>
__global__ __launch_bounds__(THREADS, WAVES_PER_SIMD) void analysis_kernel(const float* __restrict__ x, const float* __restrict__ mask,
                                                                          const float* __restrict__ Tf, float4* __restrict__ rec, long nbatch,
                                                                          const float* __restrict__ params, int nfeature) {
  static_assert(MASK != 2, "bit masks exist on the 64^3 grid only");
  constexpr bool MASKED = MASK == 1 || MASK == 4;
  __shared__ __attribute__((aligned(16))) float2 work[LDS_ELEMS];
  __shared__ __attribute__((aligned(16))) float2 quad[QUAD_ELEMS];
  const long z = volume_of_block(nbatch);
  if (z < 0) return;
  const int t = threadIdx.x;
  const int lo = t & 31, d = t >> 5;
  Twiddles tw;
  make_twiddles<false>(tw);
  for (int i = t; i < QUAD_ELEMS; i += THREADS) quad[i] = make_float2(0.f, 0.f);    // the -a half of a = 0 is never written and reads as zero
  float pr_a = 0.f, pr_b = 0.f, pr_p = 0.f, pr_q = 0.f;
  if constexpr (MASK >= 3) {
    const int c = (int)(z % nfeature);
    pr_a = params[c];
    pr_b = params[nfeature + c];
    if constexpr (MASK == 4) { pr_p = params[2 * nfeature + c]; pr_q = params[3 * nfeature + c]; }
  }
  // quad address of the item (complex index), bit 31 = sign bit of (-1)^n
  unsigned adr[NA];
#pragma unroll
  for (int it = 0; it < NA; ++it) {
    int c, a, n;
    decode_item(it * THREADS + t, c, a, n);
    adr[it] = (unsigned)(quad_row(a) + 4 * n) | ((unsigned)(n & 1) << 31);
  }
  // last gamma pass (threads t < 128: row slot lo, k1 = d): where the outputs of row m = index_of(lo) go
  const int m = index_of(lo);
  const int am = m <= 16 ? m : 32 - m;
  const int qa = quad_row(am);
  const int pos_lo = m > 16 ? 2 : 0;                    // place of an output with n >= 0
  const int pos_hi = (m > 16 || m == 0) ? 1 : 3;        // place of an output with n < 0 (m = 0 counts as -0 there)

  float2 accp[NA][4], accm[NA][4];
#pragma unroll
  for (int it = 0; it < NA; ++it)
#pragma unroll
    for (int u = 0; u < 4; ++u) { accp[it][u] = make_float2(0.f, 0.f); accm[it][u] = make_float2(0.f, 0.f); }

  const __amdgpu_buffer_rsrc_t rx = make_rsrc(x + (size_t)z * (N * N * N), N * N * N * 4);
  const __amdgpu_buffer_rsrc_t rm = make_rsrc((MASKED ? mask : x) + (size_t)z * (N * N * N), N * N * N * 4);
  const __amdgpu_buffer_rsrc_t rt = make_rsrc(Tf, (unsigned)(PACKED_FLOATS * 4));
  const unsigned xoff = t * 4;           // + (beta * 1024 + j1 * 256) * 4: row alpha = 8 j1 + d, column gamma = lo
  const unsigned toff = t * 16;
  float pa[4], pb[4];
  float ma[MASKED ? 4 : 1], mb[MASKED ? 4 : 1];
  float4 t1[NA], t2[NA];

  auto load_planes = [&](int j) {        // rows 8 j1 + d of the planes j and 31 - j: 256 contiguous bytes per wave and load
#pragma unroll
    for (int j1 = 0; j1 < 4; ++j1) {
      pa[j1] = buf_load_f32(rx, xoff, (j * 1024 + j1 * 256) * 4);
      pb[j1] = buf_load_f32(rx, xoff, ((31 - j) * 1024 + j1 * 256) * 4);
      if constexpr (MASKED) {
        ma[j1] = buf_load_f32(rm, xoff, (j * 1024 + j1 * 256) * 4);
        mb[j1] = buf_load_f32(rm, xoff, ((31 - j) * 1024 + j1 * 256) * 4);
      }
    }
  };
  auto load_table = [&](int j) {
#pragma unroll
    for (int it = 0; it < NA; ++it) {
      t1[it] = buf_load_f32x4(rt, toff, ((j * NIT + it) * 2 + 0) * (THREADS * 16));
      t2[it] = buf_load_f32x4(rt, toff, ((j * NIT + it) * 2 + 1) * (THREADS * 16));
    }
  };
  // pass A of the alpha axis out of the registers: 4-point transforms over j1, twiddle, -> work[8 k1 + d][lo]
  auto stage_c1 = [&]() {
    float2 v[4];
#pragma unroll
    for (int j1 = 0; j1 < 4; ++j1) {
      if constexpr (MASK == 1) v[j1] = make_float2(s2cnn::relu_pass(pa[j1], ma[j1]), s2cnn::relu_pass(pb[j1], mb[j1]));
      else if constexpr (MASK == 3) v[j1] = make_float2(s2cnn::affine_relu(pa[j1], pr_a, pr_b), s2cnn::affine_relu(pb[j1], pr_a, pr_b));
      else if constexpr (MASK == 4) v[j1] = make_float2(s2cnn::bn_relu_grad(pa[j1], ma[j1], pr_a, pr_b, pr_p, pr_q),
                                                        s2cnn::bn_relu_grad(pb[j1], mb[j1], pr_a, pr_b, pr_p, pr_q));
      else v[j1] = make_float2(pa[j1], pb[j1]);
    }
    fft4<false>(v[0], v[1], v[2], v[3]);
    float2* col = work + d * PITCH + lo;
    col[0] = v[0];
    col[8 * PITCH] = twmul(v[1], tw, 1);
    col[16 * PITCH] = twmul(v[2], tw, 2);
    col[24 * PITCH] = twmul(v[3], tw, 3);
  };
  // pass B of the gamma axis: row slot lo, inputs at slots 8 k1 + j2, outputs n = k1 + 4 k2 -> quad layout
  auto stage_r2 = [&]() {
    float2 v[8];
    const float2* line = work + lo * PITCH + 8 * d;
#pragma unroll
    for (int j2 = 0; j2 < 8; ++j2) v[j2] = line[j2];
    fft8<false>(v);
#pragma unroll
    for (int k2 = 0; k2 < 4; ++k2) quad[qa + 4 * (d + 4 * k2) + pos_lo] = v[k2];                 // n = d + 4 k2 >= 0
#pragma unroll
    for (int k2 = 4; k2 < 8; ++k2) quad[qa + 4 * (32 - d - 4 * k2) + pos_hi] = v[k2];            // the bins -n', n' = 32 - n > 0
    if (d == 0) quad[qa + pos_hi] = v[0];                                                         // n = 0 again as -0
  };
  auto accumulate = [&](int it) {
    const float4* src = reinterpret_cast<const float4*>(quad + (adr[it] & 0x7fffffffu));
    const float4 za = src[0], zb = src[1];              // Z[+a,n], Z[-a,-n] | Z[-a,n], Z[+a,-n]
    const unsigned sb = adr[it] & 0x80000000u;
    // twice the separated planes (the table carries 1/2): P = Z[m,n] + conj Z[-m,-n], P' = (Z[m,n] - conj Z[-m,-n]) / i times (-1)^n
    const float2 Pp = make_float2(za.x + za.z, za.y - za.w);
    const float2 Qp = make_float2(flip(za.y + za.w, sb), flip(za.z - za.x, sb));
    const float2 Pm = make_float2(zb.x + zb.z, zb.y - zb.w);
    const float2 Qm = make_float2(flip(zb.y + zb.w, sb), flip(zb.z - zb.x, sb));
    const float a1[4] = {t1[it].x, t1[it].y, t1[it].z, t1[it].w};
    const float a2[4] = {t2[it].x, t2[it].y, t2[it].z, t2[it].w};
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      // (-1)^(l-n) = (-1)^u (-1)^n for l = 4c+u: the sign of odd u goes into the table operand
      const float b1 = (u & 1) ? -a1[u] : a1[u], b2 = (u & 1) ? -a2[u] : a2[u];
      accp[it][u].x = fmaf(b2, Qp.x, fmaf(a1[u], Pp.x, accp[it][u].x));
      accp[it][u].y = fmaf(b2, Qp.y, fmaf(a1[u], Pp.y, accp[it][u].y));
      accm[it][u].x = fmaf(b1, Qm.x, fmaf(a2[u], Pm.x, accm[it][u].x));
      accm[it][u].y = fmaf(b1, Qm.y, fmaf(a2[u], Pm.y, accm[it][u].y));
    }
  };

  load_planes(0);
  load_table(0);
  __syncthreads();                                  // cleared quads
  for (int j = 0; j < NJ; ++j) {
    stage_c1();
    load_planes(j + 1 < NJ ? j + 1 : NJ - 1);       // clamped, not branched: in flight during the step
    __syncthreads();
    if (t >= THREADS / 2) pass_b_cols<false>(work, t - THREADS / 2);
    __syncthreads();
    pass_a<false, true>(work, tw);
    __syncthreads();
    if (t < THREADS / 2) stage_r2();
    __syncthreads();
#pragma unroll
    for (int it = 0; it < NA; ++it) accumulate(it);
    load_table(j + 1 < NJ ? j + 1 : NJ - 1);
  }

  const __amdgpu_buffer_rsrc_t rr = make_rsrc(rec + (size_t)z * REC_F4, (unsigned)REC_BYTES);
#pragma unroll
  for (int it = 0; it < NA; ++it) {                 // the pass that follows reads these rounds only
    buf_store_f32x4(make_float4(accp[it][0].x, accp[it][0].y, accp[it][1].x, accp[it][1].y), rr, toff, (it * 4 + 0) * (THREADS * 16));
    buf_store_f32x4(make_float4(accp[it][2].x, accp[it][2].y, accp[it][3].x, accp[it][3].y), rr, toff, (it * 4 + 1) * (THREADS * 16));
    buf_store_f32x4(make_float4(accm[it][0].x, accm[it][0].y, accm[it][1].x, accm[it][1].y), rr, toff, (it * 4 + 2) * (THREADS * 16));
    buf_store_f32x4(make_float4(accm[it][2].x, accm[it][2].y, accm[it][3].x, accm[it][3].y), rr, toff, (it * 4 + 3) * (THREADS * 16));
  }
}

// ---------------------------------------------------------------------------------------------
// synthesis: records of the symmetrised spectrum -> y [nbatch][32][32][32] real
//
// Every item adds its share of the bins of a plane pair to a place of its own in a staging area (480 places); a
// reduction sums the places of each column (a, n), one per degree group c >= max(a, n) / 4, in that order, into the plane.
// bias, relu, MOM, moments, yref, params: as fused64::synthesis_kernel (no bit masks).
// ---------------------------------------------------------------------------------------------
__host__ __device__ constexpr int stage_offset(int c) { return c == 0 ? 0 : c == 1 ? 16 : c == 2 ? 80 : 224; }   // sum_{c' < c} (4c'+4)^2

template <int NA, int MOM>
__global__ __launch_bounds__(THREADS, WAVES_PER_SIMD) void synthesis_kernel(const float4* __restrict__ rec, const float* __restrict__ Tf,
                                                                           float* __restrict__ y, long nbatch, const float* __restrict__ bias,
                                                                           int nfeature, int relu, float2* __restrict__ moments,
                                                                           const float* __restrict__ yref, const float* __restrict__ params) {
  __shared__ __attribute__((aligned(16))) float2 work[LDS_ELEMS];
  // places 0 .. NITEMS-1: one per item; ZERO_PLACE: never written, read for the degree groups a column does not have;
  // DUMP_PLACE: written by the threads without an item, never read
  constexpr int ZERO_PLACE = NITEMS, DUMP_PLACE = NITEMS + 1, NPLACES = NITEMS + 2;
  __shared__ __attribute__((aligned(16))) float4 stg_p[NPLACES];     // the item's share of the bins [+a,n], [-a,-n]
  __shared__ __attribute__((aligned(16))) float4 stg_m[NPLACES];     //                              [-a,n], [+a,-n]
  const long z = volume_of_block(nbatch);
  if (z < 0) return;
  const int t = threadIdx.x;
  const int lo = t & 31;
  const float bz = bias ? bias[z % nfeature] : 0.f;
  float ms1 = 0.f, ms2 = 0.f;
  [[maybe_unused]] float mpivot = 0.f;
  Twiddles tw;
  make_twiddles<true>(tw);
  for (int i = t; i < LDS_ELEMS; i += THREADS) work[i] = make_float2(0.f, 0.f);
  for (int i = t; i < NPLACES; i += THREADS) { stg_p[i] = make_float4(0.f, 0.f, 0.f, 0.f); stg_m[i] = make_float4(0.f, 0.f, 0.f, 0.f); }   // places of skipped rounds stay zero

  const __amdgpu_buffer_rsrc_t rr = make_rsrc(rec + (size_t)z * REC_F4, (unsigned)REC_BYTES);
  const __amdgpu_buffer_rsrc_t rt = make_rsrc(Tf, (unsigned)(PACKED_FLOATS * 4));
  const __amdgpu_buffer_rsrc_t ry = make_rsrc(y + (size_t)z * (N * N * N), N * N * N * 4);
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(MOM == 2 ? yref + (size_t)z * (N * N * N) : y, MOM == 2 ? N * N * N * 4 : 0);
  const unsigned toff = t * 16;
  float mom_a = 0.f, mom_b = 0.f;
  if constexpr (MOM == 2) { mom_a = params[z % nfeature]; mom_b = params[nfeature + z % nfeature]; }

  float2 xp[NA][4], xm[NA][4];
  int place[NA];                 // staging place of the item; bit 30: n is odd
#pragma unroll
  for (int it = 0; it < NA; ++it) {
    int c, a, n;
    const bool ok = decode_item(it * THREADS + t, c, a, n);
    place[it] = ok ? (stage_offset(c) + a * (4 * c + 4) + n) | ((n & 1) << 30) : DUMP_PLACE;
    const float4 v0 = buf_load_f32x4(rr, toff, (it * 4 + 0) * (THREADS * 16)), v1 = buf_load_f32x4(rr, toff, (it * 4 + 1) * (THREADS * 16));
    const float4 v2 = buf_load_f32x4(rr, toff, (it * 4 + 2) * (THREADS * 16)), v3 = buf_load_f32x4(rr, toff, (it * 4 + 3) * (THREADS * 16));
    xp[it][0] = make_float2(v0.x, v0.y); xp[it][1] = make_float2(v0.z, v0.w);
    xp[it][2] = make_float2(v1.x, v1.y); xp[it][3] = make_float2(v1.z, v1.w);
    xm[it][0] = make_float2(v2.x, v2.y); xm[it][1] = make_float2(v2.z, v2.w);
    xm[it][2] = make_float2(v3.x, v3.y); xm[it][3] = make_float2(v3.z, v3.w);
  }
  float4 t1[NA], t2[NA];
  auto load_table = [&](int j) {
#pragma unroll
    for (int it = 0; it < NA; ++it) {
      t1[it] = buf_load_f32x4(rt, toff, ((j * NIT + it) * 2 + 0) * (THREADS * 16));
      t2[it] = buf_load_f32x4(rt, toff, ((j * NIT + it) * 2 + 1) * (THREADS * 16));
    }
  };
  // the item's share of a plane pair: S = sum_l t1 xs, S' = sum_l s t2 xs at (+a, n), t1 <-> t2 at (-a, n);
  // complex plane Z = S + i S' at [m,n], its Hermitian partner conj S + i conj S' at [-m,-n]
  auto contribute = [&](int it) {
    const float a1[4] = {t1[it].x, t1[it].y, t1[it].z, t1[it].w};
    const float a2[4] = {t2[it].x, t2[it].y, t2[it].z, t2[it].w};
    float2 Sp = make_float2(0.f, 0.f), Qp = Sp, Sm = Sp, Qm = Sp;
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float b1 = (u & 1) ? -a1[u] : a1[u], b2 = (u & 1) ? -a2[u] : a2[u];
      Sp.x = fmaf(a1[u], xp[it][u].x, Sp.x); Sp.y = fmaf(a1[u], xp[it][u].y, Sp.y);
      Qp.x = fmaf(b2, xp[it][u].x, Qp.x);    Qp.y = fmaf(b2, xp[it][u].y, Qp.y);
      Sm.x = fmaf(a2[u], xm[it][u].x, Sm.x); Sm.y = fmaf(a2[u], xm[it][u].y, Sm.y);
      Qm.x = fmaf(b1, xm[it][u].x, Qm.x);    Qm.y = fmaf(b1, xm[it][u].y, Qm.y);
    }
    const unsigned sb = ((unsigned)place[it] << 1) & 0x80000000u;
    const int pos = place[it] & 0xffff;
    const float qpx = flip(Qp.x, sb), qpy = flip(Qp.y, sb), qmx = flip(Qm.x, sb), qmy = flip(Qm.y, sb);
    stg_p[pos] = make_float4(Sp.x - qpy, Sp.y + qpx, Sp.x + qpy, qpx - Sp.y);
    stg_m[pos] = make_float4(Sm.x - qmy, Sm.y + qmx, Sm.x + qmy, qmx - Sm.y);
  };
  // staging -> work (natural order): thread t takes the column a = t / 16, n = t % 16.  No branches: a degree group the
  // column does not have reads the zero place, a bin that does not exist (-0) goes to the pad column of its row.
  int red_pos[NA == 1 ? 3 : 4], red_dst[4];
  {
    const int a = t >> 4, n = t & 15;
    const int cmin = (a > n ? a : n) >> 2;
#pragma unroll
    for (int c = 0; c < (NA == 1 ? 3 : 4); ++c) red_pos[c] = c >= cmin ? stage_offset(c) + a * (4 * c + 4) + n : ZERO_PLACE;
    const int rp = a * PITCH, rm = ((32 - a) & 31) * PITCH;
    red_dst[0] = rp + n;                                  // [+a, n]
    red_dst[1] = n > 0 ? rm + 32 - n : rm + 32;           // [-a,-n]
    red_dst[2] = a > 0 ? rm + n : rp + 32;                // [-a, n]
    red_dst[3] = a > 0 && n > 0 ? rp + 32 - n : rp + 32;  // [+a,-n]
  }
  auto reduce = [&]() {
    float4 s0 = make_float4(0.f, 0.f, 0.f, 0.f), s1 = s0;
#pragma unroll
    for (int c = 0; c < (NA == 1 ? 3 : 4); ++c) {
      const float4 u0 = stg_p[red_pos[c]], u1 = stg_m[red_pos[c]];
      s0 = make_float4(s0.x + u0.x, s0.y + u0.y, s0.z + u0.z, s0.w + u0.w);
      s1 = make_float4(s1.x + u1.x, s1.y + u1.y, s1.z + u1.z, s1.w + u1.w);
    }
    work[red_dst[0]] = make_float2(s0.x, s0.y);
    work[red_dst[1]] = make_float2(s0.z, s0.w);
    work[red_dst[2]] = make_float2(s1.x, s1.y);
    work[red_dst[3]] = make_float2(s1.z, s1.w);
    // the bins of m = 16 and n = 16 hold what the last transform left there: cleared again
    if (t < 32) { work[16 * PITCH + t] = make_float2(0.f, 0.f); work[t * PITCH + 16] = make_float2(0.f, 0.f); }
  };
  // pass B of the alpha axis by the threads u = t - 128 = (gamma = u % 32, k1 = u / 32): the column of sample gamma sits at
  // slot_of(gamma); outputs rows alpha = k1 + 4 k2.  Real part -> plane j, imaginary part -> plane 31 - j; a wave stores
  // two adjacent rows (256 bytes) at once.
  auto stage_c2_store = [&](int j) {
    const int u = t - THREADS / 2;
    const unsigned yoff = u * 4;                  // + (beta * 1024 + k2 * 128) * 4
    float2 v[8];
    [[maybe_unused]] float2 w[8];
    if constexpr (MOM == 2) {
#pragma unroll
      for (int k = 0; k < 8; ++k)
        w[k] = make_float2(buf_load_f32(rw, yoff, (j * 1024 + k * 128) * 4), buf_load_f32(rw, yoff, ((31 - j) * 1024 + k * 128) * 4));
    }
    const float2* line = work + slot_of(lo) + 8 * (u >> 5) * PITCH;
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = line[k * PITCH];
    fft8<true>(v);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      float ra = v[k].x + bz, rb = v[k].y + bz;
      if constexpr (MOM == 1) {
        if (j == 0 && k == 0) mpivot = ra;
        const float da = ra - mpivot, db = rb - mpivot;
        ms1 += da + db; ms2 = fmaf(da, da, fmaf(db, db, ms2));
      }
      if constexpr (MOM == 2) {
        const float ga = s2cnn::relu_pass(ra, fmaf(mom_a, w[k].x, mom_b)), gb = s2cnn::relu_pass(rb, fmaf(mom_a, w[k].y, mom_b));
        ms1 += ga + gb; ms2 = fmaf(ga, w[k].x, fmaf(gb, w[k].y, ms2));
      }
      if (relu) { ra = s2cnn::relu_f(ra); rb = s2cnn::relu_f(rb); }
      buf_store_f32(ra, ry, yoff, (j * 1024 + k * 128) * 4);
      buf_store_f32(rb, ry, yoff, ((31 - j) * 1024 + k * 128) * 4);
    }
  };

  load_table(0);
  __syncthreads();                                  // cleared work and staging
#pragma unroll
  for (int it = 0; it < NA; ++it) contribute(it);
  load_table(1);
  __syncthreads();
  reduce();
  __syncthreads();
  for (int j = 0; j < NJ; ++j) {
    if (j + 1 < NJ) {                               // the shares of pair j + 1, while pair j is in the plane
#pragma unroll
      for (int it = 0; it < NA; ++it) contribute(it);
      load_table(j + 2 < NJ ? j + 2 : NJ - 1);
    }
    pass_a<true, true>(work, tw);
    __syncthreads();
    if (t < THREADS / 2) pass_b_rows<true>(work, t);
    __syncthreads();
    pass_a<true, false>(work, tw);
    __syncthreads();
    if (t >= THREADS / 2) stage_c2_store(j);
    if (j + 1 < NJ) {
      __syncthreads();
      reduce();
      __syncthreads();
    }
  }
  constexpr int HALF = THREADS / 2;                 // the threads that hold samples: 2 x 8 x 16 each
  if constexpr (MOM == 1) {                         // (mean, squared deviations) per thread, merged pairwise in float64
    __syncthreads();
    double* red = reinterpret_cast<double*>(work);
    constexpr double NT_SAMPLES = 2.0 * 8.0 * NJ;
    if (t >= HALF) {
      red[t - HALF] = (double)mpivot + (double)ms1 / NT_SAMPLES;
      red[t] = (double)ms2 - (double)ms1 * (double)ms1 / NT_SAMPLES;
    }
    __syncthreads();
    double cnt = NT_SAMPLES;
    for (int s = HALF / 2; s > 0; s >>= 1) {
      if (t < s) {
        const double dm = red[t + s] - red[t];
        red[HALF + t] += red[HALF + t + s] + dm * dm * (0.5 * cnt);
        red[t] = 0.5 * (red[t] + red[t + s]);
      }
      cnt *= 2.0;
      __syncthreads();
    }
    if (t == 0) moments[z] = make_float2((float)(red[0] * cnt), (float)red[HALF]);
  }
  if constexpr (MOM == 2) {                         // the threads' partial sums through LDS, pairwise, always in the same order
    __syncthreads();
    float* red = reinterpret_cast<float*>(work);
    if (t >= HALF) { red[t - HALF] = ms1; red[t] = ms2; }
    __syncthreads();
    for (int s = HALF / 2; s > 0; s >>= 1) {
      if (t < s) { red[t] += red[t + s]; red[HALF + t] += red[HALF + t + s]; }
      __syncthreads();
    }
    if (t == 0) moments[z] = make_float2(red[0], red[HALF]);
  }
}

template <int MASK>
inline void launch_analysis_m(int nl, hipStream_t st, const s2cnn::Input& in, const float* Tf, float4* rec, long nbatch) {
  const dim3 grid(grid_size(nbatch)), block(THREADS);
  if (nl <= 12) hipLaunchKernelGGL((analysis_kernel<1, MASK>), grid, block, 0, st, in.x, in.w, Tf, rec, nbatch, in.params, in.nfeature);
  else hipLaunchKernelGGL((analysis_kernel<2, MASK>), grid, block, 0, st, in.x, in.w, Tf, rec, nbatch, in.params, in.nfeature);
}

// in: the signal and what is done to it in the loads (s2cnn::Input; not PRO_BITS)
inline void launch_analysis(int nl, hipStream_t st, const s2cnn::Input& in, const float* Tf, float4* rec, long nbatch) {
  switch (in.kind) {
    case s2cnn::PRO_MASK: launch_analysis_m<1>(nl, st, in, Tf, rec, nbatch); break;
    case s2cnn::PRO_AFFINE_RELU: launch_analysis_m<3>(nl, st, in, Tf, rec, nbatch); break;
    case s2cnn::PRO_BN_RELU_GRAD: launch_analysis_m<4>(nl, st, in, Tf, rec, nbatch); break;
    default: launch_analysis_m<0>(nl, st, in, Tf, rec, nbatch);
  }
}

template <int MOM>
inline void launch_synthesis_m(int nl, hipStream_t st, const float4* rec, const float* Tf, float* y, long nbatch, const float* bias,
                               int nfeature, int relu, float2* moments, const float* yref, const float* params) {
  const dim3 grid(grid_size(nbatch)), block(THREADS);
  if (nl <= 12) hipLaunchKernelGGL((synthesis_kernel<1, MOM>), grid, block, 0, st, rec, Tf, y, nbatch, bias, nfeature, relu, moments, yref, params);
  else hipLaunchKernelGGL((synthesis_kernel<2, MOM>), grid, block, 0, st, rec, Tf, y, nbatch, bias, nfeature, relu, moments, yref, params);
}

// moments: NULL, or two sums per volume: those of the output, or, with yref and params, those of the gradient of a normalisation
inline void launch_synthesis(int nl, hipStream_t st, const float4* rec, const float* Tf, float* y, long nbatch, const float* bias,
                             int nfeature, int relu, float2* moments = nullptr, const float* yref = nullptr, const float* params = nullptr) {
  if (moments && yref) launch_synthesis_m<2>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, moments, yref, params);
  else if (moments) launch_synthesis_m<1>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, moments, nullptr, nullptr);
  else launch_synthesis_m<0>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, nullptr, nullptr, nullptr);
}

}  // namespace fused32
