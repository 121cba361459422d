// SO(3) analysis and synthesis of real signals on the 64^3 grid (bandwidth 32) as ONE kernel each:
// a workgroup owns one volume, keeps its whole half spectrum in registers and walks over beta, so
// the transformed planes never leave the compute unit (no intermediate in HBM).
//
// Per step the workgroup takes the two planes beta_j and beta_{63-j} (j < 32) as one complex plane,
// transforms it inside LDS (radix 8 x 8, see so3_plane_fft64.h) and contracts it with the Wigner
// table.  The table is needed for j < 32 only, because on the SOFT grid beta_{63-j} = pi - beta_j and
//     d^l_{mn}(pi - beta) = (-1)^(l-n) d^l_{-m,n}(beta)          (weights symmetric in j as well),
// and for n >= 0 only, because spectra of real signals obey X[l,-m,-n] = (-1)^(m-n) conj X[l,m,n].
//
// Work decomposition: an ITEM is (c, a, n) = four consecutive degrees l = 4c..4c+3 of the two columns
// (m = +a, n) and (m = -a, n), 0 <= a, n <= 4c+3.  There are sum_c (4c+4)^2 = 3264 items for c < 8;
// a thread owns 7 of them (one per ROUND), i.e. 7 x 4 x 2 complex values in registers.  Which ones is a table
// (so3_fused64_items.h, written by gen_fused64_items.py): consecutive rounds of a thread hold the same column (a, n)
// where they can, because the bins of a column are then read (analysis) or written (synthesis) once for the whole
// RUN of rounds instead of once per item, and items of low degree sit in the first rounds, so that a truncated
// spectrum skips the later ones.  Nothing below depends on the assignment beyond what the table says.
// With P = plane of beta_j, P' = plane of beta_{63-j}, t1 = T[j,l,+a,n], t2 = T[j,l,-a,n], s = (-1)^(l-n):
//   analysis : X[l,+a,n] += t1 P[+a,n] + s t2 P'[+a,n]      X[l,-a,n] += t2 P[-a,n] + s t1 P'[-a,n]
//   synthesis: S[+a,n] = sum_l t1 xs[l,+a,n]   S'[+a,n] = sum_l s t2 xs[l,+a,n]   (and -a with t1 <-> t2)
// The packed table holds t1/2, t2/2 per (j, item, degree) in the order the threads load it.
//
// The two halves of a step overlap: while plane pair j is contracted out of one LDS buffer, pair j+1 is
// transformed in the other, stage by stage between the same barriers.
//
// A spectral row holds ONE 8-byte entry per volume, so a workgroup never touches the spectrum itself:
// it exchanges its registers with a per-volume record in scratch memory (coalesced), and
// spectrum_scatter / spectrum_gather move tiles of 16 volumes between the records and the rows
// (128-byte pieces, mirror half and symmetrisation included).
#pragma once
#include <hip/hip_runtime.h>
#include "so3_plane_fft64.h"
#include "so3_fused64_items.h"

namespace fused64 {

using fft64::N;
using fft64::PITCH;
using fft64::LDS_ELEMS;
using fft64::sigma;

constexpr int THREADS = 512;
constexpr int NIT = 7;             // items per thread
constexpr int NITEMS = 3264;       // sum_{c<8} (4c+4)^2
constexpr int NJ = 32;             // beta pairs
constexpr size_t PACKED_FLOATS = (size_t)NJ * NIT * 2 * THREADS * 4;

// Buffer addressing (uniform descriptor in SGPRs + one 32-bit lane offset + a scalar offset): the bases are
// uniform per workgroup, so no 64-bit address arithmetic is left in vector registers.  Offsets in bytes.
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* base, unsigned bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(base), 0, (int)bytes, 0x00020000);
}
__device__ __forceinline__ float buf_load_f32(__amdgpu_buffer_rsrc_t r, unsigned voff, unsigned soff) {
  return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, (int)soff, 0));
}
// a load with the non-temporal hint: input that is read once (a transform's signal planes)
__device__ __forceinline__ float buf_load_f32_stream(__amdgpu_buffer_rsrc_t r, unsigned voff, unsigned soff) {
  return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, (int)soff, 2));
}
__device__ __forceinline__ float4 buf_load_f32x4(__amdgpu_buffer_rsrc_t r, unsigned voff, unsigned soff) {
  const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)soff, 0);
  return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
}
__device__ __forceinline__ void buf_store_f32(float x, __amdgpu_buffer_rsrc_t r, unsigned voff, unsigned soff) {
  __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(x), r, (int)voff, (int)soff, 0);
}
// the hint chosen at run time by a uniform flag (the instruction carries it as an immediate, so there are two of them)
__device__ __forceinline__ float buf_load_f32_policy(__amdgpu_buffer_rsrc_t r, unsigned voff, unsigned soff, bool stream) {
  return stream ? buf_load_f32_stream(r, voff, soff) : buf_load_f32(r, voff, soff);
}
// the same store with the non-temporal hint (cache policy bit 1): for output that this kernel and the next ones on the
// stream do not find in a cache anyway (a transform's result planes)
__device__ __forceinline__ void buf_store_f32_stream(float x, __amdgpu_buffer_rsrc_t r, unsigned voff, unsigned soff) {
  __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(x), r, (int)voff, (int)soff, 2);
}
__device__ __forceinline__ void buf_store_f32_policy(float x, __amdgpu_buffer_rsrc_t r, unsigned voff, unsigned soff, bool stream) {
  if (stream) buf_store_f32_stream(x, r, voff, soff);
  else buf_store_f32(x, r, voff, soff);
}
using s2cnn::STREAM_BYTES;
__device__ __forceinline__ void buf_store_f32x4(float4 x, __amdgpu_buffer_rsrc_t r, unsigned voff, unsigned soff) {
  u32x4 v; v.x = __float_as_uint(x.x); v.y = __float_as_uint(x.y); v.z = __float_as_uint(x.z); v.w = __float_as_uint(x.w);
  __builtin_amdgcn_raw_buffer_store_b128(v, r, (int)voff, (int)soff, 0);
}

// x with its sign flipped where `signbit` (0 or 0x80000000) is set
__device__ __forceinline__ float flip(float x, unsigned signbit) { return __uint_as_float(__float_as_uint(x) ^ signbit); }

__host__ __device__ inline int lmn_index(int l, int m, int n) { return l * (4 * l * l - 1) / 3 + (l + m) * (2 * l + 1) + (l + n); }

// place i = round * THREADS + thread -> its item (c, a, n); false for a place without an item (a, n then name the
// column of the neighbouring round, so that the place starts no run of its own)
__device__ __forceinline__ bool decode_item(int i, int& c, int& a, int& n) {
  const unsigned e = ITEM_TABLE[i];
  n = (int)(e & 31u); a = (int)((e >> 5) & 31u); c = (int)((e >> 10) & 7u);
  return (e >> 13) & 1u;
}

// Packed table: float index ((((j*NIT + it)*2 + h)*THREADS + t)*4 + u) holds
//   0.5 * T[j, l = 4c+u, m = (h ? -a : +a), n]   for the item (c, a, n) of place it*THREADS + t,
// zero where l < max(a, n), l >= nl, or the slot is padding.  T is [64][nspec_stride].
__global__ void pack_table(const float* __restrict__ T, float* __restrict__ Tf, long nspec_stride, int nl) {
  for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < PACKED_FLOATS; e += (size_t)gridDim.x * blockDim.x) {
    const int u = (int)(e & 3);
    const int t = (int)((e >> 2) & (THREADS - 1));
    const int h = (int)((e >> 11) & 1);
    const int r = (int)(e >> 12);
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

// w64^(d k), k = 0..7, for this wave's d = threadIdx.x / 64 (conjugated for the inverse) as wave-uniform values: they
// live in scalar registers, so the twiddled passes read nothing but their data from LDS.
struct Twiddles { float c[8], s[8]; };
__device__ __forceinline__ float uniform(float x) { return __uint_as_float(__builtin_amdgcn_readfirstlane(__float_as_uint(x))); }
template <bool INV>
__device__ __forceinline__ void make_twiddles(Twiddles& tw) {
  const int d = threadIdx.x >> 6;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    float s, c;
    sincospif((float)(d * k) / 32.0f, &s, &c);   // angle 2 pi d k / 64
    tw.c[k] = uniform(c);
    tw.s[k] = uniform(INV ? s : -s);
  }
}
__device__ __forceinline__ float2 twmul(float2 v, const Twiddles& tw, int k) {
  return make_float2(v.x * tw.c[k] - v.y * tw.s[k], v.x * tw.s[k] + v.y * tw.c[k]);
}

// One radix-8 pass of the in-place 2-D transform of a 64x64 complex plane in LDS by 512 threads
// (natural order in, sigma order out on both axes): P = 0, 1 rows, P = 2, 3 columns.
// A barrier must follow each pass.
template <bool INV, int P>
__device__ __forceinline__ void fft_pass(float2* buf, const Twiddles& tw) {
  using namespace fft64;
  const int lo = threadIdx.x & 63;   // line
  const int d = threadIdx.x >> 6;    // j2 in the first pass of an axis, k1 in the second
  float2* line = P == 0 ? buf + lo * PITCH + d : P == 1 ? buf + lo * PITCH + 8 * d : P == 2 ? buf + lo + d * PITCH : buf + lo + 8 * d * PITCH;
  constexpr int stride = P == 0 ? 8 : P == 1 ? 1 : P == 2 ? 8 * PITCH : PITCH;
  float2 v[8];
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = line[j * stride];
  fft8<INV>(v);
  if (P == 0 || P == 2) {
#pragma unroll
    for (int j = 1; j < 8; ++j) v[j] = twmul(v[j], tw, j);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) line[j * stride] = v[j];
}

// The same pass in two halves, so that independent work can be placed between the LDS reads and their use.
template <int P>
__device__ __forceinline__ void fft_pass_load(const float2* buf, float2 (&v)[8]) {
  using namespace fft64;
  const int lo = threadIdx.x & 63, d = threadIdx.x >> 6;
  const float2* line = P == 0 ? buf + lo * PITCH + d : P == 1 ? buf + lo * PITCH + 8 * d : P == 2 ? buf + lo + d * PITCH : buf + lo + 8 * d * PITCH;
  constexpr int stride = P == 0 ? 8 : P == 1 ? 1 : P == 2 ? 8 * PITCH : PITCH;
#pragma unroll
  for (int j = 0; j < 8; ++j) v[j] = line[j * stride];
}
template <bool INV, int P>
__device__ __forceinline__ void fft_pass_finish(float2* buf, const Twiddles& tw, float2 (&v)[8]) {
  using namespace fft64;
  const int lo = threadIdx.x & 63, d = threadIdx.x >> 6;
  float2* line = P == 0 ? buf + lo * PITCH + d : P == 1 ? buf + lo * PITCH + 8 * d : P == 2 ? buf + lo + d * PITCH : buf + lo + 8 * d * PITCH;
  constexpr int stride = P == 0 ? 8 : P == 1 ? 1 : P == 2 ? 8 * PITCH : PITCH;
  fft8<INV>(v);
  if (P == 0 || P == 2) {
#pragma unroll
    for (int j = 1; j < 8; ++j) v[j] = twmul(v[j], tw, j);
  }
#pragma unroll
  for (int j = 0; j < 8; ++j) line[j * stride] = v[j];
}

// Workgroup -> volume.  Consecutive workgroups go round-robin over the 8 XCDs; the workgroups of one
// XCD take consecutive volumes (neighbouring records, and the same table slab at the same time).
__device__ __forceinline__ long volume_of_block(long nbatch) {
  const long zper = (nbatch + 7) / 8;
  const long xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const long z = xcd * zper + slot;
  return (slot < zper && z < nbatch) ? z : -1;
}
inline unsigned grid_size(long nbatch) { return (unsigned)(8 * ((nbatch + 7) / 8)); }

// Per-volume record in scratch memory: [k = 4 it + q][t] float4, q = 0: (+a) degrees u = 0, 1 as
// (re, im, re, im); q = 1: (+a) u = 2, 3; q = 2, 3: the same for (-a).
constexpr int REC_F4 = NIT * 4 * THREADS;                 // float4 per record
constexpr size_t REC_BYTES = (size_t)REC_F4 * 16;         // 229376
// workgroups per volume: a power of two, at least four beta pairs each, no more than fill the chip once
inline int parts(long nbatch) {
  int p = 1;
  while (2 * p * 4 <= NJ && 2 * p * nbatch <= 256) p *= 2;
  return p;
}
inline size_t scratch_bytes(long nbatch) { return (size_t)nbatch * parts(nbatch) * REC_BYTES; }

// ---------------------------------------------------------------------------------------------
// analysis: x [nbatch][64][64][64] real -> records of the half spectrum n >= 0
//
// Plane pair j+1 goes global -> registers -> first alpha stage -> `work` (LDS) -> second alpha stage ->
// two gamma stages, the last of which writes the QUAD layout: the four bins an item reads,
// Z[+a,n], Z[-a,-n], Z[-a,n], Z[+a,-n], side by side at quad[a][n][0..3].  Meanwhile pair j is
// contracted out of the other quad buffer, two items per stage.
// ---------------------------------------------------------------------------------------------
// NR: frequencies 0 <= a, n < NR are kept.  32 in general; a spectrum truncated below degree 24 (NA = 3 item rounds) needs
// 24 only, which lets the two quad buffers and the plane of such a kernel fit the LDS of a CU twice: two workgroups (two
// volumes in different phases of their steps) per CU.
constexpr int rows_kept(int NA) { return NA <= 3 ? 24 : 32; }
// waves per SIMD the kernels are compiled for: 4 (two workgroups per CU) where the registers of the truncated kernel allow
// it without spilling more than a few values: `lean` = the variant loads no second tensor / forms no sums
constexpr int waves_per_simd(int NA, bool lean) { return NA <= 3 && lean ? 4 : 2; }
// complex numbers per a-row of the quad layout: NR quads + one more (the unused n = NR) + room for the skew
constexpr int quad_pitch(int NR) { return NR * 4 + 14; }
constexpr int quad_elems(int NR) { return (NR + 1) * quad_pitch(NR); }     // row NR takes what is not kept (the dump row)
// Row a starts 2 (a / 8) complex numbers late.  The last gamma stage writes the rows 8r + s (r = lane % 8) at once; a pitch
// that keeps rows 16-byte aligned puts rows 8 apart into the same banks, the skew moves them 4 banks apart instead.
template <int NR> __host__ __device__ constexpr int quad_row(int a) { return a * quad_pitch(NR) + 2 * (a >> 3); }
// table registers: four slots, item it in slot it % 4; a slot is refilled right after its item has been used:
//   after item 0, 1, 2: items 4, 5, 6 of the same plane pair;  after 3, 4, 5, 6: items 3, 0, 1, 2 of the next pair
__device__ constexpr int table_slot(int it) { return it & 3; }

// NA: item rounds that carry degrees below the output bandwidth (the item table puts the low degree groups into the
// first rounds, so a truncated spectrum leaves the later rounds without work: NA = 3 covers l < 24, 6 covers l < 28, 7
// everything).
// MASK: what is done to x as it is loaded, one of s2cnn::Prologue: 0: nothing; 1: x where mask > 0 and zero elsewhere
// (mask: a tensor of the shape of x); 2: the same with `mask` holding one BIT per sample instead (bits_index below), as
// the synthesis writes them; 3: max(a x + b, 0); 4: a (a mask + b > 0 ? x : 0) + p + q mask, with a, b, p, q of the
// volume's feature z % nfeature in params [.][nfeature].
constexpr int BITS_WORDS = N * N;      // 64-bit words per volume: [beta][alpha % 8][alpha / 8], bit = gamma
__host__ __device__ inline size_t bits_index(long z, int beta, int d) { return ((size_t)z * N + beta) * N + 8 * d; }   // + alpha / 8
// PROBE (measurement only, results meaningless): 1: the Wigner contraction of an item reduced to one add per table
// operand (table loads, LDS reads of the quads and everything else kept); 2: the table loads gone as well.  What is left
// is the plane pipeline: loads, the 2-D transform through LDS with its barriers, the quad layout, the record.
template <int NA, int MASK, int PROBE = 0, bool SPLIT = false, bool STREAM = false>
__global__ __launch_bounds__(THREADS, waves_per_simd(NA, MASK == 0 || MASK == 2 || MASK == 3)) void analysis_kernel(const float* __restrict__ x, const float* __restrict__ mask,
                                                           const float* __restrict__ Tf, float4* __restrict__ rec, long nbatch,
                                                           const float* __restrict__ params, int nfeature, int nparts) {
  constexpr bool MASKED = MASK == 1 || MASK == 4;      // a second tensor is loaded beside x
  using namespace fft64;
  __shared__ __attribute__((aligned(16))) float2 work[LDS_ELEMS];
  constexpr int NR = rows_kept(NA), QUAD_ELEMS = quad_elems(NR);
  __shared__ __attribute__((aligned(16))) float2 quad[2][QUAD_ELEMS];
  // nparts workgroups per volume (few volumes do not fill the chip with one each): part p takes the beta pairs
  // p NJ / nparts .. (p+1) NJ / nparts - 1 and writes a record of its own, [volume][part]; spectrum_scatter adds them
  const long vp = volume_of_block(nbatch * nparts);
  if (vp < 0) return;
  const long z = SPLIT ? vp / nparts : vp;
  const int j0 = SPLIT ? (int)(vp - z * nparts) * NJ / nparts : 0, j1 = SPLIT ? ((int)(vp - z * nparts) + 1) * NJ / nparts : NJ;
  constexpr bool stream = STREAM;        // the signal passes no cache (see s2cnn::STREAM_BYTES): non-temporal loads / stores
  const int t = threadIdx.x;
  const int lo = t & 63, d = t >> 6;
  Twiddles twl;
  make_twiddles<false>(twl);
  for (int i = t; i < 2 * QUAD_ELEMS; i += THREADS) (&quad[0][0])[i] = make_float2(0.f, 0.f);   // places nobody writes (the -a half of a = 0) read as zero
  float pr_a = 0.f, pr_b = 0.f, pr_p = 0.f, pr_q = 0.f;      // the feature's constants: the same for the whole workgroup
  if constexpr (MASK >= 3) {
    const int c = (int)(z % nfeature);
    pr_a = params[c];
    pr_b = params[nfeature + c];
    if constexpr (MASK == 4) { pr_p = params[2 * nfeature + c]; pr_q = params[3 * nfeature + c]; }
  }

  // quad address of the item (complex index), bit 31 = sign bit of (-1)^n
  unsigned adr[NIT];
#pragma unroll
  for (int it = 0; it < NIT; ++it) {
    int c, a, n;
    decode_item(it * THREADS + t, c, a, n);
    adr[it] = it < NA ? (unsigned)(quad_row<NR>(a) + 4 * n) | ((unsigned)(n & 1) << 31) : 0u;   // active rounds hold a, n < NR
  }

  // where this thread's outputs of the last gamma stage go: row slot lo holds m = sigma(lo)
  const int m = sigma(lo);
  // quad[a][n] = { Z[+a,n], Z[-a,-n], Z[-a,n], Z[+a,-n] }; +0 and -0 are the same frequency, so
  //   m = 0 counts as -0 when n < 0 (the item (0, n) then finds Z[0,n], Z[0,-n] in its first two places) and
  //   n = 0 is written to the place of -0 as well (the one extra store below, by the wave d = 0).
  const int am = m <= 32 ? m : 64 - m;
  // Rows that are not kept (am >= NR; m = 32 always) go to the dump row, every lane to places of its own there whatever
  // the column is (nmul = 0): no branch, and no two lanes at the same address.
  const bool keep = am < NR;
  const int qa = keep ? quad_row<NR>(am) : quad_row<NR>(NR) + 4 * (am - NR);
  const int nmul = keep ? 4 : 0;
  const int pos_lo = m > 32 ? 2 : 0;                  // place of an output with n >= 0
  const int pos_hi = (m > 32 || m == 0) ? 1 : 3;      // place of an output with n < 0
  const int extra = d == 0 ? qa + pos_hi : quad_row<NR>(NR) + 4 * NR + 2;   // n = 0 again as -0; other waves: the pad of the dump row

  float2 accp[NIT][4], accm[NIT][4];
#pragma unroll
  for (int it = 0; it < NIT; ++it)
#pragma unroll
    for (int u = 0; u < 4; ++u) { accp[it][u] = make_float2(0.f, 0.f); accm[it][u] = make_float2(0.f, 0.f); }

  const __amdgpu_buffer_rsrc_t rx = make_rsrc(x + (size_t)z * (N * N * N), N * N * N * 4);
  const __amdgpu_buffer_rsrc_t rm = make_rsrc((MASKED ? mask : x) + (size_t)z * (N * N * N), N * N * N * 4);
  const __amdgpu_buffer_rsrc_t rt = make_rsrc(Tf, (unsigned)(PACKED_FLOATS * 4));
  const unsigned xoff = (d * N + lo) * 4;        // + (beta * 4096 + j1 * 512) * 4: row alpha = 8 j1 + d, column gamma = lo
  const unsigned toff = t * 16;
  float pa[8], pb[8];
  float ma[MASKED ? 8 : 1], mb[MASKED ? 8 : 1];
  // bit masks of the wave's eight rows of either plane: uniform over the wave (scalar loads), one lane mask per row
  unsigned long long ba[MASK == 2 ? 8 : 1], bb[MASK == 2 ? 8 : 1];
  const unsigned long long* const bits = reinterpret_cast<const unsigned long long*>(mask);
  const int du = __builtin_amdgcn_readfirstlane(d);
  float4 t1[4], t2[4];

  auto load_rows = [&](int j, int j1) {      // row 8 j1 + d of the planes j and 63-j: one full row (256 bytes) per wave and load
    pa[j1] = buf_load_f32_policy(rx, xoff, (j * 4096 + j1 * 512) * 4, stream);
    pb[j1] = buf_load_f32_policy(rx, xoff, ((63 - j) * 4096 + j1 * 512) * 4, stream);
    if constexpr (MASKED) {
      ma[j1] = buf_load_f32_policy(rm, xoff, (j * 4096 + j1 * 512) * 4, stream);
      mb[j1] = buf_load_f32_policy(rm, xoff, ((63 - j) * 4096 + j1 * 512) * 4, stream);
    }
    if constexpr (MASK == 2) {
      ba[j1] = bits[bits_index(z, j, du) + j1];
      bb[j1] = bits[bits_index(z, 63 - j, du) + j1];
    }
  };
  auto load_planes = [&](int j) {
#pragma unroll
    for (int j1 = 0; j1 < 8; ++j1) load_rows(j, j1);
  };
  auto load_planes_part = [&](int j, int g) {   // a quarter of load_planes
#pragma unroll
    for (int j1 = 2 * g; j1 < 2 * g + 2; ++j1) load_rows(j, j1);
  };
  auto load_table = [&](int j, int it) {
    if constexpr (PROBE == 2) {
      t1[table_slot(it)] = make_float4(1.f * j, 0.f, 0.f, 0.f);
      t2[table_slot(it)] = make_float4(1.f * it, 0.f, 0.f, 0.f);
      return;
    }
    t1[table_slot(it)] = buf_load_f32x4(rt, toff, ((j * NIT + it) * 2 + 0) * (THREADS * 16));
    t2[table_slot(it)] = buf_load_f32x4(rt, toff, ((j * NIT + it) * 2 + 1) * (THREADS * 16));
  };
  // first alpha stage, out of the registers: 8-point transforms over j1, twiddle, -> work[8 k1 + d][lo]
  auto stage_c1 = [&]() {
    float2 v[8];
#pragma unroll
    for (int j1 = 0; j1 < 8; ++j1) {
      if constexpr (MASK == 1) v[j1] = make_float2(s2cnn::relu_pass(pa[j1], ma[j1]), s2cnn::relu_pass(pb[j1], mb[j1]));
      else if constexpr (MASK == 3) v[j1] = make_float2(s2cnn::affine_relu(pa[j1], pr_a, pr_b), s2cnn::affine_relu(pb[j1], pr_a, pr_b));
      else if constexpr (MASK == 4) v[j1] = make_float2(s2cnn::bn_relu_grad(pa[j1], ma[j1], pr_a, pr_b, pr_p, pr_q),
                                                        s2cnn::bn_relu_grad(pb[j1], mb[j1], pr_a, pr_b, pr_p, pr_q));
      else if constexpr (MASK == 2) v[j1] = make_float2(__builtin_amdgcn_inverse_ballot_w64(ba[j1]) ? pa[j1] : 0.f,
                                                        __builtin_amdgcn_inverse_ballot_w64(bb[j1]) ? pb[j1] : 0.f);
      else v[j1] = make_float2(pa[j1], pb[j1]);
    }
    fft8<false>(v);
#pragma unroll
    for (int k = 1; k < 8; ++k) v[k] = twmul(v[k], twl, k);
#pragma unroll
    for (int k = 0; k < 8; ++k) work[(8 * k + d) * PITCH + lo] = v[k];
  };
  // second gamma stage: row slot lo, inputs at slots 8 d + j2, outputs n = d + 8 k2 -> quad layout
  auto stage_r2 = [&](float2* q) {
    float2 v[8];
    const float2* line = work + lo * PITCH + 8 * d;
#pragma unroll
    for (int j2 = 0; j2 < 8; ++j2) v[j2] = line[j2];
    fft8<false>(v);
    // outputs n = d + 8 k2 >= 0 and n' = 64 - d - 8 k2 > 0 (the bins -n'); those that are not kept are not written (d is
    // uniform over the wave); n' = NR lands in the pad of the row
    // (which outputs are kept is known at compile time: d + 8 k2 < NR for every d < 8, or for none)
#pragma unroll
    for (int k2 = 0; k2 < 4; ++k2)
      if (8 * k2 + 7 < NR) q[qa + nmul * (d + 8 * k2) + pos_lo] = v[k2];
#pragma unroll
    for (int k2 = 4; k2 < 8; ++k2)
      if (64 - 8 * k2 <= NR) q[qa + nmul * (64 - d - 8 * k2) + pos_hi] = v[k2];
    q[extra] = v[0];
  };
  // fresh: the rounds in which some thread of this half of the workgroup starts another column (FRESH_LO, FRESH_HI of the
  // item table, compile-time): the quad is read and separated there and serves the rounds that follow
  float2 Pp, Qp, Pm, Qm;          // the separated bins of the column of the current run
  auto accumulate = [&](const float2* q, int it, unsigned fresh) {
    if (it == 0 || ((fresh >> it) & 1u)) {
      const float4* src = reinterpret_cast<const float4*>(q + (adr[it] & 0x7fffffffu));
      const float4 za = src[0], zb = src[1];              // Z[+a,n], Z[-a,-n] | Z[-a,n], Z[+a,-n]
      const unsigned sb = adr[it] & 0x80000000u;
      // twice the separated planes (the table carries the factor 1/2):
      // P = Z[m,n] + conj Z[-m,-n],  P' = (Z[m,n] - conj Z[-m,-n]) / i, the latter times (-1)^n
      Pp = make_float2(za.x + za.z, za.y - za.w);
      Qp = make_float2(flip(za.y + za.w, sb), flip(za.z - za.x, sb));
      Pm = make_float2(zb.x + zb.z, zb.y - zb.w);
      Qm = make_float2(flip(zb.y + zb.w, sb), flip(zb.z - zb.x, sb));
    }
    const float4 ta = t1[table_slot(it)], tb = t2[table_slot(it)];
    if constexpr (PROBE == 1 || PROBE == 2) {
      const float4 za = make_float4(Pp.x, Pp.y, Qp.x, Qp.y), zb = make_float4(Pm.x, Pm.y, Qm.x, Qm.y);
      accp[it][0].x += za.x + ta.x; accm[it][0].x += zb.x + tb.x;
      return;
    }
    const float a1[4] = {ta.x, ta.y, ta.z, ta.w};
    const float a2[4] = {tb.x, tb.y, tb.z, tb.w};
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

  // first plane pair: transformed alone
  load_planes(j0);
  load_table(j0, 0);
  if constexpr (NA > 1) load_table(j0, 1);
  if constexpr (NA > 2) load_table(j0, 2);
  if constexpr (NA > 3) load_table(j0, 3);
  __syncthreads();                              // cleared quads
  stage_c1();
  load_planes(j0 + 1);                          // a part has at least two pairs
  __syncthreads();
  fft_pass<false, 3>(work, twl); __syncthreads();
  fft_pass<false, 0>(work, twl); __syncthreads();
  stage_r2(quad[j0 & 1]); __syncthreads();

  // step j: contract pair j out of quad[j & 1] while pair j+1 is transformed into quad[(j+1) & 1].
  // The scheduling fences keep the parts of a stage in program order.
#define S2CNN_FENCE() __builtin_amdgcn_sched_barrier(0)
  // contract item k, then refill its table slot with the item that uses the slot next; plane loads in quarters:
  // memory instructions are spread over the step so that their queue never fills up
#define S2CNN_ACC(k, jl, il)                                                                             \
  if constexpr ((k) < NA) {                                                                              \
    accumulate(cur, k, FR); S2CNN_FENCE();                                                               \
    if constexpr ((k) + 4 < NA) load_table(j, (k) + 4); else load_table(j + 1, (k) & 3);                 \
    S2CNN_FENCE();                                                                                       \
  }
#define S2CNN_PLANES(g) load_planes_part(jp, g); S2CNN_FENCE();
  // Waves d < 4 transform first and contract second, waves d >= 4 the other way round: each SIMD holds one
  // wave of either kind, so its LDS-bound and its FMA-bound half of a stage overlap.
  if (d < 4) {
    constexpr unsigned FR = FRESH_LO;
    for (int j = j0; j < j1 - 1; ++j) {
      const float2* cur = quad[j & 1];
      float2* nxt = quad[(j + 1) & 1];
      const int jp = j + 2 < j1 ? j + 2 : j1 - 1;     // clamped, not branched: a branch would make the loads synchronous
      stage_c1(); S2CNN_FENCE();
      S2CNN_PLANES(0) S2CNN_ACC(0, j, 4) S2CNN_PLANES(1) S2CNN_ACC(1, j, 5)
      __syncthreads();
      fft_pass<false, 3>(work, twl); S2CNN_FENCE();
      S2CNN_PLANES(2) S2CNN_ACC(2, j, 6) S2CNN_PLANES(3) S2CNN_ACC(3, j + 1, 3)
      __syncthreads();
      fft_pass<false, 0>(work, twl); S2CNN_FENCE();
      S2CNN_ACC(4, j + 1, 0) S2CNN_ACC(5, j + 1, 1)
      __syncthreads();
      stage_r2(nxt); S2CNN_FENCE();
      S2CNN_ACC(6, j + 1, 2)
      __syncthreads();
    }
  } else {
    constexpr unsigned FR = FRESH_HI;
    for (int j = j0; j < j1 - 1; ++j) {
      const float2* cur = quad[j & 1];
      float2* nxt = quad[(j + 1) & 1];
      const int jp = j + 2 < j1 ? j + 2 : j1 - 1;
      S2CNN_ACC(0, j, 4) S2CNN_ACC(1, j, 5)
      stage_c1(); S2CNN_FENCE();
      S2CNN_PLANES(0) S2CNN_PLANES(1)
      __syncthreads();
      {
        float2 fv[8];
        fft_pass_load<3>(work, fv); S2CNN_FENCE();          // in flight during the two items
        S2CNN_ACC(2, j, 6) S2CNN_PLANES(2) S2CNN_ACC(3, j + 1, 3) S2CNN_PLANES(3)
        fft_pass_finish<false, 3>(work, twl, fv);
      }
      __syncthreads();
      {
        float2 fv[8];
        fft_pass_load<0>(work, fv); S2CNN_FENCE();
        S2CNN_ACC(4, j + 1, 0) S2CNN_ACC(5, j + 1, 1)
        fft_pass_finish<false, 0>(work, twl, fv);
      }
      __syncthreads();
      S2CNN_ACC(6, j + 1, 2)
      stage_r2(nxt);
      __syncthreads();
    }
  }
  {
    const float2* cur = quad[(j1 - 1) & 1];
#define S2CNN_LAST(k)                                                                                    \
  if constexpr ((k) < NA) {                                                                              \
    accumulate(cur, k, FRESH_LO | FRESH_HI);                                                             \
    if constexpr ((k) + 4 < NA) { S2CNN_FENCE(); load_table(j1 - 1, (k) + 4); S2CNN_FENCE(); }           \
  }
    S2CNN_LAST(0) S2CNN_LAST(1) S2CNN_LAST(2) S2CNN_LAST(3) S2CNN_LAST(4) S2CNN_LAST(5) S2CNN_LAST(6)
#undef S2CNN_LAST
  }
#undef S2CNN_ACC
#undef S2CNN_PLANES
#undef S2CNN_FENCE

  const __amdgpu_buffer_rsrc_t rr = make_rsrc(rec + (size_t)vp * REC_F4, (unsigned)REC_BYTES);      // record [z][part]
#pragma unroll
  for (int it = 0; it < NA; ++it) {            // the pass that follows reads these rounds only
    buf_store_f32x4(make_float4(accp[it][0].x, accp[it][0].y, accp[it][1].x, accp[it][1].y), rr, toff, (it * 4 + 0) * (THREADS * 16));
    buf_store_f32x4(make_float4(accp[it][2].x, accp[it][2].y, accp[it][3].x, accp[it][3].y), rr, toff, (it * 4 + 1) * (THREADS * 16));
    buf_store_f32x4(make_float4(accm[it][0].x, accm[it][0].y, accm[it][1].x, accm[it][1].y), rr, toff, (it * 4 + 2) * (THREADS * 16));
    buf_store_f32x4(make_float4(accm[it][2].x, accm[it][2].y, accm[it][3].x, accm[it][3].y), rr, toff, (it * 4 + 3) * (THREADS * 16));
  }
}

// ---------------------------------------------------------------------------------------------
// records <-> spectral rows, for a tile of 16 volumes and 32 items per workgroup (256 threads).
// grid (ceil(nbatch / 16), rounds * G::THREADS / 32).  Row kinds of an item and degree: 0 (+a, n)  1 (-a, n)
// 2 (-a,-n)  3 (+a,-n); kinds 2, 3 are (-1)^(a-n) conj of kinds 0, 1 in a spectrum of a real signal.
// ---------------------------------------------------------------------------------------------
constexpr int ZT = 16;              // volumes per tile: one 128-byte piece of a spectral row
constexpr int IT_TILE = 32;         // items per tile
constexpr int VLD = 16 * ZT + 1;    // LDS floats per item: 16 components x 16 volumes, padded

// What these passes need to know of the kernels whose records they read and write: threads per volume, the size of a
// record and the item of every place.  The per-volume kernels of another grid (so3_fused32.h) bring their own.
struct Geometry {
  static constexpr int THREADS = fused64::THREADS;
  static constexpr int REC_F4 = fused64::REC_F4;
  static __device__ __forceinline__ bool decode(int i, int& c, int& a, int& n) { return decode_item(i, c, a, n); }
};

template <class G>
__device__ __forceinline__ int pack_item_info(int i) {
  int c, a, n;
  const bool ok = G::decode(i, c, a, n);
  return c | (a << 8) | (n << 16) | (ok ? 1 << 24 : 0);
}

// rows of item `info`, degree offset u, kind k: spectral index, or -1 if there is no such row
__device__ __forceinline__ int row_index(int info, int u, int kind, int nl) {
  const int c = info & 0xff, a = (info >> 8) & 0xff, n = (info >> 16) & 0xff;
  const int l = 4 * c + u;
  const bool ok = (info >> 24) && l >= a && l >= n && l < nl && (!(kind & 1) || a > 0) && (kind < 2 || n > 0) &&
                  (kind != 3 || a > 0);
  if (!ok) return -1;
  const int m = (kind == 1 || kind == 2) ? -a : a;
  return lmn_index(l, m, kind >= 2 ? -n : n);
}

// nparts: records per volume ([volume][part], see so3_fused4r.h); their sum is the volume's record
template <class G = Geometry>
__global__ __launch_bounds__(256) void spectrum_scatter(const float4* __restrict__ rec, float2* __restrict__ out, int nl, long nbatch, int nparts) {
  constexpr int THREADS = G::THREADS, REC_F4 = G::REC_F4, TILES = THREADS / IT_TILE;
  __shared__ float vals[IT_TILE * VLD];
  __shared__ int info[IT_TILE];
  const int th = threadIdx.x;
  const long z0 = (long)blockIdx.x * ZT;
  const int it = blockIdx.y / TILES, t0 = (blockIdx.y % TILES) * IT_TILE;
  if (th < IT_TILE) info[th] = pack_item_info<G>(it * THREADS + t0 + th);
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int e = th + 256 * r;
    const int item = e & 31, q = (e >> 5) & 3, zz = e >> 7;
    // a volume past the end reads the last one (its values are not stored): no branch around the loads
    const size_t zc = (size_t)(z0 + zz < nbatch ? z0 + zz : nbatch - 1);
    float4 v = rec[zc * nparts * REC_F4 + (it * 4 + q) * THREADS + t0 + item];
    for (int p = 1; p < nparts; ++p) {
      const float4 w = rec[(zc * nparts + p) * REC_F4 + (it * 4 + q) * THREADS + t0 + item];
      v = make_float4(v.x + w.x, v.y + w.y, v.z + w.z, v.w + w.w);
    }
    float* d = vals + item * VLD + (4 * q) * ZT + zz;
    d[0] = v.x; d[ZT] = v.y; d[2 * ZT] = v.z; d[3 * ZT] = v.w;
  }
  __syncthreads();
  const int zz = th & 15, u = th >> 6, kind = (th >> 4) & 3;
  if (z0 + zz >= nbatch) return;
  const int comp = 4 * ((kind & 1) * 2 + (u >> 1)) + 2 * (u & 1);
  for (int item = 0; item < IT_TILE; ++item) {
    const int inf = info[item];
    const int row = row_index(inf, u, kind, nl);
    if (row < 0) continue;
    float re = vals[item * VLD + comp * ZT + zz], im = vals[item * VLD + (comp + 1) * ZT + zz];
    if (kind >= 2) {
      const float sg = (((inf >> 8) - (inf >> 16)) & 1) ? -1.f : 1.f;
      re *= sg; im *= -sg;
    }
    out[(size_t)row * nbatch + z0 + zz] = make_float2(re, im);
  }
}

// xh [nspec][nbatch] complex (any symmetry) -> records of the symmetrised spectrum
//   xs[l,m,n] = xh[l,m,n] + (-1)^(m-n) conj xh[l,-m,-n]   (twice the Hermitian part: the table carries 1/2),
// zero where there is no such degree; the (-a) half of items with a = 0 is zero (it is the (+a) half).
template <class G = Geometry>
__global__ __launch_bounds__(256) void spectrum_gather(const float2* __restrict__ xh, float4* __restrict__ rec, int nl, long nbatch) {
  constexpr int THREADS = G::THREADS, REC_F4 = G::REC_F4, TILES = THREADS / IT_TILE;
  __shared__ float vals[IT_TILE * VLD];
  __shared__ int info[IT_TILE];
  const int th = threadIdx.x;
  const long z0 = (long)blockIdx.x * ZT;
  const int it = blockIdx.y / TILES, t0 = (blockIdx.y % TILES) * IT_TILE;
  if (th < IT_TILE) info[th] = pack_item_info<G>(it * THREADS + t0 + th);
  __syncthreads();
  {
    const int zz = th & 15, u = (th >> 4) & 3, pm = (th >> 6) & 1, sub = th >> 7;
    const int comp = 4 * (pm * 2 + (u >> 1)) + 2 * (u & 1);
    const long zc = z0 + zz < nbatch ? z0 + zz : nbatch - 1;
    // all loads of the thread's items first (an entry that does not exist reads row 0 instead and is not used), so that
    // their latencies overlap; then the sums
    constexpr int NI = IT_TILE / 2;
    float2 v0[NI], v1[NI];
    float sg[NI];                                               // 0: no such entry
#pragma unroll
    for (int k = 0; k < NI; ++k) {
      const int inf = info[sub + 2 * k];
      const int r0 = row_index(inf, u, pm, nl);                 // (+-a, n)
      const int a = (inf >> 8) & 0xff, n = (inf >> 16) & 0xff;
      const int l = 4 * (inf & 0xff) + u;
      const int r1 = r0 >= 0 ? lmn_index(l, pm ? a : -a, -n) : 0;   // the partner (-+a, -n); exists for every n
      v0[k] = xh[(size_t)(r0 < 0 ? 0 : r0) * nbatch + zc];
      v1[k] = xh[(size_t)r1 * nbatch + zc];
      sg[k] = r0 < 0 ? 0.f : ((a - n) & 1) ? -1.f : 1.f;
    }
#pragma unroll
    for (int k = 0; k < NI; ++k) {
      const int item = sub + 2 * k;
      const bool has = sg[k] != 0.f;
      vals[item * VLD + comp * ZT + zz] = has ? v0[k].x + sg[k] * v1[k].x : 0.f;
      vals[item * VLD + (comp + 1) * ZT + zz] = has ? v0[k].y - sg[k] * v1[k].y : 0.f;
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int e = th + 256 * r;
    const int item = e & 31, q = (e >> 5) & 3, zz = e >> 7;
    if (z0 + zz >= nbatch) continue;
    const float* d = vals + item * VLD + (4 * q) * ZT + zz;
    rec[(size_t)(z0 + zz) * REC_F4 + (it * 4 + q) * THREADS + t0 + item] = make_float4(d[0], d[ZT], d[2 * ZT], d[3 * ZT]);
  }
}

// ---------------------------------------------------------------------------------------------
// The same two passes for a spectrum kept in the REAL basis (see so3_real_basis.hip: R = Re(U X U^H),
// one float per entry).  With A = X[l,+a,n], C = X[l,-a,n] of a real signal, s = (-1)^a:
//     R[+a,+n] = A.re + s C.re     R[+a,-n] = -A.im - s C.im
//     R[-a,+n] = A.im - s C.im     R[-a,-n] =  A.re - s C.re          (a, n > 0)
//     a = 0: sqrt2 A.re, -sqrt2 A.im      n = 0: (A.re + s C.re)/sqrt2, (A.im - s C.im)/sqrt2      a = n = 0: A.re
// and backwards (records hold twice the complex value, the table carries 1/2):
//     2 A = (cc + ss, sc - cs)   2 C = s (cc - ss, -(cs + sc))   with cc, cs, sc, ss = R[+a,+n], R[+a,-n], R[-a,+n], R[-a,-n]
//     a = 0: sqrt2 (cc, -cs), C unused     n = 0: sqrt2 (cc, sc), s sqrt2 (cc, -sc)     a = n = 0: (2 cc, 0)
// Tiles of ZR volumes (4 ZR-byte pieces of a row) and IT_TILE_R items; grid (ceil(nbatch / ZR), rounds * G::THREADS / IT_TILE_R).
// ---------------------------------------------------------------------------------------------
constexpr int ZR = 32;                      // volumes per tile: 32 or 64
constexpr int IT_TILE_R = 512 / ZR;         // items per tile: the tile holds 512 x 16 floats
static_assert(IT_TILE_R * 16 <= 256 && 4 * ZR <= 256 && 256 % ZR == 0 && 16 % (256 / ZR) == 0, "thread mappings of the real-basis record passes");
constexpr int VLD_R = 16 * ZR + 1;
constexpr float SQRT2 = 1.41421356237309504880f, RSQRT2 = 0.70710678118654752440f;

// where one output row of the tile comes from: out[row] = alpha * vals[comp] + beta * vals[comp + 8] (row < 0: no such row)
struct RowRule { int row, comp; float alpha, beta; };

// rule of row slot rs = 4 u + kind (degree 4 c + u; kind: 0 (+a,+n)  1 (+a,-n)  2 (-a,+n)  3 (-a,-n)) of an item
__device__ __forceinline__ RowRule row_rule(int inf, int rs, int nl) {
  const int u = rs >> 2, kind = rs & 3;
  const int c = inf & 0xff, a = (inf >> 8) & 0xff, n = (inf >> 16) & 0xff;
  const int l = 4 * c + u;
  RowRule r{-1, 0, 0.f, 0.f};
  if (!(inf >> 24) || l < a || l < n || l >= nl || ((kind & 1) && n == 0) || ((kind & 2) && a == 0)) return r;
  r.row = lmn_index(l, (kind & 2) ? -a : a, (kind & 1) ? -n : n);
  // A = (+a) half: components 4 (u / 2) + 2 (u % 2) + (0 re, 1 im);  C = (-a) half: the same + 8
  r.comp = 4 * (u >> 1) + 2 * (u & 1) + ((kind == 1 || kind == 2) ? 1 : 0);
  const float s = (a & 1) ? -1.f : 1.f;
  r.alpha = kind == 1 ? -1.f : 1.f;
  r.beta = (kind == 0) ? s : -s;
  if (a == 0) { r.alpha *= SQRT2; r.beta = 0.f; if (n == 0) r.alpha = 1.f; }
  else if (n == 0) { r.alpha *= RSQRT2; r.beta *= RSQRT2; }
  return r;
}

template <class G = Geometry>
__global__ __launch_bounds__(256) void spectrum_scatter_real(const float4* __restrict__ rec, float* __restrict__ out, int nl, long nbatch, int nparts) {
  constexpr int THREADS = G::THREADS, REC_F4 = G::REC_F4, TILES = THREADS / IT_TILE_R;
  __shared__ float vals[IT_TILE_R * VLD_R];
  __shared__ RowRule rules[IT_TILE_R * 16];
  const int th = threadIdx.x;
  const long z0 = (long)blockIdx.x * ZR;
  const int it = blockIdx.y / TILES, t0 = (blockIdx.y % TILES) * IT_TILE_R;
  if (th < IT_TILE_R * 16) rules[th] = row_rule(pack_item_info<G>(it * THREADS + t0 + (th >> 4)), th & 15, nl);   // items x 16 row slots: one per thread
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int e = th + 256 * r;
    const int item = e % IT_TILE_R, q = (e / IT_TILE_R) & 3, zz = e / (4 * IT_TILE_R);
    // a volume past the end reads the last one (its values are not stored): no branch around the loads, so the eight of
    // a thread are in flight together
    const size_t zc = (size_t)(z0 + zz < nbatch ? z0 + zz : nbatch - 1);
    float4 v = rec[zc * nparts * REC_F4 + (it * 4 + q) * THREADS + t0 + item];
    for (int p = 1; p < nparts; ++p) {
      const float4 w = rec[(zc * nparts + p) * REC_F4 + (it * 4 + q) * THREADS + t0 + item];
      v = make_float4(v.x + w.x, v.y + w.y, v.z + w.z, v.w + w.w);
    }
    float* d = vals + item * VLD_R + (4 * q) * ZR + zz;
    d[0] = v.x; d[ZR] = v.y; d[2 * ZR] = v.z; d[3 * ZR] = v.w;
  }
  __syncthreads();
  constexpr int NSLOT = 256 / ZR;              // row slots at a time, ZR volumes (4 ZR bytes of a row) each
  const int zz = th % ZR, sub = th / ZR;
  if (z0 + zz >= nbatch) return;
  float* dst = out + z0 + zz;
  for (int p = 0; p < (16 / NSLOT) * IT_TILE_R; ++p) {
    const int item = p / (16 / NSLOT);
    const RowRule r = rules[item * 16 + (p % (16 / NSLOT)) * NSLOT + sub];
    if (r.row < 0) continue;
    const float* v = vals + item * VLD_R + r.comp * ZR + zz;
    dst[(size_t)r.row * nbatch] = r.alpha * v[0] + r.beta * v[8 * ZR];
  }
}

// the four rows R[+a,+n], R[+a,-n], R[-a,+n], R[-a,-n] of degree 4 c + u of an item (-1: none; rows[0] < 0: no such degree)
struct QuadRows { int rows[4]; float s; };

__device__ __forceinline__ QuadRows quad_rows(int inf, int u, int nl) {
  const int c = inf & 0xff, a = (inf >> 8) & 0xff, n = (inf >> 16) & 0xff;
  const int l = 4 * c + u;
  QuadRows q{{-1, -1, -1, -1}, (a & 1) ? -1.f : 1.f};
  if ((inf >> 24) && l >= a && l >= n && l < nl) {
    q.rows[0] = lmn_index(l, a, n);
    if (n > 0) q.rows[1] = lmn_index(l, a, -n);
    if (a > 0) q.rows[2] = lmn_index(l, -a, n);
    if (a > 0 && n > 0) q.rows[3] = lmn_index(l, -a, -n);
  }
  return q;
}

template <class G = Geometry>
__global__ __launch_bounds__(256) void spectrum_gather_real(const float* __restrict__ rr, float4* __restrict__ rec, int nl, long nbatch) {
  constexpr int THREADS = G::THREADS, REC_F4 = G::REC_F4, TILES = THREADS / IT_TILE_R;
  __shared__ float vals[IT_TILE_R * VLD_R];
  __shared__ QuadRows quads[IT_TILE_R * 4];
  const int th = threadIdx.x;
  const long z0 = (long)blockIdx.x * ZR;
  const int it = blockIdx.y / TILES, t0 = (blockIdx.y % TILES) * IT_TILE_R;
  if (th < IT_TILE_R * 4) quads[th] = quad_rows(pack_item_info<G>(it * THREADS + t0 + (th >> 2)), th & 3, nl);
  __syncthreads();
  {
    constexpr int NSUB = 256 / (4 * ZR), NI = IT_TILE_R / NSUB;      // items per thread
    const int zz = th % ZR, u = (th / ZR) & 3, sub = th / (4 * ZR);
    const long zc = z0 + zz < nbatch ? z0 + zz : nbatch - 1;
    const float* src = rr + zc;
    // all loads of the thread's items first (a row that does not exist reads row 0 instead: a valid address, and the
    // value is not used), so that their latencies overlap; then the combinations
    QuadRows qs[NI];
    float cc[NI], cs[NI], sc[NI], ss[NI];
#pragma unroll
    for (int k = 0; k < NI; ++k) {
      qs[k] = quads[(sub + k * NSUB) * 4 + u];
      const QuadRows& q = qs[k];
      cc[k] = src[(size_t)(q.rows[0] < 0 ? 0 : q.rows[0]) * nbatch];
      cs[k] = src[(size_t)(q.rows[1] < 0 ? 0 : q.rows[1]) * nbatch];
      sc[k] = src[(size_t)(q.rows[2] < 0 ? 0 : q.rows[2]) * nbatch];
      ss[k] = src[(size_t)(q.rows[3] < 0 ? 0 : q.rows[3]) * nbatch];
    }
#pragma unroll
    for (int k = 0; k < NI; ++k) {
      const QuadRows& q = qs[k];
      float2 A = make_float2(0.f, 0.f), C = A;
      if (q.rows[0] >= 0) {
        const bool hn = q.rows[1] >= 0, ha = q.rows[2] >= 0;
        const float s = q.s;
        if (ha && hn) { A = make_float2(cc[k] + ss[k], sc[k] - cs[k]); C = make_float2(s * (cc[k] - ss[k]), -s * (cs[k] + sc[k])); }
        else if (ha)  { A = make_float2(SQRT2 * cc[k], SQRT2 * sc[k]); C = make_float2(s * SQRT2 * cc[k], -s * SQRT2 * sc[k]); }
        else if (hn)  { A = make_float2(SQRT2 * cc[k], -SQRT2 * cs[k]); }
        else          { A = make_float2(2.f * cc[k], 0.f); }
      }
      const int comp = 4 * (u >> 1) + 2 * (u & 1);
      float* d = vals + (sub + k * NSUB) * VLD_R + comp * ZR + zz;
      d[0] = A.x; d[ZR] = A.y; d[8 * ZR] = C.x; d[9 * ZR] = C.y;
    }
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 8; ++r) {
    const int e = th + 256 * r;
    const int item = e % IT_TILE_R, q = (e / IT_TILE_R) & 3, zz = e / (4 * IT_TILE_R);
    if (z0 + zz >= nbatch) continue;
    const float* d = vals + item * VLD_R + (4 * q) * ZR + zz;
    rec[(size_t)(z0 + zz) * REC_F4 + (it * 4 + q) * THREADS + t0 + item] = make_float4(d[0], d[ZR], d[2 * ZR], d[3 * ZR]);
  }
}

// ---------------------------------------------------------------------------------------------
// synthesis: records of the symmetrised spectrum -> y [nbatch][64][64][64] real
//
// While plane pair j is transformed in `work` (two gamma stages, two alpha stages, the last one
// straight into the global stores), the shares of the items in the bins of pair j+1 are summed in registers
// over each RUN of rounds that hold the same column, and leave for a staging area when the run ends.  The
// item table cuts a column into at most two runs; the staging area has one place per column and run, and
// a reduction over the two places fills `work` for the next step.
// Sums are formed in a fixed order: results are reproducible bit for bit.
// ---------------------------------------------------------------------------------------------
// bias: NULL, or one value per feature added to every sample of volume z (feature = z % nfeature)
// relu: nonzero = negative samples (after the bias) are stored as zero
// NA as in analysis_kernel
// PROBE (measurement only, results meaningless): 1: an item's share of a plane pair reduced to one add per table operand.
// MOM: the kernel also writes two sums over the volume it produces, formed in a fixed order, to moments[z]:
//   1: (sum v, sum (v - mean of the volume)^2) of the output v (bias included, before the activation): the statistics of
//      a batch normalisation that follows, without a read of their own.  Every thread sums its squares around a pivot (its
//      first sample); the threads' sums are moved to their means and merged pairwise in float64, so a mean that is large
//      against the spread costs the variance no digits;
//   2: (sum v m, sum v m w) with w = yref at the same sample and m = (a w + b > 0), a = params[f], b = params[nfeature + f],
//      f = z % nfeature: the two reductions of the gradient of such a normalisation followed by max(., 0), with the
//      output as the incoming gradient (s2cnn::bn_relu_grad).
template <int NA, int PROBE = 0, int MOM = 0, bool SPLIT = false, bool STREAM = false>
__global__ __launch_bounds__(THREADS, waves_per_simd(NA, MOM == 0)) void synthesis_kernel(const float4* __restrict__ rec, const float* __restrict__ Tf,
                                                            float* __restrict__ y, long nbatch, const float* __restrict__ bias, int nfeature,
                                                            int relu, unsigned long long* __restrict__ bits, float2* __restrict__ moments,
                                                            const float* __restrict__ yref, const float* __restrict__ params, int nparts) {
  using namespace fft64;
  __shared__ __attribute__((aligned(16))) float2 work[LDS_ELEMS];
  float ms1 = 0.f, ms2 = 0.f;
  [[maybe_unused]] float mpivot = 0.f;
  constexpr int NR = rows_kept(NA);                                           // frequencies a, n < NR carry degrees of the input (see analysis_kernel)
  constexpr int NCOL = NR * NR;                                               // columns (a, n)
  __shared__ __attribute__((aligned(16))) float4 stg_p[2 * NCOL];             // [run of the column][NR a + n]: the run's share of the bins [+a,n], [-a,-n]
  __shared__ __attribute__((aligned(16))) float4 stg_m[2 * NCOL];             //                                                            [-a,n], [+a,-n]
  // nparts workgroups per volume (1 with MOM): part p reads the volume's record and writes the planes of its beta pairs
  const long vp = volume_of_block(nbatch * nparts);
  if (vp < 0) return;
  const long z = SPLIT ? vp / nparts : vp;
  const int j0 = SPLIT ? (int)(vp - z * nparts) * NJ / nparts : 0, j1 = SPLIT ? ((int)(vp - z * nparts) + 1) * NJ / nparts : NJ;
  constexpr bool stream = STREAM;        // the signal passes no cache (see s2cnn::STREAM_BYTES): non-temporal loads / stores
  const int t = threadIdx.x;
  const int lo = t & 63, d = t >> 6;
  const float bz = bias ? bias[z % nfeature] : 0.f;
  Twiddles twl;
  make_twiddles<true>(twl);
  for (int i = t; i < LDS_ELEMS; i += THREADS) work[i] = make_float2(0.f, 0.f);   // bins of m = 32 and n = 32 stay zero ... until a transform overwrites them: cleared again in reduce()
  // places of the staging area that no run writes (the second place of a column with one run, the columns beyond a
  // truncated spectrum) are read by reduce() all the same: they stay zero
  for (int i = t; i < 2 * NCOL; i += THREADS) { stg_p[i] = make_float4(0.f, 0.f, 0.f, 0.f); stg_m[i] = make_float4(0.f, 0.f, 0.f, 0.f); }

  float2 xp[NIT][4], xm[NIT][4];
  // the table entries of this thread's places, two per word: bits 0-9 the column 32 a + n (bit 0 = n odd), bit 14 which of
  // the column's two runs this one is, bit 15 the run ends with this round
  unsigned ent[(NIT + 1) / 2];
#pragma unroll
  for (int w = 0; w < (NIT + 1) / 2; ++w) ent[w] = 0;
  const __amdgpu_buffer_rsrc_t rr = make_rsrc(rec + (size_t)z * REC_F4, (unsigned)REC_BYTES);
  const __amdgpu_buffer_rsrc_t rt = make_rsrc(Tf, (unsigned)(PACKED_FLOATS * 4));
  const __amdgpu_buffer_rsrc_t ry = make_rsrc(y + (size_t)z * (N * N * N), N * N * N * 4);
  const unsigned toff = t * 16;
  const unsigned yoff = (d * N + lo) * 4;          // + (beta * 4096 + k * 512) * 4: row alpha = d + 8 k, column gamma = lo
  const __amdgpu_buffer_rsrc_t rw = make_rsrc(MOM == 2 ? yref + (size_t)z * (N * N * N) : y, MOM == 2 ? N * N * N * 4 : 0);
  float mom_a = 0.f, mom_b = 0.f;
  if constexpr (MOM == 2) { mom_a = params[z % nfeature]; mom_b = params[nfeature + z % nfeature]; }
#pragma unroll
  for (int it = 0; it < NA; ++it) {
    ent[it >> 1] |= (unsigned)ITEM_TABLE[it * THREADS + t] << (16 * (it & 1));
    const float4 v0 = buf_load_f32x4(rr, toff, (it * 4 + 0) * (THREADS * 16)), v1 = buf_load_f32x4(rr, toff, (it * 4 + 1) * (THREADS * 16));
    const float4 v2 = buf_load_f32x4(rr, toff, (it * 4 + 2) * (THREADS * 16)), v3 = buf_load_f32x4(rr, toff, (it * 4 + 3) * (THREADS * 16));
    xp[it][0] = make_float2(v0.x, v0.y); xp[it][1] = make_float2(v0.z, v0.w);
    xp[it][2] = make_float2(v1.x, v1.y); xp[it][3] = make_float2(v1.z, v1.w);
    xm[it][0] = make_float2(v2.x, v2.y); xm[it][1] = make_float2(v2.z, v2.w);
    xm[it][2] = make_float2(v3.x, v3.y); xm[it][3] = make_float2(v3.z, v3.w);
  }
  float4 t1[4], t2[4];
  auto load_table = [&](int j, int it) {
    t1[table_slot(it)] = buf_load_f32x4(rt, toff, ((j * NIT + it) * 2 + 0) * (THREADS * 16));
    t2[table_slot(it)] = buf_load_f32x4(rt, toff, ((j * NIT + it) * 2 + 1) * (THREADS * 16));
  };
  // the item's share of a plane pair: S = sum_l t1 xs, S' = sum_l s t2 xs at (+a, n), t1 <-> t2 at (-a, n);
  // complex plane Z = S + i S' at [m,n], its Hermitian partner conj S + i conj S' at [-m,-n]
  // the sums of the current run: S = sum_l t1 xs, S' = sum_l s t2 xs at (+a, n), t1 <-> t2 at (-a, n)
  float2 Sp = make_float2(0.f, 0.f), Qp = make_float2(0.f, 0.f), Sm = make_float2(0.f, 0.f), Qm = make_float2(0.f, 0.f);
  typedef float macc_t __attribute__((ext_vector_type(4)));
  [[maybe_unused]] macc_t macc[4] = {};
  // fresh: as in analysis_kernel; a run can only end in front of a round that starts one, or in the last round
  auto contribute = [&](int it, unsigned fresh) {
    const float4 ta = t1[table_slot(it)], tb = t2[table_slot(it)];
    const float a1[4] = {ta.x, ta.y, ta.z, ta.w};
    const float a2[4] = {tb.x, tb.y, tb.z, tb.w};
    if constexpr (PROBE == 2) {
      // what the contraction would cost on the matrix pipe: 4 groups of 16 items x 4 degrees, one 4x4x1 instruction each
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        macc[0] = __builtin_amdgcn_mfma_f32_4x4x1f32(a1[u], xp[it][u].x, macc[0], 0, 0, 0);
        macc[1] = __builtin_amdgcn_mfma_f32_4x4x1f32(a2[u], xp[it][u].y, macc[1], 0, 0, 0);
        macc[2] = __builtin_amdgcn_mfma_f32_4x4x1f32(a1[u], xm[it][u].x, macc[2], 0, 0, 0);
        macc[3] = __builtin_amdgcn_mfma_f32_4x4x1f32(a2[u], xm[it][u].y, macc[3], 0, 0, 0);
      }
    } else if constexpr (PROBE != 0) {
      Sp.x += a1[0] + xp[it][0].x; Sm.x += a2[0] + xm[it][0].x;
    } else {
#pragma unroll
      for (int u = 0; u < 4; ++u) {
        const float b1 = (u & 1) ? -a1[u] : a1[u], b2 = (u & 1) ? -a2[u] : a2[u];
        Sp.x = fmaf(a1[u], xp[it][u].x, Sp.x); Sp.y = fmaf(a1[u], xp[it][u].y, Sp.y);
        Qp.x = fmaf(b2, xp[it][u].x, Qp.x);    Qp.y = fmaf(b2, xp[it][u].y, Qp.y);
        Sm.x = fmaf(a2[u], xm[it][u].x, Sm.x); Sm.y = fmaf(a2[u], xm[it][u].y, Sm.y);
        Qm.x = fmaf(b1, xm[it][u].x, Qm.x);    Qm.y = fmaf(b1, xm[it][u].y, Qm.y);
      }
    }
    // the run ends here (in the last round every run does): complex plane Z = S + i S' at [m,n], its Hermitian partner
    // conj S + i conj S' at [-m,-n], the factor (-1)^n of S' in the sign bit; then the sums start again
    if (it != NA - 1 && !((fresh >> (it + 1)) & 1u)) return;
    const unsigned e = (ent[it >> 1] >> (16 * (it & 1))) & 0xffffu;
    if (it == NA - 1 || (e >> 15)) {
      const unsigned sb = (e & 1u) << 31;
      const float qpx = flip(Qp.x, sb), qpy = flip(Qp.y, sb), qmx = flip(Qm.x, sb), qmy = flip(Qm.y, sb);
      const unsigned col32 = e & 0x3ffu;                                        // 32 a + n
      const unsigned pos = ((e >> 14) & 1u) * NCOL + col32 - (32 - NR) * (col32 >> 5);
      if constexpr (PROBE == 2) {
        stg_p[pos] = make_float4(macc[0].x - macc[1].y, macc[0].y + macc[1].x, macc[0].x + macc[1].y, macc[1].x - macc[0].y);
        stg_m[pos] = make_float4(macc[2].x - macc[3].y, macc[2].y + macc[3].x, macc[2].x + macc[3].y, macc[3].x - macc[2].y);
#pragma unroll
        for (int g = 0; g < 4; ++g) macc[g] = macc_t{qpx, qpy, qmx, qmy};
      } else {
      stg_p[pos] = make_float4(Sp.x - qpy, Sp.y + qpx, Sp.x + qpy, qpx - Sp.y);
      stg_m[pos] = make_float4(Sm.x - qmy, Sm.y + qmx, Sm.x + qmy, qmx - Sm.y);
      }
      Sp = make_float2(0.f, 0.f); Qp = Sp; Sm = Sp; Qm = Sp;
    }
  };
  // staging -> work (natural order): the two runs of each column, in that order; thread t takes the columns t and t + 512
  auto reduce = [&]() {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const int col = t + h * THREADS;
      if (NCOL < 2 * THREADS && col >= NCOL) break;
      const int a = col / NR, n = col - a * NR;
      const float4 u0 = stg_p[col], v0 = stg_p[NCOL + col], u1 = stg_m[col], v1 = stg_m[NCOL + col];
      const float4 s0 = make_float4(u0.x + v0.x, u0.y + v0.y, u0.z + v0.z, u0.w + v0.w);
      const float4 s1 = make_float4(u1.x + v1.x, u1.y + v1.y, u1.z + v1.z, u1.w + v1.w);
      const int rp = a * PITCH, rm = ((64 - a) & 63) * PITCH;
      work[rp + n] = make_float2(s0.x, s0.y);
      if (n > 0) work[rm + 64 - n] = make_float2(s0.z, s0.w);
      if (a > 0) {
        work[rm + n] = make_float2(s1.x, s1.y);
        if (n > 0) work[rp + 64 - n] = make_float2(s1.z, s1.w);
      }
    }
    // the bins that no column fills hold what the last transform left there: cleared again
    if constexpr (NR == 32) {
      if (t < 64) { work[32 * PITCH + t] = make_float2(0.f, 0.f); work[t * PITCH + 32] = make_float2(0.f, 0.f); }
    } else {
      constexpr int GAP = 64 - 2 * NR + 1;                  // frequencies NR .. 64 - NR on either axis
      for (int i = t; i < GAP * 64; i += THREADS) work[(NR + (i >> 6)) * PITCH + (i & 63)] = make_float2(0.f, 0.f);
      for (int i = t; i < (64 - GAP) * GAP; i += THREADS) {
        const int rr = i / GAP, c = NR + (i - rr * GAP);
        work[(rr < NR ? rr : rr + GAP) * PITCH + c] = make_float2(0.f, 0.f);
      }
    }
  };
  // second alpha stage: lane lo takes the column slot sigma(lo), i.e. column gamma = lo; inputs at row slots
  // 8 d + j, outputs rows alpha = d + 8 k.  Real part -> plane j, imaginary part -> plane 63-j, one whole 256-byte row
  // per wave and store.
  auto stage_c2_store = [&](int j) {
    float2 v[8];
    [[maybe_unused]] float2 w[8];
    if constexpr (MOM == 2) {
#pragma unroll
      for (int k = 0; k < 8; ++k)
        w[k] = make_float2(buf_load_f32_policy(rw, yoff, (j * 4096 + k * 512) * 4, stream), buf_load_f32_policy(rw, yoff, ((63 - j) * 4096 + k * 512) * 4, stream));
    }
    const float2* line = work + sigma(lo) + 8 * d * PITCH;
#pragma unroll
    for (int k = 0; k < 8; ++k) v[k] = line[k * PITCH];
    fft8<true>(v);
    unsigned long long wa = 0, wb = 0;               // lane k: which samples of row d + 8 k are positive (one bit per column)
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      float ra = v[k].x + bz, rb = v[k].y + bz;
      if constexpr (MOM == 1) {
        if (j == j0 && k == 0) mpivot = ra;
        const float da = ra - mpivot, db = rb - mpivot;
        ms1 += da + db; ms2 = fmaf(da, da, fmaf(db, db, ms2));
      }
      if constexpr (MOM == 2) {
        const float ga = s2cnn::relu_pass(ra, fmaf(mom_a, w[k].x, mom_b)), gb = s2cnn::relu_pass(rb, fmaf(mom_a, w[k].y, mom_b));
        ms1 += ga + gb; ms2 = fmaf(ga, w[k].x, fmaf(gb, w[k].y, ms2));
      }
      if (relu) { ra = s2cnn::relu_f(ra); rb = s2cnn::relu_f(rb); }
      buf_store_f32_policy(ra, ry, yoff, (j * 4096 + k * 512) * 4, stream);
      buf_store_f32_policy(rb, ry, yoff, ((63 - j) * 4096 + k * 512) * 4, stream);
      if (bits) {                                   // the gradient of max(., 0) passes where the output is not <= 0 (a NaN passes)
        const unsigned long long qa = __ballot(!(ra <= 0.f)), qb = __ballot(!(rb <= 0.f));
        if (lo == k) { wa = qa; wb = qb; }
      }
    }
    if (bits && lo < 8) {                           // 64 contiguous bytes per plane and wave
      bits[bits_index(z, j, d) + lo] = wa;
      bits[bits_index(z, 63 - j, d) + lo] = wb;
    }
  };

#define S2CNN_FENCE() __builtin_amdgcn_sched_barrier(0)
  // the item's share, then its table slot is refilled with the item that uses the slot next (see table_slot)
  // (pair P being contributed; the slot then takes item k + 4 of the same pair or item k % 4 of the next one)
#define S2CNN_CON(k, P)                                                                                  \
  if constexpr ((k) < NA) {                                                                              \
    contribute(k, FR); S2CNN_FENCE();                                                                    \
    if constexpr ((k) + 4 < NA) load_table((P) < j1 ? (P) : j1 - 1, (k) + 4);                            \
    else load_table((P) + 1 < j1 ? (P) + 1 : j1 - 1, (k) & 3);                                           \
    S2CNN_FENCE();                                                                                       \
  }
  load_table(j0, 0);
  if constexpr (NA > 1) load_table(j0, 1);
  if constexpr (NA > 2) load_table(j0, 2);
  if constexpr (NA > 3) load_table(j0, 3);
  __syncthreads();
  {
    constexpr unsigned FR = FRESH_LO | FRESH_HI;
    S2CNN_CON(0, j0) S2CNN_CON(1, j0) S2CNN_CON(2, j0) S2CNN_CON(3, j0) S2CNN_CON(4, j0) S2CNN_CON(5, j0) S2CNN_CON(6, j0)
  }
  __syncthreads();
  reduce();
  __syncthreads();

  // step j: transform pair j in `work` and write it out, while the shares of pair j+1 go to the staging area.
  // Waves d < 4 transform first, waves d >= 4 last: each SIMD holds one wave of either kind, so the LDS-bound
  // and the FMA-bound half of a stage overlap.
  if (d < 4) {
    constexpr unsigned FR = FRESH_LO;
    for (int j = j0; j < j1 - 1; ++j) {
      fft_pass<true, 0>(work, twl); S2CNN_FENCE();
      S2CNN_CON(0, j + 1) S2CNN_CON(1, j + 1)
      __syncthreads();
      fft_pass<true, 1>(work, twl); S2CNN_FENCE();
      S2CNN_CON(2, j + 1) S2CNN_CON(3, j + 1)
      __syncthreads();
      fft_pass<true, 2>(work, twl); S2CNN_FENCE();
      S2CNN_CON(4, j + 1) S2CNN_CON(5, j + 1)
      __syncthreads();
      stage_c2_store(j); S2CNN_FENCE();
      S2CNN_CON(6, j + 1)
      __syncthreads();
      reduce();
      __syncthreads();
    }
  } else {
    constexpr unsigned FR = FRESH_HI;
    for (int j = j0; j < j1 - 1; ++j) {
      S2CNN_CON(0, j + 1) S2CNN_CON(1, j + 1)
      fft_pass<true, 0>(work, twl);
      __syncthreads();
      S2CNN_CON(2, j + 1) S2CNN_CON(3, j + 1)
      fft_pass<true, 1>(work, twl);
      __syncthreads();
      S2CNN_CON(4, j + 1) S2CNN_CON(5, j + 1)
      fft_pass<true, 2>(work, twl);
      __syncthreads();
      S2CNN_CON(6, j + 1)
      stage_c2_store(j);
      __syncthreads();
      reduce();
      __syncthreads();
    }
  }
#undef S2CNN_CON
#undef S2CNN_FENCE
  fft_pass<true, 0>(work, twl); __syncthreads();
  fft_pass<true, 1>(work, twl); __syncthreads();
  fft_pass<true, 2>(work, twl); __syncthreads();
  stage_c2_store(j1 - 1);
  if constexpr (MOM == 1) {                         // (mean, squared deviations) of every thread's 2 x 8 x 32 samples, merged pairwise in float64
    __syncthreads();
    double* red = reinterpret_cast<double*>(work);
    constexpr double NT_SAMPLES = 2.0 * 8.0 * NJ;
    red[t] = (double)mpivot + (double)ms1 / NT_SAMPLES;
    red[THREADS + t] = (double)ms2 - (double)ms1 * (double)ms1 / NT_SAMPLES;
    __syncthreads();
    double cnt = NT_SAMPLES;                        // samples behind each entry at this level
    for (int s = THREADS / 2; s > 0; s >>= 1) {
      if (t < s) {
        const double dm = red[t + s] - red[t];
        red[THREADS + t] += red[THREADS + t + s] + dm * dm * (0.5 * cnt);
        red[t] = 0.5 * (red[t] + red[t + s]);
      }
      cnt *= 2.0;
      __syncthreads();
    }
    if (t == 0) moments[z] = make_float2((float)(red[0] * cnt), (float)red[THREADS]);
  }
  if constexpr (MOM == 2) {                         // the threads' partial sums through LDS, pairwise, always in the same order
    __syncthreads();
    float* red = reinterpret_cast<float*>(work);
    red[t] = ms1; red[THREADS + t] = ms2;
    __syncthreads();
    for (int s = THREADS / 2; s > 0; s >>= 1) {
      if (t < s) { red[t] += red[t + s]; red[THREADS + t] += red[THREADS + t + s]; }
      __syncthreads();
    }
    if (t == 0) moments[z] = make_float2(red[0], red[THREADS]);
  }
}

// item rounds that carry degrees below nl (the template argument NA of the kernels below)
inline int active_rounds(int nl) { return nl <= 24 ? 3 : nl <= 28 ? 6 : NIT; }

// Launchers: the instantiation whose item rounds cover the nl degrees present.
template <int MASK, bool SPLIT, bool STREAM>
inline void launch_analysis_ms(int nl, hipStream_t st, const s2cnn::Input& in, const float* Tf, float4* rec, long nbatch, int nparts) {
  const dim3 grid(grid_size(nbatch * nparts)), block(THREADS);
  if (nl <= 24) hipLaunchKernelGGL((analysis_kernel<3, MASK, 0, SPLIT, STREAM>), grid, block, 0, st, in.x, in.w, Tf, rec, nbatch, in.params, in.nfeature, nparts);
  else if (nl <= 28) hipLaunchKernelGGL((analysis_kernel<6, MASK, 0, SPLIT, STREAM>), grid, block, 0, st, in.x, in.w, Tf, rec, nbatch, in.params, in.nfeature, nparts);
  else hipLaunchKernelGGL((analysis_kernel<7, MASK, 0, SPLIT, STREAM>), grid, block, 0, st, in.x, in.w, Tf, rec, nbatch, in.params, in.nfeature, nparts);
}

// a signal of s2cnn::STREAM_BYTES or more passes no cache: the instantiations with non-temporal loads / stores
inline bool streamed(long nbatch) { return (size_t)nbatch * (N * N * N * 4) >= s2cnn::STREAM_BYTES; }

// one workgroup per volume runs the instantiation whose plane loop has constant bounds
template <int MASK>
inline void launch_analysis_m(int nl, hipStream_t st, const s2cnn::Input& in, const float* Tf, float4* rec, long nbatch, int nparts) {
  if (nparts > 1) launch_analysis_ms<MASK, true, false>(nl, st, in, Tf, rec, nbatch, nparts);
  else if (streamed(nbatch)) launch_analysis_ms<MASK, false, true>(nl, st, in, Tf, rec, nbatch, 1);
  else launch_analysis_ms<MASK, false, false>(nl, st, in, Tf, rec, nbatch, 1);
}

// in: the signal and what is done to it in the loads (s2cnn::Input)
inline void launch_analysis(int nl, hipStream_t st, const s2cnn::Input& in, const float* Tf, float4* rec, long nbatch, int nparts = 1) {
  switch (in.kind) {
    case s2cnn::PRO_MASK: launch_analysis_m<1>(nl, st, in, Tf, rec, nbatch, nparts); break;
    case s2cnn::PRO_BITS: launch_analysis_m<2>(nl, st, in, Tf, rec, nbatch, nparts); break;
    case s2cnn::PRO_AFFINE_RELU: launch_analysis_m<3>(nl, st, in, Tf, rec, nbatch, nparts); break;
    case s2cnn::PRO_BN_RELU_GRAD: launch_analysis_m<4>(nl, st, in, Tf, rec, nbatch, nparts); break;
    default: launch_analysis_m<0>(nl, st, in, Tf, rec, nbatch, nparts);
  }
}

// bits: NULL, or BITS_WORDS 64-bit words per volume that receive one bit per sample: the output is not <= 0
// degrees up to which the kernel has registers to spare for the second operand of the sums of MOM = 2
constexpr int GRAD_MOMENTS_MAX_NL = 28;

// moments: NULL, or two sums per volume (see MOM): those of the output, or, with yref and params (nl <= GRAD_MOMENTS_MAX_NL
// only), those of the gradient of a normalisation
// nparts: workgroups per volume where no sums are formed (one with `moments`)
template <int MOM, bool SPLIT, bool STREAM>
inline void launch_synthesis_ms(int nl, hipStream_t st, const float4* rec, const float* Tf, float* y, long nbatch, const float* bias,
                                int nfeature, int relu, unsigned long long* bits, float2* moments, const float* yref, const float* params, int nparts) {
  const dim3 grid(grid_size(nbatch * nparts)), block(THREADS);
  if (nl <= 24) hipLaunchKernelGGL((synthesis_kernel<3, 0, MOM, SPLIT, STREAM>), grid, block, 0, st, rec, Tf, y, nbatch, bias, nfeature, relu, bits, moments, yref, params, nparts);
  else if (nl <= 28 || MOM == 2) hipLaunchKernelGGL((synthesis_kernel<6, 0, MOM, SPLIT, STREAM>), grid, block, 0, st, rec, Tf, y, nbatch, bias, nfeature, relu, bits, moments, yref, params, nparts);
  else hipLaunchKernelGGL((synthesis_kernel<(MOM == 2 ? 6 : 7), 0, MOM, SPLIT, STREAM>), grid, block, 0, st, rec, Tf, y, nbatch, bias, nfeature, relu, bits, moments, yref, params, nparts);
}
template <int MOM>
inline void launch_synthesis_m(int nl, hipStream_t st, const float4* rec, const float* Tf, float* y, long nbatch, const float* bias,
                               int nfeature, int relu, unsigned long long* bits, float2* moments, const float* yref, const float* params, int nparts) {
  if (MOM == 0 && nparts > 1) launch_synthesis_ms<0, true, false>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, bits, nullptr, nullptr, nullptr, nparts);
  else if (streamed(nbatch)) launch_synthesis_ms<MOM, false, true>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, bits, moments, yref, params, 1);
  else launch_synthesis_ms<MOM, false, false>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, bits, moments, yref, params, 1);
}
inline void launch_synthesis(int nl, hipStream_t st, const float4* rec, const float* Tf, float* y, long nbatch, const float* bias,
                             int nfeature, int relu, unsigned long long* bits, float2* moments = nullptr, const float* yref = nullptr,
                             const float* params = nullptr, int nparts = 1) {
  if (moments && yref) launch_synthesis_m<2>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, bits, moments, yref, params, 1);      // nl <= GRAD_MOMENTS_MAX_NL
  else if (moments) launch_synthesis_m<1>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, bits, moments, nullptr, nullptr, 1);
  else launch_synthesis_m<0>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, bits, nullptr, nullptr, nullptr, nparts);
}

}  // namespace fused64
