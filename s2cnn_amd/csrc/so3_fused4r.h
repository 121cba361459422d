// SO(3) analysis and synthesis of real signals on a grid of N = 4 R points per axis (bandwidth 2 R) as ONE kernel each, in
// the form of the 64^3 kernels of so3_fused64.h: a workgroup owns one volume, keeps its half spectrum in registers and
// walks over beta, so the transformed planes never leave the compute unit.  What is the same (the beta fold, the sign
// rules, the ITEMS, the quad layout, the per-volume records and the passes between records and spectral rows) is described
// there; this file says what differs.  Instantiated for the grids 20^3 (R = 5, bandwidth 10), 32^3 (R = 8, bandwidth 16)
// and 44^3 (R = 11, bandwidth 22).
//
// A volume of these grids is a fraction of the work of a 64^3 volume, so SEVERAL volumes are resident on a compute unit at
// once, each in another phase of its step: what the 64^3 kernels arrange inside one workgroup (two halves of the waves in
// different phases, two quad buffers) the hardware scheduler does here between workgroups, and a step is a plain
// sequence: transform a plane pair, barrier, contract it.
//
// An N-point line is 4 x R: with j = R j1 + j2 in, k = k1 + 4 k2 out,
//   X[k1 + 4 k2] = sum_{j2 < R} wR^{j2 k2} ( wN^{j2 k1} sum_{j1 < 4} x[R j1 + j2] w4^{j1 k1} ):
// pass A (N R threads = (line, j2)) does the 4-point sums and the twiddle in place (slots R j1 + j2 -> R k1 + j2), pass B
// (4 N threads = (line, k1)) the R-point sums in place (slots R k1 + j2 -> R k1 + k2): bin k sits at slot
// R (k % 4) + k / 4.  The R-point transform is the 8-point butterfly, or for other R a sum folded over j <-> R - j
// (half the multiplications of the plain sum).  The B passes of the two axes go to different waves of the workgroup.
//
// ITEMS (c, a, n) in the order of c, then a, then n; place p (round p / THREADS, thread p % THREADS) holds item p, so a
// spectrum cut off at a low degree leaves the later rounds without work, and an item's place in the staging area of the
// synthesis is its own number.
#pragma once
#include <hip/hip_runtime.h>
#include "so3_fused64.h"

namespace fused4r {

using fft64::fft4;
using fft64::fft8;
using fused64::buf_load_f32;
using fused64::buf_load_f32_stream;
using fused64::buf_load_f32_policy;
using fused64::buf_store_f32_policy;
using fused64::STREAM_BYTES;
using fused64::buf_load_f32x4;
using fused64::buf_store_f32;
using fused64::buf_store_f32_stream;
using fused64::buf_store_f32x4;
using fused64::flip;
using fused64::lmn_index;
using fused64::make_rsrc;
using fused64::volume_of_block;
using fused64::grid_size;

// sin and cos at compile time (|x| <= 2 pi): the constants of the folded R-point sums
constexpr double CX_PI = 3.14159265358979323846264338327950288;
constexpr double cx_sin_series(double x) {
  double term = x, sum = x;
  for (int k = 1; k < 16; ++k) { term *= -x * x / ((2 * k) * (2 * k + 1)); sum += term; }
  return sum;
}
constexpr double cx_sin(double x) {      // reduced to [-pi/2, pi/2]
  while (x > CX_PI) x -= 2 * CX_PI;
  while (x < -CX_PI) x += 2 * CX_PI;
  if (x > CX_PI / 2) x = CX_PI - x;
  if (x < -CX_PI / 2) x = -CX_PI - x;
  return cx_sin_series(x);
}
constexpr double cx_cos(double x) { return cx_sin(x + CX_PI / 2); }
template <int R, int Q> struct Trig {
  static constexpr float c = (float)cx_cos(2 * CX_PI * (Q % R) / R);
  static constexpr float s = (float)cx_sin(2 * CX_PI * (Q % R) / R);
};

// R-point DFT out of registers, natural order in; every output X[k] is handed to emit(k, X[k]) as soon as it is formed, so
// no second set of registers holds the outputs.  Sign of the exponent: - (forward) / + (INV).
// X[k] = v0 + sum_{j=1..H} ( p_j cos(2 pi j k / R) -+ i m_j sin(2 pi j k / R) ) for odd R,
// p_j = v_j + v_{R-j}, m_j = v_j - v_{R-j} (formed in place: v_j <- p_j, v_{R-j} <- m_j), H = (R - 1) / 2; X[R - k] has the
// other sign of the sine part.
template <int R, int K, int J>
__device__ __forceinline__ void dft_fold_term(const float2 (&v)[R], float2& C, float2& S) {
  if constexpr (J <= (R - 1) / 2) {
    constexpr float c = Trig<R, J * K>::c, s = Trig<R, J * K>::s;
    C.x = fmaf(v[J].x, c, C.x); C.y = fmaf(v[J].y, c, C.y);
    S.x = fmaf(v[R - J].x, s, S.x); S.y = fmaf(v[R - J].y, s, S.y);
    dft_fold_term<R, K, J + 1>(v, C, S);
  }
}
template <int R, bool INV, int K, class Emit>
__device__ __forceinline__ void dft_fold_outputs(const float2 (&v)[R], Emit& emit) {
  if constexpr (K <= (R - 1) / 2) {
    float2 C = v[0], S = make_float2(0.f, 0.f);
    dft_fold_term<R, K, 1>(v, C, S);
    // forward: X[K] = C - i S, X[R-K] = C + i S; inverse: the other way round
    const float2 lo = make_float2(C.x + S.y, C.y - S.x), hi = make_float2(C.x - S.y, C.y + S.x);
    emit(K, INV ? hi : lo);
    emit(R - K, INV ? lo : hi);
    dft_fold_outputs<R, INV, K + 1>(v, emit);
  }
}
template <int R, bool INV, class Emit>
__device__ __forceinline__ void dft_r(float2 (&v)[R], Emit emit) {
  if constexpr (R == 8) {
    fft8<INV>(v);
#pragma unroll
    for (int k = 0; k < 8; ++k) emit(k, v[k]);
  } else {
    static_assert(R % 2 == 1, "the folded sum is written for odd R");
    constexpr int H = (R - 1) / 2;
    float2 sum = v[0];
#pragma unroll
    for (int j = 1; j <= H; ++j) {
      const float2 a = v[j], b = v[R - j];
      v[j] = make_float2(a.x + b.x, a.y + b.y);
      v[R - j] = make_float2(a.x - b.x, a.y - b.y);
      sum.x += v[j].x; sum.y += v[j].y;
    }
    emit(0, sum);
    dft_fold_outputs<R, INV, 1>(v, emit);
  }
}

// The grid of N = 4 R points per axis and how a workgroup of T threads (a power of two) is laid over it;
// W = waves per SIMD the kernels are compiled for (workgroups per compute unit x T / 256).
// DMA: the analysis sends the loads of the next plane pair straight to LDS (buffer loads with the lds bit: lane i of a wave
// writes word i of a 256-byte row of its own), so no registers hold them while they are in flight; a wave waits for its own
// loads and reads back its own rows.
template <int R_, int T, int W, bool DMA_ = false>
struct Grid {
  static constexpr bool DMA = DMA_;
  static constexpr int R = R_;
  static constexpr int N = 4 * R;
  static constexpr int H = N / 2;               // bandwidth: frequencies 0 <= a, n < H; also the number of beta pairs
  static constexpr int NJ = H;
  static constexpr int NR = H;
  static constexpr int PITCH = N + 1;           // row pitch of the plane in complex elements (odd); column N is a pad
  static constexpr int LDS_ELEMS = N * PITCH;
  static constexpr int THREADS = T;
  static constexpr int WAVES_PER_SIMD = W;
  static constexpr int A_THREADS = N * R;       // threads of a pass A (and of the plane loads): (line, j2)
  static constexpr int B_THREADS = 4 * N;       // threads of a pass B: (line, k1)
  static constexpr int B_COLS_FIRST = (T - B_THREADS) / 64 * 64;     // the pass B of the column axis takes the last waves
  static constexpr int NCG = (NR + 3) / 4;      // degree groups c
  static __host__ __device__ constexpr int width(int c) { return 4 * c + 4 < NR ? 4 * c + 4 : NR; }     // a, n < width(c) in group c
  static __host__ __device__ constexpr int offset(int c) { int o = 0; for (int q = 0; q < c; ++q) o += width(q) * width(q); return o; }
  static constexpr int NITEMS = offset(NCG);
  static constexpr int NIT = (NITEMS + T - 1) / T;          // item rounds
  static constexpr size_t PACKED_FLOATS = (size_t)NJ * NIT * 2 * T * 4;
  static constexpr int REC_F4 = NIT * 4 * T;
  static constexpr size_t REC_BYTES = (size_t)REC_F4 * 16;
  static constexpr int QUAD_PITCH = NR * 4 + 14;
  static constexpr int QUAD_ELEMS = (NR + 1) * QUAD_PITCH;  // row NR takes the bins of m = N / 2, which nobody reads
  static_assert((T & (T - 1)) == 0 && A_THREADS <= T && NR * NR <= T && B_THREADS <= T / 2 + 64, "workgroup too small for the grid");
  static_assert((NR + 1) * 4 + 2 * (NR >> 3) <= QUAD_PITCH, "quad rows overlap");

  static __host__ __device__ constexpr int quad_row(int a) { return a * QUAD_PITCH + 2 * (a >> 3); }
  static __host__ __device__ constexpr int slot_of(int k) { return R * (k & 3) + (k >> 2); }     // where bin (or sample) k of a line sits
  static __host__ __device__ constexpr int index_of(int s) { return s / R + 4 * (s % R); }       // which bin (or sample) slot s holds
  // place p = round * THREADS + thread -> its item (c, a, n); false for a place without an item
  static __host__ __device__ inline bool decode(int p, int& c, int& a, int& n) {
    c = 0; a = 0; n = 0;
    if (p >= NITEMS) return false;
    for (int q = 1; q < NCG; ++q)
      if (p >= offset(q)) c = q;
    const int r = p - offset(c);
    a = r / width(c); n = r - a * width(c);
    return true;
  }
  // workgroups per volume: a power of two, at least four beta pairs each, no more than fill the chip once
  static int parts(long nbatch) {
    int p = 1;
    while (2 * p * 4 <= NJ && 2 * p * nbatch <= 256) p *= 2;
    return p;
  }
  static size_t scratch_bytes(long nbatch) { return (size_t)nbatch * parts(nbatch) * REC_BYTES; }
  // item rounds that carry degrees below nl
  static int active_rounds(int nl) {
    const int groups = nl >= NR ? NCG : (nl + 3) / 4;
    return (offset(groups) + T - 1) / T;
  }
};

using Grid20 = Grid<5, 128, 4>;                    // 20^3: eight
using Grid32 = Grid<8, 256, 4>;                    // 32^3: four workgroups per compute unit, plane loads through registers
using Grid44 = Grid<11, 512, 4, true>;       // 44^3: two (one, with all the registers it wants, is slower)

// Packed table, as fused64::pack_table: float index ((((j*NIT + it)*2 + h)*THREADS + t)*4 + u) holds
// 0.5 * T[j, l = 4c+u, m = (h ? -a : +a), n] for the item of place it*THREADS + t.  T is [N][nspec_stride].
template <class G>
__global__ void pack_table(const float* __restrict__ T, float* __restrict__ Tf, long nspec_stride, int nl) {
  for (size_t e = blockIdx.x * (size_t)blockDim.x + threadIdx.x; e < G::PACKED_FLOATS; e += (size_t)gridDim.x * blockDim.x) {
    const int u = (int)(e & 3);
    const int t = (int)((e >> 2) % G::THREADS);
    const int h = (int)((e / (4 * G::THREADS)) & 1);
    const int r = (int)(e / (8 * G::THREADS));
    const int it = r % G::NIT, j = r / G::NIT;
    int c, a, n;
    float v = 0.f;
    if (G::decode(it * G::THREADS + t, c, a, n)) {
      const int l = 4 * c + u;
      if (l >= a && l >= n && l < nl) v = 0.5f * T[(size_t)j * nspec_stride + lmn_index(l, h ? -a : a, n)];
    }
    Tf[e] = v;
  }
}

// wN^(d k), k = 1..3, for this thread's d = threadIdx.x / N (conjugated for the inverse)
struct Twiddles { float c[3], s[3]; };
template <class G, bool INV>
__device__ __forceinline__ void make_twiddles(Twiddles& tw) {
  const int d = threadIdx.x / G::N;
#pragma unroll
  for (int k = 1; k < 4; ++k) {
    float s, c;
    sincospif((float)(2 * d * k) / (float)G::N, &s, &c);     // angle 2 pi d k / N
    tw.c[k - 1] = c;
    tw.s[k - 1] = INV ? s : -s;
  }
}
__device__ __forceinline__ float2 twmul(float2 v, const Twiddles& tw, int k) {
  return make_float2(v.x * tw.c[k - 1] - v.y * tw.s[k - 1], v.x * tw.s[k - 1] + v.y * tw.c[k - 1]);
}

// pass A of an axis in place, by the threads (line lo, j2 = d): ROWS: elements along row lo; else along column lo
template <class G, bool INV, bool ROWS>
__device__ __forceinline__ void pass_a(float2* buf, const Twiddles& tw, int lo, int d) {
  if (G::A_THREADS < G::THREADS && threadIdx.x >= G::A_THREADS) return;
  float2* line = ROWS ? buf + lo * G::PITCH + d : buf + lo + d * G::PITCH;
  constexpr int stride = ROWS ? G::R : G::R * G::PITCH;
  float2 v0 = line[0], v1 = line[stride], v2 = line[2 * stride], v3 = line[3 * stride];
  fft4<INV>(v0, v1, v2, v3);
  line[0] = v0; line[stride] = twmul(v1, tw, 1); line[2 * stride] = twmul(v2, tw, 2); line[3 * stride] = twmul(v3, tw, 3);
}
// pass B in place, by the thread u = (line u % N, k1 = u / N) of its B_THREADS threads
template <class G, bool INV, bool ROWS>
__device__ __forceinline__ void pass_b(float2* buf, int u) {
  const int lo = u % G::N, k1 = u / G::N;
  float2* line = ROWS ? buf + lo * G::PITCH + G::R * k1 : buf + lo + G::R * k1 * G::PITCH;
  constexpr int stride = ROWS ? 1 : G::PITCH;
  float2 v[G::R];
#pragma unroll
  for (int j = 0; j < G::R; ++j) v[j] = line[j * stride];
  dft_r<G::R, INV>(v, [&](int k, float2 x) { line[k * stride] = x; });      // the thread's own slots: all of them are in registers by now
}

// ---------------------------------------------------------------------------------------------
// analysis: x [nbatch][N][N][N] real -> records of the half spectrum n >= 0
// NA: item rounds with degrees below the output bandwidth; MASK: s2cnn::Prologue (bit masks, 2, are not supported)
// nparts: workgroups per volume.  Few volumes do not fill the chip with one workgroup each: part p of a volume then takes
// the beta pairs p NJ / nparts .. (p+1) NJ / nparts - 1 and writes a record of its own ([volume][part]); the pass to the
// spectral rows adds the parts in their order.
// ---------------------------------------------------------------------------------------------
template <class G, int NA, int MASK, bool STREAM>
__global__ __launch_bounds__(G::THREADS, G::WAVES_PER_SIMD) void analysis_kernel(const float* __restrict__ x, const float* __restrict__ mask,
                                                                                const float* __restrict__ Tf, float4* __restrict__ rec,
                                                                                long nbatch, const float* __restrict__ params, int nfeature,
                                                                                int nparts) {
  static_assert(MASK != 2, "bit masks exist on the 64^3 grid only");
  constexpr bool MASKED = MASK == 1 || MASK == 4;
  constexpr int N = G::N, R = G::R, PITCH = G::PITCH, THREADS = G::THREADS, NJ = G::NJ, NR = G::NR, NIT = G::NIT;
  __shared__ __attribute__((aligned(16))) float2 work[G::LDS_ELEMS];
  __shared__ __attribute__((aligned(16))) float2 quad[G::QUAD_ELEMS];
  const long vp = volume_of_block(nbatch * nparts);
  if (vp < 0) return;
  const long z = vp / nparts;
  const int part = (int)(vp - z * nparts);
  const int j0 = part * NJ / nparts, j1 = (part + 1) * NJ / nparts;
  constexpr bool stream = STREAM;        // the signal passes no cache (see s2cnn::STREAM_BYTES): non-temporal loads / stores
  const int t = threadIdx.x;
  const int lo = t % N, d = t / N;
  const bool in_a = G::A_THREADS == THREADS || t < G::A_THREADS;
  Twiddles tw;
  make_twiddles<G, false>(tw);
  for (int i = t; i < G::QUAD_ELEMS; i += THREADS) quad[i] = make_float2(0.f, 0.f);    // the -a half of a = 0 is never written and reads as zero
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
    G::decode(it * THREADS + t, c, a, n);
    adr[it] = (unsigned)(G::quad_row(a) + 4 * n) | ((unsigned)(n & 1) << 31);
  }
  // last gamma pass (threads t < B_THREADS: row slot t % N, k1 = t / N): where the outputs of row m = index_of(slot) go
  const int m = G::index_of(lo);
  const int am = m <= N / 2 ? m : N - m;
  const int qa = G::quad_row(am);
  const int pos_lo = m > N / 2 ? 2 : 0;                    // place of an output with n >= 0
  const int pos_hi = (m > N / 2 || m == 0) ? 1 : 3;        // place of an output with n < 0 (m = 0 counts as -0 there)

  float2 accp[NA][4], accm[NA][4];
#pragma unroll
  for (int it = 0; it < NA; ++it)
#pragma unroll
    for (int u = 0; u < 4; ++u) { accp[it][u] = make_float2(0.f, 0.f); accm[it][u] = make_float2(0.f, 0.f); }

  const __amdgpu_buffer_rsrc_t rx = make_rsrc(x + (size_t)z * (N * N * N), N * N * N * 4);
  const __amdgpu_buffer_rsrc_t rm = make_rsrc((MASKED ? mask : x) + (size_t)z * (N * N * N), N * N * N * 4);
  const __amdgpu_buffer_rsrc_t rt = make_rsrc(Tf, (unsigned)(G::PACKED_FLOATS * 4));
  const unsigned xoff = t * 4;           // + (beta N^2 + j1 R N) * 4: row alpha = R j1 + d, column gamma = lo (d N + lo = t)
  const unsigned toff = t * 16;
  float pa[4], pb[4];
  float ma[MASKED ? 4 : 1], mb[MASKED ? 4 : 1];
  // DMA: [tensor][plane][j1][thread] words, filled by the loads themselves
  __shared__ __attribute__((aligned(16))) float landing[G::DMA ? (MASKED ? 16 : 8) * THREADS : 1];
  const int wave_first = __builtin_amdgcn_readfirstlane(t & ~63);       // first thread of this wave
  float4 t1[NA], t2[NA];

  auto load_planes = [&](int j) {        // rows R j1 + d of the planes j and N-1-j: contiguous over the workgroup
    if constexpr (G::DMA) {
      typedef __attribute__((address_space(3))) void* lds_ptr;
      if constexpr (stream) {       // the cache policy is an immediate of the instruction
#pragma unroll
        for (int j1 = 0; j1 < 4; ++j1) {
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr)(landing + (0 + j1) * THREADS + wave_first), 4, (int)xoff, (j * N * N + j1 * R * N) * 4, 0, 2);
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr)(landing + (4 + j1) * THREADS + wave_first), 4, (int)xoff, ((N - 1 - j) * N * N + j1 * R * N) * 4, 0, 2);
          if constexpr (MASKED) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rm, (lds_ptr)(landing + (8 + j1) * THREADS + wave_first), 4, (int)xoff, (j * N * N + j1 * R * N) * 4, 0, 2);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rm, (lds_ptr)(landing + (12 + j1) * THREADS + wave_first), 4, (int)xoff, ((N - 1 - j) * N * N + j1 * R * N) * 4, 0, 2);
          }
        }
      } else {
#pragma unroll
        for (int j1 = 0; j1 < 4; ++j1) {
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr)(landing + (0 + j1) * THREADS + wave_first), 4, (int)xoff, (j * N * N + j1 * R * N) * 4, 0, 0);
          __builtin_amdgcn_raw_ptr_buffer_load_lds(rx, (lds_ptr)(landing + (4 + j1) * THREADS + wave_first), 4, (int)xoff, ((N - 1 - j) * N * N + j1 * R * N) * 4, 0, 0);
          if constexpr (MASKED) {
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rm, (lds_ptr)(landing + (8 + j1) * THREADS + wave_first), 4, (int)xoff, (j * N * N + j1 * R * N) * 4, 0, 0);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rm, (lds_ptr)(landing + (12 + j1) * THREADS + wave_first), 4, (int)xoff, ((N - 1 - j) * N * N + j1 * R * N) * 4, 0, 0);
          }
        }
      }
      return;
    }
#pragma unroll
    for (int j1 = 0; j1 < 4; ++j1) {
      pa[j1] = buf_load_f32_policy(rx, xoff, (j * N * N + j1 * R * N) * 4, stream);
      pb[j1] = buf_load_f32_policy(rx, xoff, ((N - 1 - j) * N * N + j1 * R * N) * 4, stream);
      if constexpr (MASKED) {
        ma[j1] = buf_load_f32_policy(rm, xoff, (j * N * N + j1 * R * N) * 4, stream);
        mb[j1] = buf_load_f32_policy(rm, xoff, ((N - 1 - j) * N * N + j1 * R * N) * 4, stream);
      }
    }
  };
  auto load_table = [&](int j, int it) {
    t1[it] = buf_load_f32x4(rt, toff, ((j * NIT + it) * 2 + 0) * (THREADS * 16));
    t2[it] = buf_load_f32x4(rt, toff, ((j * NIT + it) * 2 + 1) * (THREADS * 16));
  };
  // pass A of the alpha axis out of the registers: 4-point transforms over j1, twiddle, -> work[R k1 + d][lo]
  auto stage_c1 = [&]() {
    float2 v[4];
    if constexpr (G::DMA) {        // this wave's loads have landed (vmcnt = 0), then its own words are read back
      __builtin_amdgcn_s_waitcnt(0x0F70);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int j1 = 0; j1 < 4; ++j1) {
        pa[j1] = landing[(0 + j1) * THREADS + t];
        pb[j1] = landing[(4 + j1) * THREADS + t];
        if constexpr (MASKED) { ma[j1] = landing[(8 + j1) * THREADS + t]; mb[j1] = landing[(12 + j1) * THREADS + t]; }
      }
    }
#pragma unroll
    for (int j1 = 0; j1 < 4; ++j1) {
      if constexpr (MASK == 1) v[j1] = make_float2(s2cnn::relu_pass(pa[j1], ma[j1]), s2cnn::relu_pass(pb[j1], mb[j1]));
      else if constexpr (MASK == 3) v[j1] = make_float2(s2cnn::affine_relu(pa[j1], pr_a, pr_b), s2cnn::affine_relu(pb[j1], pr_a, pr_b));
      else if constexpr (MASK == 4) v[j1] = make_float2(s2cnn::bn_relu_grad(pa[j1], ma[j1], pr_a, pr_b, pr_p, pr_q),
                                                        s2cnn::bn_relu_grad(pb[j1], mb[j1], pr_a, pr_b, pr_p, pr_q));
      else v[j1] = make_float2(pa[j1], pb[j1]);
    }
    fft4<false>(v[0], v[1], v[2], v[3]);
    if (!in_a) return;
    float2* col = work + d * PITCH + lo;
    col[0] = v[0];
    col[R * PITCH] = twmul(v[1], tw, 1);
    col[2 * R * PITCH] = twmul(v[2], tw, 2);
    col[3 * R * PITCH] = twmul(v[3], tw, 3);
  };
  // pass B of the gamma axis: row slot lo, inputs at slots R k1 + j2 (k1 = d), outputs n = k1 + 4 k2 -> quad layout:
  // n < N/2 to the place of +n, n > N/2 to the place of -(N - n); n = N/2 lands in the spare quad of the row
  auto stage_r2 = [&]() {
    float2 v[R];
    const float2* line = work + lo * PITCH + R * d;
#pragma unroll
    for (int j2 = 0; j2 < R; ++j2) v[j2] = line[j2];
    dft_r<R, false>(v, [&](int k2, float2 x) {
      if (4 * k2 + 3 < N / 2) {
        quad[qa + 4 * (d + 4 * k2) + pos_lo] = x;
      } else if (4 * k2 > N / 2) {
        quad[qa + 4 * (N - d - 4 * k2) + pos_hi] = x;
      } else {                                   // the group of four that holds n = N/2: which side depends on k1
        const int n = d + 4 * k2;
        const bool neg = n > N / 2;
        quad[qa + 4 * (neg ? N - n : n) + (neg ? pos_hi : pos_lo)] = x;
      }
      if (k2 == 0 && d == 0) quad[qa + pos_hi] = x;          // n = 0 again as -0
    });
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

  // The barriers of a step order LDS accesses only.  With loads on their way to LDS, __syncthreads() would wait for them
  // too (its fence covers every write to LDS): there the barrier is taken once this wave's own LDS accesses are done.
  auto step_barrier = [&]() {
    if constexpr (G::DMA) {
      asm volatile("" ::: "memory");                // the compiler moves no memory access across the barrier ...
      __builtin_amdgcn_s_waitcnt(0xC07F);           // lgkmcnt(0)
      __builtin_amdgcn_s_barrier();
      asm volatile("" ::: "memory");                // ... in either direction
    } else {
      __syncthreads();
    }
  };
  __syncthreads();                                  // cleared quads
  load_planes(j0);
  for (int j = j0; j < j1; ++j) {
    stage_c1();
    // the next plane pair, in flight during the step.  Into registers: clamped, not branched (a branch would make the loads
    // synchronous); into LDS: none after the last pair (nothing would read them)
    if constexpr (!G::DMA) load_planes(j + 1 < j1 ? j + 1 : j1 - 1);
    else { __builtin_amdgcn_sched_barrier(0); if (j + 1 < j1) load_planes(j + 1); }
    step_barrier();
    if (t >= G::B_COLS_FIRST && t < G::B_COLS_FIRST + G::B_THREADS) pass_b<G, false, false>(work, t - G::B_COLS_FIRST);
    step_barrier();
    pass_a<G, false, true>(work, tw, lo, d);
    step_barrier();
    if (t < G::B_THREADS) stage_r2();
#pragma unroll
    for (int it = 0; it < NA; ++it) load_table(j, it);        // only now: their registers are not held through the transform
    step_barrier();
#pragma unroll
    for (int it = 0; it < NA; ++it) accumulate(it);
  }

  const __amdgpu_buffer_rsrc_t rr = make_rsrc(rec + (size_t)vp * G::REC_F4, (unsigned)G::REC_BYTES);      // record [z][part]
#pragma unroll
  for (int it = 0; it < NA; ++it) {                 // the pass that follows reads these rounds only
    buf_store_f32x4(make_float4(accp[it][0].x, accp[it][0].y, accp[it][1].x, accp[it][1].y), rr, toff, (it * 4 + 0) * (THREADS * 16));
    buf_store_f32x4(make_float4(accp[it][2].x, accp[it][2].y, accp[it][3].x, accp[it][3].y), rr, toff, (it * 4 + 1) * (THREADS * 16));
    buf_store_f32x4(make_float4(accm[it][0].x, accm[it][0].y, accm[it][1].x, accm[it][1].y), rr, toff, (it * 4 + 2) * (THREADS * 16));
    buf_store_f32x4(make_float4(accm[it][2].x, accm[it][2].y, accm[it][3].x, accm[it][3].y), rr, toff, (it * 4 + 3) * (THREADS * 16));
  }
}

// ---------------------------------------------------------------------------------------------
// synthesis: records of the symmetrised spectrum -> y [nbatch][N][N][N] real
//
// Every item adds its share of the bins of a plane pair to a place of its own in a staging area (its number); a reduction
// sums the places of each column (a, n), one per degree group c >= max(a, n) / 4, in that order, into the plane.
// bias, relu, MOM, moments, yref, params: as fused64::synthesis_kernel (no bit masks).
// nparts: workgroups per volume (1 with MOM): part p reads the volume's record and writes the planes of its beta pairs.
// ---------------------------------------------------------------------------------------------
template <class G, int NA, int MOM, bool STREAM>
__global__ __launch_bounds__(G::THREADS, G::WAVES_PER_SIMD) void synthesis_kernel(const float4* __restrict__ rec, const float* __restrict__ Tf,
                                                                                 float* __restrict__ y, long nbatch, const float* __restrict__ bias,
                                                                                 int nfeature, int relu, float2* __restrict__ moments,
                                                                                 const float* __restrict__ yref, const float* __restrict__ params,
                                                                                 int nparts) {
  constexpr int N = G::N, R = G::R, PITCH = G::PITCH, THREADS = G::THREADS, NJ = G::NJ, NR = G::NR, NIT = G::NIT;
  __shared__ __attribute__((aligned(16))) float2 work[G::LDS_ELEMS];
  // places 0 .. NITEMS-1: one per item; ZERO_PLACE: never written, read for the degree groups a column does not have;
  // DUMP_PLACE: written by the threads without an item, never read
  constexpr int ZERO_PLACE = G::NITEMS, DUMP_PLACE = G::NITEMS + 1, NPLACES = G::NITEMS + 2;
  // degree groups that the NA rounds hold at least in part (the others are zero)
  constexpr int GROUPS = [] { int g = 0; for (int c = 0; c < G::NCG; ++c) if (G::offset(c) < NA * THREADS) g = c + 1; return g; }();
  __shared__ __attribute__((aligned(16))) float4 stg[2 * NPLACES];
  float4* const stg_p = stg;                 // the item's share of the bins [+a,n], [-a,-n]
  float4* const stg_m = stg + NPLACES;       //                              [-a,n], [+a,-n]
  const long vp = volume_of_block(nbatch * nparts);
  if (vp < 0) return;
  const long z = vp / nparts;
  const int part = (int)(vp - z * nparts);
  const int j0 = part * NJ / nparts, j1 = (part + 1) * NJ / nparts;
  constexpr bool stream = STREAM;        // the signal passes no cache (see s2cnn::STREAM_BYTES): non-temporal loads / stores
  const int t = threadIdx.x;
  const int lo = t % N, d = t / N;
  const float bz = bias ? bias[z % nfeature] : 0.f;
  float ms1 = 0.f, ms2 = 0.f;
  [[maybe_unused]] float mpivot = 0.f;
  Twiddles tw;
  make_twiddles<G, true>(tw);
  for (int i = t; i < G::LDS_ELEMS; i += THREADS) work[i] = make_float2(0.f, 0.f);
  for (int i = t; i < NPLACES; i += THREADS) { stg_p[i] = make_float4(0.f, 0.f, 0.f, 0.f); stg_m[i] = make_float4(0.f, 0.f, 0.f, 0.f); }   // places of skipped rounds stay zero

  const __amdgpu_buffer_rsrc_t rr = make_rsrc(rec + (size_t)z * G::REC_F4, (unsigned)G::REC_BYTES);
  const __amdgpu_buffer_rsrc_t rt = make_rsrc(Tf, (unsigned)(G::PACKED_FLOATS * 4));
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
    const bool ok = G::decode(it * THREADS + t, c, a, n);
    place[it] = ok ? (it * THREADS + t) | ((n & 1) << 30) : DUMP_PLACE;
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
  // staging -> work (natural order): thread t < NR^2 takes the column a = t / NR, n = t % NR.  No branches inside: a
  // degree group the column does not have reads the zero place, a bin that does not exist (-0) goes to the pad column.
  // the thread's reduction indices, kept in LDS where registers are short (three item rounds): [index][thread] words
  constexpr bool RED_LDS = NA >= 3;
  __shared__ unsigned short red_tab[RED_LDS ? (GROUPS + 4) * THREADS : 1];
  int red_pos[GROUPS], red_dst[4];
  const bool in_red = NR * NR == THREADS || t < NR * NR;
  {
    const int a = in_red ? t / NR : 0, n = in_red ? t % NR : 0;
    const int cmin = (a > n ? a : n) >> 2;
#pragma unroll
    for (int c = 0; c < GROUPS; ++c) red_pos[c] = c >= cmin ? G::offset(c) + a * G::width(c) + n : ZERO_PLACE;
    const int rp = a * PITCH, rm = ((N - a) % N) * PITCH;
    red_dst[0] = rp + n;                                  // [+a, n]
    red_dst[1] = n > 0 ? rm + N - n : rm + N;             // [-a,-n]
    red_dst[2] = a > 0 ? rm + n : rp + N;                 // [-a, n]
    red_dst[3] = a > 0 && n > 0 ? rp + N - n : rp + N;    // [+a,-n]
    if constexpr (RED_LDS) {
#pragma unroll
      for (int c = 0; c < GROUPS; ++c) red_tab[c * THREADS + t] = (unsigned short)red_pos[c];
#pragma unroll
      for (int q = 0; q < 4; ++q) red_tab[(GROUPS + q) * THREADS + t] = (unsigned short)red_dst[q];
    }
  }
  auto reduce = [&]() {
    if (in_red) {
      float4 s0 = make_float4(0.f, 0.f, 0.f, 0.f), s1 = s0;
#pragma unroll
      for (int c = 0; c < GROUPS; ++c) {
        const int pos = RED_LDS ? (int)red_tab[c * THREADS + t] : red_pos[c];
        const float4 u0 = stg_p[pos], u1 = stg_m[pos];
        s0 = make_float4(s0.x + u0.x, s0.y + u0.y, s0.z + u0.z, s0.w + u0.w);
        s1 = make_float4(s1.x + u1.x, s1.y + u1.y, s1.z + u1.z, s1.w + u1.w);
      }
      work[RED_LDS ? (int)red_tab[(GROUPS + 0) * THREADS + t] : red_dst[0]] = make_float2(s0.x, s0.y);
      work[RED_LDS ? (int)red_tab[(GROUPS + 1) * THREADS + t] : red_dst[1]] = make_float2(s0.z, s0.w);
      work[RED_LDS ? (int)red_tab[(GROUPS + 2) * THREADS + t] : red_dst[2]] = make_float2(s1.x, s1.y);
      work[RED_LDS ? (int)red_tab[(GROUPS + 3) * THREADS + t] : red_dst[3]] = make_float2(s1.z, s1.w);
    }
    // the bins of m = N/2 and n = N/2 hold what the last transform left there: cleared again
    if (t < N) { work[(N / 2) * PITCH + t] = make_float2(0.f, 0.f); work[t * PITCH + N / 2] = make_float2(0.f, 0.f); }
  };
  // pass B of the alpha axis by the threads u = (gamma = u % N, k1 = u / N): the column of sample gamma sits at
  // slot_of(gamma); outputs rows alpha = k1 + 4 k2.  Real part -> plane j, imaginary part -> plane N-1-j; the stores of
  // the workgroup cover four adjacent rows at once.
  auto stage_c2_store = [&](int j, int u) {
    const unsigned yoff = u * 4;                  // + (beta N^2 + k2 4 N) * 4   (k1 N + gamma = u)
    float2 v[R];
    [[maybe_unused]] float2 w[R];
    if constexpr (MOM == 2) {
#pragma unroll
      for (int k = 0; k < R; ++k)
        w[k] = make_float2(buf_load_f32_policy(rw, yoff, (j * N * N + k * 4 * N) * 4, stream), buf_load_f32_policy(rw, yoff, ((N - 1 - j) * N * N + k * 4 * N) * 4, stream));
    }
    const float2* line = work + G::slot_of(u % N) + R * (u / N) * PITCH;
#pragma unroll
    for (int k = 0; k < R; ++k) v[k] = line[k * PITCH];
    dft_r<R, true>(v, [&](int k, float2 x) {
      float ra = x.x + bz, rb = x.y + bz;
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
      buf_store_f32_policy(ra, ry, yoff, (j * N * N + k * 4 * N) * 4, stream);
      buf_store_f32_policy(rb, ry, yoff, ((N - 1 - j) * N * N + k * 4 * N) * 4, stream);
    });
  };
  const bool in_store = t >= G::B_COLS_FIRST && t < G::B_COLS_FIRST + G::B_THREADS;

  load_table(j0);
  __syncthreads();                                  // cleared work and staging
#pragma unroll
  for (int it = 0; it < NA; ++it) contribute(it);
  if (G::B_COLS_FIRST < (G::B_THREADS + 63) / 64 * 64) load_table(j0 + 1 < j1 ? j0 + 1 : j1 - 1);
  __syncthreads();
  reduce();
  __syncthreads();
  // The shares of pair j + 1 are formed while pair j is in the plane.  Where the B passes of the two axes have waves of
  // their own (SPLIT), every wave forms its shares while it would otherwise wait for one of them: the waves beyond those
  // of the row pass B during that pass, the others during the last pass and its stores; their table values are loaded
  // right before.
  constexpr int ROW_B_END = (G::B_THREADS + 63) / 64 * 64;
  constexpr bool SPLIT = ROW_B_END <= G::B_COLS_FIRST;
  const bool early = t >= ROW_B_END;
  for (int j = j0; j < j1; ++j) {
    const bool more = j + 1 < j1;
    if (!SPLIT && more) {
#pragma unroll
      for (int it = 0; it < NA; ++it) contribute(it);
    }
    if (SPLIT && more && early) load_table(j + 1);
    pass_a<G, true, true>(work, tw, lo, d);
    __syncthreads();
    if (t < G::B_THREADS) pass_b<G, true, true>(work, t);
    if (SPLIT && more) {
      if (early) {
#pragma unroll
        for (int it = 0; it < NA; ++it) contribute(it);
      } else {
        load_table(j + 1);
      }
    }
    __syncthreads();
    pass_a<G, true, false>(work, tw, lo, d);
    __syncthreads();
    if (in_store) stage_c2_store(j, t - G::B_COLS_FIRST);
    if (SPLIT && more && !early) {
#pragma unroll
      for (int it = 0; it < NA; ++it) contribute(it);
    }
    if (more) {
      if (!SPLIT) load_table(j + 2 < j1 ? j + 2 : j1 - 1);      // only now: its registers are not held through the transform
      __syncthreads();
      reduce();
      __syncthreads();
    }
  }
  // the sums of the B_THREADS threads that hold samples (2 R NJ each) through LDS, pairwise, always in the same order;
  // threads without samples enter with a count of zero
  constexpr int PAD = G::B_THREADS <= 128 ? 128 : G::B_THREADS <= 256 ? 256 : 512;
  static_assert(PAD <= THREADS && 3 * PAD * 8 <= (int)sizeof(stg), "reduction does not fit");
  if constexpr (MOM == 1) {                         // (mean, squared deviations, count) per thread, merged in float64
    __syncthreads();
    double* red = reinterpret_cast<double*>(stg);    // [3][PAD]: mean, M2, count
    constexpr double NT_SAMPLES = 2.0 * R * NJ;
    if (t < PAD) { red[t] = 0.0; red[PAD + t] = 0.0; red[2 * PAD + t] = 0.0; }
    __syncthreads();
    if (in_store) {
      const int u = t - G::B_COLS_FIRST;
      red[u] = (double)mpivot + (double)ms1 / NT_SAMPLES;
      red[PAD + u] = (double)ms2 - (double)ms1 * (double)ms1 / NT_SAMPLES;
      red[2 * PAD + u] = NT_SAMPLES;
    }
    __syncthreads();
    for (int s = PAD / 2; s > 0; s >>= 1) {
      if (t < s) {
        const double na = red[2 * PAD + t], nb = red[2 * PAD + t + s], n = na + nb;
        if (nb > 0.0) {
          const double dm = red[t + s] - red[t];
          red[PAD + t] += red[PAD + t + s] + dm * dm * (na * nb / n);
          red[t] += dm * (nb / n);
          red[2 * PAD + t] = n;
        }
      }
      __syncthreads();
    }
    if (t == 0) moments[z] = make_float2((float)(red[0] * red[2 * PAD]), (float)red[PAD]);
  }
  if constexpr (MOM == 2) {
    __syncthreads();
    float* red = reinterpret_cast<float*>(stg);
    if (t < PAD) { red[t] = 0.f; red[PAD + t] = 0.f; }
    __syncthreads();
    if (in_store) { red[t - G::B_COLS_FIRST] = ms1; red[PAD + t - G::B_COLS_FIRST] = ms2; }
    __syncthreads();
    for (int s = PAD / 2; s > 0; s >>= 1) {
      if (t < s) { red[t] += red[t + s]; red[PAD + t] += red[PAD + t + s]; }
      __syncthreads();
    }
    if (t == 0) moments[z] = make_float2(red[0], red[PAD]);
  }
}

// Launchers: the instantiation whose item rounds cover the nl degrees present.
template <class G, int MASK, bool STREAM>
inline void launch_analysis_ms(int nl, hipStream_t st, const s2cnn::Input& in, const float* Tf, float4* rec, long nbatch, int nparts) {
  const dim3 grid(grid_size(nbatch * nparts)), block(G::THREADS);
  const int na = G::active_rounds(nl);
  static_assert(G::NIT <= 3, "add the instantiations of more rounds");
  if (na <= 1) hipLaunchKernelGGL((analysis_kernel<G, 1, MASK, STREAM>), grid, block, 0, st, in.x, in.w, Tf, rec, nbatch, in.params, in.nfeature, nparts);
  else if (na == 2 || G::NIT < 3) hipLaunchKernelGGL((analysis_kernel<G, (G::NIT < 2 ? G::NIT : 2), MASK, STREAM>), grid, block, 0, st, in.x, in.w, Tf, rec, nbatch, in.params, in.nfeature, nparts);
  else hipLaunchKernelGGL((analysis_kernel<G, G::NIT, MASK, STREAM>), grid, block, 0, st, in.x, in.w, Tf, rec, nbatch, in.params, in.nfeature, nparts);
}
// a signal of s2cnn::STREAM_BYTES or more passes no cache: the instantiation with non-temporal loads
template <class G> inline bool streamed(long nbatch) { return (size_t)nbatch * (G::N * G::N * G::N * 4) >= s2cnn::STREAM_BYTES; }
template <class G, int MASK>
inline void launch_analysis_m(int nl, hipStream_t st, const s2cnn::Input& in, const float* Tf, float4* rec, long nbatch, int nparts) {
  if (streamed<G>(nbatch)) launch_analysis_ms<G, MASK, true>(nl, st, in, Tf, rec, nbatch, nparts);
  else launch_analysis_ms<G, MASK, false>(nl, st, in, Tf, rec, nbatch, nparts);
}

// in: the signal and what is done to it in the loads (s2cnn::Input; not PRO_BITS)
template <class G>
inline void launch_analysis(int nl, hipStream_t st, const s2cnn::Input& in, const float* Tf, float4* rec, long nbatch, int nparts) {
  switch (in.kind) {
    case s2cnn::PRO_MASK: launch_analysis_m<G, 1>(nl, st, in, Tf, rec, nbatch, nparts); break;
    case s2cnn::PRO_AFFINE_RELU: launch_analysis_m<G, 3>(nl, st, in, Tf, rec, nbatch, nparts); break;
    case s2cnn::PRO_BN_RELU_GRAD: launch_analysis_m<G, 4>(nl, st, in, Tf, rec, nbatch, nparts); break;
    default: launch_analysis_m<G, 0>(nl, st, in, Tf, rec, nbatch, nparts);
  }
}

template <class G, int MOM, bool STREAM>
inline void launch_synthesis_ms(int nl, hipStream_t st, const float4* rec, const float* Tf, float* y, long nbatch, const float* bias,
                                int nfeature, int relu, float2* moments, const float* yref, const float* params, int nparts) {
  const dim3 grid(grid_size(nbatch * nparts)), block(G::THREADS);
  const int na = G::active_rounds(nl);
  if (na <= 1) hipLaunchKernelGGL((synthesis_kernel<G, 1, MOM, STREAM>), grid, block, 0, st, rec, Tf, y, nbatch, bias, nfeature, relu, moments, yref, params, nparts);
  else if (na == 2 || G::NIT < 3) hipLaunchKernelGGL((synthesis_kernel<G, (G::NIT < 2 ? G::NIT : 2), MOM, STREAM>), grid, block, 0, st, rec, Tf, y, nbatch, bias, nfeature, relu, moments, yref, params, nparts);
  else hipLaunchKernelGGL((synthesis_kernel<G, G::NIT, MOM, STREAM>), grid, block, 0, st, rec, Tf, y, nbatch, bias, nfeature, relu, moments, yref, params, nparts);
}
template <class G, int MOM>
inline void launch_synthesis_m(int nl, hipStream_t st, const float4* rec, const float* Tf, float* y, long nbatch, const float* bias,
                               int nfeature, int relu, float2* moments, const float* yref, const float* params, int nparts) {
  if (streamed<G>(nbatch)) launch_synthesis_ms<G, MOM, true>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, moments, yref, params, nparts);
  else launch_synthesis_ms<G, MOM, false>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, moments, yref, params, nparts);
}

// moments: NULL, or two sums per volume: those of the output, or, with yref and params, those of the gradient of a normalisation
// (one workgroup per volume then, whatever nparts says)
template <class G>
inline void launch_synthesis(int nl, hipStream_t st, const float4* rec, const float* Tf, float* y, long nbatch, const float* bias,
                             int nfeature, int relu, int nparts, float2* moments = nullptr, const float* yref = nullptr, const float* params = nullptr) {
  if (moments && yref) launch_synthesis_m<G, 2>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, moments, yref, params, 1);
  else if (moments) launch_synthesis_m<G, 1>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, moments, nullptr, nullptr, 1);
  else launch_synthesis_m<G, 0>(nl, st, rec, Tf, y, nbatch, bias, nfeature, relu, nullptr, nullptr, nullptr, nparts);
}

}  // namespace fused4r
