// Block-diagonal REAL products over the (2l+1)x(2l+1) blocks of an SO(3) spectrum held in the real
// basis (see so3_real_basis.hip), on the fp32 matrix cores of gfx950 (v_mfma_f32_32x32x2_f32).
//
// The spectrum of a real signal on SO(3) obeys x[l,-m,-n] = (-1)^(m-n) conj(x[l,m,n]); a fixed unitary
// change of basis per degree turns every such block into a real matrix, and the complex product
// z = x y^H of two such spectra into the real product z_r = x_r y_r^T: a quarter of the multiply-adds.
//
//   fwd   : Z [(m,i),(n,j)] = sum_{(p,k)} X [(m,i),(p,k)] * Y [(p,k),(n,j)]
//   gradx : GX[(m,i),(p,k)] = sum_{(n,j)} GZ[(m,i),(n,j)] * Y [(n,j),(p,k)]
//   grady : GY[(p,k),(n,j)] = sum_{(m,i)} X [(p,k),(m,i)] * GZ[(m,i),(n,j)]
//
// with tensors stored as [l, spectral row, spectral col, feature row, feature col] (the layout of the
// complex product without the trailing pair).  As there, an operand is an L x L grid of dense feature
// blocks in which either the contraction index ("K-contiguous") or the free index ("MN-contiguous") is
// the fast one, and each tile sits in LDS in the orientation it has in memory.
//
// One MFMA 32x32x2 takes two contraction steps, one per half-wave; a lane reads four consecutive steps
// at once (k = 8s + 4h .. +3) and feeds them to four consecutive MFMAs.
//
// Tiling.  A workgroup (4 waves) owns TM x TN = (64 NRB) x (64 NCB) outputs (NCB = 2, or 1 when the 128 x 128 tiles
// of a small problem would leave CUs without work); wave (wm, wn) takes row
// blocks wm + 2i and column blocks wn + 2j (interleaved, so ragged tiles still split evenly).  The grid
// lists exactly the tiles of all degrees, heaviest degree first.
#include <type_traits>
#include "common.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int NRB = 2;            // 32-row blocks per wave
constexpr int TM = 64 * NRB;
constexpr int BSTR = 64, WSTR = 32;
constexpr int TK = 32;            // contraction steps per LDS stage
constexpr int NT = 256;
constexpr int KC_LD = TK + 4;     // leading dim of a K-contiguous LDS tile: 144 B rows
constexpr int SMALL_GRID = 512;   // workgroups that fill the chip (2 per CU)

enum Mode { FWD = 0, GRADX = 1, GRADY = 2 };

struct MmParams {
  const float* A;
  const float* B;
  float* C;
  int nl;
  int RI;  // feature rows per block of C (and of A)
  int CI;  // feature cols per block of C (and of B)
  int KI;  // contraction features per block
};

template <int MODE> struct Cfg;
// A block (rb,kb) at rb*L+kb (MNMAJ) or kb*L+rb; same for B with (cb,kb); C (rb,cb) at rb*L+cb or cb*L+rb.
template <> struct Cfg<FWD>   { static constexpr bool A_KC = true,  B_KC = false, A_MNMAJ = true,  B_MNMAJ = true,  C_RMAJ = true;  };
template <> struct Cfg<GRADX> { static constexpr bool A_KC = true,  B_KC = true,  A_MNMAJ = true,  B_MNMAJ = false, C_RMAJ = true;  };
template <> struct Cfg<GRADY> { static constexpr bool A_KC = false, B_KC = false, A_MNMAJ = false, B_MNMAJ = false, C_RMAJ = false; };

template <bool KC, int EXT> struct TileShape {
  static constexpr int LD = KC ? KC_LD : EXT;
  static constexpr int ELEMS = KC ? EXT * KC_LD : TK * EXT;
};

template <int VEC> struct VecT { typedef float type; };
template <> struct VecT<2> { typedef float2 type; };
template <> struct VecT<4> { typedef float4 type; };

// One operand's tile loader: global -> registers -> LDS.  EXT = tile extent along the free index,
// VEC = floats per access.  The contraction index is the flattened pair (block kb, feature kin): a stage
// takes the next TK values of it whatever the block size, so small blocks (a batch of 16 in grad y) fill
// whole stages and odd block sizes pad only the very last stage.  load() fetches the current stage and
// steps to the next one.
//
// FAST: the block size KI along the contraction and the stage length TK divide one another, so every stage
// starts at the same position inside a block for every thread.  Then the per-thread offsets are fixed at
// init, the stage advances by a wave-uniform step (scalar arithmetic), rows outside the matrix are clamped
// to a valid row (their products land in accumulators that are never stored) and only a ragged LAST stage
// (TK a multiple of KI, odd number of blocks) is masked: the loop body is loads and LDS writes, nothing else.
//
// FAST = 2: KI >= TK but not a multiple of it (100 features), KI a multiple of VEC.  A stage then starts anywhere inside
// a block and may run over ONE block boundary.  Where the stage starts is still uniform (scalar offset, scalar
// bookkeeping); a thread only has to know whether ITS contraction steps lie behind the boundary, which is one compare
// with a uniform value and the (uniform) distance between the end of a block and the start of the next added to its
// offset: the same loop body as FAST = 1 plus a compare, a select and an add per slot.
template <bool KC, bool MNMAJ, int EXT, int VEC, int FAST>
struct TileLoader {
  static constexpr int NSLOT = EXT * TK / (NT * VEC);
  static constexpr int LD = TileShape<KC, EXT>::LD;
  static constexpr int KSTEP = NT * VEC / EXT;     // MN-contiguous: contraction steps between slots
  typedef typename VecT<VEC>::type vec_t;
  static_assert(NSLOT >= 1 && NSLOT <= 32, "tile does not fit the workgroup");

  const float* base;    // start of degree l
  int off[KC ? NSLOT : 1];
  unsigned valid_mn;    // bit q: slot q's row is inside the matrix (KC) / bit 0 (MN-contiguous)
  int kb, kin;          // block and feature of this thread's first contraction step in the current stage
  int lds_off;
  int blk_k_stride;
  int MNI, KI, L;
  vec_t reg[NSLOT];
  // FAST only
  unsigned foff[FAST ? NSLOT : 1];   // per-slot BYTE offset: row/column block, row inside it, position inside the stage
  __amdgpu_buffer_rsrc_t rsrc;  // the operand of this degree as a buffer: scalar base, per-slot offsets in VGPRs
  unsigned soff;                // uniform: byte offset of the current stage (scalar offset of the loads)
  int sub, nsub, step_in, step_cross;
  int stage_i, last_ragged;     // last_ragged: index of the one masked stage, or -1
  unsigned tail_ok;             // bit q: slot q lies inside the matrix in that stage
  // FAST = 2 only
  int kin_s;                    // uniform: position inside its block at which the current stage starts
  int kk0;                      // this thread's first contraction step inside a stage
  unsigned cross_bytes;         // uniform: what a step behind the block boundary adds to the offset

  typedef unsigned u32x4 __attribute__((ext_vector_type(4)));
  static __device__ __forceinline__ vec_t buffer_load(__amdgpu_buffer_rsrc_t r, unsigned voff, unsigned so) {
    if constexpr (VEC == 4) {
      const u32x4 v = __builtin_amdgcn_raw_buffer_load_b128(r, (int)voff, (int)so, 0);
      return make_float4(__uint_as_float(v.x), __uint_as_float(v.y), __uint_as_float(v.z), __uint_as_float(v.w));
    } else if constexpr (VEC == 2) {
      typedef unsigned u32x2 __attribute__((ext_vector_type(2)));
      const u32x2 v = __builtin_amdgcn_raw_buffer_load_b64(r, (int)voff, (int)so, 0);
      return make_float2(__uint_as_float(v.x), __uint_as_float(v.y));
    } else {
      return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, (int)voff, (int)so, 0));
    }
  }

  __device__ __forceinline__ void init(const float* base_l, int L_, int MNI_, int KI_, int tile0) {
    base = base_l; MNI = MNI_; KI = KI_; L = L_;
    const int t = threadIdx.x;
    const int blk_elems = MNI * KI;
    const int blk_mn_stride = (MNMAJ ? L : 1) * blk_elems;
    blk_k_stride = (MNMAJ ? 1 : L) * blk_elems;
    if (FAST) {
      const int unit = KC ? 1 : MNI;                       // stride of one contraction step inside a block
      const int K = L * KI, nstage = (K + TK - 1) / TK, ktail = K - (nstage - 1) * TK;
      rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(base_l), 0, 4 * L * L * MNI * KI, 0x00020000);
      soff = 0; sub = 0; stage_i = 0;
      if (FAST == 2) { nsub = 1; step_in = TK * unit; step_cross = 0; kin_s = 0; cross_bytes = 4u * (unsigned)(blk_k_stride - KI * unit); }
      else if (KI >= TK) { nsub = KI / TK; step_in = TK * unit; step_cross = blk_k_stride - (KI - TK) * unit; }
      else { nsub = 1; step_in = 0; step_cross = (TK / KI) * blk_k_stride; }
      last_ragged = ktail < TK ? nstage - 1 : -1;
      tail_ok = 0;
      const int last = L * MNI - 1;
      if (KC) {
        constexpr int TPR = TK / VEC;
        const int kk = (t % TPR) * VEC, r0 = t / TPR;
        const int kbl = KI >= TK ? 0 : kk / KI, kin = kk - kbl * KI;
        lds_off = r0 * LD + kk;
        kk0 = kk;
#pragma unroll
        for (int q = 0; q < NSLOT; ++q) {
          int row = tile0 + r0 + q * (NT / TPR);
          row = row > last ? last : row;
          const int mb = row / MNI, mi = row - mb * MNI;
          foff[q] = 4u * (unsigned)(mb * blk_mn_stride + mi * KI + kbl * blk_k_stride + kin);
          if (kk < ktail) tail_ok |= 1u << q;
        }
      } else {
        constexpr int TPR = EXT / VEC;
        int mn = tile0 + (t % TPR) * VEC;
        mn = mn > last ? 0 : mn;
        const int kk = t / TPR;
        lds_off = kk * LD + (t % TPR) * VEC;
        kk0 = kk;
        const int mb = mn / MNI, mi = mn - mb * MNI;
#pragma unroll
        for (int q = 0; q < NSLOT; ++q) {
          const int k = kk + q * KSTEP;
          const int kbl = KI >= TK ? 0 : k / KI, kin = k - kbl * KI;
          foff[q] = 4u * (unsigned)(mb * blk_mn_stride + mi + kbl * blk_k_stride + kin * MNI);
          if (k < ktail) tail_ok |= 1u << q;
        }
      }
      return;
    }
    valid_mn = 0;
    int kk;
    if (KC) {
      constexpr int TPR = TK / VEC;
      kk = (t % TPR) * VEC;
      const int r0 = t / TPR;
      lds_off = r0 * LD + kk;
#pragma unroll
      for (int q = 0; q < NSLOT; ++q) {
        const int row = tile0 + r0 + q * (NT / TPR);
        const int mb = row / MNI, mi = row - mb * MNI;
        off[q] = mb * blk_mn_stride + mi * KI;
        if (row < L * MNI) valid_mn |= 1u << q;
      }
    } else {
      constexpr int TPR = EXT / VEC;
      const int mn = tile0 + (t % TPR) * VEC;
      kk = t / TPR;
      lds_off = kk * LD + (t % TPR) * VEC;
      const int mb = mn / MNI, mi = mn - mb * MNI;
      off[0] = mb * blk_mn_stride + mi;
      if (mn < L * MNI) valid_mn = 1u;
    }
    kb = kk / KI;
    kin = kk - kb * KI;
  }

  // clamped address + select instead of a predicated load: all loads of a stage are in flight together
  __device__ __forceinline__ void load() {
    if (FAST == 2) {
      const int room = KI - kin_s;                     // contraction steps of this stage that still lie in the current block
      if (stage_i == last_ragged) {
#pragma unroll
        for (int q = 0; q < NSLOT; ++q) {
          const int k = KC ? kk0 : kk0 + q * KSTEP;
          const vec_t v = buffer_load(rsrc, foff[q] + (k >= room ? cross_bytes : 0u), soff);
          reg[q] = ((tail_ok >> q) & 1u) ? v : vec_t{};
        }
      } else {
#pragma unroll
        for (int q = 0; q < NSLOT; ++q) {
          const int k = KC ? kk0 : kk0 + q * KSTEP;    // KC: a thread's VEC steps never straddle a block (KI is a multiple of VEC)
          reg[q] = buffer_load(rsrc, foff[q] + (k >= room ? cross_bytes : 0u), soff);
        }
      }
      ++stage_i;
      kin_s += TK;
      soff += 4u * (unsigned)step_in;
      if (kin_s >= KI) { kin_s -= KI; soff += cross_bytes; }
      return;
    }
    if (FAST) {
      if (stage_i == last_ragged) {
#pragma unroll
        for (int q = 0; q < NSLOT; ++q) {
          const bool ok = (tail_ok >> q) & 1u;
          const vec_t v = buffer_load(rsrc, foff[q], soff);
          reg[q] = ok ? v : vec_t{};
        }
      } else {
#pragma unroll
        for (int q = 0; q < NSLOT; ++q) reg[q] = buffer_load(rsrc, foff[q], soff);
      }
      ++stage_i;
      if (++sub == nsub) { sub = 0; soff += 4u * (unsigned)step_cross; }
      else soff += 4u * (unsigned)step_in;
      return;
    }
    if (KC) {
      const bool kvalid = kb < L;
      const int koff = kb * blk_k_stride + kin;
#pragma unroll
      for (int q = 0; q < NSLOT; ++q) {
        const bool ok = kvalid && ((valid_mn >> q) & 1u);
        const vec_t v = *reinterpret_cast<const vec_t*>(base + (ok ? off[q] + koff : 0));
        reg[q] = ok ? v : vec_t{};
      }
    } else {
      int b = kb, k = kin;
#pragma unroll
      for (int q = 0; q < NSLOT; ++q) {
        const bool ok = valid_mn && b < L;
        const vec_t v = *reinterpret_cast<const vec_t*>(base + (ok ? b * blk_k_stride + off[0] + k * MNI : 0));
        reg[q] = ok ? v : vec_t{};
        k += KSTEP;
        if (KI >= KSTEP) { if (k >= KI) { k -= KI; ++b; } }
        else { const int w = k / KI; b += w; k -= w * KI; }
      }
    }
    kin += TK;
    if (KI >= TK) { if (kin >= KI) { kin -= KI; ++kb; } }
    else { const int w = kin / KI; kb += w; kin -= w * KI; }
  }

  __device__ __forceinline__ void store(float* tile) const {
    constexpr int QSTEP = KC ? NT * VEC / TK : KSTEP;   // rows (KC) or k-rows between slots
#pragma unroll
    for (int q = 0; q < NSLOT; ++q)
      *reinterpret_cast<vec_t*>(tile + lds_off + q * QSTEP * LD) = reg[q];
  }
};

// the four consecutive contraction steps k0 .. k0+3 of tile row/col `idx`
template <bool KC, int LD>
__device__ __forceinline__ float4 fetch_operand(const float* tile, int idx, int k0) {
  if (KC) {
    return *reinterpret_cast<const float4*>(tile + idx * LD + k0);
  } else {
    const float* q = tile + k0 * LD + idx;
    return make_float4(q[0], q[LD], q[2 * LD], q[3 * LD]);
  }
}

template <typename C_, int NCB, int NI, int NJ>
__device__ __forceinline__ void stage_mma(const float* As, const float* Bs, v16f (&acc)[NRB][NCB], int arow, int bcol, int h) {
  constexpr int TN = 64 * NCB;
  constexpr int ALD = TileShape<C_::A_KC, TM>::LD, BLD = TileShape<C_::B_KC, TN>::LD;
  constexpr int NS = TK / 8;
  float4 a[2][NI], b[2][NJ];
#pragma unroll
  for (int i = 0; i < NI; ++i) a[0][i] = fetch_operand<C_::A_KC, ALD>(As, arow + BSTR * i, 4 * h);
#pragma unroll
  for (int j = 0; j < NJ; ++j) b[0][j] = fetch_operand<C_::B_KC, BLD>(Bs, bcol + BSTR * j, 4 * h);
#pragma unroll
  for (int s = 0; s < NS; ++s) {
    const int cur = s & 1, nxt = cur ^ 1;
    if (s + 1 < NS) {
#pragma unroll
      for (int i = 0; i < NI; ++i) a[nxt][i] = fetch_operand<C_::A_KC, ALD>(As, arow + BSTR * i, 8 * (s + 1) + 4 * h);
#pragma unroll
      for (int j = 0; j < NJ; ++j) b[nxt][j] = fetch_operand<C_::B_KC, BLD>(Bs, bcol + BSTR * j, 8 * (s + 1) + 4 * h);
    }
    __builtin_amdgcn_sched_barrier(0);   // keep the LDS reads of the next step ahead of this step's MFMAs
#pragma unroll
    for (int t = 0; t < 4; ++t)
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          const float av = t == 0 ? a[cur][i].x : t == 1 ? a[cur][i].y : t == 2 ? a[cur][i].z : a[cur][i].w;
          const float bv = t == 0 ? b[cur][j].x : t == 1 ? b[cur][j].y : t == 2 ? b[cur][j].z : b[cur][j].w;
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av, bv, acc[i][j], 0, 0, 0);
        }
  }
}

// Double-buffered LDS: while the matrix cores consume stage s from one buffer, the operands of stage s+1
// (fetched during stage s-1) are written to the other and the global loads of stage s+2 are issued; one
// barrier per stage.
template <typename C_, int NCB, int NI, int NJ, typename LA, typename LB>
__device__ __forceinline__ void contract(LA& la, LB& lb, float* As, float* Bs, v16f (&acc)[NRB][NCB],
                                         int nstage, int arow, int bcol, int h) {
  constexpr int TN = 64 * NCB;
  constexpr int AEL = TileShape<C_::A_KC, TM>::ELEMS, BEL = TileShape<C_::B_KC, TN>::ELEMS;
  la.load();
  lb.load();
  la.store(As);
  lb.store(Bs);
  if (nstage > 1) {
    la.load();
    lb.load();
  }
  __syncthreads();
  for (int stage = 0; stage < nstage; ++stage) {
    const int cur = stage & 1;
    if (stage + 1 < nstage) {
      la.store(As + (cur ^ 1) * AEL);       // that buffer was last read in stage - 1, which every wave has left
      lb.store(Bs + (cur ^ 1) * BEL);
      if (stage + 2 < nstage) {
        la.load();
        lb.load();
      }
    }
    if (NI > 0 && NJ > 0)
      stage_mma<C_, NCB, (NI > 0 ? NI : 1), (NJ > 0 ? NJ : 1)>(As + cur * AEL, Bs + cur * BEL, acc, arow, bcol, h);
    __syncthreads();
  }
}

__host__ __device__ inline void tile_counts(int L, int RI, int CI, int TN, int& tm, int& tn, int& slots) {
  tm = s2cnn::ceil_div(L * RI, TM);
  tn = s2cnn::ceil_div(L * CI, TN);
  slots = tm * tn;
}

template <int MODE, int VA, int VB, int FAST, int NCB>
__global__ __launch_bounds__(NT) void so3_block_mm_real_kernel(MmParams p) {
  typedef Cfg<MODE> C_;
  constexpr int TN = 64 * NCB;

  __shared__ __attribute__((aligned(16))) float As[2 * TileShape<C_::A_KC, TM>::ELEMS];
  __shared__ __attribute__((aligned(16))) float Bs[2 * TileShape<C_::B_KC, TN>::ELEMS];

  int t = blockIdx.x;
  int l = p.nl - 1, tm = 0, tn = 0, slots = 0;
  for (;; --l) {
    tile_counts(2 * l + 1, p.RI, p.CI, TN, tm, tn, slots);
    if (t < slots || l == 0) break;
    t -= slots;
  }
  const int tile_nq = t / tm;
  const int L = 2 * l + 1;
  const int tile_m = (t % tm) * TM;
  const int tile_n = tile_nq * TN;
  const size_t L0 = (size_t)l * (4 * l * l - 1) / 3;
  const int M = L * p.RI, N = L * p.CI;

  TileLoader<C_::A_KC, C_::A_MNMAJ, TM, VA, FAST> la;
  TileLoader<C_::B_KC, C_::B_MNMAJ, TN, VB, FAST> lb;
  la.init(p.A + L0 * p.RI * p.KI, L, p.RI, p.KI, tile_m);
  lb.init(p.B + L0 * p.CI * p.KI, L, p.CI, p.KI, tile_n);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r32 = lane & 31, h = lane >> 5;
  const int wrow = (wave >> 1) * WSTR, wcol = (wave & 1) * WSTR;

  v16f acc[NRB][NCB];
#pragma unroll
  for (int i = 0; i < NRB; ++i)
#pragma unroll
    for (int j = 0; j < NCB; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int remr = M - tile_m - wrow, remc = N - tile_n - wcol;
  int ni = remr <= 0 ? 0 : (remr + BSTR - 1) / BSTR, nj = remc <= 0 ? 0 : (remc + BSTR - 1) / BSTR;
  ni = ni > NRB ? NRB : ni;
  nj = nj > NCB ? NCB : nj;
  if (ni == 0 || nj == 0) ni = nj = 0;

  const int nstage = s2cnn::ceil_div(L * p.KI, TK);
#define S2CNN_CONTRACT(I, J) contract<C_, NCB, I, J>(la, lb, As, Bs, acc, nstage, wrow + r32, wcol + r32, h)
  if (nj == NCB) {
    switch (ni) {
      case 4: if (NRB >= 4) { S2CNN_CONTRACT((NRB >= 4 ? 4 : 1), NCB); } break;
      case 3: if (NRB >= 3) { S2CNN_CONTRACT((NRB >= 3 ? 3 : 1), NCB); } break;
      case 2: if (NRB >= 2) { S2CNN_CONTRACT((NRB >= 2 ? 2 : 1), NCB); } break;
      case 1: S2CNN_CONTRACT(1, NCB); break;
      default: S2CNN_CONTRACT(0, 0); break;
    }
  } else if (nj == 0) {
    S2CNN_CONTRACT(0, 0);
  } else if constexpr (NCB > 1) {
    switch (ni) {
      case 4: if (NRB >= 4) { S2CNN_CONTRACT((NRB >= 4 ? 4 : 1), 1); } break;
      case 3: if (NRB >= 3) { S2CNN_CONTRACT((NRB >= 3 ? 3 : 1), 1); } break;
      case 2: if (NRB >= 2) { S2CNN_CONTRACT((NRB >= 2 ? 2 : 1), 1); } break;
      default: S2CNN_CONTRACT(1, 1); break;
    }
  }
#undef S2CNN_CONTRACT

  // Accumulator register v of lane (r32, h) holds row 8*(v/4) + 4*h + v%4 and column r32 of its 32x32 block.
  float* Cl = p.C + L0 * p.RI * p.CI;
  const int blk_elems = p.RI * p.CI;
#pragma unroll
  for (int j = 0; j < NCB; ++j) {
    const int col = tile_n + wcol + BSTR * j + r32;
    if (j >= nj || col >= N) continue;
    const int cb = col / p.CI, ci = col - cb * p.CI;
#pragma unroll
    for (int i = 0; i < NRB; ++i) {
      if (i >= ni) continue;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = tile_m + wrow + BSTR * i + 8 * (v / 4) + 4 * h + (v % 4);
        if (row < M) {
          const int rb = row / p.RI, ri = row - rb * p.RI;
          const int blk = C_::C_RMAJ ? rb * L + cb : cb * L + rb;
          Cl[(size_t)blk * blk_elems + ri * p.CI + ci] = acc[i][j][v];
        }
      }
    }
  }
}

int total_slots(int nl, int RI, int CI, int TN) {
  long n = 0;
  for (int l = 0; l < nl; ++l) {
    int tm, tn, slots;
    tile_counts(2 * l + 1, RI, CI, TN, tm, tn, slots);
    n += slots;
  }
  return n > 0x7fffffffL ? -1 : (int)n;
}

inline bool aligned4(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 3u) == 0; }

template <int MODE>
int run(const float* a, const float* b, float* c, int nl, int RI, int CI, int KI, void* stream) {
  if (!a || !b || !c || nl < 1 || RI < 1 || CI < 1 || KI < 1) return S2CNN_EINVAL;
  if (nl > 512 || (long)RI * KI > (1L << 24) || (long)CI * KI > (1L << 24) || (long)RI * CI > (1L << 24)) return S2CNN_EINVAL;
  const long Lmax = 2L * nl - 1;
  if (Lmax * Lmax * RI * KI >= (1L << 31) || Lmax * Lmax * CI * KI >= (1L << 31)) return S2CNN_EINVAL;
  if (!aligned4(a) || !aligned4(b) || !aligned4(c)) return S2CNN_EALIGN;
  // 128 x 128 tiles unless they are too few to give every CU its two workgroups: then 128 x 64
  const bool narrow = total_slots(nl, RI, CI, 128) < SMALL_GRID;
  const int grid = total_slots(nl, RI, CI, narrow ? 64 : 128);
  if (grid < 1) return S2CNN_EINVAL;
  MmParams p{a, b, c, nl, RI, CI, KI};
  typedef Cfg<MODE> C_;
  // four (two) floats per access need the fast index of the operand to be a multiple of 4 (2) and a 16-byte (8-byte) base
  const int afast = C_::A_KC ? KI : RI, bfast = C_::B_KC ? KI : CI;
  const bool a4 = afast % 4 == 0 && s2cnn::aligned16(a);
  const bool b4 = bfast % 4 == 0 && s2cnn::aligned16(b);
  const bool a2 = a4 || (afast % 2 == 0 && s2cnn::aligned8(a));
  const bool b2 = b4 || (bfast % 2 == 0 && s2cnn::aligned8(b));
  hipStream_t st = static_cast<hipStream_t>(stream);
  // the fast loaders address a degree with 32-bit byte offsets
  const bool small = Lmax * Lmax * RI * KI < (1L << 30) && Lmax * Lmax * CI * KI < (1L << 30);
  const bool divides = (KI % TK == 0 || TK % KI == 0) && small;                 // block size and K stage divide one another
  const bool crosses = !divides && KI > TK && small;                           // 100 features: stages that run over a block boundary
  const bool fast = a4 && b4 && divides;
  const bool fast2 = a4 && b4 && crosses && KI % 4 == 0;
  // the same two loaders with 8-byte accesses: even sizes that are no multiples of four (50, 70 features)
  const bool fast_v2 = !fast && a2 && b2 && divides && KI % 2 == 0;
  const bool fast2_v2 = !fast2 && a2 && b2 && crosses && KI % 2 == 0;
#define S2CNN_LAUNCH(VA, VB, FAST)                                                                                    \
  do {                                                                                                                \
    if (narrow) hipLaunchKernelGGL((so3_block_mm_real_kernel<MODE, VA, VB, FAST, 1>), dim3(grid), dim3(NT), 0, st, p); \
    else hipLaunchKernelGGL((so3_block_mm_real_kernel<MODE, VA, VB, FAST, 2>), dim3(grid), dim3(NT), 0, st, p);        \
  } while (0)
  if (fast) S2CNN_LAUNCH(4, 4, 1);
  else if (fast2) S2CNN_LAUNCH(4, 4, 2);
  else if (fast_v2) S2CNN_LAUNCH(2, 2, 1);
  else if (fast2_v2) S2CNN_LAUNCH(2, 2, 2);
  else if (a4 && b4) S2CNN_LAUNCH(4, 4, 0);
  else if (a4 && b2) S2CNN_LAUNCH(4, 2, 0);
  else if (a2 && b4) S2CNN_LAUNCH(2, 4, 0);
  else if (a2 && b2) S2CNN_LAUNCH(2, 2, 0);      // even feature counts (50, 70, 350 in the reference's shape network)
  else if (a4) S2CNN_LAUNCH(4, 1, 0);
  else if (b4) S2CNN_LAUNCH(1, 4, 0);
  else S2CNN_LAUNCH(1, 1, 0);
#undef S2CNN_LAUNCH
  return s2cnn::launch_status();
}

}  // namespace

extern "C" int s2cnn_so3_mm_real_fwd(const float* x, const float* y, float* z, int nl, int nbatch, int f_in,
                                     int f_out, void* stream) {
  s2cnn::clear_stale_error();
  return run<FWD>(x, y, z, nl, nbatch, f_out, f_in, stream);
}

extern "C" int s2cnn_so3_mm_real_gradx(const float* gz, const float* y, float* gx, int nl, int nbatch, int f_in,
                                       int f_out, void* stream) {
  s2cnn::clear_stale_error();
  return run<GRADX>(gz, y, gx, nl, nbatch, f_in, f_out, stream);
}

extern "C" int s2cnn_so3_mm_real_grady(const float* gz, const float* x, float* gy, int nl, int nbatch, int f_in,
                                       int f_out, void* stream) {
  s2cnn::clear_stale_error();
  return run<GRADY>(x, gz, gy, nl, f_in, f_out, nbatch, stream);
}
