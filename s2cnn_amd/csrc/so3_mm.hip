// Block-diagonal complex products over the (2l+1)x(2l+1) blocks of an SO(3) spectrum,
// on the fp32 matrix cores of gfx950 (v_mfma_f32_32x32x2_f32).
//
// For one degree l (L = 2l+1) each of the three products is a complex GEMM whose three
// index spaces are pairs (spectral index, feature index):
//
//   fwd   : Z[(m,i),(n,j)] = sum_{(p,k)} X [(m,i),(p,k)] * conj(Y[(p,k),(n,j)])
//   gradx : GX[(m,i),(p,k)] = sum_{(n,j)} GZ[(m,i),(n,j)] *      Y[(n,j),(p,k)]
//   grady : GY[(p,k),(n,j)] = sum_{(m,i)} X [(p,k),(m,i)] * conj(GZ[(m,i),(n,j)])
//
// with tensors stored as [l, spectral row, spectral col, feature row, feature col, 2].
// An operand is therefore an L x L grid of dense feature blocks; within a block either the
// contraction index ("K-contiguous") or the free index ("MN-contiguous") is the fast one.
// The kernel keeps each operand tile in LDS in the orientation it has in memory, so loads
// from HBM are coalesced and nothing is transposed on the way.
//
// Complex arithmetic on a real matrix core, three real products per complex one (Gauss): with
// b = br + i bi' (bi' = -bi where the operand is conjugated)
//     P1 = sum ar br,   P2 = sum ai bi',   P3 = sum (ar + ai)(br + bi')
//     re = P1 - P2,     im = P3 - P1 - P2.
// One MFMA 32x32x2 takes two contraction steps, one per half-wave; a lane holds two consecutive complex
// steps of its row / column (four floats), forms the two sums in registers and feeds six MFMAs: 1.5 per
// complex multiply-add instead of the 2 of the direct form, at the price of a third accumulator per block.
// The sums are formed in fp32 before the product, so the imaginary part carries a rounding error of the
// size of |a||b| eps rather than of its own size: the same bound as any fp32 complex product.
//
// Tiling.  A workgroup (4 waves) owns 128 rows x 64 columns = 4 x 2 blocks of 32.  Wave (wm, wn)
// takes row blocks wm, wm+2 and column block wn, so a ragged tile (fewer live blocks) still
// splits evenly over the waves; blocks that lie wholly outside the matrix are skipped per wave.
// The grid lists exactly the tiles of all degrees, heaviest degree first (no idle workgroups:
// a workgroup that exits at once still waits for a full slot and stalls the in-order dispatch).
#include <type_traits>
#include "common.h"

namespace {

typedef float v16f __attribute__((ext_vector_type(16)));

constexpr int NRB = 2;            // 32-row blocks per wave
constexpr int NCB = 1;            // 32-column blocks per wave (three accumulators per block: 96 registers per wave)
constexpr int TM = 64 * NRB;      // tile rows   (flattened (spectral, feature) index): 2 waves x NRB blocks
constexpr int TN = 64 * NCB;      // tile cols
constexpr int BSTR = 64, WSTR = 32;   // a wave's blocks are 64 apart, the two waves of a dimension offset by 32
constexpr int TK = 16;            // complex contraction steps per LDS stage
constexpr int NT = 256;           // threads: 4 waves
constexpr int KC_LD = TK + 2;     // leading dim (complex) of a K-contiguous LDS tile: 144 B rows

enum Mode { FWD = 0, GRADX = 1, GRADY = 2 };

struct MmParams {
  const float2* A;
  const float2* B;
  float2* C;
  int nl;
  int RI;  // feature rows per block of C (and of A)
  int CI;  // feature cols per block of C (and of B)
  int KI;  // contraction features per block
};

template <int MODE> struct Cfg;
// A block (rb,kb) at rb*L+kb (MNMAJOR) or kb*L+rb; same for B with (cb,kb); C (rb,cb) at rb*L+cb or cb*L+rb.
template <> struct Cfg<FWD>   { static constexpr bool A_KC = true,  B_KC = false, A_MNMAJ = true,  B_MNMAJ = true,  C_RMAJ = true,  CONJ = true;  };
template <> struct Cfg<GRADX> { static constexpr bool A_KC = true,  B_KC = true,  A_MNMAJ = true,  B_MNMAJ = false, C_RMAJ = true,  CONJ = false; };
template <> struct Cfg<GRADY> { static constexpr bool A_KC = false, B_KC = false, A_MNMAJ = false, B_MNMAJ = false, C_RMAJ = false, CONJ = true;  };

template <bool KC, int EXT> struct TileShape {
  static constexpr int LD = KC ? KC_LD : EXT;             // LDS leading dimension (complex)
  static constexpr int ELEMS = KC ? EXT * KC_LD : TK * EXT;
};

// One operand's tile loader: global -> registers -> LDS.  EXT = tile extent along the free index,
// VEC = complex numbers per access.
template <bool KC, bool MNMAJ, int EXT, int VEC>
struct TileLoader {
  static constexpr int NSLOT = EXT * TK / (NT * VEC);
  static constexpr int LD = TileShape<KC, EXT>::LD;
  typedef typename std::conditional<VEC == 2, float4, float2>::type vec_t;
  static_assert(NSLOT >= 1, "tile too small for the workgroup");

  const float2* base;   // start of degree l
  int off[KC ? NSLOT : 1];
  unsigned valid_mn;    // bit q: slot q's row is inside the matrix (KC) / bit 0 (MN-contiguous)
  int kk;               // KC: this thread's k inside the stage; else k of slot 0
  int lds_off;          // LDS offset (complex) of slot 0
  int blk_k_stride;     // elements between consecutive contraction blocks
  int MNI, KI;
  vec_t reg[NSLOT];

  __device__ void init(const float2* base_l, int L, int MNI_, int KI_, int tile0) {
    base = base_l; MNI = MNI_; KI = KI_;
    const int t = threadIdx.x;
    const int blk_elems = MNI * KI;
    const int blk_mn_stride = (MNMAJ ? L : 1) * blk_elems;
    blk_k_stride = (MNMAJ ? 1 : L) * blk_elems;
    valid_mn = 0;
    if (KC) {
      constexpr int TPR = TK / VEC;          // threads per tile row
      kk = (t % TPR) * VEC;
      const int r0 = t / TPR;
      lds_off = r0 * LD + kk;
#pragma unroll
      for (int q = 0; q < NSLOT; ++q) {
        const int row = tile0 + r0 + q * (NT / TPR);
        const int mb = row / MNI, mi = row - mb * MNI;
        off[q] = mb * blk_mn_stride + mi * KI + kk;
        if (row < L * MNI) valid_mn |= 1u << q;
      }
    } else {
      constexpr int TPR = EXT / VEC;         // threads per k-row of the tile
      const int mn = tile0 + (t % TPR) * VEC;
      kk = t / TPR;
      lds_off = kk * LD + (t % TPR) * VEC;
      const int mb = mn / MNI, mi = mn - mb * MNI;
      off[0] = mb * blk_mn_stride + mi;
      if (mn < L * MNI) valid_mn = 1u;
    }
  }

  // clamped address + select instead of a predicated load: all loads of a stage are in flight together
  __device__ void load(int kb, int k0) {
    const float2* p = base + (size_t)kb * blk_k_stride;
    if (KC) {
      const bool kvalid = (k0 + kk) < KI;
#pragma unroll
      for (int q = 0; q < NSLOT; ++q) {
        const bool ok = kvalid && ((valid_mn >> q) & 1u);
        const vec_t v = *reinterpret_cast<const vec_t*>(p + (ok ? off[q] + k0 : 0));
        reg[q] = ok ? v : vec_t{};
      }
    } else {
      constexpr int KSTEP = NT * VEC / EXT;
#pragma unroll
      for (int q = 0; q < NSLOT; ++q) {
        const int k = k0 + kk + q * KSTEP;
        const bool ok = valid_mn && k < KI;
        const vec_t v = *reinterpret_cast<const vec_t*>(p + (ok ? off[0] + k * MNI : 0));
        reg[q] = ok ? v : vec_t{};
      }
    }
  }

  __device__ void store(float2* tile) const {
    if (KC) {
      constexpr int RSTEP = NT * VEC / TK;
#pragma unroll
      for (int q = 0; q < NSLOT; ++q)
        *reinterpret_cast<vec_t*>(tile + lds_off + q * RSTEP * LD) = reg[q];
    } else {
      constexpr int KSTEP = NT * VEC / EXT;
#pragma unroll
      for (int q = 0; q < NSLOT; ++q)
        *reinterpret_cast<vec_t*>(tile + lds_off + q * KSTEP * LD) = reg[q];
    }
  }
};

// The four reals (re k0, im k0, re k0+1, im k0+1) of tile row/col `idx` and the lane's pair of
// contraction steps k0 = 4s + 2h.
template <bool KC, int LD>
__device__ __forceinline__ float4 fetch_operand(const float2* tile, int idx, int k0) {
  if (KC) {
    return *reinterpret_cast<const float4*>(tile + idx * LD + k0);
  } else {
    const float2 a = tile[k0 * LD + idx];
    const float2 b = tile[(k0 + 1) * LD + idx];
    return make_float4(a.x, a.y, b.x, b.y);
  }
}

// the three accumulators of a 32x32 block of complex outputs
struct Acc3 { v16f p1, p2, p3; };

// All matrix-core work of one LDS stage for a wave with NI live row blocks (rows arow + 64 i) and NJ
// live column blocks (columns bcol + 64 j).  Operand registers are double buffered: the LDS reads of
// step s+1 are issued before the MFMAs of step s.
template <typename C_, int NI, int NJ>
__device__ __forceinline__ void stage_mma(const float2* As, const float2* Bs, Acc3 (&acc)[NRB][NCB], int arow, int bcol, int h) {
  constexpr int ALD = TileShape<C_::A_KC, TM>::LD, BLD = TileShape<C_::B_KC, TN>::LD;
  float4 a[2][NI], b[2][NJ];
#pragma unroll
  for (int i = 0; i < NI; ++i) a[0][i] = fetch_operand<C_::A_KC, ALD>(As, arow + BSTR * i, 2 * h);
#pragma unroll
  for (int j = 0; j < NJ; ++j) b[0][j] = fetch_operand<C_::B_KC, BLD>(Bs, bcol + BSTR * j, 2 * h);
#pragma unroll
  for (int s = 0; s < TK / 4; ++s) {
    const int cur = s & 1, nxt = cur ^ 1;
    if (s + 1 < TK / 4) {
#pragma unroll
      for (int i = 0; i < NI; ++i) a[nxt][i] = fetch_operand<C_::A_KC, ALD>(As, arow + BSTR * i, 4 * (s + 1) + 2 * h);
#pragma unroll
      for (int j = 0; j < NJ; ++j) b[nxt][j] = fetch_operand<C_::B_KC, BLD>(Bs, bcol + BSTR * j, 4 * (s + 1) + 2 * h);
    }
    __builtin_amdgcn_sched_barrier(0);   // keep the LDS reads of the next step ahead of this step's MFMAs
    float2 asum[NI], bim[NJ], bsum[NJ];  // per contraction step of the lane's pair: ar + ai | bi' | br + bi'
#pragma unroll
    for (int i = 0; i < NI; ++i) asum[i] = make_float2(a[cur][i].x + a[cur][i].y, a[cur][i].z + a[cur][i].w);
#pragma unroll
    for (int j = 0; j < NJ; ++j) {
      const float4 v = b[cur][j];
      bim[j] = C_::CONJ ? make_float2(-v.y, -v.w) : make_float2(v.y, v.w);
      bsum[j] = make_float2(v.x + bim[j].x, v.z + bim[j].y);
    }
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < NI; ++i)
#pragma unroll
        for (int j = 0; j < NJ; ++j) {
          const float ar = t == 0 ? a[cur][i].x : a[cur][i].z, ai = t == 0 ? a[cur][i].y : a[cur][i].w;
          const float br = t == 0 ? b[cur][j].x : b[cur][j].z;
          acc[i][j].p1 = __builtin_amdgcn_mfma_f32_32x32x2f32(ar, br, acc[i][j].p1, 0, 0, 0);
          acc[i][j].p2 = __builtin_amdgcn_mfma_f32_32x32x2f32(ai, t == 0 ? bim[j].x : bim[j].y, acc[i][j].p2, 0, 0, 0);
          acc[i][j].p3 = __builtin_amdgcn_mfma_f32_32x32x2f32(t == 0 ? asum[i].x : asum[i].y, t == 0 ? bsum[j].x : bsum[j].y,
                                                              acc[i][j].p3, 0, 0, 0);
        }
  }
}

// The contraction loop of one tile.  LDS is double buffered: while the matrix cores consume stage s from one
// buffer, the operands of stage s+1 (fetched during stage s-1) are written to the other and the global loads
// of stage s+2 are issued; one barrier per stage.
template <typename C_, int NI, int NJ, typename LA, typename LB>
__device__ __forceinline__ void contract(LA& la, LB& lb, float2* As, float2* Bs, Acc3 (&acc)[NRB][NCB],
                                         int nstage, int nkc, int arow, int bcol, int h) {
  constexpr int AEL = TileShape<C_::A_KC, TM>::ELEMS, BEL = TileShape<C_::B_KC, TN>::ELEMS;
  int kb = 0, kc = 0;
  auto advance = [&]() { if (++kc == nkc) { kc = 0; ++kb; } };
  la.load(0, 0);
  lb.load(0, 0);
  la.store(As);
  lb.store(Bs);
  advance();
  if (nstage > 1) {
    la.load(kb, kc * TK);
    lb.load(kb, kc * TK);
  }
  __syncthreads();
  for (int stage = 0; stage < nstage; ++stage) {
    const int cur = stage & 1;
    if (stage + 1 < nstage) {
      la.store(As + (cur ^ 1) * AEL);       // that buffer was last read in stage - 1, which every wave has left
      lb.store(Bs + (cur ^ 1) * BEL);
      advance();
      if (stage + 2 < nstage) {
        la.load(kb, kc * TK);
        lb.load(kb, kc * TK);
      }
    }
    if (NI > 0 && NJ > 0)
      stage_mma<C_, (NI > 0 ? NI : 1), (NJ > 0 ? NJ : 1)>(As + cur * AEL, Bs + cur * BEL, acc, arow, bcol, h);
    __syncthreads();
  }
}

__host__ __device__ inline void tile_counts(int L, int RI, int CI, int& tm, int& tn, int& slots) {
  tm = s2cnn::ceil_div(L * RI, TM);
  tn = s2cnn::ceil_div(L * CI, TN);
  slots = tm * tn;   // every workgroup of the grid has a tile: idle workgroups stall the dispatcher
}

template <int MODE, int VEC>
__global__ __launch_bounds__(NT, MODE == GRADX ? 2 : 3) void so3_block_mm_kernel(MmParams p) {   // grad x: two K-contiguous tiles leave LDS for two workgroups
  typedef Cfg<MODE> C_;
  __shared__ __attribute__((aligned(16))) float2 As[2 * TileShape<C_::A_KC, TM>::ELEMS];
  __shared__ __attribute__((aligned(16))) float2 Bs[2 * TileShape<C_::B_KC, TN>::ELEMS];

  // ---- which tile: degrees in descending order so the heaviest tiles are dispatched first
  int t = blockIdx.x;
  int l = p.nl - 1, tm = 0, tn = 0, slots = 0;
  for (;; --l) {
    tile_counts(2 * l + 1, p.RI, p.CI, tm, tn, slots);
    if (t < slots || l == 0) break;
    t -= slots;
  }
  const int r = t;                                  // row tiles run fastest within a degree
  const int tile_nq = r / tm;
  const int L = 2 * l + 1;
  const int tile_m = (r % tm) * TM;
  const int tile_n = tile_nq * TN;
  const size_t L0 = (size_t)l * (4 * l * l - 1) / 3;
  const int M = L * p.RI, N = L * p.CI;

  TileLoader<C_::A_KC, C_::A_MNMAJ, TM, VEC> la;
  TileLoader<C_::B_KC, C_::B_MNMAJ, TN, VEC> lb;
  la.init(p.A + L0 * p.RI * p.KI, L, p.RI, p.KI, tile_m);
  lb.init(p.B + L0 * p.CI * p.KI, L, p.CI, p.KI, tile_n);

  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r32 = lane & 31, h = lane >> 5;
  const int wrow = (wave >> 1) * WSTR, wcol = (wave & 1) * WSTR;

  Acc3 acc[NRB][NCB];
#pragma unroll
  for (int i = 0; i < NRB; ++i)
#pragma unroll
    for (int j = 0; j < NCB; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) { acc[i][j].p1[v] = 0.f; acc[i][j].p2[v] = 0.f; acc[i][j].p3[v] = 0.f; }

  // live blocks of this wave: rows tile_m + wrow + 64 i < M, columns tile_n + wcol + 64 j < N (prefixes of i, j)
  const int remr = M - tile_m - wrow, remc = N - tile_n - wcol;
  int ni = remr <= 0 ? 0 : (remr + BSTR - 1) / BSTR, nj = remc <= 0 ? 0 : (remc + BSTR - 1) / BSTR;
  ni = ni > NRB ? NRB : ni;
  nj = nj > NCB ? NCB : nj;
  if (ni == 0 || nj == 0) ni = nj = 0;

  const int nkc = s2cnn::ceil_div(p.KI, TK);
  const int nstage = L * nkc;
  // one specialised copy of the whole contraction loop per count of live blocks (wave-uniform choice)
#define S2CNN_CONTRACT(I, J) contract<C_, I, J>(la, lb, As, Bs, acc, nstage, nkc, wrow + r32, wcol + r32, h)
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
  } else if constexpr (NCB > 1) {  // one live column block of two
    switch (ni) {
      case 4: if (NRB >= 4) { S2CNN_CONTRACT((NRB >= 4 ? 4 : 1), 1); } break;
      case 3: if (NRB >= 3) { S2CNN_CONTRACT((NRB >= 3 ? 3 : 1), 1); } break;
      case 2: if (NRB >= 2) { S2CNN_CONTRACT((NRB >= 2 ? 2 : 1), 1); } break;
      default: S2CNN_CONTRACT(1, 1); break;
    }
  }
#undef S2CNN_CONTRACT

  // ---- write the sub-tile.  Accumulator register v of lane (r32, h) holds row 8*(v/4) + 4*h + v%4
  // and column r32 of its 32x32 block.
  float2* Cl = p.C + L0 * p.RI * p.CI;
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
          const float p1 = acc[i][j].p1[v], p2 = acc[i][j].p2[v];
          Cl[(size_t)blk * blk_elems + ri * p.CI + ci] = make_float2(p1 - p2, acc[i][j].p3[v] - p1 - p2);
        }
      }
    }
  }
}

int total_slots(int nl, int RI, int CI) {
  long n = 0;
  for (int l = 0; l < nl; ++l) {
    int tm, tn, slots;
    tile_counts(2 * l + 1, RI, CI, tm, tn, slots);
    n += slots;
  }
  return n > 0x7fffffffL ? -1 : (int)n;
}

template <int MODE>
int run(const float* a, const float* b, float* c, int nl, int RI, int CI, int KI, void* stream) {
  if (!a || !b || !c || nl < 1 || RI < 1 || CI < 1 || KI < 1) return S2CNN_EINVAL;
  if (nl > 512 || (long)RI * KI > (1L << 24) || (long)CI * KI > (1L << 24) || (long)RI * CI > (1L << 24)) return S2CNN_EINVAL;
  // per-degree operand slabs are indexed with 32-bit offsets
  const long Lmax = 2L * nl - 1;
  if (Lmax * Lmax * RI * KI >= (1L << 31) || Lmax * Lmax * CI * KI >= (1L << 31)) return S2CNN_EINVAL;
  if (!s2cnn::aligned8(a) || !s2cnn::aligned8(b) || !s2cnn::aligned8(c)) return S2CNN_EALIGN;
  const int grid = total_slots(nl, RI, CI);
  if (grid < 1) return S2CNN_EINVAL;
  MmParams p{reinterpret_cast<const float2*>(a), reinterpret_cast<const float2*>(b),
             reinterpret_cast<float2*>(c), nl, RI, CI, KI};
  typedef Cfg<MODE> C_;
  // two complex numbers per access need the fast index of each operand to be even and 16-byte bases
  const bool a_even = C_::A_KC ? (KI % 2 == 0) : (RI % 2 == 0);
  const bool b_even = C_::B_KC ? (KI % 2 == 0) : (CI % 2 == 0);
  const bool vec2 = a_even && b_even && s2cnn::aligned16(a) && s2cnn::aligned16(b);
  hipStream_t st = static_cast<hipStream_t>(stream);
  if (vec2)
    hipLaunchKernelGGL((so3_block_mm_kernel<MODE, 2>), dim3(grid), dim3(NT), 0, st, p);
  else
    hipLaunchKernelGGL((so3_block_mm_kernel<MODE, 1>), dim3(grid), dim3(NT), 0, st, p);
  return s2cnn::launch_status();
}

}  // namespace

extern "C" int s2cnn_so3_mm_fwd(const float* x, const float* y, float* z, int nl, int nbatch, int f_in,
                                int f_out, void* stream) {
  s2cnn::clear_stale_error();
  return run<FWD>(x, y, z, nl, nbatch, f_out, f_in, stream);
}

extern "C" int s2cnn_so3_mm_gradx(const float* gz, const float* y, float* gx, int nl, int nbatch, int f_in,
                                  int f_out, void* stream) {
  s2cnn::clear_stale_error();
  return run<GRADX>(gz, y, gx, nl, nbatch, f_in, f_out, stream);
}

extern "C" int s2cnn_so3_mm_grady(const float* gz, const float* x, float* gy, int nl, int nbatch, int f_in,
                                  int f_out, void* stream) {
  s2cnn::clear_stale_error();
  return run<GRADY>(x, gz, gy, nl, f_in, f_out, nbatch, stream);
}
