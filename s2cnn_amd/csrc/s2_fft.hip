// S^2 Fourier analysis and synthesis on the SOFT grid.
//
// Analysis   out[l,m,z] = sum_beta T[beta,lm] X[z,beta,m],  X[z,beta,m] = sum_alpha x[z,beta,alpha] e^{-i m alpha}
// Synthesis  y[z,beta,alpha] = sum_m e^{+i m alpha} S[z,beta,m],  S[z,beta,m] = sum_{l>=|m|} T[beta,lm] xhat[l,m,z]
//
// T holds the column n = 0 of the Wigner small-d matrices.  Only |m| < nb = min(b_in, b_out)
// is consumed, so the alpha transform is a DFT pruned to 2nb-1 bins; the intermediate lives in a
// workspace [z][beta][mi], mi = m + nb - 1.
#include "common.h"
#include "s2_fft_real.h"

namespace {

__device__ inline float2 cmul(float2 a, float2 b) { return make_float2(a.x * b.x - a.y * b.y, a.x * b.y + a.y * b.x); }

// one workgroup per (z,beta) row
template <bool CPLX>
__global__ __launch_bounds__(256) void s2_row_dft_fwd(const float* __restrict__ x, float2* __restrict__ X, int n2, int nb) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float2* w = reinterpret_cast<float2*>(smem);
  float* row = smem + 2 * n2;
  const size_t r = blockIdx.x;
  const int nin = (CPLX ? 2 : 1) * n2;
  for (int k = threadIdx.x; k < n2; k += blockDim.x) {
    float s, c;
    sincospif(2.0f * (float)k / (float)n2, &s, &c);
    w[k] = make_float2(c, -s);
  }
  for (int i = threadIdx.x; i < nin; i += blockDim.x) row[i] = x[r * nin + i];
  __syncthreads();
  const int MW = 2 * nb - 1;
  for (int mi = threadIdx.x; mi < MW; mi += blockDim.x) {
    const int m = mi - (nb - 1);
    const int step = ((m % n2) + n2) % n2;
    int tw = 0;
    float2 acc = make_float2(0.f, 0.f);
    for (int a = 0; a < n2; ++a) {
      const float2 t = w[tw];
      if (CPLX) {
        const float2 pr = cmul(reinterpret_cast<const float2*>(row)[a], t);
        acc.x += pr.x; acc.y += pr.y;
      } else {
        acc.x += row[a] * t.x; acc.y += row[a] * t.y;
      }
      tw += step; if (tw >= n2) tw -= n2;
    }
    X[r * MW + mi] = acc;
  }
}

// thread per (z, lm): lanes along z
__global__ __launch_bounds__(256) void s2_wigner_fwd(const float2* __restrict__ X, const float* __restrict__ T,
                                                     float2* __restrict__ out, int n2, int nb, int b_out, long nbatch) {
  const long z = (long)blockIdx.x * blockDim.x + threadIdx.x;
  const int lm = blockIdx.y;
  if (z >= nbatch) return;
  int l = (int)sqrtf((float)lm);
  while (l * l > lm) --l;
  while ((l + 1) * (l + 1) <= lm) ++l;
  const int m = lm - l * l - l;
  const int MW = 2 * nb - 1;
  const int nspec = b_out * b_out;
  const float2* xp = X + (size_t)z * n2 * MW + (m + nb - 1);
  float2 acc = make_float2(0.f, 0.f);
  for (int bt = 0; bt < n2; ++bt) {
    const float t = T[(size_t)bt * nspec + lm];
    const float2 v = xp[(size_t)bt * MW];
    acc.x += t * v.x; acc.y += t * v.y;
  }
  out[(size_t)lm * nbatch + z] = acc;
}

// thread per (z, beta*MW + mi): S[z][beta][mi] = sum_l T[beta,lm] xhat[lm][z]
__global__ __launch_bounds__(256) void s2_wigner_inv(const float2* __restrict__ xh, const float* __restrict__ T,
                                                     float2* __restrict__ S, int n2, int nb, long nbatch) {
  const long z = (long)blockIdx.x * blockDim.x + threadIdx.x;
  if (z >= nbatch) return;
  const int MW = 2 * nb - 1;
  const int bt = blockIdx.y / MW, mi = blockIdx.y - bt * MW;
  const int m = mi - (nb - 1);
  const int nspec = nb * nb;
  float2 acc = make_float2(0.f, 0.f);
  for (int l = abs(m); l < nb; ++l) {
    const int lm = l * l + l + m;
    const float t = T[(size_t)bt * nspec + lm];
    const float2 v = xh[(size_t)lm * nbatch + z];
    acc.x += t * v.x; acc.y += t * v.y;
  }
  S[((size_t)z * n2 + bt) * MW + mi] = acc;
}

// one workgroup per (z,beta) row: y[alpha] = sum_mi S[mi] e^{+i m alpha}
template <bool CPLX>
__global__ __launch_bounds__(256) void s2_row_dft_inv(const float2* __restrict__ S, float* __restrict__ y, int n2, int nb) {
  extern __shared__ __attribute__((aligned(16))) float smem[];
  float2* w = reinterpret_cast<float2*>(smem);
  float2* row = w + n2;
  const size_t r = blockIdx.x;
  const int MW = 2 * nb - 1;
  for (int k = threadIdx.x; k < n2; k += blockDim.x) {
    float s, c;
    sincospif(2.0f * (float)k / (float)n2, &s, &c);
    w[k] = make_float2(c, s);  // e^{+2 pi i k / n2}
  }
  for (int i = threadIdx.x; i < MW; i += blockDim.x) row[i] = S[r * MW + i];
  __syncthreads();
  for (int a = threadIdx.x; a < n2; a += blockDim.x) {
    int tw = (int)(((long)(-(nb - 1)) * a) % n2); if (tw < 0) tw += n2;
    float2 acc = make_float2(0.f, 0.f);
    for (int mi = 0; mi < MW; ++mi) {
      const float2 pr = cmul(row[mi], w[tw]);
      acc.x += pr.x; acc.y += pr.y;
      tw += a; if (tw >= n2) tw -= n2;
    }
    if (CPLX) reinterpret_cast<float2*>(y)[r * n2 + a] = acc;
    else y[r * n2 + a] = acc.x;
  }
}

size_t ws_bytes(int b_grid, int b_spec, long nbatch) {
  if (b_grid < 1 || b_spec < 1 || nbatch < 1) return 0;
  const long nb = b_grid < b_spec ? b_grid : b_spec;
  return (size_t)nbatch * (2 * b_grid) * (2 * nb - 1) * sizeof(float2);
}

bool sizes_ok(int b_grid, int b_spec, long nbatch) {
  return b_grid >= 1 && b_spec >= 1 && b_spec <= b_grid && b_grid <= 2048 && nbatch >= 1 &&
         nbatch * 2L * b_grid < (1L << 31) && 2L * b_grid * (2L * b_spec - 1) <= 65535 && (long)b_spec * b_spec <= 65535;
}

}  // namespace

// The analysis of few real signals is split along beta and writes one partial spectrum per split into the workspace:
// the size covers them (complex_in = 0), so that a split is never dropped for want of room.
extern "C" size_t s2cnn_s2_analysis_workspace(int b_in, int b_out, long nbatch, int complex_in) {
  size_t need = ws_bytes(b_in, b_out, nbatch);
  if (need && !complex_in && b_out <= b_in) {
    const s2_real::Plan plan = s2_real::plan_fwd(2 * b_in, b_out);
    if (plan.rb > 0) {
      const size_t split = (size_t)s2_real::splits_for(2 * b_in, plan.rb, nbatch) * b_out * b_out * nbatch * sizeof(float2);
      if (split > need) need = split;
    }
  }
  return need;
}
extern "C" size_t s2cnn_s2_synthesis_workspace(int b_in, int b_out, long nbatch, int) { return ws_bytes(b_out, b_in, nbatch); }

extern "C" int s2cnn_s2_analysis(const float* x, const float* table, float* out, void* workspace, size_t workspace_bytes,
                                 int b_in, int b_out, long nbatch, int complex_in, void* stream) {
  s2cnn::clear_stale_error();
  if (!x || !table || !out || !sizes_ok(b_in, b_out, nbatch)) return S2CNN_EINVAL;
  if (!s2cnn::aligned8(out) || (complex_in && !s2cnn::aligned8(x))) return S2CNN_EALIGN;
  if (!workspace || workspace_bytes < ws_bytes(b_in, b_out, nbatch) || !s2cnn::aligned8(workspace)) return S2CNN_EWORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int n2 = 2 * b_in, nb = b_out;
  if (!complex_in) {   // real signals, b_out <= 32: one kernel, one workgroup per signal
    const s2_real::Plan plan = s2_real::plan_fwd(n2, nb);
    if (plan.rb > 0) {
      if (plan.lds > 48 * 1024) (void)hipFuncSetAttribute((const void*)s2_real::analysis_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)plan.lds);
      // few signals: split along beta, partial spectra in the workspace, added up in a fixed order
      int nsplit = s2_real::splits_for(n2, plan.rb, nbatch);
      const size_t nout = (size_t)nb * nb * nbatch;
      if (nsplit > 1 && nsplit * nout * sizeof(float2) > workspace_bytes)      // a workspace sized for the two-kernel path only:
        nsplit = (int)(workspace_bytes / (nout * sizeof(float2)));              // as many splits as it holds
      if (nsplit < 2) nsplit = 1;
      float2* dst = nsplit > 1 ? static_cast<float2*>(workspace) : reinterpret_cast<float2*>(out);
      hipLaunchKernelGGL(s2_real::analysis_kernel, dim3((unsigned)nbatch, nsplit), dim3(s2_real::NT), plan.lds, st, x, table,
                         dst, n2, nb, nbatch, plan.rb);
      if (nsplit > 1)
        hipLaunchKernelGGL(s2_real::reduce_splits, dim3((unsigned)((nout + 255) / 256 < 1024 ? (nout + 255) / 256 : 1024)), dim3(256), 0, st,
                           dst, reinterpret_cast<float2*>(out), (long)nout, nsplit);
      return s2cnn::launch_status();
    }
  }
  float2* X = static_cast<float2*>(workspace);
  const size_t lds = sizeof(float) * (2 * n2 + (complex_in ? 2 : 1) * n2);
  const unsigned rows = (unsigned)(nbatch * n2);
  if (complex_in) hipLaunchKernelGGL(s2_row_dft_fwd<true>, dim3(rows), dim3(64), lds, st, x, X, n2, nb);
  else hipLaunchKernelGGL(s2_row_dft_fwd<false>, dim3(rows), dim3(64), lds, st, x, X, n2, nb);
  int rc = s2cnn::launch_status();
  if (rc) return rc;
  dim3 grid((unsigned)((nbatch + 63) / 64), b_out * b_out);
  hipLaunchKernelGGL(s2_wigner_fwd, grid, dim3(64), 0, st, X, table, reinterpret_cast<float2*>(out), n2, nb, b_out, nbatch);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_s2_synthesis(const float* xhat, const float* table, float* out, void* workspace, size_t workspace_bytes,
                                  int b_in, int b_out, long nbatch, int complex_out, void* stream) {
  s2cnn::clear_stale_error();
  if (!xhat || !table || !out || !sizes_ok(b_out, b_in, nbatch)) return S2CNN_EINVAL;
  if (!s2cnn::aligned8(xhat) || (complex_out && !s2cnn::aligned8(out))) return S2CNN_EALIGN;
  if (!workspace || workspace_bytes < ws_bytes(b_out, b_in, nbatch) || !s2cnn::aligned8(workspace)) return S2CNN_EWORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int n2 = 2 * b_out, nb = b_in;
  if (!complex_out) {
    const s2_real::Plan plan = s2_real::plan_inv(n2, nb);
    if (plan.rb > 0) {
      if (plan.lds > 48 * 1024) (void)hipFuncSetAttribute((const void*)s2_real::synthesis_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)plan.lds);
      hipLaunchKernelGGL(s2_real::synthesis_kernel, dim3((unsigned)nbatch, s2_real::splits_for(n2, 64, nbatch)), dim3(s2_real::NT), plan.lds, st,
                         reinterpret_cast<const float2*>(xhat), table, out, n2, nb, nbatch);
      return s2cnn::launch_status();
    }
  }
  const int MW = 2 * nb - 1;
  float2* S = static_cast<float2*>(workspace);
  dim3 grid((unsigned)((nbatch + 63) / 64), n2 * MW);
  hipLaunchKernelGGL(s2_wigner_inv, grid, dim3(64), 0, st, reinterpret_cast<const float2*>(xhat), table, S, n2, nb, nbatch);
  int rc = s2cnn::launch_status();
  if (rc) return rc;
  const size_t lds = sizeof(float2) * (n2 + MW);
  const unsigned rows = (unsigned)(nbatch * n2);
  if (complex_out) hipLaunchKernelGGL(s2_row_dft_inv<true>, dim3(rows), dim3(64), lds, st, S, out, n2, nb);
  else hipLaunchKernelGGL(s2_row_dft_inv<false>, dim3(rows), dim3(64), lds, st, S, out, n2, nb);
  return s2cnn::launch_status();
}
