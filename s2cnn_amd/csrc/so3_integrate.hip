// Haar integral over SO(3) on the SOFT grid and its adjoint:
//   out[z] = sum_beta w[beta] sum_{alpha,gamma} x[z,beta,alpha,gamma]
//   gx[z,beta,alpha,gamma] = g[z] w[beta]
// A pure read-reduce (write-broadcast) pass: one workgroup per volume.
#include "common.h"

namespace {

// AFFINE: the integrand is max(a x + b, 0) with a = params[z % nfeature], b = params[nfeature + z % nfeature] of volume z
template <bool AFFINE>
__global__ __launch_bounds__(256) void so3_integrate_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                                            float* __restrict__ out, int n2, const float* __restrict__ params,
                                                            int nfeature) {
  __shared__ float part[256];
  const size_t plane = (size_t)n2 * n2;
  const float* xs = x + blockIdx.x * plane * n2;
  float pa = 1.f, pb = 0.f;
  if constexpr (AFFINE) { pa = params[blockIdx.x % nfeature]; pb = params[nfeature + blockIdx.x % nfeature]; }
  auto f = [&](float v) { return AFFINE ? s2cnn::affine_relu(v, pa, pb) : v; };
  auto f4 = [&](float4 v) { return AFFINE ? make_float4(f(v.x), f(v.y), f(v.z), f(v.w)) : v; };
  float acc = 0.f;
  if (plane % 4096 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
    // 16-byte loads, four in flight per thread (4 KB per workgroup and step)
    const bool stream = (size_t)gridDim.x * plane * n2 * 4 >= s2cnn::STREAM_BYTES;     // a tensor that passes no cache
    const float4* x4 = reinterpret_cast<const float4*>(xs);
    const size_t p4 = plane / 4;
    for (int bt = 0; bt < n2; ++bt) {
      float4 s0 = make_float4(0.f, 0.f, 0.f, 0.f), s1 = s0, s2 = s0, s3 = s0;
      const float4* pl = x4 + bt * p4 + threadIdx.x;
      for (size_t i = 0; i < p4; i += 1024) {
        const float4 v0 = f4(s2cnn::load_policy(pl + i, stream)), v1 = f4(s2cnn::load_policy(pl + i + 256, stream)), v2 = f4(s2cnn::load_policy(pl + i + 512, stream)), v3 = f4(s2cnn::load_policy(pl + i + 768, stream));
        s0.x += v0.x; s0.y += v0.y; s0.z += v0.z; s0.w += v0.w;
        s1.x += v1.x; s1.y += v1.y; s1.z += v1.z; s1.w += v1.w;
        s2.x += v2.x; s2.y += v2.y; s2.z += v2.z; s2.w += v2.w;
        s3.x += v3.x; s3.y += v3.y; s3.z += v3.z; s3.w += v3.w;
      }
      acc += w[bt] * (((s0.x + s0.y) + (s0.z + s0.w)) + ((s1.x + s1.y) + (s1.z + s1.w)) + ((s2.x + s2.y) + (s2.z + s2.w)) + ((s3.x + s3.y) + (s3.z + s3.w)));
    }
  } else if ((reinterpret_cast<uintptr_t>(x) & 15u) == 0) {
    // any other grid: n2 is even, so planes and volumes are whole numbers of 16-byte words
    const float4* x4 = reinterpret_cast<const float4*>(xs);
    const int p4 = (int)(plane / 4);
    for (int bt = 0; bt < n2; ++bt) {
      float4 s0 = make_float4(0.f, 0.f, 0.f, 0.f), s1 = s0;
      const float4* pl = x4 + (size_t)bt * p4;
      for (int i = threadIdx.x; i < p4; i += 512) {
        const float4 v0 = f4(pl[i]);
        const float4 v1 = i + 256 < p4 ? f4(pl[i + 256]) : make_float4(0.f, 0.f, 0.f, 0.f);
        s0.x += v0.x; s0.y += v0.y; s0.z += v0.z; s0.w += v0.w;
        s1.x += v1.x; s1.y += v1.y; s1.z += v1.z; s1.w += v1.w;
      }
      acc += w[bt] * (((s0.x + s0.y) + (s0.z + s0.w)) + ((s1.x + s1.y) + (s1.z + s1.w)));
    }
  } else {
    for (int bt = 0; bt < n2; ++bt) {
      float s = 0.f;
      for (size_t i = threadIdx.x; i < plane; i += blockDim.x) s += f(xs[bt * plane + i]);
      acc += w[bt] * s;
    }
  }
  part[threadIdx.x] = acc;
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) part[threadIdx.x] += part[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[blockIdx.x] = part[0];
}

__global__ __launch_bounds__(256) void so3_integrate_grad_kernel(const float* __restrict__ g, const float* __restrict__ w,
                                                                 float* __restrict__ gx, int n2) {
  const size_t plane = (size_t)n2 * n2;
  float* dst = gx + blockIdx.x * plane * n2;
  const float gv = g[blockIdx.x];
  if ((reinterpret_cast<uintptr_t>(gx) & 15u) == 0) {      // n2 is even: every plane is a whole number of 16-byte words
    float4* dst4 = reinterpret_cast<float4*>(dst);
    const int p4 = (int)(plane / 4);
    const bool stream = (size_t)gridDim.x * plane * n2 * 4 >= s2cnn::STREAM_BYTES;     // a tensor that passes no cache
    for (int bt = 0; bt < n2; ++bt) {
      const float v = gv * w[bt];
      const float4 v4 = make_float4(v, v, v, v);
      for (int i = threadIdx.x; i < p4; i += blockDim.x) s2cnn::store_policy(v4, dst4 + (size_t)bt * p4 + i, stream);
    }
    return;
  }
  for (int bt = 0; bt < n2; ++bt) {
    const float v = gv * w[bt];
    for (size_t i = threadIdx.x; i < plane; i += blockDim.x) dst[bt * plane + i] = v;
  }
}

// Two sums per volume in one read, in a fixed order (bit-reproducible): what a batch normalisation over the volumes
// of a feature needs of them.
//   GRAD = false: out[z] = (sum x, sum (x - mean_z)^2), mean_z the mean of the volume.  The squares are summed around a
//                 pivot (the volume's first sample) and moved to the mean in float64, so a mean that is large against the
//                 spread costs the variance no digits (E[x^2] - mean^2 in float32 would).
//   GRAD = true : out[z] = (sum g m, sum g m y) with m = (a y + b > 0), a = params[z % F], b = params[F + z % F]
template <bool GRAD>
__global__ __launch_bounds__(256) void volume_moments_kernel(const float* __restrict__ x, const float* __restrict__ y,
                                                             const float* __restrict__ params, int nfeature,
                                                             float2* __restrict__ out, long n) {
  __shared__ double part[2][256];
  const long z = blockIdx.x;
  const float* xs = x + z * n;
  const float* ys = GRAD ? y + z * n : nullptr;
  float a = 0.f, b = 0.f;
  if constexpr (GRAD) { a = params[z % nfeature]; b = params[nfeature + z % nfeature]; }
  const float pivot = GRAD ? 0.f : xs[0];
  auto term = [&](float xv, float yv, float& s1, float& s2) {
    if constexpr (GRAD) {
      const float gm = s2cnn::relu_pass(xv, fmaf(a, yv, b));
      s1 += gm; s2 = fmaf(gm, yv, s2);
    } else {
      const float dv = xv - pivot;
      s1 += dv; s2 = fmaf(dv, dv, s2);
    }
  };
  float s1[4] = {0.f, 0.f, 0.f, 0.f}, s2[4] = {0.f, 0.f, 0.f, 0.f};
  const bool wide = n % 4 == 0 && (reinterpret_cast<uintptr_t>(x) & 15u) == 0 && (!GRAD || (reinterpret_cast<uintptr_t>(y) & 15u) == 0);
  if (wide) {
    const float4* x4 = reinterpret_cast<const float4*>(xs);
    const float4* y4 = reinterpret_cast<const float4*>(ys);
    const long n4 = n / 4;
    for (long i = threadIdx.x; i < n4; i += 256) {
      const float4 xv = x4[i];
      const float4 yv = GRAD ? y4[i] : xv;
      term(xv.x, yv.x, s1[0], s2[0]); term(xv.y, yv.y, s1[1], s2[1]);
      term(xv.z, yv.z, s1[2], s2[2]); term(xv.w, yv.w, s1[3], s2[3]);
    }
  } else {
    for (long i = threadIdx.x; i < n; i += 256) term(xs[i], GRAD ? ys[i] : 0.f, s1[0], s2[0]);
  }
  part[0][threadIdx.x] = ((double)s1[0] + (double)s1[1]) + ((double)s1[2] + (double)s1[3]);
  part[1][threadIdx.x] = ((double)s2[0] + (double)s2[1]) + ((double)s2[2] + (double)s2[3]);
  __syncthreads();
  for (int s = 128; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) {
      part[0][threadIdx.x] += part[0][threadIdx.x + s];
      part[1][threadIdx.x] += part[1][threadIdx.x + s];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    if constexpr (GRAD) out[z] = make_float2((float)part[0][0], (float)part[1][0]);
    else out[z] = make_float2((float)(part[0][0] + (double)n * (double)pivot), (float)(part[1][0] - part[0][0] * part[0][0] / (double)n));
  }
}

// The per-feature arithmetic of the normalisation on the sums of volume_moments_kernel, one workgroup per feature, float64:
//   forward : mom [batch][F][parts][2] = (sum y, sum (y - mean of the part)^2), `parts` partial sums per volume of equal counts  ->  mean, biased variance, 1/sqrt(var + eps) of the statistics in use
//             (the batch's when training, else the running ones), ab = (a, b) with a = weight / sqrt(var + eps),
//             b = bias - mean a; when training, the running averages move by `momentum` (unbiased variance).
//   backward: mom = (sum g m, sum g m y)  ->  params (a, b, p, q) of the load-time gradient, and the gradients of weight and bias.
// The two sums of feature f over its batch x parts partials, by one workgroup of 64 threads in a fixed order (float64).
__device__ __forceinline__ void feature_sums(const float2* __restrict__ mom, int batch, int nf, int parts, int f, double& s1, double& s2) {
  __shared__ double red[2][64];
  double a1 = 0.0, a2 = 0.0;
  const int total = batch * parts;
  for (int i = threadIdx.x; i < total; i += 64) {
    const int b = i / parts, p = i - b * parts;
    const float2 v = mom[((size_t)b * nf + f) * parts + p];
    a1 += v.x; a2 += v.y;
  }
  red[0][threadIdx.x] = a1; red[1][threadIdx.x] = a2;
  __syncthreads();
  for (int s = 32; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) { red[0][threadIdx.x] += red[0][threadIdx.x + s]; red[1][threadIdx.x] += red[1][threadIdx.x + s]; }
    __syncthreads();
  }
  s1 = red[0][0]; s2 = red[1][0];
}

__global__ void bn_forward_kernel(const float2* __restrict__ mom, int batch, int nf, int parts, double count, const float* __restrict__ weight,
                                  const float* __restrict__ bias, float* __restrict__ running_mean, float* __restrict__ running_var,
                                  double eps, double momentum, int training, float* __restrict__ ab, float* __restrict__ stats) {
  const int f = blockIdx.x;
  double s1, s2;
  feature_sums(mom, batch, nf, parts, f, s1, s2);          // sum of the samples, sum of the parts' squared deviations from their own means
  const double mean = s1 / count;
  // ... plus what the parts' means deviate from the mean of all: sum over the parts of n_part (mean_part - mean)^2
  const double npart = count / ((double)batch * parts);
  __shared__ double spread[64];
  double d2 = 0.0;
  for (int i = threadIdx.x; i < batch * parts; i += 64) {
    const int b = i / parts, p = i - b * parts;
    const double dm = (double)mom[((size_t)b * nf + f) * parts + p].x / npart - mean;
    d2 += dm * dm;
  }
  spread[threadIdx.x] = d2;
  __syncthreads();
  for (int s = 32; s > 0; s >>= 1) {
    if ((int)threadIdx.x < s) spread[threadIdx.x] += spread[threadIdx.x + s];
    __syncthreads();
  }
  if (threadIdx.x != 0) return;
  double var = (s2 + npart * spread[0]) / count;
  var = var < 0.0 ? 0.0 : var;
  double use_mean = mean, use_var = var;
  if (!training) { use_mean = running_mean[f]; use_var = running_var[f]; }
  const double invstd = 1.0 / sqrt(use_var + eps);
  const double a = (weight ? (double)weight[f] : 1.0) * invstd;
  ab[f] = (float)a;
  ab[nf + f] = (float)((bias ? (double)bias[f] : 0.0) - use_mean * a);
  stats[f] = (float)mean;                 // of the batch, for the caller's own bookkeeping
  stats[nf + f] = (float)var;
  stats[2 * nf + f] = (float)use_mean;    // in use
  stats[3 * nf + f] = (float)invstd;
  if (training && running_mean && running_var) {
    running_mean[f] = (float)((1.0 - momentum) * running_mean[f] + momentum * mean);
    running_var[f] = (float)((1.0 - momentum) * running_var[f] + momentum * var * (count / (count > 1.0 ? count - 1.0 : 1.0)));
  }
}

__global__ void bn_backward_kernel(const float2* __restrict__ mom, int batch, int nf, int parts, double count, const float* __restrict__ ab,
                                   const float* __restrict__ stats, int training, float* __restrict__ params, float* __restrict__ gwb) {
  const int f = blockIdx.x;
  double d1, d2;
  feature_sums(mom, batch, nf, parts, f, d1, d2);
  if (threadIdx.x != 0) return;
  const double mean = stats[2 * nf + f], invstd = stats[3 * nf + f], a = ab[f];
  const double gw = invstd * (d2 - mean * d1);          // sum g m (y - mean) / std
  double p = 0.0, q = 0.0;
  if (training) {
    const double k2 = invstd * gw / count;
    p = -a * d1 / count + a * k2 * mean;
    q = -a * k2;
  }
  params[f] = ab[f];
  params[nf + f] = ab[nf + f];
  params[2 * nf + f] = (float)p;
  params[3 * nf + f] = (float)q;
  gwb[f] = (float)gw;
  gwb[nf + f] = (float)d1;
}

}  // namespace

extern "C" int s2cnn_bn_forward_from_moments(const float* moments, int batch, int nfeature, int parts, double count, const float* weight,
                                             const float* bias, float* running_mean, float* running_var, double eps,
                                             double momentum, int training, float* ab, float* stats, void* stream) {
  s2cnn::clear_stale_error();
  if (!moments || !ab || !stats || batch < 1 || nfeature < 1 || parts < 1 || count < 1.0) return S2CNN_EINVAL;
  if (!training && (!running_mean || !running_var)) return S2CNN_EINVAL;
  if (!s2cnn::aligned8(moments)) return S2CNN_EALIGN;
  hipLaunchKernelGGL(bn_forward_kernel, dim3((unsigned)nfeature), dim3(64), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<const float2*>(moments), batch, nfeature, parts, count, weight, bias, running_mean, running_var, eps, momentum,
                     training, ab, stats);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_bn_backward_from_moments(const float* moments, int batch, int nfeature, int parts, double count, const float* ab,
                                              const float* stats, int training, float* params, float* gwb, void* stream) {
  s2cnn::clear_stale_error();
  if (!moments || !ab || !stats || !params || !gwb || batch < 1 || nfeature < 1 || parts < 1 || count < 1.0) return S2CNN_EINVAL;
  if (!s2cnn::aligned8(moments)) return S2CNN_EALIGN;
  hipLaunchKernelGGL(bn_backward_kernel, dim3((unsigned)nfeature), dim3(64), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<const float2*>(moments), batch, nfeature, parts, count, ab, stats, training, params, gwb);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_volume_moments(const float* x, float* out, long nvol, long n, void* stream) {
  s2cnn::clear_stale_error();
  if (!x || !out || nvol < 1 || nvol >= (1L << 31) || n < 1) return S2CNN_EINVAL;
  if (!s2cnn::aligned8(out)) return S2CNN_EALIGN;
  hipLaunchKernelGGL(volume_moments_kernel<false>, dim3((unsigned)nvol), dim3(256), 0, static_cast<hipStream_t>(stream), x, nullptr, nullptr, 1,
                     reinterpret_cast<float2*>(out), n);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_bn_relu_grad_moments(const float* g, const float* y, const float* params, int nfeature, float* out, long nvol, long n,
                                          void* stream) {
  s2cnn::clear_stale_error();
  if (!g || !y || !params || !out || nfeature < 1 || nvol < 1 || nvol >= (1L << 31) || nvol % nfeature != 0 || n < 1) return S2CNN_EINVAL;
  if (!s2cnn::aligned8(out)) return S2CNN_EALIGN;
  hipLaunchKernelGGL(volume_moments_kernel<true>, dim3((unsigned)nvol), dim3(256), 0, static_cast<hipStream_t>(stream), g, y, params, nfeature,
                     reinterpret_cast<float2*>(out), n);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_so3_integrate(const float* x, const float* w, float* out, int b, long n, void* stream) {
  s2cnn::clear_stale_error();
  if (!x || !w || !out || b < 1 || b > 1024 || n < 1 || n >= (1L << 31)) return S2CNN_EINVAL;
  hipLaunchKernelGGL(so3_integrate_kernel<false>, dim3((unsigned)n), dim3(256), 0, static_cast<hipStream_t>(stream), x, w, out, 2 * b, nullptr, 1);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_so3_integrate_affine_relu(const float* x, const float* params, int nfeature, const float* w, float* out, int b,
                                               long n, void* stream) {
  s2cnn::clear_stale_error();
  if (!x || !params || !w || !out || b < 1 || b > 1024 || n < 1 || n >= (1L << 31) || nfeature < 1 || n % nfeature != 0) return S2CNN_EINVAL;
  hipLaunchKernelGGL(so3_integrate_kernel<true>, dim3((unsigned)n), dim3(256), 0, static_cast<hipStream_t>(stream), x, w, out, 2 * b, params,
                     nfeature);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_so3_integrate_grad(const float* g, const float* w, float* gx, int b, long n, void* stream) {
  s2cnn::clear_stale_error();
  if (!g || !w || !gx || b < 1 || b > 1024 || n < 1 || n >= (1L << 31)) return S2CNN_EINVAL;
  hipLaunchKernelGGL(so3_integrate_grad_kernel, dim3((unsigned)n), dim3(256), 0, static_cast<hipStream_t>(stream), g, w, gx, 2 * b);
  return s2cnn::launch_status();
}

extern "C" int s2cnn_abi_version(void) { return 1; }

extern "C" const char* s2cnn_strerror(int code) {
  switch (code) {
    case S2CNN_OK: return "ok";
    case S2CNN_EINVAL: return "a size is out of range or inconsistent, or a pointer is NULL";
    case S2CNN_EWORKSPACE: return "workspace is NULL, misaligned or smaller than the *_workspace() size";
    case S2CNN_EALIGN: return "a pointer does not meet the alignment documented for this entry (4, 8 or 16 bytes)";
    case S2CNN_ETOOBIG: return "the sizes need more scratch than the library's static buffer holds (S2CNN_STATIC_SCRATCH_BYTES)";
    default: return code > 0 ? hipGetErrorString(static_cast<hipError_t>(code)) : "unknown s2cnn error";
  }
}
