// Measurement library (libs2cnn_probe.so), built on request only (`python -m s2cnn_amd.csrc.build --probes`) and never
// loaded by the package: the per-volume kernels of the 64^3 grid instantiated with parts of them compiled out
// (template argument PROBE of fused64::analysis_kernel / synthesis_kernel), so that `bench.py --floor` can time what the
// rest of the kernel costs.  With probe != 0 the results are meaningless.
#include "common.h"
#include "so3_fused64.h"
#include "s2cnn_hip_probe.h"

extern "C" int s2cnn_so3_fft64_probe(const float* x, float* y, const float* packed_table, void* workspace, size_t workspace_bytes,
                                     long nbatch, int direction, int probe, void* stream) {
  using namespace fused64;
  s2cnn::clear_stale_error();
  if (!packed_table || nbatch < 1 || direction < 0 || direction > 1 || probe < 0 || probe > 2) return S2CNN_EINVAL;
  if ((direction == 0 && !x) || (direction == 1 && !y)) return S2CNN_EINVAL;
  if (!s2cnn::aligned16(x) || !s2cnn::aligned16(y) || !s2cnn::aligned16(packed_table)) return S2CNN_EALIGN;
  if (!workspace || workspace_bytes < scratch_bytes(nbatch) || (reinterpret_cast<uintptr_t>(workspace) & 255u)) return S2CNN_EWORKSPACE;
  hipStream_t st = static_cast<hipStream_t>(stream);
  float4* rec = static_cast<float4*>(workspace);
  const dim3 grid(grid_size(nbatch)), block(THREADS);
  if (direction == 0) {
    if (probe == 1) hipLaunchKernelGGL((analysis_kernel<7, 0, 1>), grid, block, 0, st, x, nullptr, packed_table, rec, nbatch, nullptr, 1, 1);
    else if (probe == 2) hipLaunchKernelGGL((analysis_kernel<7, 0, 2>), grid, block, 0, st, x, nullptr, packed_table, rec, nbatch, nullptr, 1, 1);
    else hipLaunchKernelGGL((analysis_kernel<7, 0, 0>), grid, block, 0, st, x, nullptr, packed_table, rec, nbatch, nullptr, 1, 1);
  } else {
    if (probe == 2) hipLaunchKernelGGL((synthesis_kernel<7, 2>), grid, block, 0, st, rec, packed_table, y, nbatch, nullptr, 1, 0, nullptr, nullptr, nullptr, nullptr, 1);
    else if (probe == 1) hipLaunchKernelGGL((synthesis_kernel<7, 1>), grid, block, 0, st, rec, packed_table, y, nbatch, nullptr, 1, 0, nullptr, nullptr, nullptr, nullptr, 1);
    else hipLaunchKernelGGL((synthesis_kernel<7, 0>), grid, block, 0, st, rec, packed_table, y, nbatch, nullptr, 1, 0, nullptr, nullptr, nullptr, nullptr, 1);
  }
  return s2cnn::launch_status();
}
