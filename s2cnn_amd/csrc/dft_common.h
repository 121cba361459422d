// Helpers shared by the folded plane / row transforms (so3_plane_dft_real.h, s2_fft_real.h).
#pragma once
#include <hip/hip_runtime.h>

namespace dft_common {

__host__ __device__ inline int pad(int v, int q) { return (v + q - 1) / q * q; }

// (cos, sin)(2 pi j k / n2)
__device__ __forceinline__ float2 cs_entry(int j, int k, int n2) {
  float s, c;
  sincospif(2.0f * (float)((j * k) % n2) / (float)n2, &s, &c);
  return make_float2(c, s);
}

// e -> (row, col) = (e / w, e % w) for e = e0, e0 + stride, e0 + 2 stride, ... without a division per step
struct Walk2 {
  int row, col, drow, dcol, w;
  __device__ __forceinline__ void init(int e0, int stride, int width) {
    w = width; row = e0 / w; col = e0 - row * w; drow = stride / w; dcol = stride - drow * w;
  }
  __device__ __forceinline__ void step() {
    row += drow; col += dcol;
    if (col >= w) { col -= w; ++row; }
  }
};

}  // namespace dft_common
