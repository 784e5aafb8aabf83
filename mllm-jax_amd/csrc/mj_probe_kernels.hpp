// mj_probe_kernels.hpp -- measurement support: an MFMA-only loop (no memory traffic in the timed part)
// that shows what the matrix cores of this GPU sustain under its power cap, with operands that change
// on every instruction (random bf16 data) or with all-zero operands.
#pragma once
#include "gemm_tn.hpp"

namespace mj {

// One workgroup = 4 wavefronts, each with the register tile of the product kernels: 4 x 4 blocks of
// v_mfma_f32_32x32x16_bf16, 256 accumulators.  Two operand sets alternate so that consecutive
// instructions never see the same inputs.  2 * 16 * 32768 flop per wavefront and iteration.
__global__ __launch_bounds__(256) void k_probe_mfma(const bf16x8* src, float* out, int iters) {
  bf16x8 a[2][4], b[2][4];
  const int t = threadIdx.x + blockIdx.x * 256;
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      a[s][i] = src[(t * 16 + s * 4 + i) & 65535];
      b[s][i] = src[(t * 16 + 8 + s * 4 + i) & 65535];
    }
  f32x16 acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 2; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s][i], b[s][j], acc[i][j], 0, 0, 0);
  }
  float sum = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) sum += acc[i][j][r];
  out[t] = sum;
}

}  // namespace mj
