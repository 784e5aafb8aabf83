// mj_norm_kernels.hpp -- RMSNorm that produces the loss path's `hidden` (forward and backward).
//
// Reference: LlamaRMSNorm (MLLM_JAX/language/llama/llama.py:426-452), instantiated as the final
// norm of the backbone (qwen2/modular_qwen2.py:76, :128): in float32,
//   y = x * rsqrt(mean(x^2) + eps) * scale, cast back to the activation dtype.
// Both kernels are HBM-bound row reductions: one wavefront per row, 16-byte accesses, reductions
// across lanes with shuffles (no LDS traffic in the forward).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mj {

typedef uint32_t nu32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float norm_bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float norm_bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }
__device__ __forceinline__ uint32_t norm_pack_bf16(float a, float b) {   // round to nearest even, finite inputs
  uint32_t x = __float_as_uint(a), y = __float_as_uint(b);
  x += 0x7fffu + ((x >> 16) & 1u);
  y += 0x7fffu + ((y >> 16) & 1u);
  return (x >> 16) | (y & 0xffff0000u);
}
__device__ __forceinline__ void norm_unpack8(nu32x4 v, float* f) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = norm_bf16_lo(v[j]);
    f[2 * j + 1] = norm_bf16_hi(v[j]);
  }
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
  return v;
}

struct NormFwdArgs {
  const uint16_t* x;   // [n, ld_x] bf16
  const float* scale;  // [H]
  uint16_t* y;         // [n, ld_y] bf16
  float* rstd;         // [n] or null
  int64_t ld_x, ld_y;
  int n, H;
  float eps;
};

// block = 4 wavefronts = 4 rows; MAXC 16-byte chunks per lane (H <= 512 * MAXC) stay in registers
template <int MAXC>
__global__ __launch_bounds__(256) void k_rmsnorm_fwd(NormFwdArgs p) {
  const int lane = threadIdx.x & 63, row = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= p.n) return;
  const int chunks = p.H >> 3;
  const nu32x4* xr = (const nu32x4*)(p.x + (int64_t)row * p.ld_x);
  nu32x4 v[MAXC];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int c = lane + 64 * i;
    if (c < chunks) {
      v[i] = xr[c];
      float f[8];
      norm_unpack8(v[i], f);
#pragma unroll
      for (int j = 0; j < 8; ++j) ss = fmaf(f[j], f[j], ss);
    }
  }
  ss = wave_sum(ss);
  const float r = rsqrtf(ss / (float)p.H + p.eps);
  if (p.rstd != nullptr && lane == 0) p.rstd[row] = r;
  nu32x4* yr = (nu32x4*)(p.y + (int64_t)row * p.ld_y);
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const int c = lane + 64 * i;
    if (c < chunks) {
      float f[8];
      norm_unpack8(v[i], f);
      const float4 s0 = *(const float4*)(p.scale + c * 8), s1 = *(const float4*)(p.scale + c * 8 + 4);
      nu32x4 o;
      o[0] = norm_pack_bf16(f[0] * r * s0.x, f[1] * r * s0.y);
      o[1] = norm_pack_bf16(f[2] * r * s0.z, f[3] * r * s0.w);
      o[2] = norm_pack_bf16(f[4] * r * s1.x, f[5] * r * s1.y);
      o[3] = norm_pack_bf16(f[6] * r * s1.z, f[7] * r * s1.w);
      yr[c] = o;
    }
  }
}

struct NormBwdArgs {
  const uint16_t *dy, *x;   // [n, ld] bf16
  const float* scale;       // [H]
  uint16_t* dx;             // [n, ld_dx] bf16
  float* part;              // [gridDim.x, H] per-workgroup partial sums of dscale
  int64_t ld_dy, ld_x, ld_dx;
  int n, H;
  float eps;
};

// With r = rsqrt(mean(x^2) + eps) and gs = dy * scale:
//   dx = r * gs - x * r^3 * mean(gs * x),   dscale[h] = sum over rows of dy * x * r.
// Each wavefront walks rows with the grid's stride, keeps its share of dscale in registers, and
// the workgroup's four wavefronts are added through LDS into one partial row (fixed order).
template <int MAXC>
__global__ __launch_bounds__(256) void k_rmsnorm_bwd(NormBwdArgs p) {
  extern __shared__ float sh[];   // [3][H]: partial rows of wavefronts 1..3
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int chunks = p.H >> 3;
  float ds[MAXC][8];
#pragma unroll
  for (int i = 0; i < MAXC; ++i)
#pragma unroll
    for (int j = 0; j < 8; ++j) ds[i][j] = 0.f;
  for (int row = blockIdx.x * 4 + wave; row < p.n; row += gridDim.x * 4) {
    const nu32x4* xr = (const nu32x4*)(p.x + (int64_t)row * p.ld_x);
    const nu32x4* gr = (const nu32x4*)(p.dy + (int64_t)row * p.ld_dy);
    float ss = 0.f, t = 0.f;
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = lane + 64 * i;
      if (c < chunks) {
        float fx[8], fg[8];
        norm_unpack8(xr[c], fx);
        norm_unpack8(gr[c], fg);
        const float4 s0 = *(const float4*)(p.scale + c * 8), s1 = *(const float4*)(p.scale + c * 8 + 4);
        const float s[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          ss = fmaf(fx[j], fx[j], ss);
          t = fmaf(fg[j] * s[j], fx[j], t);
        }
      }
    }
    ss = wave_sum(ss);
    t = wave_sum(t);
    const float r = rsqrtf(ss / (float)p.H + p.eps);
    const float k = r * r * r * t / (float)p.H;
    nu32x4* dr = (nu32x4*)(p.dx + (int64_t)row * p.ld_dx);
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = lane + 64 * i;
      if (c < chunks) {
        float fx[8], fg[8], o[8];
        norm_unpack8(xr[c], fx);      // second read of the row: served by the cache
        norm_unpack8(gr[c], fg);
        const float4 s0 = *(const float4*)(p.scale + c * 8), s1 = *(const float4*)(p.scale + c * 8 + 4);
        const float s[8] = {s0.x, s0.y, s0.z, s0.w, s1.x, s1.y, s1.z, s1.w};
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          o[j] = r * fg[j] * s[j] - fx[j] * k;
          ds[i][j] = fmaf(fg[j] * fx[j], r, ds[i][j]);
        }
        nu32x4 ov;
#pragma unroll
        for (int j = 0; j < 4; ++j) ov[j] = norm_pack_bf16(o[2 * j], o[2 * j + 1]);
        dr[c] = ov;
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = lane + 64 * i;
      if (c < chunks)
#pragma unroll
        for (int j = 0; j < 8; ++j) sh[(wave - 1) * p.H + c * 8 + j] = ds[i][j];
    }
  }
  __syncthreads();
  if (wave == 0) {
#pragma unroll
    for (int i = 0; i < MAXC; ++i) {
      const int c = lane + 64 * i;
      if (c < chunks)
#pragma unroll
        for (int j = 0; j < 8; ++j) {
          const int h = c * 8 + j;
          p.part[(int64_t)blockIdx.x * p.H + h] = ((ds[i][j] + sh[h]) + sh[p.H + h]) + sh[2 * p.H + h];
        }
    }
  }
}

// dscale[h] (+)= sum over partial rows, fixed order.  Block = 64 columns x 4 row lanes; lane r
// adds the partial rows r, r+4, ... (eight loads in flight), the four lanes are added through LDS.
__global__ __launch_bounds__(256) void k_rmsnorm_dscale(const float* part, int parts, int H, float* dscale,
                                                        int accumulate) {
  __shared__ float sh[3][64];
  const int cx = threadIdx.x & 63, ry = threadIdx.x >> 6;
  const int h = blockIdx.x * 64 + cx;
  float a = 0.f;
  if (h < H) {
    int q = ry;
    for (; q + 28 < parts; q += 32) {
      float v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = part[(int64_t)(q + 4 * u) * H + h];
#pragma unroll
      for (int u = 0; u < 8; ++u) a += v[u];
    }
    for (; q < parts; q += 4) a += part[(int64_t)q * H + h];
  }
  if (ry > 0) sh[ry - 1][cx] = a;
  __syncthreads();
  if (ry == 0 && h < H) {
    a = ((a + sh[0][cx]) + sh[1][cx]) + sh[2][cx];
    dscale[h] = accumulate ? dscale[h] + a : a;
  }
}

}  // namespace mj
