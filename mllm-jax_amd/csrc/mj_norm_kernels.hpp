// mj_norm_kernels.hpp -- RMSNorm that produces the loss path's `hidden` (forward and backward).
//
// Reference: LlamaRMSNorm (MLLM_JAX/language/llama/llama.py:426-452), instantiated as the final
// norm of the backbone (qwen2/modular_qwen2.py:76, :128): in float32,
//   y = x * rsqrt(mean(x^2) + eps) * scale, cast back to the activation dtype.
// Both kernels are HBM-bound row reductions with 16-byte accesses: the forward gives a row to one
// wavefront (reductions across lanes with shuffles, no LDS traffic), the backward to one workgroup.
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
// A workgroup walks rows with the grid's stride; thread t owns the 16-byte chunks t, t + 256, ... of
// every row (CPT of them, H <= 2048 * CPT), so its share of dscale and of `scale` is CPT * 8
// registers each and a whole row never sits in one wavefront's registers: ~80 registers per thread,
// four to eight workgroups per CU to hide the latency of the single read of each row (the next row's
// loads are issued before the current row is worked on).  The two row sums cross the four
// wavefronts through LDS, one barrier per row (the slots alternate with the row's parity).  Each
// workgroup ends with one partial row of dscale; k_rmsnorm_dscale adds them in a fixed order.
template <int CPT>
__global__ __launch_bounds__(256) void k_rmsnorm_bwd(NormBwdArgs p) {
  __shared__ float s_sum[2][4][2];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int chunks = p.H >> 3;
  float sc[CPT][8], ds[CPT][8];
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int c = tid + 256 * i;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      sc[i][j] = c < chunks ? p.scale[c * 8 + j] : 0.f;
      ds[i][j] = 0.f;
    }
  }
  auto load_row = [&](int row, nu32x4 (&vx)[CPT], nu32x4 (&vg)[CPT]) {
    const nu32x4* xr = (const nu32x4*)(p.x + (int64_t)row * p.ld_x);
    const nu32x4* gr = (const nu32x4*)(p.dy + (int64_t)row * p.ld_dy);
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + 256 * i;
      if (c < chunks) { vx[i] = xr[c]; vg[i] = gr[c]; }
      else { vx[i] = nu32x4{0u, 0u, 0u, 0u}; vg[i] = nu32x4{0u, 0u, 0u, 0u}; }
    }
  };
  auto work_row = [&](int row, int parity, const nu32x4 (&vx)[CPT], const nu32x4 (&vg)[CPT]) {
    float fx[CPT][8], fg[CPT][8];
    float ss = 0.f, t = 0.f;
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      norm_unpack8(vx[i], fx[i]);
      norm_unpack8(vg[i], fg[i]);
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        ss = fmaf(fx[i][j], fx[i][j], ss);
        t = fmaf(fg[i][j] * sc[i][j], fx[i][j], t);
      }
    }
    ss = wave_sum(ss);
    t = wave_sum(t);
    if (lane == 0) { s_sum[parity][wave][0] = ss; s_sum[parity][wave][1] = t; }
    __syncthreads();
    ss = ((s_sum[parity][0][0] + s_sum[parity][1][0]) + s_sum[parity][2][0]) + s_sum[parity][3][0];
    t = ((s_sum[parity][0][1] + s_sum[parity][1][1]) + s_sum[parity][2][1]) + s_sum[parity][3][1];
    const float r = rsqrtf(ss / (float)p.H + p.eps);
    const float k = r * r * r * t / (float)p.H;
    nu32x4* dr = (nu32x4*)(p.dx + (int64_t)row * p.ld_dx);
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int c = tid + 256 * i;
      float o[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        o[j] = r * fg[i][j] * sc[i][j] - fx[i][j] * k;
        ds[i][j] = fmaf(fg[i][j] * fx[i][j], r, ds[i][j]);
      }
      nu32x4 ov;
#pragma unroll
      for (int j = 0; j < 4; ++j) ov[j] = norm_pack_bf16(o[2 * j], o[2 * j + 1]);
      if (c < chunks) dr[c] = ov;
    }
  };

  // The prefetch is unconditional (past the end it reads the last row again): a fixed number of
  // loads between a row's loads and its use lets the wait count leave the newer ones in flight.
  const int stride = gridDim.x, last = p.n - 1;
  int row = blockIdx.x;
  nu32x4 ax[CPT], ag[CPT], bx[CPT], bg[CPT];
  if (row < p.n) load_row(row, ax, ag);
  while (row < p.n) {
    load_row(min(row + stride, last), bx, bg);
    work_row(row, 0, ax, ag);
    row += stride;
    if (row >= p.n) break;
    load_row(min(row + stride, last), ax, ag);
    work_row(row, 1, bx, bg);
    row += stride;
  }
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int c = tid + 256 * i;
    if (c < chunks) {
      float4* out = (float4*)(p.part + (int64_t)blockIdx.x * p.H + c * 8);
      out[0] = float4{ds[i][0], ds[i][1], ds[i][2], ds[i][3]};
      out[1] = float4{ds[i][4], ds[i][5], ds[i][6], ds[i][7]};
    }
  }
}

// dscale[h] (+)= sum over partial rows, fixed order.  Block = 16 column quads x 16 row lanes; lane r
// adds the partial rows r, r+16, ... (eight 16-byte loads in flight), the sixteen lanes are added
// through LDS in lane order.
__global__ __launch_bounds__(256) void k_rmsnorm_dscale(const float* part, int parts, int H, float* dscale,
                                                        int accumulate) {
  __shared__ float4 sh[15][16];
  const int cx = threadIdx.x & 15, ry = threadIdx.x >> 4;
  const int h = blockIdx.x * 64 + cx * 4;            // H % 8 == 0: a quad is inside or outside as a whole
  float4 a = {0.f, 0.f, 0.f, 0.f};
  auto add = [](float4& s, const float4 v) { s.x += v.x; s.y += v.y; s.z += v.z; s.w += v.w; };
  if (h < H) {
    int q = ry;
    for (; q + 7 * 16 < parts; q += 8 * 16) {
      float4 v[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) v[u] = *(const float4*)(part + (int64_t)(q + 16 * u) * H + h);
#pragma unroll
      for (int u = 0; u < 8; ++u) add(a, v[u]);
    }
    for (; q < parts; q += 16) add(a, *(const float4*)(part + (int64_t)q * H + h));
  }
  if (ry > 0) sh[ry - 1][cx] = a;
  __syncthreads();
  if (ry == 0 && h < H) {
#pragma unroll
    for (int r = 0; r < 15; ++r) add(a, sh[r][cx]);
    float4* out = (float4*)(dscale + h);
    if (accumulate) add(a, *out);
    *out = a;
  }
}

}  // namespace mj
