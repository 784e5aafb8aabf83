// mj_grpo_kernels.hpp -- device kernels of the fused GRPO loss path (gfx950).
//
// Per token chunk of n rows (n <= chunk_tokens):
//   k_logits_stats  : logits^T tile = Wt * hidden^T on MFMA; epilogue applies the softcap,
//                     reduces (max, sum exp, sum exp*z) per token over the tile's vocab rows
//                     and (training) stores the capped logits as IEEE half, transposed [V, n].
//   k_target_logit  : z[t, y_t] = <hidden[t,:], Wt[y_t,:]> in fp32 (one wavefront per token).
//   k_finalize      : merges the per-tile statistics -> lse, logp, entropy, ratio / clip /
//                     min surrogate, per-token loss term and dloss/dlogp.
//   k_dz            : dZt = g * (onehot - exp(z - lse)) * softcap', in place, plus the
//                     token-major copy dZ[n, V] for the dHidden product.
//   k_dhidden, k_dw : the two backward contractions.
// Nothing here allocates; all buffers come from the caller's workspace.
#pragma once
#include "gemm_tn.hpp"

namespace mj {

constexpr float kLog2e = 1.4426950408889634f;
// Stand-in logit for vocab rows past V.  A power of two, so that kNegBig * kLog2e is exact and
// fma(z, kLog2e, -max * kLog2e) is exactly 0 when a whole half-tile holds only stand-ins.
constexpr float kNegBig = -0x1p100f;

MJ_DEV float bf16_to_f32(uint16_t v) { return __uint_as_float((uint32_t)v << 16); }
MJ_DEV uint16_t f32_to_bf16(float f) {   // round to nearest even; inputs are finite
  uint32_t u = __float_as_uint(f);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}
// The logits kept for the backward pass are IEEE half, not bf16: they feed exp(z - lse), where an
// absolute error of ulp(z)/2 becomes a relative error of the probability (|z| < 8: 2^-9 in half
// against 2^-6 in bf16).  Values are clamped to the finite half range first.
MJ_DEV uint16_t f32_to_f16_bits(float f) {
  const _Float16 h = (_Float16)__builtin_amdgcn_fmed3f(f, -65504.f, 65504.f);
  return __builtin_bit_cast(uint16_t, h);
}
MJ_DEV float f16_bits_to_f32(uint16_t v) { return (float)__builtin_bit_cast(_Float16, v); }
MJ_DEV float softcap_apply(float z, float cap, float inv_cap) {
  // cap * tanh(z / cap), tanh(x) = 1 - 2 / (1 + e^{2x})
  const float e = __builtin_amdgcn_exp2f(z * inv_cap * (2.f * kLog2e));
  return cap * (1.f - 2.f * __builtin_amdgcn_rcpf(1.f + e));
}

// ----------------------------------------------------------------------------- logits + stats
struct LogitsArgs {
  const __bf16* wt;      // [V, H] (ld = ld_wt)
  const __bf16* hid;     // chunk origin, [n, ld_hid]
  int64_t ld_wt, ld_hid;
  int V, n, H;
  float cap;             // 0 = off
  uint16_t* zt;          // [V, ld_z] half logits^T of the chunk, or nullptr (forward only)
  int64_t ld_z;
  float *pm, *pl, *ps;   // per (vocab half-tile, token) partial max / sum e / sum e*z, ld = ld_p
  int64_t ld_p;
};

template <int BM, int BN>
__global__ __launch_bounds__(kThreads) void k_logits_stats(LogitsArgs p, TileMap<4, 8> map) {
  using G = GemmTN<BM, BN>;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  int tm, tn;
  if (!map.tile(blockIdx.x, tm, tn)) return;
  const int m0 = tm * BM, n0 = tn * BN;
  G g;
  g.run(p.wt + (int64_t)m0 * p.ld_wt, p.V - m0, p.ld_wt, p.hid + (int64_t)n0 * p.ld_hid, p.n - n0,
        p.ld_hid, p.H, smem);

  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave & 1, wn = wave >> 1, l31 = lane & 31, lhi = lane >> 5;
  const int vbase = m0 + wm * G::WM + lhi * 4;   // + mi*32 + (r/4)*8 + r%4
  const bool tail = (m0 + BM > p.V);
  const float inv_cap = p.cap > 0.f ? 1.f / p.cap : 0.f;
#pragma unroll
  for (int ni = 0; ni < G::NI; ++ni) {
    const int col = n0 + wn * G::WN + ni * 32 + l31;
    float mx = kNegBig;
#pragma unroll
    for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        float z = g.acc[mi][ni][r];
        if (p.cap > 0.f) z = softcap_apply(z, p.cap, inv_cap);
        if (tail && (vbase + mi * 32 + (r >> 2) * 8 + (r & 3)) >= p.V) z = kNegBig;
        g.acc[mi][ni][r] = z;
        mx = fmaxf(mx, z);
      }
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    float l = 0.f, s = 0.f;
    const float mxl = mx * kLog2e;
#pragma unroll
    for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const float z = g.acc[mi][ni][r];
        const float e = __builtin_amdgcn_exp2f(fmaf(z, kLog2e, -mxl));
        l += e;
        s = fmaf(e, z, s);
      }
    l += __shfl_xor(l, 32);
    s += __shfl_xor(s, 32);
    if (lhi == 0) {
      const int64_t o = (int64_t)(tm * 2 + wm) * p.ld_p + col;
      p.pm[o] = mx;
      p.pl[o] = l;
      p.ps[o] = s;
    }
    if (p.zt != nullptr) {
#pragma unroll
      for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int v = vbase + mi * 32 + (r >> 2) * 8 + (r & 3);
          if (!tail || v < p.V) p.zt[(int64_t)v * p.ld_z + col] = f32_to_f16_bits(g.acc[mi][ni][r]);
        }
    }
  }
}

// ----------------------------------------------------------------------------- target logit
// One wavefront per token: zy[t] = softcap(<hid[t,:], wt[y_t,:]>).
__global__ __launch_bounds__(256) void k_target_logit(const __bf16* hid, int64_t ld_hid,
                                                      const __bf16* wt, int64_t ld_wt,
                                                      const int32_t* targets, int n, int H, int V,
                                                      float cap, float* zy) {
  const int t = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (t >= n) return;
  int y = targets[t];
  y = y < 0 ? 0 : (y >= V ? V - 1 : y);
  const uint16_t* a = (const uint16_t*)hid + (int64_t)t * ld_hid;
  const uint16_t* b = (const uint16_t*)wt + (int64_t)y * ld_wt;
  float acc = 0.f;
  for (int k = lane * 8; k < H; k += 512) {
    const u32x4 av = *(const u32x4*)(a + k), bv = *(const u32x4*)(b + k);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      acc = fmaf(__uint_as_float(av[i] << 16), __uint_as_float(bv[i] << 16), acc);
      acc = fmaf(__uint_as_float(av[i] & 0xffff0000u), __uint_as_float(bv[i] & 0xffff0000u), acc);
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
  if (lane == 0) zy[t] = cap > 0.f ? softcap_apply(acc, cap, 1.f / cap) : acc;
}

// ----------------------------------------------------------------------------- finalize
struct FinalizeArgs {
  const float *pm, *pl, *ps;   // [parts, ld_p]
  int64_t ld_p;
  int parts, n, n_pad;         // tokens in chunk, padded count (g is written for all n_pad)
  const float* zy;             // [n] chunk-local
  const float *old_logp, *adv, *mask;   // chunk origin; old_logp may be null
  float eps_low, eps_high, inv_tv, gscale;
  int sft;
  float *logp, *lse, *ent;     // chunk origin outputs (ent may be null)
  float* term;                 // per-token loss term
  float* g;                    // [n_pad] dloss/dlogp * gscale, or null (forward only)
};

// block = (64 tokens) x (4 slices of the partial list)
__global__ __launch_bounds__(256) void k_finalize(FinalizeArgs p) {
  __shared__ float sm[4][64], sl[4][64], ss[4][64];
  const int tx = threadIdx.x & 63, ty = threadIdx.x >> 6;
  const int t = blockIdx.x * 64 + tx;
  float m = kNegBig, l = 0.f, s = 0.f;
  if (t < p.n) {
    for (int q = ty; q < p.parts; q += 4) {
      const int64_t o = (int64_t)q * p.ld_p + t;
      const float mq = p.pm[o], lq = p.pl[o], sq = p.ps[o];
      const float mn = fmaxf(m, mq);
      const float a = __expf(m - mn), b = __expf(mq - mn);
      l = l * a + lq * b;
      s = s * a + sq * b;
      m = mn;
    }
  }
  sm[ty][tx] = m; sl[ty][tx] = l; ss[ty][tx] = s;
  __syncthreads();
  if (ty != 0) return;
  if (t >= p.n) {
    if (p.g != nullptr && t < p.n_pad) p.g[t] = 0.f;
    return;
  }
  float M = fmaxf(fmaxf(sm[0][tx], sm[1][tx]), fmaxf(sm[2][tx], sm[3][tx]));
  float L = 0.f, S = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float w = __expf(sm[i][tx] - M);
    L += sl[i][tx] * w;
    S += ss[i][tx] * w;
  }
  const float lse = M + __logf(L);
  const float logp = p.zy[t] - lse;
  p.lse[t] = lse;
  p.logp[t] = logp;
  if (p.ent != nullptr) p.ent[t] = lse - S / L;   // = -sum p log p  (reference adds 1e-9 inside the log)
  const float mk = p.mask[t];
  float term, g;
  if (p.sft) {
    term = -logp * mk * p.inv_tv;
    g = -mk * p.inv_tv;
  } else {
    const float adv = p.adv[t];
    const float ratio = p.old_logp != nullptr ? __expf(logp - p.old_logp[t]) : 1.f;
    const float lo = 1.f - p.eps_low, hi = 1.f + p.eps_high;
    const float clipped = fminf(fmaxf(ratio, lo), hi);
    term = -fminf(ratio * adv, clipped * adv) * mk * p.inv_tv;
    const bool active = (ratio >= lo && ratio <= hi) || (ratio > hi && adv < 0.f) || (ratio < lo && adv > 0.f);
    g = active ? -mk * p.inv_tv * adv * ratio : 0.f;
  }
  p.term[t] = term;
  if (p.g != nullptr) p.g[t] = g * p.gscale;
}

// dloss/dlogp from a saved forward (separate backward entry point)
__global__ __launch_bounds__(256) void k_coeff_from_saved(const float* logp, const float* old_logp,
                                                          const float* adv, const float* mask, int n,
                                                          int n_pad, float eps_low, float eps_high,
                                                          float inv_tv, float gscale, int sft, float* g) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= n_pad) return;
  float out = 0.f;
  if (t < n) {
    const float mk = mask[t];
    if (sft) {
      out = -mk * inv_tv;
    } else {
      const float a = adv[t];
      const float ratio = old_logp != nullptr ? __expf(logp[t] - old_logp[t]) : 1.f;
      const float lo = 1.f - eps_low, hi = 1.f + eps_high;
      const bool active = (ratio >= lo && ratio <= hi) || (ratio > hi && a < 0.f) || (ratio < lo && a > 0.f);
      out = active ? -mk * inv_tv * a * ratio : 0.f;
    }
  }
  g[t] = out * gscale;
}

// Deterministic single-workgroup sum of the per-token loss terms.
__global__ __launch_bounds__(1024) void k_reduce_loss(const float* term, int n, float* loss) {
  __shared__ float sh[1024];
  float a = 0.f;
  for (int i = threadIdx.x; i < n; i += 1024) a += term[i];
  sh[threadIdx.x] = a;
  __syncthreads();
  for (int o = 512; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) sh[threadIdx.x] += sh[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) loss[0] = sh[0];
}

// ----------------------------------------------------------------------------- dZ
struct DzArgs {
  uint16_t* zt;        // [V, ld_z] in: capped logits^T (half); out: dZ^T (bf16)
  int64_t ld_z;
  uint16_t* dz;        // [n_pad, ld_dz] out: dZ token-major
  int64_t ld_dz;
  const float *lse, *g;    // chunk-local [n_pad] (lse valid for t < n)
  const int32_t* targets;  // chunk origin
  int V, n, n_pad;
  float cap;
};

// block: 64 vocab rows x 64 tokens
__global__ __launch_bounds__(256) void k_dz(DzArgs p) {
  __shared__ uint16_t tile[64][72];   // [v][token], padded
  const int v0 = blockIdx.x * 64, t0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 7, ty = threadIdx.x >> 3;   // 8 token-octets x 32 rows
  const float inv_cap2 = p.cap > 0.f ? 1.f / (p.cap * p.cap) : 0.f;
  float lse[8], g[8];
  int y[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int t = t0 + tx * 8 + i;
    const bool in = t < p.n;
    lse[i] = in ? p.lse[t] : 0.f;
    g[i] = in ? p.g[t] : 0.f;
    y[i] = in ? p.targets[t] : -1;
  }
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int vl = ty + pass * 32, v = v0 + vl;
    u32x4 out = {0u, 0u, 0u, 0u};
    if (v < p.V) {
      uint16_t* src = p.zt + (int64_t)v * p.ld_z + t0 + tx * 8;
      const u32x4 in = *(const u32x4*)src;
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t w = in[i >> 1];
        const float z = f16_bits_to_f32((uint16_t)((i & 1) ? (w >> 16) : (w & 0xffffu)));
        float d = -__builtin_amdgcn_exp2f((z - lse[i]) * kLog2e);
        if (v == y[i]) d += 1.f;
        d *= g[i];
        if (p.cap > 0.f) d *= 1.f - z * z * inv_cap2;
        if (!(g[i] != 0.f)) d = 0.f;   // masked or padding token: exactly zero, whatever z holds
        const uint32_t b = f32_to_bf16(d);
        out[i >> 1] |= (i & 1) ? (b << 16) : b;
      }
      *(u32x4*)src = out;
    }
    *(u32x4*)&tile[vl][tx * 8] = out;
  }
  __syncthreads();
  // transposed write: thread -> token tl, 8 consecutive vocab rows per 16-byte store
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int tl = ty + pass * 32, t = t0 + tl;
    const int vv = tx * 8;
    if (t < p.n_pad && v0 + vv < p.V) {
      u32x4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        o[i] = (uint32_t)tile[vv + 2 * i][tl] | ((uint32_t)tile[vv + 2 * i + 1][tl] << 16);
      *(u32x4*)(p.dz + (int64_t)t * p.ld_dz + v0 + vv) = o;
    }
  }
}

// ----------------------------------------------------------------------------- backward products
struct DhArgs {
  const __bf16* dz;   // [n, ld_dz]
  const __bf16* w;    // [H, ld_w]
  int64_t ld_dz, ld_w;
  int n, H, V;
  uint16_t* dh;       // chunk origin [n, ld_dh] bf16
  int64_t ld_dh;
};

template <int BM, int BN>
__global__ __launch_bounds__(kThreads) void k_dhidden(DhArgs p, TileMap<4, 8> map) {
  using G = GemmTN<BM, BN>;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  int tm, tn;
  if (!map.tile(blockIdx.x, tm, tn)) return;
  const int m0 = tm * BM, n0 = tn * BN;
  G g;
  g.run(p.dz + (int64_t)m0 * p.ld_dz, p.n - m0, p.ld_dz, p.w + (int64_t)n0 * p.ld_w, p.H - n0, p.ld_w,
        p.V, smem);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave & 1, wn = wave >> 1, l31 = lane & 31, lhi = lane >> 5;
#pragma unroll
  for (int ni = 0; ni < G::NI; ++ni) {
    const int col = n0 + wn * G::WN + ni * 32 + l31;
    if (col >= p.H) continue;
#pragma unroll
    for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * G::WM + mi * 32 + (r >> 2) * 8 + lhi * 4 + (r & 3);
        if (row < p.n) p.dh[(int64_t)row * p.ld_dh + col] = f32_to_bf16(g.acc[mi][ni][r]);
      }
  }
}

struct DwArgs {
  const __bf16* ht;    // chunk origin inside hiddenT [H, ld_ht]
  const __bf16* dzt;   // [V, ld_z]
  int64_t ld_ht, ld_z;
  int H, V, K;         // K = chunk tokens rounded up to 8 (padding holds zeros)
  float* dw;           // [H, ld_w] f32
  int64_t ld_dw;
  int accumulate;
};

template <int BM, int BN>
__global__ __launch_bounds__(kThreads) void k_dw(DwArgs p, TileMap<4, 8> map) {
  using G = GemmTN<BM, BN>;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  int tm, tn;
  if (!map.tile(blockIdx.x, tm, tn)) return;
  const int m0 = tm * BM, n0 = tn * BN;
  G g;
  g.run(p.ht + (int64_t)m0 * p.ld_ht, p.H - m0, p.ld_ht, p.dzt + (int64_t)n0 * p.ld_z, p.V - n0, p.ld_z,
        p.K, smem);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int wm = wave & 1, wn = wave >> 1, l31 = lane & 31, lhi = lane >> 5;
#pragma unroll
  for (int ni = 0; ni < G::NI; ++ni) {
    const int col = n0 + wn * G::WN + ni * 32 + l31;
    if (col >= p.V) continue;
#pragma unroll
    for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int row = m0 + wm * G::WM + mi * 32 + (r >> 2) * 8 + lhi * 4 + (r & 3);
        if (row < p.H) {
          float* dst = p.dw + (int64_t)row * p.ld_dw + col;
          *dst = p.accumulate ? *dst + g.acc[mi][ni][r] : g.acc[mi][ni][r];
        }
      }
  }
}

// ----------------------------------------------------------------------------- transpose
// dst[c, r] = src[r, c] for r < R, c < C; dst columns R..R_pad-1 are zero-filled.
// Requires C % 8 == 0, ld_dst % 8 == 0, R_pad % 8 == 0.  Block: 64 x 64 tile.
__global__ __launch_bounds__(256) void k_transpose_bf16(const uint16_t* src, int64_t ld_src,
                                                        uint16_t* dst, int64_t ld_dst, int R, int C,
                                                        int R_pad) {
  __shared__ uint16_t tile[64][72];
  const int r0 = blockIdx.x * 64, c0 = blockIdx.y * 64;
  const int tx = threadIdx.x & 7, ty = threadIdx.x >> 3;
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int rl = ty + pass * 32, r = r0 + rl, c = c0 + tx * 8;
    u32x4 v = {0u, 0u, 0u, 0u};
    if (r < R && c < C) v = *(const u32x4*)(src + (int64_t)r * ld_src + c);
    *(u32x4*)&tile[rl][tx * 8] = v;
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 2; ++pass) {
    const int cl = ty + pass * 32, c = c0 + cl, r = r0 + tx * 8;
    if (c < C && r < R_pad) {
      u32x4 o;
#pragma unroll
      for (int i = 0; i < 4; ++i)
        o[i] = (uint32_t)tile[tx * 8 + 2 * i][cl] | ((uint32_t)tile[tx * 8 + 2 * i + 1][cl] << 16);
      *(u32x4*)(dst + (int64_t)c * ld_dst + r) = o;
    }
  }
}

}  // namespace mj
