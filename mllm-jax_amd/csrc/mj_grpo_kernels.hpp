// mj_grpo_kernels.hpp -- device kernels of the fused GRPO loss path (gfx950).
//
// Per token chunk of n rows (n <= chunk_tokens):
//   k_logits_stats  : logits^T tile [vocab x tokens] = W^T * hidden^T on MFMA, W and hidden read in
//                     place; the epilogue applies the softcap, reduces (sum exp, sum exp*z) per token
//                     over the tile's vocab rows, picks out the sampled token's logit and (training)
//                     stores a 16-bit row-major [n, V] matrix for the backward (see StatsMode).
//   k_finalize      : adds up the per-tile statistics -> lse, logp, entropy, ratio / clip / min
//                     surrogate, per-token loss term, dloss/dlogp, the row scale of E and its
//                     one-hot patch.
//   k_dhidden       : dHidden[n,H] = rowscale * (E or dZ) * W^T, optionally split over the vocab into
//                     fp32 partial sums that k_dhidden_reduce adds up.
//   k_scale_hidden  : (rs * hidden)^T, or hidden^T behind a kStatsMax pass: the token-side operand of
//                     the dW product with the tokens contiguous, [H, n_pad] bf16.
//   k_dw            : dW^T tile [vocab x hidden] = (E or dZ)^T * (rs * hidden or hidden), written /
//                     accumulated into dW[H,V] with 16-byte accesses.
//   k_dz            : only behind a kStatsMax pass: in place, logits -> dZ (bf16).
// Nothing here allocates; all buffers come from the caller's workspace.
#pragma once
#include "gemm_tn.hpp"

namespace mj {

constexpr float kLog2e = 1.4426950408889634f;
constexpr float kLn2 = 0.6931471805599453f, kLn2Sq = 0.4804530139182014f;
// Stand-in logit for vocab rows past V.  A power of two, so that kNegBig * kLog2e is exact and
// fma(z, kLog2e, -max * kLog2e) is exactly 0 when a whole half-tile holds only stand-ins.
constexpr float kNegBig = -0x1p100f;

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

// Epilogue stores go through buffer descriptors: the row part of the address is a scalar offset,
// the lane part is computed once, and rows past the end of the output fall outside the
// descriptor's range and are dropped -- no per-store address arithmetic or branches.
MJ_DEV void store_b16(uint16_t v, __amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  __builtin_amdgcn_raw_buffer_store_b16((short)v, r, voff, soff, 0);
}
MJ_DEV void store_b32(float v, __amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  __builtin_amdgcn_raw_buffer_store_b32(__float_as_uint(v), r, voff, soff, 0);
}
MJ_DEV void store_b128(f32x4 v, __amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(u32x4, v), r, voff, soff, 0);
}
MJ_DEV float load_b32(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  return __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, voff, soff, 0));
}
MJ_DEV f32x4 load_b128(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
  return __builtin_bit_cast(f32x4, __builtin_amdgcn_raw_buffer_load_b128(r, voff, soff, 0));
}

// Target ids outside [0, V) select the nearest valid id, in the forward and the backward alike.
MJ_DEV int clamp_target(int y, int V) { return min(max(y, 0), V - 1); }

// Tokens of a chunk that take part in the backward pass, rounded up to whole 256-token tiles:
// all n_pad of them, or -- when the caller compacted the tokens that carry a gradient to the
// front -- those up to the device-side count.
MJ_DEV int live_pad(const int* n_live, int c0, int n_pad) {
  if (n_live == nullptr) return n_pad;
  const int left = __builtin_amdgcn_readfirstlane(*n_live) - c0;
  return min(n_pad, max(left + 255, 0) & ~255);
}

// ----------------------------------------------------------------------------- logits + stats
// What the epilogue of the logits product keeps for a chunk of tokens:
//   kStatsExp  : per (vocab half-tile, token) the sums of e = exp(z) and e * z with NO running
//                maximum (valid while logsumexp(z) stays within +-60, which k_finalize checks for
//                every token) and, when a backward follows, the row-major 16-bit matrix
//                E[t, v] = bf16(exp(z) * cap'(z)); rows of masked tokens are not written.  Since
//                dZ[t, v] = rs_t * (E[t, v] - onehot patch) with rs_t = -g_t / sum_v exp(z), the two
//                backward products read E as it is: k_dhidden scales its output rows by rs_t, k_dw
//                reads rs_t * hidden, and no pass over [n, V] is needed to form dZ.
//   kStatsMax  : the same sums relative to the per-tile maximum (any logit range) and the capped
//                logits as IEEE half; k_dz turns those into dZ in place.  Used with the entropy
//                bonus and as the rescue when kStatsExp's range check fails.
//   kStatsGrad : backward from a saved forward: lse and dloss/dlogp are inputs, so the epilogue writes
//                dZ = -g * p * cap' directly (k_patch_grad adds the one-hot term).
// state[0] tells the backward products what the 16-bit matrix holds: 0 = E (scale by rs, read
// rs * hidden), 1 = dZ itself.  Either way the rows of tokens without a gradient (dloss/dlogp and
// the entropy-bonus coefficient both 0: masked tokens, zero advantages) are never read: one bit
// per token, 64-bit words (`dead`), tells the loaders of the backward products to fill those rows
// with zeros instead of fetching them.  The products still multiply the zeros.
enum StatsMode { kStatsExp = 0, kStatsMax = 1, kStatsGrad = 2 };

constexpr float kExpSumMin = 0x1p-86f, kExpSumMax = 0x1p86f;   // logsumexp within about +-59.6

struct LogitsArgs {
  const __bf16* w;       // lm_head [H, ld_w]
  const __bf16* hid;     // chunk origin, [n, ld_hid]
  int64_t ld_w, ld_hid;
  int V, n, H;
  float cap;             // 0 = off
  uint16_t* zt;          // [n, ld_z] 16-bit rows of the chunk (see StatsMode), or nullptr (forward only)
  int64_t ld_z;
  float *pm, *pl, *ps;   // per (vocab half-tile, token) partial max / sum e / sum e*z, ld = ld_p
  float* plt;            // temperature != 1 only: sum e^((z-max)/T), and ps then holds sum e^((z-max)/T)*z (max = 0 in kStatsExp)
  float inv_t;           // 1 / temperature
  int64_t ld_p;
  const int32_t* targets;   // chunk origin
  float* zy;                // chunk origin: capped logit of the sampled token
  const int* n_live;        // null, or device count of leading tokens (from token c0 on) that need a backward
  int c0;
  const float* mask;        // chunk origin; rows of tokens with mask == 0 are not stored
  const float *lse, *g;     // kStatsGrad: chunk-local saved logsumexp [n] and dloss/dlogp [n_pad]
  int* state;
};

MJ_DEV uint32_t pack_bf16(float a, float b) {
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2{a, b}, bf16x2));
}
MJ_DEV uint32_t pack_f16(float a, float b) {   // clamped to the finite half range, round to nearest even
  typedef __attribute__((ext_vector_type(2))) float f32x2;
  typedef __attribute__((ext_vector_type(2))) _Float16 f16x2;
  const f32x2 v = {__builtin_amdgcn_fmed3f(a, -65504.f, 65504.f), __builtin_amdgcn_fmed3f(b, -65504.f, 65504.f)};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2));
}

// Eight values of one token: a lane's rows 0..3 of two consecutive 8-row groups of the MFMA layout.
// The lanes l and l + 32 hold rows 4..7 of the same groups for the same token; after exchanging
// one half with the partner each lane owns eight CONSECUTIVE vocab entries and stores them with
// one 16-byte access (`voff` carries the lane's 16 bytes of the 32).
template <bool HALF>
MJ_DEV void store_rows8(const float (&v)[8], __amdgpu_buffer_rsrc_t rs, uint32_t voff, uint32_t soff) {
  uint32_t a0, a1, b0, b1;
  if (HALF) {
    a0 = pack_f16(v[0], v[1]); a1 = pack_f16(v[2], v[3]); b0 = pack_f16(v[4], v[5]); b1 = pack_f16(v[6], v[7]);
  } else {
    a0 = pack_bf16(v[0], v[1]); a1 = pack_bf16(v[2], v[3]); b0 = pack_bf16(v[4], v[5]); b1 = pack_bf16(v[6], v[7]);
  }
  // v_permlane32_swap: the first operand of lanes 32..63 <-> the second operand of lanes 0..31
  const auto s0 = __builtin_amdgcn_permlane32_swap(a0, b0, false, false);
  const auto s1 = __builtin_amdgcn_permlane32_swap(a1, b1, false, false);
  const u32x4 out = {s0[0], s1[0], s0[1], s1[1]};
  __builtin_amdgcn_raw_buffer_store_b128(out, rs, voff, soff, 0);
}

// One 256 x 256 tile: logits^T [vocab x tokens] = W^T * hidden^T on MFMA, then the epilogue of MODE
// (kStatsMax, kStatsGrad; kStatsExp has a tile of its own, logits_tile16).
template <int BM, int BN, int MODE, bool CAP>
MJ_DEV void logits_tile(const LogitsArgs& p, int tm, int tn, char* smem, int tid) {
  using G = GemmTN<BM, BN, kKRow, kRowK>;
  const int m0 = tm * BM, n0 = tn * BN;
  G g;
  g.run(p.w + m0, p.V - m0, p.ld_w, p.hid + (int64_t)n0 * p.ld_hid, p.n - n0, p.ld_hid, p.H, smem, tid);

  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keeps descriptors in SGPRs
  const int wm = wave & 1, wn = wave >> 1, l31 = lane & 31, lhi = lane >> 5;
  const int vwave = m0 + wm * G::WM;             // first vocab row of this wavefront
  const int vbase = vwave + lhi * 4;             // + mi*32 + (r/4)*8 + r%4
  const int t0 = n0 + wn * G::WN;                // first token of this wavefront
  const bool tail = (m0 + BM > p.V);
  const float inv_cap = CAP ? 1.f / p.cap : 0.f;
  const float inv_cap2 = inv_cap * inv_cap;
  const int zt_cols = live_pad(p.n_live, p.c0, (p.n + 255) & ~255);
  // this wavefront's 128 token rows of the 16-bit matrix; rows at or past n fall outside and are dropped
  const uint32_t ldz2 = (uint32_t)p.ld_z * 2;
  const int trows = min(max(p.n - t0, 0), G::WN);
  const __amdgpu_buffer_rsrc_t zrs =
      make_rsrc_wave(p.zt == nullptr ? nullptr : p.zt + (int64_t)t0 * p.ld_z, (int64_t)trows * ldz2);
#pragma unroll
  for (int ni = 0; ni < G::NI; ++ni) {
    const int col = t0 + ni * 32 + l31;
    // Softcap (CAP: a kernel of its own, so that the uncapped one carries none of this).  While every
    // logit of the block is small against the cap -- checked per wavefront -- tanh is its odd series
    // to u^7 (|u| <= 0.25: error below 1e-7 of u, five multiply-adds instead of an exp and a reciprocal).
    static_assert(MODE != kStatsExp, "kStatsExp runs on logits_tile16");
    if (CAP) {
      float big = 0.f;
#pragma unroll
      for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
        for (int r = 0; r < 16; ++r) big = fmaxf(big, fabsf(g.acc[mi][ni][r]));
      if (__all(big * inv_cap <= 0.25f)) {
        // z P(z^2),  P(w) = k (1 - w / (3 c^2) + 2 w^2 / (15 c^4) - 17 w^3 / (315 c^6)),  k = log2(e) or 1
        const float k0 = 1.f;
        const float c1 = k0 * (-1.f / 3.f) * inv_cap2, c2 = k0 * (2.f / 15.f) * inv_cap2 * inv_cap2;
        const float c3 = k0 * (-17.f / 315.f) * inv_cap2 * inv_cap2 * inv_cap2;
#pragma unroll
        for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float z = g.acc[mi][ni][r], w = z * z;
            g.acc[mi][ni][r] = z * fmaf(w, fmaf(w, fmaf(w, c3, c2), c1), k0);
          }
      } else {
#pragma unroll
        for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float zc = softcap_apply(g.acc[mi][ni][r], p.cap, inv_cap);
            g.acc[mi][ni][r] = zc;
          }
      }
    }
    // An opaque use of the block's 64 accumulators: with it the register allocator moves them out of
    // the accumulation registers here, one block at a time, instead of parking 32 of them in scratch
    // memory at the start of the epilogue (no scratch access is left in the kernel; measured 1 % faster).
#pragma unroll
    for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
      for (int r = 0; r < 16; ++r) asm volatile("" : "+v"(g.acc[mi][ni][r]));
    // The stand-in for rows past V is a rare, wave-uniform case behind a real scalar branch (the
    // empty asm keeps the compiler from flattening it into per-element selects).
    if (tail) {
      asm volatile("");
#pragma unroll
      for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if ((vbase + mi * 32 + (r >> 2) * 8 + (r & 3)) >= p.V) g.acc[mi][ni][r] = kNegBig;
    }
    // where this lane's eight-entry groups go: token row, then the lane's half of a 16-entry span
    const bool store = p.zt != nullptr && (t0 + ni * 32) < zt_cols;   // tokens past the live ones are never read
    const uint32_t voff = (uint32_t)((ni * 32 + l31) * ldz2 + (vwave + lhi * 8) * 2);
    // Rows of tokens that cannot carry a gradient (mask 0; in kStatsGrad: dloss/dlogp 0) are not
    // written at all: the backward products know them from the dead-token bits and do not read them.
    bool keep = true;
    if (store) keep = MODE == kStatsGrad ? (col < p.n && p.g[col] != 0.f) : (col < p.n && p.mask[col] != 0.f);
    auto group_off = [&](int mi, int qp) {      // kOob when the lane's eight entries lie past V (V % 8 == 0)
      return (keep && (vwave + mi * 32 + qp * 16 + lhi * 8) < p.V) ? voff : kOob;
    };

    if (MODE == kStatsMax) {
      float mx = kNegBig;
#pragma unroll
      for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, g.acc[mi][ni][r]);
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
      float lt = 0.f;
      if (p.inv_t != 1.f) {
        // The reference takes the log-prob from softmax(z) but the entropy from softmax(z / T)
        // (train_modules/__init__.py:124-126, :136): a second pair of sums, only when T != 1.
        asm volatile("");
        const float kt = kLog2e * p.inv_t, mxt = mx * kt;
        s = 0.f;
#pragma unroll
        for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
          for (int r = 0; r < 16; ++r) {
            const float z = g.acc[mi][ni][r];
            const float e = __builtin_amdgcn_exp2f(fmaf(z, kt, -mxt));
            lt += e;
            s = fmaf(e, z, s);
          }
        lt += __shfl_xor(lt, 32);
        s += __shfl_xor(s, 32);
      }
      if (lhi == 0) {
        const int64_t o = (int64_t)(tm * 2 + wm) * p.ld_p + col;
        p.pm[o] = mx;
        p.pl[o] = l;
        p.ps[o] = s;
        if (p.inv_t != 1.f) p.plt[o] = lt;
      }
      if (store) {
#pragma unroll
        for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
          for (int qp = 0; qp < 2; ++qp) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) v[j] = g.acc[mi][ni][qp * 8 + j];
            store_rows8<true>(v, zrs, group_off(mi, qp), (uint32_t)(mi * 32 + qp * 16) * 2);
          }
      }
    } else {   // kStatsGrad
      const float lse2 = col < p.n ? p.lse[col] * kLog2e : 0.f;
      const float gneg = col < p.n ? -p.g[col] : 0.f;
      if (store) {
#pragma unroll
        for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
          for (int qp = 0; qp < 2; ++qp) {
            float v[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
              const float z = g.acc[mi][ni][qp * 8 + j];
              const float d = gneg * __builtin_amdgcn_exp2f(fmaf(z, kLog2e, -lse2));
              v[j] = CAP ? d * (1.f - z * z * inv_cap2) : d;
            }
            store_rows8<false>(v, zrs, group_off(mi, qp), (uint32_t)(mi * 32 + qp * 16) * 2);
          }
      }
    }
    // The sampled token's logit: exactly one lane of one tile holds it.  Few wavefronts have a
    // hit at all (32 tokens x 128 rows out of V), so the register search sits behind a vote.
    {
      const int y = col < p.n ? clamp_target(p.targets[col], p.V) : -1;
      const int d = y - vwave;                       // row inside the wavefront's 128
      const bool hit = y >= 0 && d >= 0 && d < G::WM && ((d >> 2) & 1) == lhi;
      if (__any(hit)) {
        const int flat = (d >> 5) * 16 + ((d >> 3) & 3) * 4 + (d & 3);   // mi*16 + r
        float zy = 0.f;
#pragma unroll
        for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
          for (int r = 0; r < 16; ++r) zy = (flat == mi * 16 + r) ? g.acc[mi][ni][r] : zy;
        if (hit) p.zy[col] = zy;
      }
    }
  }
}

// Sum of x over the four 16-lane rows of a wavefront, in every lane, without a trip through the LDS
// crossbar: v_permlane16_swap pairs the rows (0,1) and (2,3), v_permlane32_swap the two halves.
MJ_DEV float sum_rows16(float x) {
  const uint32_t a = __float_as_uint(x);
  const auto p = __builtin_amdgcn_permlane16_swap(a, a, false, false);
  const uint32_t b = __float_as_uint(__uint_as_float(p[0]) + __uint_as_float(p[1]));
  const auto q = __builtin_amdgcn_permlane32_swap(b, b, false, false);
  return __uint_as_float(q[0]) + __uint_as_float(q[1]);
}

// The kStatsExp tile on the chained 16 x 16 x 32 engine (GemmTN16).  A lane holds, for the token
// ni*16 + lane%16, the four vocab rows mi*16 + (lane/16)*4 + 0..3 of each of the eight blocks mi.
// Two blocks at a time, the lanes l and l + 16 exchange one packed half (v_permlane16_swap) so that
// each owns eight CONSECUTIVE vocab entries of one block and stores them with one 16-byte access.
// The per-token inputs of the epilogue (mask, sampled token) are requested before the k loop, one
// token per thread, and handed to the lanes that need them through kTileExtraLds bytes of LDS behind
// the two stages: requested in the epilogue they cost a memory round trip per tile (2.6 us of a
// tile's 95 at 16384 x 3584 x 152064).
constexpr int kTileExtraLds = 2048;
template <int BM, int BN, bool CAP>
MJ_DEV void logits_tile16(const LogitsArgs& p, int tm, int tn, char* smem, int tid) {
  using G = GemmTN16<BM, BN, kKRow, kRowK>;
  static_assert(BN == kThreads, "one token of the tile per thread");
  const int m0 = tm * BM, n0 = tn * BN;
  const int tok = n0 + tid;
  const float mask_t = tok < p.n ? p.mask[tok] : 0.f;
  const int target_t = tok < p.n ? clamp_target(p.targets[tok], p.V) : -1;
  G g;
  g.run(p.w + m0, p.V - m0, p.ld_w, p.hid + (int64_t)n0 * p.ld_hid, p.n - n0, p.ld_hid, p.H, smem, tid);
  float* tile_mask = (float*)(smem + G::kLdsBytes);
  int* tile_target = (int*)(tile_mask + BN);
  tile_mask[tid] = mask_t;
  tile_target[tid] = target_t;
  __syncthreads();

  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keeps descriptors in SGPRs
  const int wm = wave & 1, wn = wave >> 1, l15 = lane & 15, lq = lane >> 4;
  const int vwave = m0 + wm * G::WM;             // first vocab row of this wavefront
  const int vbase = vwave + lq * 4;              // + mi*16 + r
  const int t0 = n0 + wn * G::WN;                // first token of this wavefront
  const bool tail = (m0 + BM > p.V);
  const float inv_cap = CAP ? 1.f / p.cap : 0.f;
  const float inv_cap2 = inv_cap * inv_cap;
  const int zt_cols = live_pad(p.n_live, p.c0, (p.n + 255) & ~255);
  const uint32_t ldz2 = (uint32_t)p.ld_z * 2;
  const int trows = min(max(p.n - t0, 0), G::WN);
  const __amdgpu_buffer_rsrc_t zrs =
      make_rsrc_wave(p.zt == nullptr ? nullptr : p.zt + (int64_t)t0 * p.ld_z, (int64_t)trows * ldz2);
  float mk[G::NI];
  int tg[G::NI];
#pragma unroll
  for (int ni = 0; ni < G::NI; ++ni) {
    mk[ni] = tile_mask[wn * G::WN + ni * 16 + l15];
    tg[ni] = tile_target[wn * G::WN + ni * 16 + l15];
  }
#pragma unroll
  for (int ni = 0; ni < G::NI; ++ni) {
    const int col = t0 + ni * 16 + l15;
    // softcap: see logits_tile (series while every logit of the wavefront's block column is small
    // against the cap; the capped logit is kept in units of log2)
    if (CAP) {
      float big = 0.f;
#pragma unroll
      for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
        for (int r = 0; r < 4; ++r) big = fmaxf(big, fabsf(g.acc[mi][ni][r]));
      if (__all(big * inv_cap <= 0.25f)) {
        const float c1 = kLog2e * (-1.f / 3.f) * inv_cap2, c2 = kLog2e * (2.f / 15.f) * inv_cap2 * inv_cap2;
        const float c3 = kLog2e * (-17.f / 315.f) * inv_cap2 * inv_cap2 * inv_cap2;
#pragma unroll
        for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float z = g.acc[mi][ni][r], w = z * z;
            g.acc[mi][ni][r] = z * fmaf(w, fmaf(w, fmaf(w, c3, c2), c1), kLog2e);
          }
      } else {
#pragma unroll
        for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
          for (int r = 0; r < 4; ++r) g.acc[mi][ni][r] = softcap_apply(g.acc[mi][ni][r], p.cap, inv_cap) * kLog2e;
      }
    }
    // an opaque use of the column's 32 accumulators: the register allocator then moves them out of the
    // accumulation registers here, one column at a time, instead of parking some in scratch memory
#pragma unroll
    for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
      for (int r = 0; r < 4; ++r) asm volatile("" : "+v"(g.acc[mi][ni][r]));
    if (tail) {
      asm volatile("");
#pragma unroll
      for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
        for (int r = 0; r < 4; ++r)
          if ((vbase + mi * 16 + r) >= p.V) g.acc[mi][ni][r] = kNegBig;
    }
    // where this lane's eight-entry groups go: token row; lanes of odd 16-lane rows own the second
    // block of a pair, lanes of the upper two rows the upper eight entries of a block
    const bool store = p.zt != nullptr && (t0 + ni * 16) < zt_cols;   // tokens past the live ones are never read
    const uint32_t voff = (uint32_t)((ni * 16 + l15) * ldz2 + (vwave + (lq & 1) * 16 + (lq >> 1) * 8) * 2);
    bool keep = true;
    if (store) keep = mk[ni] != 0.f;                        // rows of masked tokens are not written
    auto group_off = [&](int mp) {      // kOob when the lane's eight entries lie past V (V % 8 == 0)
      return (keep && (vwave + (2 * mp + (lq & 1)) * 16 + (lq >> 1) * 8) < p.V) ? voff : kOob;
    };
    float l = 0.f, s = 0.f;
    if (store) {
#pragma unroll
      for (int mp = 0; mp < G::MI / 2; ++mp) {
        float v[2][4];
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
          for (int r = 0; r < 4; ++r) {
            const float z = g.acc[2 * mp + h][ni][r];                // CAP: t = cap(z) log2(e)
            const float e = __builtin_amdgcn_exp2f(CAP ? z : z * kLog2e);
            l += e;
            s = fmaf(e, z, s);
            v[h][r] = CAP ? e * fmaf(z * z, -kLn2Sq * inv_cap2, 1.f) : e;   // cap' = 1 - (cap(z) / cap)^2
          }
        const uint32_t x0 = pack_bf16(v[0][0], v[0][1]), x1 = pack_bf16(v[0][2], v[0][3]);
        const uint32_t y0 = pack_bf16(v[1][0], v[1][1]), y1 = pack_bf16(v[1][2], v[1][3]);
        // v_permlane16_swap: the first operand of the odd 16-lane rows <-> the second operand of the even ones
        const auto s0 = __builtin_amdgcn_permlane16_swap(x0, y0, false, false);
        const auto s1 = __builtin_amdgcn_permlane16_swap(x1, y1, false, false);
        const u32x4 out = {s0[0], s1[0], s0[1], s1[1]};
        __builtin_amdgcn_raw_buffer_store_b128(out, zrs, group_off(mp), (uint32_t)(mp * 32) * 2, 0);
      }
    } else {
#pragma unroll
      for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float z = g.acc[mi][ni][r];
          const float e = __builtin_amdgcn_exp2f(CAP ? z : z * kLog2e);
          l += e;
          s = fmaf(e, z, s);
        }
    }
    float lt = 0.f;
    if (p.inv_t != 1.f) {
      // the entropy is that of softmax(z / T) (train_modules/__init__.py:136): its own pair of sums,
      // behind a real scalar branch so that the usual T = 1 pays nothing for it
      asm volatile("");
      const float kt = (CAP ? 1.f : kLog2e) * p.inv_t;
      s = 0.f;
#pragma unroll
      for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const float z = g.acc[mi][ni][r];
          const float e = __builtin_amdgcn_exp2f(z * kt);
          lt += e;
          s = fmaf(e, z, s);
        }
      lt = sum_rows16(lt);
    }
    l = sum_rows16(l);
    s = sum_rows16(s);
    if (CAP) s *= kLn2;                      // sum e * cap(z) in natural units
    if (lq == 0) {
      const int64_t o = (int64_t)(tm * 2 + wm) * p.ld_p + col;
      p.pl[o] = l;
      p.ps[o] = s;
      if (p.inv_t != 1.f) p.plt[o] = lt;
    }
    // the sampled token's logit: exactly one lane of one tile holds it
    {
      const int y = tg[ni];
      const int d = y - vwave;                       // row inside the wavefront's 128
      const bool hit = y >= 0 && d >= 0 && d < G::WM && ((d >> 2) & 3) == lq;
      if (__any(hit)) {
        const int flat = (d >> 4) * 4 + (d & 3);     // mi*4 + r
        float zy = 0.f;
#pragma unroll
        for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
          for (int r = 0; r < 4; ++r) zy = (flat == mi * 4 + r) ? g.acc[mi][ni][r] : zy;
        if (hit) p.zy[col] = CAP ? zy * kLn2 : zy;
      }
    }
  }
}

// A thread index that the compiler cannot trace back to threadIdx.x: inside a loop over tiles it
// makes the per-thread address arithmetic of a tile part of that tile's code, so that none of it is
// kept in registers across the previous tile's epilogue (where the 256 accumulators leave no room).
MJ_DEV int opaque_tid() {
  int t = threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

// One workgroup per tile; RESCUE: a small grid that walks the tile list, and leaves at once unless
// the range check of the kStatsExp pass failed (state != 0).
template <int BM, int BN, int MODE, bool RESCUE, bool CAP>
__global__ __launch_bounds__(kThreads) void k_logits_stats(LogitsArgs p, TileMap map) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  int tm, tn, split;
  static_assert(!(RESCUE && MODE == kStatsExp), "the rescue pass is a kStatsMax pass");
  if constexpr (RESCUE) {
    if (__builtin_amdgcn_readfirstlane(*p.state) == 0) return;
    const int items = map.items();
    for (int item = blockIdx.x; item < items; item += gridDim.x) {
      if (map.tile(item, tm, tn, split)) logits_tile<BM, BN, MODE, CAP>(p, tm, tn, smem, opaque_tid());
      __syncthreads();      // the next tile's first LDS writes must not pass this tile's last reads
    }
  } else {
    if (MODE == kStatsExp && blockIdx.x == 0 && threadIdx.x == 0) *p.state = 0;
    if (!map.tile(blockIdx.x, tm, tn, split)) return;
    if constexpr (MODE == kStatsExp) logits_tile16<BM, BN, CAP>(p, tm, tn, smem, threadIdx.x);
    else logits_tile<BM, BN, MODE, CAP>(p, tm, tn, smem, threadIdx.x);
  }
}

// ----------------------------------------------------------------------------- finalize
struct FinalizeArgs {
  const float *pm, *pl, *ps;   // [parts, ld_p]
  const float* plt;            // [parts, ld_p], temperature != 1 only
  float inv_t;
  int64_t ld_p;
  int parts, n, n_pad;         // tokens in chunk, padded count (g is written for all n_pad)
  const float* zy;             // [n] chunk-local
  const float *old_logp, *adv, *mask;   // chunk origin; old_logp may be null
  float eps_low, eps_high, inv_tv, gscale;
  int sft;
  float *logp, *lse, *ent;     // chunk origin outputs (ent may be null)
  float* term;                 // per-token loss term
  float* g;                    // [n_pad] dloss/dlogp * gscale, or null (forward only)
  float ent_coef, inv_ent_cnt; // entropy bonus (0 = off) and its normaliser
  float* eterm;                // per-token share of the masked mean entropy
  float *ge, *hent;            // [n_pad] coef*mask*inv_ent_cnt*gscale and H_t, or null (no bonus / forward only)
  // kStatsExp with a backward: row scale of E and the one-hot patch
  float* rs;                   // [n_pad] -g / sum_v exp(z), or null
  uint16_t* zt;                // E [n, ld_z]
  int64_t ld_z;
  const int32_t* targets;      // chunk origin
  int V;
  float cap;
  int* state;
  int rescue;                  // kStatsMax launched behind a kStatsExp pass: leave unless state != 0
  uint16_t* dead;              // [n_pad / 16] dead-token bits of the chunk (bit set: no gradient), or null
};

// block = (kFinTokens tokens) x (kFinSlices slices of the partial list): few tokens per block keep a
// small chunk spread over many CUs (a 512-token chunk walks 1188 partials per token)
constexpr int kFinTokens = 16, kFinSlices = 64;
template <int MODE>
__global__ __launch_bounds__(kFinTokens * kFinSlices) void k_finalize(FinalizeArgs p) {
  __shared__ float sm[kFinSlices][kFinTokens], sl[kFinSlices][kFinTokens], ss[kFinSlices][kFinTokens], st[kFinSlices][kFinTokens];
  if (MODE == kStatsMax) {
    if (p.rescue) {
      if (__builtin_amdgcn_readfirstlane(*p.state) == 0) return;
    } else if (blockIdx.x == 0 && threadIdx.x == 0) {
      *p.state = 1;            // the 16-bit matrix of this chunk will hold dZ itself
    }
  }
  const int tx = threadIdx.x % kFinTokens, ty = threadIdx.x / kFinTokens;
  const int t = blockIdx.x * kFinTokens + tx;
  const bool tempered = p.inv_t != 1.f;   // then s and lt are sums under softmax(z / T)
  float m = kNegBig, l = 0.f, s = 0.f, lt = 0.f;
  if (t < p.n) {
    for (int q = ty; q < p.parts; q += kFinSlices) {
      const int64_t o = (int64_t)q * p.ld_p + t;
      if (MODE == kStatsExp) {
        l += p.pl[o];
        s += p.ps[o];
        if (tempered) lt += p.plt[o];
      } else {
        const float mq = p.pm[o], lq = p.pl[o], sq = p.ps[o];
        const float mn = fmaxf(m, mq);
        const float a = __expf(m - mn), b = __expf(mq - mn);
        l = l * a + lq * b;
        if (tempered) {
          const float at = __expf((m - mn) * p.inv_t), bt = __expf((mq - mn) * p.inv_t);
          lt = lt * at + p.plt[o] * bt;
          s = s * at + sq * bt;
        } else {
          s = s * a + sq * b;
        }
        m = mn;
      }
    }
  }
  sm[ty][tx] = m; sl[ty][tx] = l; ss[ty][tx] = s; st[ty][tx] = lt;
  __syncthreads();
  if (ty != 0) return;
  bool dead = true;
  if (t >= p.n) {
    if (p.g != nullptr && t < p.n_pad) p.g[t] = 0.f;
    if (p.ge != nullptr && t < p.n_pad) p.ge[t] = 0.f;
    if (MODE == kStatsExp && p.rs != nullptr && t < p.n_pad) p.rs[t] = 0.f;
  } else {
    float M = 0.f, L = 0.f, S = 0.f, LT = 0.f;
    if (MODE == kStatsExp) {
#pragma unroll
      for (int i = 0; i < kFinSlices; ++i) {
        L += sl[i][tx];
        S += ss[i][tx];
        LT += st[i][tx];
      }
      // outside the window (or not finite): the sums cannot be trusted; the kStatsMax pass redoes the chunk
      if (!(L >= kExpSumMin && L <= kExpSumMax)) *p.state = 1;
      if (tempered && !(LT >= kExpSumMin && LT <= kExpSumMax)) *p.state = 1;
    } else {
      M = sm[0][tx];
#pragma unroll
      for (int i = 1; i < kFinSlices; ++i) M = fmaxf(M, sm[i][tx]);
#pragma unroll
      for (int i = 0; i < kFinSlices; ++i) {
        const float w = __expf(sm[i][tx] - M);
        const float wt = tempered ? __expf((sm[i][tx] - M) * p.inv_t) : w;
        L += sl[i][tx] * w;
        S += ss[i][tx] * wt;
        LT += st[i][tx] * wt;
      }
    }
    const float lse = M + __logf(L);
    const float zy = p.zy[t];
    const float logp = (zy - lse) * p.inv_t;     // division after the log-softmax (:124-126)
    p.lse[t] = lse;
    p.logp[t] = logp;
    // entropy of softmax(z / T): log sum e^(z/T) - sum p z / T  (reference adds 1e-9 inside the log)
    const float H = tempered ? (M * p.inv_t + __logf(LT)) - (S / LT) * p.inv_t : lse - S / L;
    if (p.ent != nullptr) p.ent[t] = H;
    const float mk = p.mask[t];
    p.eterm[t] = H * mk * p.inv_ent_cnt;
    float ge = 0.f;
    if (p.ge != nullptr) {
      ge = p.ent_coef * mk * p.inv_ent_cnt * p.gscale;
      p.ge[t] = ge;
      p.hent[t] = H;
    }
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
    g *= p.gscale * p.inv_t;                     // dlogp/dz = (onehot - softmax(z)) / T
    if (p.g != nullptr) p.g[t] = g;
    // a row takes part in the backward products unless its whole gradient is zero; a masked token is
    // always dead (its row of the 16-bit matrix was not even written), whatever g evaluates to
    dead = mk == 0.f || (!(g != 0.f) && !(ge != 0.f));
    if (MODE == kStatsExp && p.rs != nullptr) {
      // dZ[t, v] = g (onehot - e_v / L) cap'_v = (-g / L) (E[t, v] - onehot * L * cap'_y)
      p.rs[t] = -g / L;
      if (mk != 0.f) {                           // rows of masked tokens do not exist
        const int y = clamp_target(p.targets[t], p.V);
        const float capf = p.cap > 0.f ? 1.f - (zy / p.cap) * (zy / p.cap) : 1.f;
        p.zt[(int64_t)t * p.ld_z + y] = f32_to_bf16((__builtin_amdgcn_exp2f(zy * kLog2e) - L) * capf);
      }
    }
  }
  if (p.dead != nullptr) {
    // the 16 finalising threads are lanes 0..15 of the block's first wavefront
    const uint64_t bits = __ballot(dead);
    if (tx == 0) p.dead[blockIdx.x] = (uint16_t)bits;
  }
}

// The token-side operand of the dW product, k-contiguous: ht[h, t] = c_t * hidden[t, h] as a
// [H, n_pad] bf16 matrix, c_t = rs[t] while the 16-bit matrix holds E and 1 once it holds dZ; zeros
// for t >= n.  One workgroup transposes 64 tokens x 64 columns through the LDS.
__global__ __launch_bounds__(256) void k_scale_hidden(const uint16_t* hid, int64_t ld_hid, const float* rs,
                                                  const int* state, int n, int n_pad, int H, uint16_t* ht) {
  __shared__ uint16_t tile[64][72];            // [token][column]; 144-byte rows keep the 16-byte writes aligned
  const int t0 = blockIdx.x * 64, h0 = blockIdx.y * 64;
  const bool scaled = *state == 0;
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int id = threadIdx.x + 256 * i, row = id >> 3, c = (id & 7) * 8;
    const int t = t0 + row;
    u32x4 out = {0u, 0u, 0u, 0u};
    if (t < n && h0 + c < H) {
      const float r = scaled ? rs[t] : 1.f;
      const u32x4 in = *(const u32x4*)(hid + (int64_t)t * ld_hid + h0 + c);
#pragma unroll
      for (int j = 0; j < 4; ++j)
        out[j] = pack_bf16(r * __uint_as_float(in[j] << 16), r * __uint_as_float(in[j] & 0xffff0000u));
    }
    *(u32x4*)&tile[row][c] = out;
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int id = threadIdx.x + 256 * i, h = id >> 3, c = (id & 7) * 8;
    if (h0 + h >= H) continue;
    u32x4 out;
#pragma unroll
    for (int j = 0; j < 4; ++j) out[j] = (uint32_t)tile[c + 2 * j][h] | ((uint32_t)tile[c + 2 * j + 1][h] << 16);
    *(u32x4*)(ht + (int64_t)(h0 + h) * n_pad + t0 + c) = out;
  }
}

// dloss/dlogp from a saved forward (separate backward entry point)
__global__ __launch_bounds__(256) void k_coeff_from_saved(const float* logp, const float* old_logp,
                                                          const float* adv, const float* mask, int n,
                                                          int n_pad, float eps_low, float eps_high,
                                                          float inv_tv, float gscale, int sft, float* g,
                                                          uint64_t* dead) {
  // gscale carries 1 / temperature as well (see k_finalize); n_pad is a multiple of 256 = the block
  const int t = blockIdx.x * 256 + threadIdx.x;
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
  out *= gscale;
  g[t] = out;
  const uint64_t bits = __ballot(!(out != 0.f));      // the epilogue stores the rows with g != 0
  if ((threadIdx.x & 63) == 0) dead[t >> 6] = bits;
}

// kStatsGrad: the sampled token's entry of dZ, g (1 - p_y) cap'_y, replaces the -g p_y cap'_y the
// epilogue wrote there; marks the 16-bit matrix as dZ.
__global__ __launch_bounds__(256) void k_patch_grad(uint16_t* zt, int64_t ld_z, const float* zy, const float* lse,
                                                    const float* g, const int32_t* targets, int n, int V, float cap,
                                                    int* state) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t == 0) *state = 1;
  if (t >= n) return;
  const float gt = g[t];
  if (gt == 0.f) return;                        // the row is all zeros
  const float z = zy[t];
  const float capf = cap > 0.f ? 1.f - (z / cap) * (z / cap) : 1.f;
  zt[(int64_t)t * ld_z + clamp_target(targets[t], V)] = f32_to_bf16(gt * (1.f - __expf(z - lse[t])) * capf);
}

// Deterministic single-workgroup sums: loss[1] = masked mean entropy, loss[0] = sum of the
// per-token policy terms - ent_coef * loss[1].
__global__ __launch_bounds__(1024) void k_reduce_loss(const float* term, const float* eterm, int n,
                                                      float ent_coef, float* loss) {
  __shared__ float sh[1024], se[1024];
  float a = 0.f, e = 0.f;
  for (int i = threadIdx.x; i < n; i += 1024) {
    a += term[i];
    e += eterm[i];
  }
  sh[threadIdx.x] = a;
  se[threadIdx.x] = e;
  __syncthreads();
  for (int o = 512; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) {
      sh[threadIdx.x] += sh[threadIdx.x + o];
      se[threadIdx.x] += se[threadIdx.x + o];
    }
    __syncthreads();
  }
  if (threadIdx.x == 0) {
    loss[0] = sh[0] - ent_coef * se[0];
    loss[1] = se[0];
  }
}

// ----------------------------------------------------------------------------- dZ
struct DzArgs {
  uint16_t* zt;        // [n, ld_z] in: capped logits (half); out: dZ (bf16)
  int64_t ld_z;
  const float *lse, *g;    // chunk-local (lse valid for t < n, g for t < n_pad)
  const float *ge, *hent;  // chunk-local entropy-bonus coefficient and H_t, or null
  const int32_t* targets;  // chunk origin
  const float* mask;       // chunk origin
  int V, n;
  float cap;
  const int* n_live;   // see live_pad
  int c0;
  const int* state;
  int rescue;          // launched behind a kStatsExp pass: leave unless state != 0
};

// Streaming, in place, after a kStatsMax pass.  A workgroup takes whole token rows: the per-token
// constants are loaded once, every thread moves 16 bytes per step and the 256 threads cover 4 KB
// of the row at a time.
__global__ __launch_bounds__(256) void k_dz(DzArgs p) {
  if (p.rescue && __builtin_amdgcn_readfirstlane(*p.state) == 0) return;
  const int lim = min(p.n, live_pad(p.n_live, p.c0, (p.n + 255) & ~255));
  const float inv_cap2 = p.cap > 0.f ? 1.f / (p.cap * p.cap) : 0.f;
  const bool bonus = p.ge != nullptr;
  for (int t = blockIdx.x; t < lim; t += gridDim.x) {
    const float lse = p.lse[t] * kLog2e, g = p.g[t];
    const float ge = bonus ? p.ge[t] : 0.f, hent = bonus ? p.hent[t] : 0.f;
    const int y = clamp_target(p.targets[t], p.V);
    // a token without a gradient: the backward products do not read its row (dead-token bits)
    if (p.mask[t] == 0.f || (!(g != 0.f) && !(ge != 0.f))) continue;
    uint16_t* row = p.zt + (int64_t)t * p.ld_z;
    for (int v0 = threadIdx.x * 8; v0 < p.V; v0 += 256 * 8) {
      u32x4 out = {0u, 0u, 0u, 0u};
      {
        const u32x4 in = *(const u32x4*)(row + v0);
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const uint32_t w = in[i >> 1];
          const float z = f16_bits_to_f32((uint16_t)((i & 1) ? (w >> 16) : (w & 0xffffu)));
          const float t2 = fmaf(z, kLog2e, -lse);          // log2 p
          const float pr = __builtin_amdgcn_exp2f(t2);
          float d = (v0 + i == y) ? 1.f - pr : -pr;
          d *= g;
          if (bonus) d = fmaf(ge * pr, fmaf(t2, 0.6931471805599453f, hent), d);   // coef * p * (log p + H)
          if (p.cap > 0.f) d *= 1.f - z * z * inv_cap2;
          const uint32_t b = f32_to_bf16(d);
          if (i & 1) out[i >> 1] |= b << 16; else out[i >> 1] = b;
        }
      }
      *(u32x4*)(row + v0) = out;
    }
  }
}

// ----------------------------------------------------------------------------- backward products
struct DhArgs {
  const __bf16* dzt;  // [n, ld_z] E or dZ of the chunk (see StatsMode)
  const __bf16* w;    // [H, ld_w]
  int64_t ld_z, ld_w;
  int n, n_pad, H, V;
  int splits, k_per_split;   // vocab range of split s: [s*k_per_split, min(V, (s+1)*k_per_split))
  uint16_t* dh;       // chunk origin [n, ld_dh] bf16 (splits == 1)
  int64_t ld_dh;
  float* part;        // [splits, n_pad, H] fp32 partial sums (splits > 1)
  const int* n_live;  // see live_pad
  int c0;
  const float* rs;    // [n_pad] row scale, applied when state == 0
  const int* state;
  const float *dv, *wv;   // value head (PPO critic): d_hidden[t, :] += dv[t] * wv[:]; both null = none
  const uint64_t* dead;   // [n_pad / 64] dead-token bits of the chunk
};

template <int BM, int BN>
__global__ __launch_bounds__(kThreads) void k_dhidden(DhArgs p, TileMap map) {
  using G = GemmTN16<BM, BN, kRowK, kRowK, true, false>;   // rows of dead tokens are not fetched
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const TileMap live(live_pad(p.n_live, p.c0, p.n_pad) / BM, map.tiles_n, map.n_first, map.lgm, map.splits, map.lgs);
  int tm, tn, split;
  if (!live.tile(blockIdx.x, tm, tn, split)) return;
  const int m0 = tm * BM, n0 = tn * BN;
  const int k0 = split * p.k_per_split;
  const int klen = min(p.V - k0, p.k_per_split);
  G g;
  g.run(p.dzt + (int64_t)m0 * p.ld_z + k0, p.n - m0, p.ld_z, p.w + (int64_t)n0 * p.ld_w + k0, p.H - n0, p.ld_w,
        klen, smem, threadIdx.x, p.dead + m0 / 64);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave & 1, wn = wave >> 1, l15 = lane & 15, lq = lane >> 4;
  const int row0 = m0 + wm * G::WM;
  const int rows = min(max(p.n - row0, 0), G::WM);
  if (p.splits == 1) {
    const bool scaled = __builtin_amdgcn_readfirstlane(*p.state) == 0;
    const uint32_t ld2 = (uint32_t)p.ld_dh * 2;
    const __amdgpu_buffer_rsrc_t rs = make_rsrc_wave(p.dh + (int64_t)row0 * p.ld_dh, (int64_t)rows * ld2);
    const __amdgpu_buffer_rsrc_t srs = make_rsrc_wave(p.rs + row0, (int64_t)rows * 4);
    const __amdgpu_buffer_rsrc_t dvs = make_rsrc_wave(p.dv == nullptr ? nullptr : p.dv + row0, (int64_t)rows * 4);
#pragma unroll
    for (int mi = 0; mi < G::MI; ++mi) {
      f32x4 sc = {1.f, 1.f, 1.f, 1.f}, dvr = {0.f, 0.f, 0.f, 0.f};
      if (scaled) sc = load_b128(srs, (uint32_t)(lq * 16), (uint32_t)(mi * 16) * 4);
      if (p.dv != nullptr) dvr = load_b128(dvs, (uint32_t)(lq * 16), (uint32_t)(mi * 16) * 4);
#pragma unroll
      for (int ni = 0; ni < G::NI; ++ni) {
        const int col = n0 + wn * G::WN + ni * 16 + l15;
        const uint32_t voff = col < p.H ? (uint32_t)(lq * 4 * ld2 + col * 2) : kOob;
        const float wvc = (p.dv != nullptr && col < p.H) ? p.wv[col] : 0.f;
#pragma unroll
        for (int j = 0; j < 4; ++j)
          store_b16(f32_to_bf16(fmaf(dvr[j], wvc, g.acc[mi][ni][j] * sc[j])), rs, voff, (uint32_t)(mi * 16 + j) * ld2);
      }
    }
  } else {
    const uint32_t ld4 = (uint32_t)p.H * 4;
    const __amdgpu_buffer_rsrc_t rs =
        make_rsrc_wave(p.part + ((int64_t)split * p.n_pad + row0) * p.H, (int64_t)rows * ld4);
#pragma unroll
    for (int ni = 0; ni < G::NI; ++ni) {
      const int col = n0 + wn * G::WN + ni * 16 + l15;
      const uint32_t voff = col < p.H ? (uint32_t)(lq * 4 * ld4 + col * 4) : kOob;
#pragma unroll
      for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
        for (int r = 0; r < 4; ++r) store_b32(g.acc[mi][ni][r], rs, voff, (uint32_t)(mi * 16 + r) * ld4);
    }
  }
}

// dh[row, :] = bf16(scale * sum over splits of part[s, row, :] + dv[row] * wv[:]), fixed order;
// scale = rs[row] when the 16-bit matrix held E (state == 0), else 1.
__global__ __launch_bounds__(256) void k_dhidden_reduce(const float* part, int splits, int n, int n_pad, int H,
                                                        uint16_t* dh, int64_t ld_dh, const float* rs,
                                                        const int* state, const float* dv, const float* wv) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;   // one thread = 4 columns
  const int h4 = H / 4;
  if (i >= (int64_t)n * h4) return;
  const int row = (int)(i / h4), c = (int)(i % h4) * 4;
  f32x4 a = *(const f32x4*)(part + (int64_t)row * H + c);
  for (int s = 1; s < splits; ++s) a += *(const f32x4*)(part + ((int64_t)s * n_pad + row) * H + c);
  if (*state == 0) a *= rs[row];
  if (dv != nullptr) a += dv[row] * *(const f32x4*)(wv + c);       // value head: + dv[t] * wv[:]
  uint16_t* o = dh + (int64_t)row * ld_dh + c;
  const uint32_t lo = f32_to_bf16(a[0]) | ((uint32_t)f32_to_bf16(a[1]) << 16);
  const uint32_t hi = f32_to_bf16(a[2]) | ((uint32_t)f32_to_bf16(a[3]) << 16);
  *(uint2*)o = make_uint2(lo, hi);
}

struct DwArgs {
  const __bf16* dzt;   // [n, ld_z] E or dZ of the chunk
  const __bf16* ht;    // [H, n_pad]: k_scale_hidden's matrix, the token-side operand
  int64_t ld_z;
  int H, V, n;         // n = tokens of the chunk
  void* dw;            // [H, ld_dw]: f32, or bf16 in the BF16OUT kernel
  int64_t ld_dw;
  int accumulate;
  const int* n_live;   // see live_pad
  int c0;
  const uint64_t* dead;   // [n_pad / 64] dead-token bits of the chunk
};

// Tile of dW^T: rows = vocab (MFMA row direction), columns = hidden (lanes), on the chained
// 16 x 16 x 32 engine (GemmTN16).  The token-side operand is k_scale_hidden's [H, n_pad] matrix, so
// only E / dZ (token-major in memory) goes through the transposing LDS read; the token rows of dead
// tokens are not fetched.  A lane's four accumulator rows of a block are four consecutive entries of
// one dW row: one 16-byte access per block in float32; in bf16 the lanes l and l + 16 exchange, two
// blocks at a time, so that each owns eight consecutive entries (an accumulating call adds in fp32
// and rounds once).
template <int BM, int BN, bool BF16OUT>
__global__ __launch_bounds__(kThreads) void k_dw(DwArgs p, TileMap map) {
  using G = GemmTN16<BM, BN, kKRow, kRowK, true, false>;
  extern __shared__ __attribute__((aligned(16))) char smem[];
  int tm, tn, split;
  if (!map.tile(blockIdx.x, tm, tn, split)) return;
  const int m0 = tm * BM, n0 = tn * BN;
  G g;
  const int n_pad = (p.n + 255) & ~255;
  const int kn = min(p.n, live_pad(p.n_live, p.c0, n_pad));   // tokens past the live ones have dZ = 0
  g.run(p.dzt + m0, p.V - m0, p.ld_z, p.ht + (int64_t)n0 * n_pad, p.H - n0, n_pad, kn, smem, threadIdx.x, p.dead);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);   // wave-uniform: keeps descriptors in SGPRs
  const int wm = wave & 1, wn = wave >> 1, l15 = lane & 15, lq = lane >> 4;
  const int h0 = n0 + wn * G::WN, v0 = m0 + wm * G::WM;
  const int hrows = min(max(p.H - h0, 0), G::WN);
  const int vleft = p.V - v0;                            // V % 8 == 0: groups of 4 or 8 are in or out together
  if (BF16OUT) {
    const uint32_t ld2 = (uint32_t)p.ld_dw * 2;
    const __amdgpu_buffer_rsrc_t rs =
        make_rsrc_wave((uint16_t*)p.dw + (int64_t)h0 * p.ld_dw + v0, (int64_t)hrows * ld2 - (int64_t)v0 * 2);
    const int vlane = (lq & 1) * 16 + (lq >> 1) * 8;     // the lane's eight entries of a block pair's 32
#pragma unroll
    for (int ni = 0; ni < G::NI; ++ni) {
      const uint32_t lane_off = (uint32_t)((ni * 16 + l15) * ld2 + vlane * 2);
      u32x4 old[G::MI / 2];
      if (p.accumulate) {                     // all loads of this column of blocks before its first store
#pragma unroll
        for (int mp = 0; mp < G::MI / 2; ++mp)
          old[mp] = __builtin_amdgcn_raw_buffer_load_b128(rs, (mp * 32 + vlane) < vleft ? lane_off : kOob,
                                                          (uint32_t)(mp * 32) * 2, 0);
      }
#pragma unroll
      for (int mp = 0; mp < G::MI / 2; ++mp) {
        float v[8];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          // v_permlane16_swap: the first operand of the odd 16-lane rows <-> the second operand of the even ones
          const auto sw = __builtin_amdgcn_permlane16_swap(__float_as_uint(g.acc[2 * mp][ni][r]),
                                                           __float_as_uint(g.acc[2 * mp + 1][ni][r]), false, false);
          v[r] = __uint_as_float(sw[0]);
          v[4 + r] = __uint_as_float(sw[1]);
        }
        if (p.accumulate) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            v[2 * j] += __uint_as_float(old[mp][j] << 16);
            v[2 * j + 1] += __uint_as_float(old[mp][j] & 0xffff0000u);
          }
        }
        const u32x4 out = {pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
        __builtin_amdgcn_raw_buffer_store_b128(out, rs, (mp * 32 + vlane) < vleft ? lane_off : kOob,
                                               (uint32_t)(mp * 32) * 2, 0);
      }
    }
    return;
  }
  const uint32_t ld4 = (uint32_t)p.ld_dw * 4;
  const __amdgpu_buffer_rsrc_t rs =
      make_rsrc_wave((float*)p.dw + (int64_t)h0 * p.ld_dw + v0, (int64_t)hrows * ld4 - (int64_t)v0 * 4);
#pragma unroll
  for (int ni = 0; ni < G::NI; ++ni) {
    const uint32_t lane_off = (uint32_t)((ni * 16 + l15) * ld4 + lq * 16);
    // when accumulating, the eight loads of this column of blocks are issued before the first store (a
    // store between two loads would order the second behind it: one memory round trip per 16 bytes)
    f32x4 a[G::MI];
#pragma unroll
    for (int mi = 0; mi < G::MI; ++mi) {
      if (p.accumulate) a[mi] = load_b128(rs, (mi * 16 + lq * 4) < vleft ? lane_off : kOob, (uint32_t)(mi * 16) * 4);
      else a[mi] = f32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int mi = 0; mi < G::MI; ++mi)
      store_b128(g.acc[mi][ni] + a[mi], rs, (mi * 16 + lq * 4) < vleft ? lane_off : kOob, (uint32_t)(mi * 16) * 4);
  }
}

// ----------------------------------------------------------------------------- upstream gradient
// rows x cols elements of a row-major matrix (pitch ld elements) times *scale, in place; every
// workgroup leaves at once when *scale == 1 (the usual case: the loss is what gets differentiated).
// BF16: 16-bit elements (8 per 16-byte unit), else float32 (4 per unit).  cols % 8 == 0.
template <bool BF16>
__global__ __launch_bounds__(256) void k_scale_inplace(void* data, int64_t rows, int64_t cols, int64_t ld,
                                                       const float* scale) {
  const float s = *scale;
  if (s == 1.f) return;
  constexpr int E = BF16 ? 8 : 4;
  const int64_t per_row = cols / E, units = rows * per_row;
  for (int64_t u = (int64_t)blockIdx.x * 256 + threadIdx.x; u < units; u += (int64_t)gridDim.x * 256) {
    const int64_t r = u / per_row, c = (u - r * per_row) * E;
    if (BF16) {
      u32x4* ptr = (u32x4*)((uint16_t*)data + r * ld + c);
      u32x4 v = *ptr;
#pragma unroll
      for (int j = 0; j < 4; ++j)
        v[j] = pack_bf16(s * __uint_as_float(v[j] << 16), s * __uint_as_float(v[j] & 0xffff0000u));
      *ptr = v;
    } else {
      f32x4* ptr = (f32x4*)((float*)data + r * ld + c);
      *ptr = *ptr * s;
    }
  }
}

// ----------------------------------------------------------------------------- per-sequence entropy
// MLLM_JAX/train_modules/__init__.py:141-157 on [b, t] row-major data, one wavefront per sequence:
//   entropy[s]      = sum_t(H * mask) / sum_t(mask)                      (nan for an empty row, as there)
//   entropy_loss[s] = the same mean over the window  mask == 1  and  4 <= cumsum(mask == 1) <= 100
// Lane l owns the l-th contiguous piece of the row, so the running count of valid tokens is a prefix
// sum over lanes.
__global__ __launch_bounds__(256) void k_sequence_entropy(const float* ent, const float* mask, int b, int t,
                                                          float* entropy, float* entropy_loss) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= b) return;
  const float* e = ent + (int64_t)row * t;
  const float* m = mask + (int64_t)row * t;
  const int seg = (t + 63) / 64, i0 = min(lane * seg, t), i1 = min(i0 + seg, t);
  int valid = 0;
  float sum_em = 0.f, sum_m = 0.f;
  for (int i = i0; i < i1; ++i) {
    const float mk = m[i];
    valid += mk == 1.f ? 1 : 0;
    sum_em = fmaf(e[i], mk, sum_em);
    sum_m += mk;
  }
  int before = valid;                                   // inclusive prefix over lanes ...
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int v = __shfl_up(before, o);
    if (lane >= o) before += v;
  }
  int cum = before - valid;                             // ... valid tokens before this lane's piece
  float win_e = 0.f, win_n = 0.f;
  for (int i = i0; i < i1; ++i) {
    if (m[i] == 1.f) {
      ++cum;
      if (cum >= 4 && cum <= 100) { win_e += e[i]; win_n += 1.f; }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    sum_em += __shfl_xor(sum_em, o);
    sum_m += __shfl_xor(sum_m, o);
    win_e += __shfl_xor(win_e, o);
    win_n += __shfl_xor(win_n, o);
  }
  if (lane == 0) {
    entropy[row] = sum_em / sum_m;
    entropy_loss[row] = win_e / win_n;
  }
}

// ----------------------------------------------------------------------------- value head (PPO critic)
// plugins/training/ppo/module.py:34-39, :52 (Dense(1) on the final hidden states) and :104-138 (clipped
// value loss).  values[t] = hidden[t, :] . wv + b: one wavefront per token row, fp32 accumulation.
__global__ __launch_bounds__(256) void k_value_head(const uint16_t* hid, int64_t ld_hid, int n, int H, const float* wv,
                                                    const float* bv, float* values) {
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (row >= n) return;
  const uint16_t* x = hid + (int64_t)row * ld_hid;
  float acc = 0.f;
  for (int c = lane * 8; c < H; c += 512) {
    const u32x4 v = *(const u32x4*)(x + c);
    const f32x4 w0 = *(const f32x4*)(wv + c), w1 = *(const f32x4*)(wv + c + 4);
    acc = fmaf(__uint_as_float(v[0] << 16), w0[0], acc);
    acc = fmaf(__uint_as_float(v[0] & 0xffff0000u), w0[1], acc);
    acc = fmaf(__uint_as_float(v[1] << 16), w0[2], acc);
    acc = fmaf(__uint_as_float(v[1] & 0xffff0000u), w0[3], acc);
    acc = fmaf(__uint_as_float(v[2] << 16), w1[0], acc);
    acc = fmaf(__uint_as_float(v[2] & 0xffff0000u), w1[1], acc);
    acc = fmaf(__uint_as_float(v[3] << 16), w1[2], acc);
    acc = fmaf(__uint_as_float(v[3] & 0xffff0000u), w1[3], acc);
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) acc += __shfl_xor(acc, o);
  if (lane == 0) values[row] = acc + bv[0];
}

struct ValueLossArgs {
  const float *values, *adv, *mask;
  const float *returns;      // or null: advantages + value_pred, NOT detached (module.py:107)
  const float *old_values;   // or null: stop_gradient(value_pred) (:118)
  int n;
  float inv_tv, coef, clip, gscale;
  int use_clip;              // value_clip_range is not None
  float* vterm;              // [n] value_loss_t * mask_t / tvtc
  float* dv;                 // [n] d(coef * value_loss)/d value_pred_t, times gscale
};

// Per token: max((v - R)^2, (old + clip(v - old, +-c) - R)^2) and its derivative with respect to
// v (module.py:131-138).  Where the two arguments of the maximum are equal each gets half of the
// cotangent (lax.max), which matters in the default case R = adv + v, old = v: both are adv^2.
__global__ __launch_bounds__(256) void k_value_loss(ValueLossArgs p) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= p.n) return;
  const float vp = p.values[t], mk = p.mask[t];
  const bool rt_free = p.returns == nullptr;
  const float rt = rt_free ? p.adv[t] + vp : p.returns[t];
  const float ov = p.old_values == nullptr ? vp : p.old_values[t];
  const float a = (vp - rt) * (vp - rt);
  const float da = rt_free ? 0.f : 2.f * (vp - rt);
  float vl = a, dvl = da;
  if (p.use_clip) {
    const float delta = vp - ov;
    const float clipped = ov + fminf(fmaxf(delta, -p.clip), p.clip);
    const float inside = fabsf(delta) <= p.clip ? 1.f : 0.f;
    const float b = (clipped - rt) * (clipped - rt);
    const float db = 2.f * (clipped - rt) * (inside - (rt_free ? 1.f : 0.f));
    vl = fmaxf(a, b);
    dvl = a > b ? da : (a < b ? db : 0.5f * (da + db));
  }
  p.vterm[t] = vl * mk * p.inv_tv;
  p.dv[t] = p.coef * dvl * mk * p.inv_tv * p.gscale;
}

// out[0] = sum of x[0..n), one workgroup, fixed order
__global__ __launch_bounds__(1024) void k_sum(const float* x, int n, float* out) {
  __shared__ float sh[1024];
  float a = 0.f;
  for (int i = threadIdx.x; i < n; i += 1024) a += x[i];
  sh[threadIdx.x] = a;
  __syncthreads();
  for (int o = 512; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) sh[threadIdx.x] += sh[threadIdx.x + o];
    __syncthreads();
  }
  if (threadIdx.x == 0) out[0] = sh[0];
}

// d_wv[c] = sum_t dv[t] * hidden[t, c]: a workgroup adds up kValueRows rows (8 columns per thread,
// rows in order), k_value_wgrad_reduce adds the workgroups' partial rows in fixed order.
constexpr int kValueRows = 64;
__global__ __launch_bounds__(256) void k_value_wgrad(const uint16_t* hid, int64_t ld_hid, int n, int H,
                                                     const float* dv, float* part) {
  const int r0 = blockIdx.x * kValueRows, r1 = min(r0 + kValueRows, n);
  for (int c = threadIdx.x * 8; c < H; c += 2048) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int r = r0; r < r1; ++r) {
      const float d = dv[r];
      const u32x4 v = *(const u32x4*)(hid + (int64_t)r * ld_hid + c);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        acc[2 * j] = fmaf(d, __uint_as_float(v[j] << 16), acc[2 * j]);
        acc[2 * j + 1] = fmaf(d, __uint_as_float(v[j] & 0xffff0000u), acc[2 * j + 1]);
      }
    }
    float* o = part + (int64_t)blockIdx.x * H + c;
    *(f32x4*)o = f32x4{acc[0], acc[1], acc[2], acc[3]};
    *(f32x4*)(o + 4) = f32x4{acc[4], acc[5], acc[6], acc[7]};
  }
}

__global__ __launch_bounds__(256) void k_value_wgrad_reduce(const float* part, int blocks, int H, float* d_wv) {
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= H) return;
  float a = 0.f;
  for (int b = 0; b < blocks; ++b) a += part[(int64_t)b * H + c];
  d_wv[c] = a;
}

// ----------------------------------------------------------------------------- compaction
// Optional: tokens whose gradient is zero by construction (mask 0, or advantage 0 where nothing
// else feeds the gradient) are moved behind the others so that the backward kernels can stop at
// the count of the rest.  perm[j] = original index of the token in slot j; stable on both sides.
struct CompactArgs {
  const float *mask, *adv;   // adv may be null (every unmasked token counts)
  int n;
  int* perm;                 // [n]
  int* n_live;               // [1]
};

__global__ __launch_bounds__(1024) void k_compact_plan(CompactArgs p) {
  __shared__ int cnt[1024];
  const int t = threadIdx.x;
  const int seg = (p.n + 1023) / 1024;
  const int b = min(t * seg, p.n), e = min(b + seg, p.n);
  int c = 0;
  for (int i = b; i < e; ++i) c += (p.mask[i] != 0.f && (p.adv == nullptr || p.adv[i] != 0.f)) ? 1 : 0;
  cnt[t] = c;
  __syncthreads();
  for (int o = 1; o < 1024; o <<= 1) {          // inclusive scan
    const int v = t >= o ? cnt[t - o] : 0;
    __syncthreads();
    cnt[t] += v;
    __syncthreads();
  }
  const int total = cnt[1023];
  int live = cnt[t] - c;                        // live tokens before this segment
  int dead = total + (b - live);                // slot of this segment's first dead token
  for (int i = b; i < e; ++i) {
    const bool ok = p.mask[i] != 0.f && (p.adv == nullptr || p.adv[i] != 0.f);
    if (ok) p.perm[live++] = i; else p.perm[dead++] = i;
  }
  if (t == 0) p.n_live[0] = total;
}

struct GatherArgs {
  const int* perm;
  int n, H;
  const uint16_t* hid; int64_t ld_hid;     // [n, ld_hid] -> hid_p [n, H]
  uint16_t* hid_p;
  const int32_t* tgt; int32_t* tgt_p;
  const float *f_in[6];                    // old_logp, adv, mask, saved_lse, saved_logp, dv (any may be null)
  float* f_out[6];
};

// one workgroup per slot: copies the token's hidden row (16 bytes per thread and step) and scalars
__global__ __launch_bounds__(256) void k_gather_tokens(GatherArgs p) {
  const int j = blockIdx.x, src = p.perm[j];
  const u32x4* in = (const u32x4*)(p.hid + (int64_t)src * p.ld_hid);
  u32x4* out = (u32x4*)(p.hid_p + (int64_t)j * p.H);
  for (int c = threadIdx.x; c < (p.H >> 3); c += 256) out[c] = in[c];
  if (threadIdx.x == 0) p.tgt_p[j] = p.tgt[src];
  if (threadIdx.x < 6 && p.f_in[threadIdx.x] != nullptr) p.f_out[threadIdx.x][j] = p.f_in[threadIdx.x][src];
}

struct ScatterArgs {
  const int* perm;
  const int* n_live;
  int n, H;
  const float* f_in[3];                    // logp, lse, entropy in slot order (any may be null)
  float* f_out[3];
  const uint16_t* dh_p;                    // [n, H] slot order, or null (no backward)
  uint16_t* dh; int64_t ld_dh;
};

// inverse of the gather for the outputs; tokens behind the live ones get a zero d_hidden row
__global__ __launch_bounds__(256) void k_scatter_tokens(ScatterArgs p) {
  const int j = blockIdx.x, dst = p.perm[j];
  if (threadIdx.x < 3 && p.f_in[threadIdx.x] != nullptr) p.f_out[threadIdx.x][dst] = p.f_in[threadIdx.x][j];
  if (p.dh_p == nullptr) return;
  const bool live = j < *p.n_live;
  const u32x4* in = (const u32x4*)(p.dh_p + (int64_t)j * p.H);
  u32x4* out = (u32x4*)(p.dh + (int64_t)dst * p.ld_dh);
  for (int c = threadIdx.x; c < (p.H >> 3); c += 256) out[c] = live ? in[c] : u32x4{0u, 0u, 0u, 0u};
}

// ----------------------------------------------------------------------------- sampling
// Last-position logits for the sampler, float32 row-major [n, ld_out]: same product as
// k_logits_stats (W read in place as the row operand), plain store epilogue -- a lane's four
// consecutive accumulator rows are four consecutive vocab entries of its token's row.
struct LogitsRowsArgs {
  const __bf16* w;       // lm_head [H, ld_w]
  const __bf16* hid;     // [n, ld_hid]
  int64_t ld_w, ld_hid;
  int V, n, H;
  float cap;             // final-logit softcap, 0 = off
  float* out;            // [n, ld_out]
  int64_t ld_out;
  int tile_rows;         // vocab columns per work item: a multiple of 8, <= BM
};

// A decode batch is a few rows against the whole vocabulary matrix: the product is bound by reading
// W once.  BN follows the batch (128 or 256 rows, so the MFMA work per slice does not outlast its
// loads) and a work item covers `tile_rows` <= BM vocab columns, chosen on the host so that the
// items fill whole rounds of the resident workgroups; the columns of the 256-wide tile past
// tile_rows are neither loaded (the operand's row limit) nor stored.
template <int BM, int BN>
__global__ __launch_bounds__(kThreads) void k_logits_rows(LogitsRowsArgs p, TileMap map) {
  using G = GemmTN<BM, BN, kKRow, kRowK, (BN < 256 ? 2 : 1)>;   // the narrow tiles wait on memory: three slices in flight
  extern __shared__ __attribute__((aligned(16))) char smem[];
  int tm, tn, split;
  if (!map.tile(blockIdx.x, tm, tn, split)) return;
  const int m0 = tm * p.tile_rows, n0 = tn * BN;
  const int m1 = min(p.V, m0 + p.tile_rows);
  G g;
  g.run(p.w + m0, m1 - m0, p.ld_w, p.hid + (int64_t)n0 * p.ld_hid, p.n - n0, p.ld_hid, p.H, smem);
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wm = wave & 1, wn = wave >> 1, l31 = lane & 31, lhi = lane >> 5;
  const int t0 = n0 + wn * G::WN, v0 = m0 + wm * G::WM;
  const int trows = min(max(p.n - t0, 0), G::WN);
  const uint32_t ld4 = (uint32_t)p.ld_out * 4;
  const __amdgpu_buffer_rsrc_t rs = make_rsrc_wave(p.out + (int64_t)t0 * p.ld_out + v0, (int64_t)trows * ld4 - (int64_t)v0 * 4);
  const int vleft = m1 - v0;             // columns of this work item from the wavefront's first on (may be <= 0)
  const float inv_cap = p.cap > 0.f ? 1.f / p.cap : 0.f;
#pragma unroll
  for (int ni = 0; ni < G::NI; ++ni) {
    const uint32_t lane_off = (uint32_t)((ni * 32 + l31) * ld4 + lhi * 16);
#pragma unroll
    for (int mi = 0; mi < G::MI; ++mi)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int vv = mi * 32 + q * 8;
        const uint32_t voff = (vv + lhi * 4) < vleft ? lane_off : kOob;
        f32x4 a = {g.acc[mi][ni][q * 4], g.acc[mi][ni][q * 4 + 1], g.acc[mi][ni][q * 4 + 2], g.acc[mi][ni][q * 4 + 3]};
        if (p.cap > 0.f) {
#pragma unroll
          for (int j = 0; j < 4; ++j) a[j] = softcap_apply(a[j], p.cap, inv_cap);
        }
        store_b128(a, rs, voff, (uint32_t)vv * 4);
      }
  }
}

// Top-k + categorical draw per row (MLLM_JAX/sample/sanple_utils.py:35-53): the k largest of
// logits / t in the IEEE total order (-0 below +0, NaN largest, as XLA's sort comparators order
// floats; ties: lower index first, like jax.lax.top_k), then argmax_j(top_j + noise_j) where
// noise holds the caller's Gumbel samples -- what jax.random.categorical evaluates.  One
// workgroup per row: an 8-bit-per-pass radix select over order-preserving keys finds the k-th
// largest key, elements above it are collected in any order, elements equal to it in index order.
constexpr int kTopKMax = 64;
struct TopKArgs {
  const float* logits;   // [b, ld]
  int64_t ld;
  int V, k;
  float t;                // temperature: keys are logits / t (MLLM_JAX/sample/sanple_utils.py:37)
  const float* noise;    // [b, k] or null (greedy: the largest)
  int32_t* token;        // [b]
  int32_t* top_idx;      // [b, k] or null
  float* top_val;        // [b, k] or null (logits / t, descending)
};

MJ_DEV uint32_t topk_key(float f) {   // larger float <=> larger key; -0 and +0 differ only in sign bit order
  const uint32_t u = __float_as_uint(f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}

MJ_DEV float topk_unkey(uint32_t key) {
  return __uint_as_float((key & 0x80000000u) ? (key ^ 0x80000000u) : ~key);
}

constexpr int kTopKPool = 4096;

__global__ __launch_bounds__(1024) void k_topk_sample(TopKArgs p) {
  __shared__ __attribute__((aligned(16))) uint32_t hist[4096];
  uint64_t* ranked_word = (uint64_t*)hist;      // the common path's pool; the histogram paths start by clearing hist
  __shared__ uint32_t pool_key[kTopKPool];
  __shared__ int pool_idx[kTopKPool];
  __shared__ uint32_t s_scan[1024];
  __shared__ uint32_t s_prefix, s_need, s_cnt, s_pool, s_wave[16], s_base;
  __shared__ float s_gmax[64];
  __shared__ float c_val[kTopKMax], o_val[kTopKMax];
  __shared__ int c_idx[kTopKMax], o_idx[kTopKMax];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const float* row = p.logits + (int64_t)blockIdx.x * p.ld;

  // Walks the row once, 16 bytes per lane where the row's address allows it, eight loads in flight
  // per lane (the row comes from L2 or beyond: latency, not bandwidth, is what one workgroup sees).
  const int v4 = (((uintptr_t)row & 15) == 0) ? (p.V & ~3) : 0;
  auto for_each = [&](auto&& f) {
    constexpr int U = 8;
    int i = tid * 4;
    for (; i + (U - 1) * 4096 < v4; i += U * 4096) {
      f32x4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = *(const f32x4*)(row + i + u * 4096);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int j = i + u * 4096;
        f(j, x[u][0]); f(j + 1, x[u][1]); f(j + 2, x[u][2]); f(j + 3, x[u][3]);
      }
    }
    for (; i < v4; i += 4096) {
      const f32x4 x = *(const f32x4*)(row + i);
      f(i, x[0]); f(i + 1, x[1]); f(i + 2, x[2]); f(i + 3, x[3]);
    }
    for (int j = v4 + tid; j < p.V; j += 1024) f(j, row[j]);
  };

  // ---- common case, two reads of the row, no histogram and no division per element.  Threshold:
  // the 1024 threads form 64 groups of 16 lanes; each group's largest logit belongs to some element,
  // so at least 64 >= k elements reach the smallest of the 64 group maxima, `tau` (a group without
  // elements or with nothing but NaNs leaves tau = -inf, and then every element qualifies).
  // x -> key(x / t) is non-decreasing, so the k-th largest key is at least key(tau / t), and an
  // element whose key reaches it has x >= tau up to the rounding of the two quotients: x >= tau_lo,
  // a few ulps below tau.  Second read: elements that are not below tau_lo (NaNs included: their key
  // is the largest) go to a pool with their exact keys -- a few hundred for logits of a language
  // model -- where each one's rank under (key descending, index ascending) is counted directly.
  // A pool that overflows (rows of near-equal values) takes the histogram paths below instead.
  constexpr int kRankPool = 1024;
  if (tid == 0) s_pool = 0;
  float mx = -__builtin_inff();
  for_each([&](int, float x) { mx = fmaxf(mx, x); });
#pragma unroll
  for (int o = 1; o < 16; o <<= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
  if ((lane & 15) == 0) s_gmax[wave * 4 + (lane >> 4)] = mx;
  __syncthreads();
  float tau = s_gmax[lane];
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) tau = fminf(tau, __shfl_xor(tau, o));
  const float tau_lo = tau - fmaxf(fabsf(tau) * 0x1p-20f, 0x1p-100f);
  for_each([&](int i, float x) {
    if (!(x < tau_lo)) {
      const uint32_t slot = atomicAdd(&s_pool, 1u);
      // one 64-bit word per element whose order is (key descending, index ascending); never 0
      if (slot < (uint32_t)kRankPool) ranked_word[slot] = ((uint64_t)topk_key(x / p.t) << 32) | (uint32_t)~i;
    }
  });
  __syncthreads();
  const uint32_t ranked = s_pool;
  __syncthreads();                       // every thread has read s_pool before the paths below reset it
  if (ranked <= (uint32_t)kRankPool) {
    const uint32_t padded = (ranked + 7u) & ~7u;              // zeros behind the pool: smaller than any word
    if ((uint32_t)tid >= ranked && (uint32_t)tid < padded) ranked_word[tid] = 0;
    __syncthreads();
    if ((uint32_t)tid < ranked) {
      const uint64_t mine = ranked_word[tid];
      int rank = 0;
      for (uint32_t r = 0; r < padded; r += 8) {              // eight LDS reads in flight, not one
        uint64_t w[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) w[j] = ranked_word[r + j];
#pragma unroll
        for (int j = 0; j < 8; ++j) rank += w[j] > mine ? 1 : 0;
      }
      // the rank is the final position: (key descending, index ascending) is the order of the result
      if (rank < p.k) { o_val[rank] = topk_unkey((uint32_t)(mine >> 32)); o_idx[rank] = (int)~(uint32_t)mine; }
    }
  } else {
  // ---- two reads of the row with a 12-bit histogram: finds the bin of the k-th largest
  // key; a second read sends larger keys straight to the result and the bin's keys to an LDS pool,
  // where the selection finishes.  A bin that overflows the pool (many near-equal logits) falls
  // back to the byte-wise select below.
  for (int b = tid; b < 4096; b += 1024) hist[b] = 0;
  if (tid == 0) { s_cnt = 0; s_pool = 0; s_base = 0; }
  __syncthreads();
  for (int i = tid; i < p.V; i += 1024) atomicAdd(&hist[topk_key(row[i] / p.t) >> 20], 1u);
  __syncthreads();
  {
    // suffix sums over the bins, four bins per thread (thread t owns bins 4t .. 4t+3)
    const uint32_t mine = hist[4 * tid] + hist[4 * tid + 1] + hist[4 * tid + 2] + hist[4 * tid + 3];
    s_scan[tid] = mine;
    __syncthreads();
    for (int o = 1; o < 1024; o <<= 1) {
      const uint32_t v = tid + o < 1024 ? s_scan[tid + o] : 0u;
      __syncthreads();
      s_scan[tid] += v;
      __syncthreads();
    }
    const uint32_t incl = s_scan[tid], excl = incl - mine;       // keys in bins >= 4t, and in bins > 4t+3
    if (excl < (uint32_t)p.k && incl >= (uint32_t)p.k) {         // exactly one thread
      uint32_t acc = excl;
      int bin = 4 * tid + 3;
      for (; bin > 4 * tid; --bin) {
        if (acc + hist[bin] >= (uint32_t)p.k) break;
        acc += hist[bin];
      }
      s_prefix = (uint32_t)bin;            // 12-bit bin of the k-th largest
      s_need = (uint32_t)p.k - acc;        // how many of that bin's keys belong to the top k
    }
    __syncthreads();
  }
  const uint32_t bin12 = s_prefix;
  uint32_t need = s_need;
  for (int i = tid; i < p.V; i += 1024) {
    const float v = row[i] / p.t;
    const uint32_t key = topk_key(v), hi = key >> 20;
    if (hi > bin12) {
      const uint32_t slot = atomicAdd(&s_cnt, 1u);
      c_val[slot] = v;
      c_idx[slot] = i;
    } else if (hi == bin12) {
      const uint32_t slot = atomicAdd(&s_pool, 1u);
      if (slot < (uint32_t)kTopKPool) { pool_key[slot] = key; pool_idx[slot] = i; }
    }
  }
  __syncthreads();
  const uint32_t pooled = s_pool;
  if (pooled <= (uint32_t)kTopKPool) {
    // the low 20 bits of the k-th largest key, 10 bits at a time, over the pool
    uint32_t prefix = bin12 << 20;
    for (int pass = 0; pass < 2; ++pass) {
      const int shift = 10 - 10 * pass;
      hist[tid] = 0;
      __syncthreads();
      const uint32_t hi_mask = 0xffffffffu << (shift + 10);
      for (uint32_t q = tid; q < pooled; q += 1024) {
        const uint32_t key = pool_key[q];
        if ((key & hi_mask) == prefix) atomicAdd(&hist[(key >> shift) & 1023u], 1u);
      }
      __syncthreads();
      {
        // suffix sums over the 1024 bins, one per thread: the bin where they cross `need`
        const uint32_t mine = hist[tid];
        s_scan[tid] = mine;
        __syncthreads();
        for (int o = 1; o < 1024; o <<= 1) {
          const uint32_t v = tid + o < 1024 ? s_scan[tid + o] : 0u;
          __syncthreads();
          s_scan[tid] += v;
          __syncthreads();
        }
        const uint32_t incl = s_scan[tid], excl = incl - mine;
        if (excl < need && incl >= need) {
          s_prefix = prefix | ((uint32_t)tid << shift);
          s_need = need - excl;
        }
        __syncthreads();
      }
      prefix = s_prefix;
      need = s_need;
      __syncthreads();
    }
    // pool keys above the threshold in any order; equal keys by ascending index
    const uint32_t above = s_cnt;
    __syncthreads();
    if (tid == 0) s_cnt = above + need;            // slots [above, above + need) belong to the equal keys
    __syncthreads();
    for (uint32_t q = tid; q < pooled; q += 1024) {
      const uint32_t key = pool_key[q];
      if (key > prefix) {
        const uint32_t slot = atomicAdd(&s_cnt, 1u);
        c_val[slot] = topk_unkey(key);
        c_idx[slot] = pool_idx[q];
      } else if (key == prefix) {
        const int ix = pool_idx[q];
        uint32_t rank = 0;
        for (uint32_t r = 0; r < pooled; ++r) rank += (pool_key[r] == prefix && pool_idx[r] < ix) ? 1u : 0u;
        if (rank < need) { c_val[above + rank] = topk_unkey(key); c_idx[above + rank] = ix; }
      }
    }
    __syncthreads();
  } else {
  // ---- fallback: the k-th largest key, most significant byte first, over the whole row
  uint32_t prefix = 0;
  need = (uint32_t)p.k;   // `need` keys still to find among those matching `prefix`
  for (int pass = 0; pass < 4; ++pass) {
    const int shift = 24 - 8 * pass;
    if (tid < 256) hist[tid] = 0;
    __syncthreads();
    const uint32_t hi_mask = pass == 0 ? 0u : (0xffffffffu << (shift + 8));
    for (int i = tid; i < p.V; i += 1024) {
      const uint32_t key = topk_key(row[i] / p.t);
      if ((key & hi_mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
    }
    __syncthreads();
    if (tid == 0) {
      uint32_t acc = 0;
      int bin = 255;
      for (; bin > 0; --bin) {
        if (acc + hist[bin] >= need) break;
        acc += hist[bin];
      }
      s_prefix = prefix | ((uint32_t)bin << shift);
      s_need = need - acc;
    }
    __syncthreads();
    prefix = s_prefix;
    need = s_need;
    __syncthreads();
  }
  // prefix = key of the k-th largest; `need` of the elements equal to it belong to the top k
  if (tid == 0) { s_cnt = 0; s_base = 0; }
  __syncthreads();
  for (int i = tid; i < p.V; i += 1024) {
    const float v = row[i] / p.t;
    if (topk_key(v) > prefix) {
      const uint32_t slot = atomicAdd(&s_cnt, 1u);
      c_val[slot] = v;
      c_idx[slot] = i;
    }
  }
  __syncthreads();
  const uint32_t above = s_cnt;            // == k - need
  // equal keys in index order: block-wide ranks, 1024 elements at a time, until `need` are taken
  for (int i0 = 0; i0 < p.V; i0 += 1024) {
    if (s_base >= need) break;             // uniform: s_base is read after the barrier below
    const int i = i0 + tid;
    const float v = i < p.V ? row[i] / p.t : 0.f;
    const bool eq = i < p.V && topk_key(v) == prefix;
    const unsigned long long m = __ballot(eq);
    if (lane == 0) s_wave[wave] = (uint32_t)__popcll(m);
    __syncthreads();
    uint32_t before = s_base;
    for (int w = 0; w < wave; ++w) before += s_wave[w];
    const uint32_t rank = before + (uint32_t)__popcll(m & ((1ull << lane) - 1ull));
    if (eq && rank < need) {
      c_val[above + rank] = v;
      c_idx[above + rank] = i;
    }
    __syncthreads();
    if (tid == 0) {
      uint32_t t = s_base;
      for (int w = 0; w < 16; ++w) t += s_wave[w];
      s_base = t;
    }
    __syncthreads();
  }
  }
  }
  // histogram paths: order the k candidates, key descending (-0 below +0), index ascending
  if (ranked > (uint32_t)kRankPool && tid < p.k) {
    const float v = c_val[tid];
    const uint32_t kv = topk_key(v);
    const int ix = c_idx[tid];
    int r = 0;
#pragma unroll 16
    for (int j = 0; j < kTopKMax; ++j) {       // fixed trip count: the LDS reads go out in batches
      const uint32_t kj = topk_key(c_val[j]);
      r += (j < p.k && (kj > kv || (kj == kv && c_idx[j] < ix))) ? 1 : 0;
    }
    o_val[r] = v;
    o_idx[r] = ix;
  }
  __syncthreads();
  if (tid < p.k) {
    if (p.top_idx != nullptr) p.top_idx[(int64_t)blockIdx.x * p.k + tid] = o_idx[tid];
    if (p.top_val != nullptr) p.top_val[(int64_t)blockIdx.x * p.k + tid] = o_val[tid];
    // the k noise values in one go (c_val is free again): the scan below then stays inside the LDS
    if (p.noise != nullptr) c_val[tid] = o_val[tid] + p.noise[(int64_t)blockIdx.x * p.k + tid];
  }
  __syncthreads();
  if (tid == 0) {
    int best = 0;
    if (p.noise != nullptr) {
      float sc[kTopKMax];
#pragma unroll
      for (int j = 0; j < kTopKMax; ++j) sc[j] = c_val[j];
      float bs = sc[0];
#pragma unroll
      for (int j = 1; j < kTopKMax; ++j)
        if (j < p.k && sc[j] > bs) { bs = sc[j]; best = j; }      // first maximum wins, like argmax
    }
    p.token[blockIdx.x] = o_idx[best];
  }
}

// ----------------------------------------------------------------------------- advantages
// Sequence-level advantage estimators (plugins/training/advantage/grpo.py:8-52 and
// advantage/estimators.py:37-157).  B is a batch of sequences (hundreds to thousands): one
// workgroup does everything, each thread walks the batch for its own samples; sums in double in
// index order, the remaining arithmetic in float like the NumPy originals.
enum AdvMode { kAdvGrpo = 0, kAdvGlobal = 1, kAdvRloo = 2, kAdvDapo = 3 };

struct AdvArgs {
  const float* rewards;
  const int32_t* group_ids;   // unused by kAdvGlobal
  float* adv;
  int b, mode, whiten;        // whiten: kAdvRloo only
  float eps, alpha, clip;     // clip <= 0: none
};

MJ_DEV void block_mean_std(const float* x, int n, double* sh, float& mean, float& stdv) {
  // population mean and standard deviation over x[0..n), all threads get the result
  const int t = threadIdx.x;
  double a = 0.0;
  for (int i = t; i < n; i += 1024) a += (double)x[i];
  sh[t] = a;
  __syncthreads();
  for (int o = 512; o > 0; o >>= 1) { if (t < o) sh[t] += sh[t + o]; __syncthreads(); }
  const double m = sh[0] / n;
  __syncthreads();
  double v = 0.0;
  for (int i = t; i < n; i += 1024) { const double d = (double)x[i] - m; v += d * d; }
  sh[t] = v;
  __syncthreads();
  for (int o = 512; o > 0; o >>= 1) { if (t < o) sh[t] += sh[t + o]; __syncthreads(); }
  mean = (float)m;
  stdv = (float)sqrt(sh[0] / n);
  __syncthreads();
}

__global__ __launch_bounds__(1024) void k_advantages(AdvArgs p) {
  __shared__ double sh[1024];
  float rmean = 0.f, rstd = 0.f;
  if (p.mode == kAdvGlobal || p.mode == kAdvDapo) block_mean_std(p.rewards, p.b, sh, rmean, rstd);
  for (int i = threadIdx.x; i < p.b; i += 1024) {
    const float r = p.rewards[i];
    float out;
    if (p.mode == kAdvGlobal) {
      out = (r - rmean) / (rstd + p.eps);                                   // estimators.py:52-55
    } else {
      const int gid = p.group_ids[i];
      double sum = 0.0;
      int cnt = 0;
      for (int j = 0; j < p.b; ++j)
        if (p.group_ids[j] == gid) { sum += (double)p.rewards[j]; ++cnt; }
      const float gsum = (float)sum, count = fmaxf((float)cnt, 1.f);
      if (p.mode == kAdvRloo) {                                             // estimators.py:88-97
        const float loo = (gsum - r) / fmaxf((float)cnt - 1.f, 1.f);
        out = r - (cnt > 1 ? loo : gsum / count);
      } else {                                                              // grpo.py:40-51
        const float mean = gsum / count;
        double sq = 0.0;
        for (int j = 0; j < p.b; ++j)
          if (p.group_ids[j] == gid) { const float c = p.rewards[j] - mean; sq += (double)(c * c); }
        out = (r - mean) / (sqrtf((float)sq / count) + p.eps);
        if (p.mode == kAdvDapo) out += p.alpha * ((r - rmean) / (rstd + p.eps));   // estimators.py:131-133
      }
    }
    p.adv[i] = out;
  }
  __syncthreads();
  if (p.mode == kAdvRloo && p.whiten) {                                     // estimators.py:99-102
    float m, sd;
    block_mean_std(p.adv, p.b, sh, m, sd);
    for (int i = threadIdx.x; i < p.b; i += 1024) p.adv[i] = (p.adv[i] - m) / (sd + p.eps);
    __syncthreads();
  }
  if (p.clip > 0.f)
    for (int i = threadIdx.x; i < p.b; i += 1024) p.adv[i] = fminf(fmaxf(p.adv[i], -p.clip), p.clip);
}

// Token-level GAE (advantage/estimators.py:160-240): the sequence reward sits on the last
// completion token; one thread scans its sequence backwards.
struct GaeArgs {
  const float *rewards, *values, *mask;   // [B], [B,T], [B,T]
  float *adv, *ret;                       // [B,T]
  int b, t;
  float gamma, lambda;
};

__global__ __launch_bounds__(256) void k_gae_scan(GaeArgs p) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= p.b) return;
  const float* v = p.values + (int64_t)i * p.t;
  const float* m = p.mask + (int64_t)i * p.t;
  int last = -1;
  for (int k = 0; k < p.t; ++k) if (m[k] > 0.f) last = k;
  float gae = 0.f, next_v = 0.f;
  for (int k = p.t - 1; k >= 0; --k) {
    const float rew = (k == last) ? p.rewards[i] : 0.f;
    const float delta = rew + p.gamma * next_v - v[k];
    gae = (delta + p.gamma * p.lambda * gae) * m[k];
    p.adv[(int64_t)i * p.t + k] = gae;
    p.ret[(int64_t)i * p.t + k] = gae + v[k];
    next_v = v[k] * m[k];
  }
}

// normalisation over the completion tokens (estimators.py:226-232) and the optional clip
__global__ __launch_bounds__(1024) void k_gae_normalize(float* adv, const float* mask, int64_t n, int normalize,
                                                        float eps, float clip) {
  __shared__ double sh[1024];
  __shared__ double cnt_sh[1024];
  const int t = threadIdx.x;
  if (normalize) {
    double a = 0.0, c = 0.0;
    for (int64_t i = t; i < n; i += 1024) if (mask[i] > 0.f) { a += (double)adv[i]; c += 1.0; }
    sh[t] = a; cnt_sh[t] = c;
    __syncthreads();
    for (int o = 512; o > 0; o >>= 1) { if (t < o) { sh[t] += sh[t + o]; cnt_sh[t] += cnt_sh[t + o]; } __syncthreads(); }
    const double cnt = cnt_sh[0], mean = cnt > 0 ? sh[0] / cnt : 0.0;
    __syncthreads();
    double v = 0.0;
    for (int64_t i = t; i < n; i += 1024) if (mask[i] > 0.f) { const double d = (double)adv[i] - mean; v += d * d; }
    sh[t] = v;
    __syncthreads();
    for (int o = 512; o > 0; o >>= 1) { if (t < o) sh[t] += sh[t + o]; __syncthreads(); }
    if (cnt > 0) {
      const float m = (float)mean, sd = (float)sqrt(sh[0] / cnt);
      for (int64_t i = t; i < n; i += 1024) adv[i] = mask[i] > 0.f ? (adv[i] - m) / (sd + eps) : 0.f;
    }
    __syncthreads();
  }
  if (clip > 0.f)
    for (int64_t i = t; i < n; i += 1024) adv[i] = fminf(fmaxf(adv[i], -clip), clip);
}

}  // namespace mj
