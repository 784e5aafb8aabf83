// plan.hpp -- host-side planning of the fused GRPO loss: argument checks, chunking, the split of
// the d_hidden product, workspace layout, and the tile choices of the sampler's logits product.
//
// Plain C++ (no HIP header, no device code): mj_grpo.hip includes it, and a host-only build under
// the address / undefined-behaviour sanitizers checks it on the CPU -- an indexing mistake here is
// an out-of-bounds access on the GPU.
#pragma once
#include <math.h>
#include <stdarg.h>
#include <stddef.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/mj_grpo.h"

namespace mj {
namespace host {

inline thread_local char g_err[512] = "";

inline int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

constexpr int kValueRows = 64;             // token rows per workgroup of the value head's weight gradient
constexpr int BM = 256, BN = 256;          // tile of all three contractions
constexpr int64_t kDefaultChunk = 16384;   // tokens whose logits live in the workspace at once
constexpr int kRescueGrid = 256;           // workgroups of the rescue pass (one per CU)

inline int64_t rup(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

struct Plan {
  int64_t N, H, V, chunk, n_pad, ld_z, parts;
  int dh_splits;          // vocab splits of the dHidden product (1 = none)
  int64_t dh_k_per_split;
  // byte offsets into the workspace
  size_t zy, term, eterm, pm, pl, ps, plt, g, ge, hent, state, rs, dead, hs, zt, part, total_fwd, total_bwd;
  // token compaction (MJ_GRPO_FLAG_SKIP_MASKED): slot-order copies of the inputs and outputs
  bool compact;
  size_t perm, n_live, hid_p, tgt_p, fin_p[5], fout_p[3], dh_p;
  // value head (mj_grpo_forward_backward_value): laid out behind total_bwd
  size_t v_term, v_dv, v_dv_p, v_part, total_value;
};

// Splits of the dHidden product over the vocab: its (n/256) x (H/256) tiles rarely fill the 256
// CUs in whole rounds, so K = V is cut into the fewest pieces (<= 32) that waste < 4% of a round.
inline int pick_splits(int64_t tiles) {
  int best = 1;
  double best_eff = 0.0;
  for (int s = 1; s <= 32; ++s) {
    const int64_t items = tiles * s, rounds = (items + 255) / 256;
    const double eff = (double)items / (double)(rounds * 256);
    if (eff > best_eff + 1e-9) { best_eff = eff; best = s; }
    if (eff >= 0.96) return s;
  }
  return best;
}

inline int make_plan(const MjGrpoDesc* d, Plan* p) {
  if (d == nullptr) return fail(MJ_GRPO_ERR_NULL, "desc is NULL");
  if (d->n_tokens <= 0 || d->hidden <= 0 || d->vocab <= 0)
    return fail(MJ_GRPO_ERR_SHAPE, "n_tokens/hidden/vocab must be positive (got %lld/%lld/%lld)",
                (long long)d->n_tokens, (long long)d->hidden, (long long)d->vocab);
  // 256 rows of any operand or output must fit one 2 GiB buffer descriptor
  if (d->n_tokens > (1ll << 30) || d->hidden > (1 << 20) || d->vocab > (1 << 21) || d->ld_hidden > (1 << 20) ||
      d->ld_w > (1 << 21) || d->chunk_tokens > (1 << 20))
    return fail(MJ_GRPO_ERR_SHAPE, "shape too large (hidden, ld_hidden <= 2^20; vocab, ld_w <= 2^21; chunk_tokens <= 2^20)");
  if (d->ld_hidden < d->hidden || d->ld_w < d->vocab)
    return fail(MJ_GRPO_ERR_SHAPE, "leading dimension smaller than row length");
  if (d->hidden % 8 || d->vocab % 8 || d->ld_hidden % 8 || d->ld_w % 8)
    return fail(MJ_GRPO_ERR_ALIGN, "hidden, vocab, ld_hidden and ld_w must be multiples of 8");
  if (!(d->temperature > 0.f) || !isfinite(d->temperature))
    return fail(MJ_GRPO_ERR_UNSUPPORTED, "temperature must be positive and finite (got %g)", (double)d->temperature);
  if (d->temperature != 1.0f && d->entropy_coef != 0.f)
    return fail(MJ_GRPO_ERR_UNSUPPORTED, "an entropy bonus needs temperature 1 (got %g)", (double)d->temperature);
  if (d->softcap < 0.f || !isfinite(d->softcap)) return fail(MJ_GRPO_ERR_UNSUPPORTED, "softcap must be >= 0");
  if (d->chunk_tokens < 0) return fail(MJ_GRPO_ERR_SHAPE, "chunk_tokens must be >= 0");
  if (d->flags & ~(uint32_t)(MJ_GRPO_FLAG_DW_ACCUMULATE | MJ_GRPO_FLAG_SFT | MJ_GRPO_FLAG_SKIP_MASKED | MJ_GRPO_FLAG_DW_BF16))
    return fail(MJ_GRPO_ERR_UNSUPPORTED, "unknown bits in flags (0x%x)", d->flags);
  if (!isfinite(d->inv_total_valid_tokens)) return fail(MJ_GRPO_ERR_SHAPE, "inv_total_valid_tokens not finite");
  if (!isfinite(d->entropy_coef) || !isfinite(d->inv_entropy_count) || d->inv_entropy_count < 0.f)
    return fail(MJ_GRPO_ERR_SHAPE, "entropy_coef / inv_entropy_count not finite");
  p->N = d->n_tokens; p->H = d->hidden; p->V = d->vocab;
  int64_t chunk = d->chunk_tokens > 0 ? d->chunk_tokens : kDefaultChunk;
  chunk = rup(chunk, 256);
  if (chunk > p->N) chunk = p->N;
  p->chunk = chunk;
  p->n_pad = rup(chunk, 256);
  p->ld_z = p->V;               // rows of the 16-bit matrix: V % 8 == 0 keeps them 16-byte aligned
  p->parts = 2 * ((p->V + BM - 1) / BM);
  if (d->dhidden_splits > 32) return fail(MJ_GRPO_ERR_SHAPE, "dhidden_splits must be <= 32 (got %u)", d->dhidden_splits);
  p->dh_splits = d->dhidden_splits ? (int)d->dhidden_splits : pick_splits((p->n_pad / BM) * ((p->H + BN - 1) / BN));
  p->dh_k_per_split = rup((p->V + p->dh_splits - 1) / p->dh_splits, 64);
  // pieces are whole 64-wide slices: a small vocabulary has fewer of them than the splits asked for
  p->dh_splits = (int)((p->V + p->dh_k_per_split - 1) / p->dh_k_per_split);
  size_t o = 0;
  auto take = [&](size_t bytes) { size_t at = o; o = (size_t)rup((int64_t)(o + bytes), 256); return at; };
  p->zy = take((size_t)p->N * 4);
  p->term = take((size_t)p->N * 4);
  p->eterm = take((size_t)p->N * 4);
  p->pm = take((size_t)p->parts * p->n_pad * 4);
  p->pl = take((size_t)p->parts * p->n_pad * 4);
  p->ps = take((size_t)p->parts * p->n_pad * 4);
  p->plt = take(d->temperature != 1.0f ? (size_t)p->parts * p->n_pad * 4 : 0);
  p->g = take((size_t)p->n_pad * 4);
  p->ge = take((size_t)p->n_pad * 4);
  p->hent = take((size_t)p->n_pad * 4);
  p->state = take(256);
  p->compact = (d->flags & MJ_GRPO_FLAG_SKIP_MASKED) != 0;
  if (p->compact) {
    p->perm = take((size_t)p->N * 4);
    p->n_live = take(256);
    p->hid_p = take((size_t)p->N * p->H * 2);
    p->tgt_p = take((size_t)p->N * 4);
    for (auto& f : p->fin_p) f = take((size_t)p->N * 4);
    for (auto& f : p->fout_p) f = take((size_t)p->N * 4);
  }
  p->total_fwd = o;
  p->dh_p = take(p->compact ? (size_t)p->N * p->H * 2 : 0);
  p->rs = take((size_t)p->n_pad * 4);
  p->dead = take((size_t)p->n_pad / 8);     // one bit per token of a chunk
  p->hs = take((size_t)p->n_pad * p->H * 2);
  p->zt = take((size_t)p->n_pad * p->ld_z * 2);
  p->part = take(p->dh_splits > 1 ? (size_t)p->dh_splits * p->n_pad * p->H * 4 : 0);
  p->total_bwd = o;
  p->v_term = take((size_t)p->N * 4);
  p->v_dv = take((size_t)rup(p->N, 256) * 4);
  p->v_dv_p = take(p->compact ? (size_t)rup(p->N, 256) * 4 : 0);
  p->v_part = take((size_t)((p->N + kValueRows - 1) / kValueRows) * p->H * 4);
  p->total_value = o;
  return MJ_GRPO_OK;
}

// mj_grpo_forward_noalloc: the plan whose forward workspace fits `scratch_bytes`.  chunk_tokens == 0
// picks the largest chunk (a multiple of 256 tokens, at most 16384) that fits.
inline int noalloc_plan(const MjGrpoDesc* desc, size_t scratch_bytes, MjGrpoDesc* d_out, Plan* p_out) {
  if (desc == nullptr) return fail(MJ_GRPO_ERR_NULL, "desc is NULL");
  MjGrpoDesc d = *desc;
  Plan p;
  int rc;
  if (d.chunk_tokens > 0) {
    if ((rc = make_plan(&d, &p))) return rc;
  } else {
    int64_t lo = 1, hi = (d.n_tokens + 255) / 256;   // in units of 256 tokens
    if (hi > 64) hi = 64;
    d.chunk_tokens = 256;
    if ((rc = make_plan(&d, &p))) return rc;
    while (p.total_fwd <= scratch_bytes && lo < hi) {
      const int64_t mid = (lo + hi + 1) / 2;
      MjGrpoDesc t = d;
      t.chunk_tokens = mid * 256;
      Plan q;
      if ((rc = make_plan(&t, &q))) return rc;
      if (q.total_fwd <= scratch_bytes) { lo = mid; d = t; p = q; } else { hi = mid - 1; }
    }
  }
  if (p.total_fwd > scratch_bytes)
    return fail(MJ_GRPO_ERR_WORKSPACE,
                "this shape needs %zu bytes of forward workspace with %lld-token chunks; the static array holds %zu "
                "(use mj_grpo_forward with a caller workspace)", p.total_fwd, (long long)p.chunk, scratch_bytes);
  *d_out = d;
  *p_out = p;
  return MJ_GRPO_OK;
}

// Sampler's logits product (b rows against the whole vocabulary): batch-row tile and vocab columns
// per work item -- the fewest rounds of resident workgroups (one per CU) whose items are <= 256
// columns wide.  Measured at 3584 x 152064: the 128-row tile beats both a 64-row tile with two
// workgroups per CU (0.25 against 0.23 ms at 64 rows) and, past 128 rows, is beaten by the 256-row
// tile (two 128-row tiles: 0.35 against 0.32 ms at 192 rows).
inline void sample_tiles(int64_t b, int64_t vocab, int* bn_out, int64_t* tiles_n_out, int64_t* tile_rows_out) {
  const int bn = b <= 128 ? 128 : 256;
  const int64_t tiles_n = (b + bn - 1) / bn;
  const int64_t slots = 256;
  int64_t tile_rows = BM;
  for (int64_t rounds = 1; rounds <= 4096; ++rounds) {
    const int64_t per = slots * rounds / tiles_n;            // items along the vocabulary
    if (per == 0) continue;
    const int64_t cols = rup((vocab + per - 1) / per, 8);
    if (cols <= BM) { tile_rows = cols; break; }
  }
  *bn_out = bn;
  *tiles_n_out = tiles_n;
  *tile_rows_out = tile_rows;
}

}  // namespace host
}  // namespace mj
