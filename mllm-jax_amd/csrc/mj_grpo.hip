// mj_grpo.hip -- C ABI (include/mj_grpo.h) and launch plan of the fused GRPO loss path.
#include "../../include/mj_grpo.h"
#include "../../include/mj_norm.h"
#include "../../include/mj_sample.h"

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>

#include <initializer_list>
#include <mutex>
#include <new>

#include "mj_grpo_kernels.hpp"
#include "mj_norm_kernels.hpp"
#include "plan.hpp"

namespace {

using namespace mj::host;
static_assert(mj::kValueRows == mj::host::kValueRows, "the plan sizes the value head's partial rows");

// ---- launch tracing (mj_grpo_set_trace): a callback before and after every kernel launch
struct Trace {
  MjGrpoTraceFn fn = nullptr;
  void* user = nullptr;
} g_trace;

struct Timed {
  hipStream_t st;
  int id;
  MjGrpoTraceFn fn;
  void* user;
  Timed(int kernel_id, hipStream_t s) : st(s), id(kernel_id), fn(g_trace.fn), user(g_trace.user) {
    if (fn) fn(user, id, 0, (void*)st);
  }
  ~Timed() {
    if (fn) fn(user, id, 1, (void*)st);
  }
};

bool misaligned(const void* p) { return ((uintptr_t)p & 15u) != 0; }

// Raises the dynamic LDS limit of a tile kernel (128 KB > the 64 KB default).  The attribute belongs to
// the function on a device: it is set on the first call that launches that kernel on that device,
// whatever thread makes it (one process-wide table under a mutex), never again afterwards.
constexpr int kMaxDevices = 64;
constexpr int kMaxTileKernels = 32;       // tile-kernel instantiations in this file: 15
struct LdsDone {
  const void* fn;
  bool dev[kMaxDevices];
};
std::mutex g_lds_mutex;
LdsDone g_lds_done[kMaxTileKernels] = {};

template <typename K>
int enable_lds(K kernel) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(MJ_GRPO_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(MJ_GRPO_ERR_UNSUPPORTED, "device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_lds_mutex);
  LdsDone* slot = nullptr;
  for (auto& d : g_lds_done) {
    if (d.fn == (const void*)kernel || d.fn == nullptr) { slot = &d; break; }
  }
  if (slot == nullptr) return fail(MJ_GRPO_ERR_UNSUPPORTED, "internal: more tile kernels than table slots");
  if (slot->fn == (const void*)kernel && slot->dev[dev]) return MJ_GRPO_OK;
  e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                          mj::GemmTN<BM, BN>::kLdsBytes + mj::kTileExtraLds);
  if (e != hipSuccess) return fail(MJ_GRPO_ERR_HIP, "hipFuncSetAttribute: %s", hipGetErrorString(e));
  slot->fn = (const void*)kernel;
  slot->dev[dev] = true;
  return MJ_GRPO_OK;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MJ_GRPO_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
  return MJ_GRPO_OK;
}

enum Mode { kForward, kForwardBackward, kBackwardOnly };

int run(Mode mode, const MjGrpoDesc* d, const void* hidden, const void* lm_head, const int32_t* targets,
        const float* old_logp, const float* adv, const float* mask, float* logp, float* lse,
        float* ent, float* loss, const float* saved_lse, const float* saved_logp, void* d_hidden,
        void* d_w, void* workspace, size_t ws_bytes, void* stream_v, const MjPpoValue* pv = nullptr) {
  Plan p;
  int rc = make_plan(d, &p);
  if (rc) return rc;
  const bool sft = (d->flags & MJ_GRPO_FLAG_SFT) != 0;
  const bool bwd = mode != kForward;
  const bool dw_bf16 = (d->flags & MJ_GRPO_FLAG_DW_BF16) != 0;
  if (!hidden || !lm_head || !targets || !mask) return fail(MJ_GRPO_ERR_NULL, "hidden/lm_head/targets/mask is NULL");
  if (!sft && !adv) return fail(MJ_GRPO_ERR_NULL, "advantages is NULL");
  if (mode != kBackwardOnly && (!logp || !lse || !loss)) return fail(MJ_GRPO_ERR_NULL, "logp/lse/loss output is NULL");
  if (mode == kBackwardOnly && (!saved_lse || !saved_logp)) return fail(MJ_GRPO_ERR_NULL, "saved lse/logp is NULL");
  if (mode == kBackwardOnly && d->entropy_coef != 0.f)
    return fail(MJ_GRPO_ERR_UNSUPPORTED, "the separate backward does not carry the entropy bonus (entropy_coef must be 0)");
  if (bwd && (!d_hidden || !d_w)) return fail(MJ_GRPO_ERR_NULL, "d_hidden/d_lm_head is NULL");
  if (!workspace) return fail(MJ_GRPO_ERR_WORKSPACE, "workspace is NULL");
  if (pv != nullptr) {
    if (mode != kForwardBackward) return fail(MJ_GRPO_ERR_UNSUPPORTED, "the value head needs the fused forward + backward pass");
    if (!pv->value_w || !pv->value_b || !pv->values || !pv->value_loss || !pv->d_value_w || !pv->d_value_b)
      return fail(MJ_GRPO_ERR_NULL, "value head: value_w/value_b/values/value_loss/d_value_w/d_value_b is NULL");
    if (misaligned(pv->value_w) || misaligned(pv->d_value_w))
      return fail(MJ_GRPO_ERR_ALIGN, "value head: value_w and d_value_w must be 16-byte aligned");
    if (!adv) return fail(MJ_GRPO_ERR_NULL, "value head: advantages is NULL");
    if (!isfinite(pv->value_coef) || (pv->use_clip && !(pv->value_clip >= 0.f)))
      return fail(MJ_GRPO_ERR_UNSUPPORTED, "value head: value_coef must be finite and value_clip >= 0");
  }
  const size_t need = pv != nullptr ? p.total_value : (bwd ? p.total_bwd : p.total_fwd);
  if (ws_bytes < need) return fail(MJ_GRPO_ERR_WORKSPACE, "workspace too small: %zu < %zu bytes", ws_bytes, need);
  if (misaligned(hidden) || misaligned(lm_head) || misaligned(workspace) ||
      (bwd && (misaligned(d_hidden) || misaligned(d_w))))
    return fail(MJ_GRPO_ERR_ALIGN, "hidden, lm_head, d_hidden, d_lm_head and workspace must be 16-byte aligned");

  hipStream_t st = (hipStream_t)stream_v;
  char* ws = (char*)workspace;
  const int N = (int)p.N, H = (int)p.H, V = (int)p.V;
  float* zy = (float*)(ws + p.zy);
  float* term = (float*)(ws + p.term);
  float* eterm = (float*)(ws + p.eterm);
  float* ge = (float*)(ws + p.ge);
  float* hent = (float*)(ws + p.hent);
  const bool bonus = bwd && d->entropy_coef != 0.f;
  float* pm = (float*)(ws + p.pm);
  float* pl = (float*)(ws + p.pl);
  float* ps = (float*)(ws + p.ps);
  float* plt = (float*)(ws + p.plt);
  const float inv_t = d->temperature == 1.0f ? 1.0f : 1.0f / d->temperature;
  float* g = (float*)(ws + p.g);
  uint16_t* zt = (uint16_t*)(ws + p.zt);
  float* part = (float*)(ws + p.part);
  const float gscale = d->grad_loss_scale;
  const size_t lds = mj::GemmTN<BM, BN>::kLdsBytes + mj::kTileExtraLds;   // two stages + the epilogue's hand-over

  // Which statistics the logits epilogue keeps (mj::StatsMode): sums of exp(z) without a running
  // maximum plus E = exp(z) for the backward -- with a kStatsMax rescue pass enqueued behind it that
  // leaves at once unless the range check failed -- or, where that form does not apply, kStatsMax.
  const bool exp_mode = mode != kBackwardOnly && d->entropy_coef == 0.f;
  int* state = (int*)(ws + p.state);
  float* rs = (float*)(ws + p.rs);
  uint16_t* hs = (uint16_t*)(ws + p.hs);
  uint64_t* dead = (uint64_t*)(ws + p.dead);
  // the logits kernels exist with and without the softcap code (a template parameter)
  const bool cap = d->softcap > 0.f;
  auto k_grad = cap ? mj::k_logits_stats<BM, BN, mj::kStatsGrad, false, true> : mj::k_logits_stats<BM, BN, mj::kStatsGrad, false, false>;
  auto k_exp = cap ? mj::k_logits_stats<BM, BN, mj::kStatsExp, false, true> : mj::k_logits_stats<BM, BN, mj::kStatsExp, false, false>;
  auto k_max = cap ? mj::k_logits_stats<BM, BN, mj::kStatsMax, false, true> : mj::k_logits_stats<BM, BN, mj::kStatsMax, false, false>;
  auto k_max_rescue = cap ? mj::k_logits_stats<BM, BN, mj::kStatsMax, true, true> : mj::k_logits_stats<BM, BN, mj::kStatsMax, true, false>;
  if (mode == kBackwardOnly) {
    if ((rc = enable_lds(k_grad))) return rc;
  } else {
    if (exp_mode && (rc = enable_lds(k_exp))) return rc;
    if (exp_mode && (rc = enable_lds(k_max_rescue))) return rc;
    if (!exp_mode && (rc = enable_lds(k_max))) return rc;
  }
  if (bwd) {
    if ((rc = enable_lds(mj::k_dhidden<BM, BN>))) return rc;
    if ((rc = dw_bf16 ? enable_lds(mj::k_dw<BM, BN, true>) : enable_lds(mj::k_dw<BM, BN, false>))) return rc;
  }

  // Value head (PPO critic), on the caller's token order: value_pred, the clipped value loss and
  // dv = d(value_coef * value_loss)/d value_pred; d_hidden picks dv up in the d_hidden product.
  const float* dv = nullptr;
  if (pv != nullptr) {
    float* dvw = (float*)(ws + p.v_dv);
    float* vterm = (float*)(ws + p.v_term);
    float* vpart = (float*)(ws + p.v_part);
    mj::k_value_head<<<(unsigned)((N + 3) / 4), 256, 0, st>>>((const uint16_t*)hidden, d->ld_hidden, N, H, pv->value_w,
                                                              pv->value_b, pv->values);
    mj::ValueLossArgs v;
    v.values = pv->values; v.adv = adv; v.mask = mask; v.returns = pv->returns; v.old_values = pv->old_values;
    v.n = N; v.inv_tv = d->inv_total_valid_tokens; v.coef = pv->value_coef; v.clip = pv->value_clip;
    v.use_clip = pv->use_clip; v.gscale = gscale; v.vterm = vterm; v.dv = dvw;
    mj::k_value_loss<<<(unsigned)((N + 255) / 256), 256, 0, st>>>(v);
    mj::k_sum<<<1, 1024, 0, st>>>(vterm, N, pv->value_loss);
    mj::k_sum<<<1, 1024, 0, st>>>(dvw, N, pv->d_value_b);
    const int vblocks = (N + mj::kValueRows - 1) / mj::kValueRows;
    mj::k_value_wgrad<<<vblocks, 256, 0, st>>>((const uint16_t*)hidden, d->ld_hidden, N, H, dvw, vpart);
    mj::k_value_wgrad_reduce<<<(unsigned)((H + 255) / 256), 256, 0, st>>>(vpart, vblocks, H, pv->d_value_w);
    if ((rc = check_launch("value head kernels"))) return rc;
    dv = dvw;
  }

  // Token compaction: tokens that cannot carry a gradient go behind the others; everything below
  // then works on slot-order copies and the backward kernels stop at the device-side count.
  const int* n_live = nullptr;
  const int* perm = nullptr;
  float* out_user[3] = {logp, lse, ent};
  void* dh_user = d_hidden;
  int64_t ld_hid = d->ld_hidden, ld_dh = d->ld_hidden;
  if (p.compact) {
    perm = (const int*)(ws + p.perm);
    n_live = (const int*)(ws + p.n_live);
    mj::CompactArgs c;
    // a token with advantage exactly 0 is dead only when nothing else feeds its gradient: the entropy
    // bonus and the critic's dv[t] * value_w both reach d_hidden[t, :] whatever the advantage is
    c.mask = mask; c.adv = (sft || d->entropy_coef != 0.f || pv != nullptr) ? nullptr : adv; c.n = N;
    c.perm = (int*)(ws + p.perm); c.n_live = (int*)(ws + p.n_live);
    mj::k_compact_plan<<<1, 1024, 0, st>>>(c);
    mj::GatherArgs ga;
    ga.perm = perm; ga.n = N; ga.H = H; ga.hid = (const uint16_t*)hidden; ga.ld_hid = d->ld_hidden;
    ga.hid_p = (uint16_t*)(ws + p.hid_p); ga.tgt = targets; ga.tgt_p = (int32_t*)(ws + p.tgt_p);
    const float* fin[5] = {old_logp, adv, mask, saved_lse, saved_logp};
    for (int i = 0; i < 5; ++i) { ga.f_in[i] = fin[i]; ga.f_out[i] = (float*)(ws + p.fin_p[i]); }
    ga.f_in[5] = dv; ga.f_out[5] = (float*)(ws + p.v_dv_p);
    mj::k_gather_tokens<<<N, 256, 0, st>>>(ga);
    if ((rc = check_launch("token compaction"))) return rc;
    hidden = ws + p.hid_p; ld_hid = H;
    targets = (const int32_t*)(ws + p.tgt_p);
    if (old_logp) old_logp = (const float*)(ws + p.fin_p[0]);
    if (adv) adv = (const float*)(ws + p.fin_p[1]);
    mask = (const float*)(ws + p.fin_p[2]);
    if (saved_lse) saved_lse = (const float*)(ws + p.fin_p[3]);
    if (saved_logp) saved_logp = (const float*)(ws + p.fin_p[4]);
    if (dv) dv = (const float*)(ws + p.v_dv_p);
    if (logp) logp = (float*)(ws + p.fout_p[0]);
    if (lse) lse = (float*)(ws + p.fout_p[1]);
    if (ent) ent = (float*)(ws + p.fout_p[2]);
    if (bwd) { d_hidden = ws + p.dh_p; ld_dh = H; }
  }

  for (int64_t c0 = 0; c0 < p.N; c0 += p.chunk) {
    const int nc = (int)((p.N - c0 < p.chunk) ? p.N - c0 : p.chunk);
    const int n_pad = (int)rup(nc, 256);
    const __bf16* hid_c = (const __bf16*)hidden + c0 * ld_hid;
    mj::LogitsArgs a;
    a.w = (const __bf16*)lm_head; a.hid = hid_c; a.ld_w = d->ld_w; a.ld_hid = ld_hid;
    a.V = V; a.n = nc; a.H = H; a.cap = d->softcap;
    a.zt = bwd ? zt : nullptr; a.ld_z = p.ld_z;
    a.pm = pm; a.pl = pl; a.ps = ps; a.plt = plt; a.inv_t = inv_t; a.ld_p = p.n_pad;
    a.targets = targets + c0; a.zy = zy + c0; a.n_live = n_live; a.c0 = (int)c0;
    a.mask = mask + c0; a.lse = nullptr; a.g = g; a.state = state;
    const mj::TileMap map = mj::TileMap::pick_shape((V + BM - 1) / BM, (nc + BN - 1) / BN, 1, 1);

    mj::FinalizeArgs f;
    f.pm = pm; f.pl = pl; f.ps = ps; f.plt = plt; f.inv_t = inv_t; f.ld_p = p.n_pad; f.parts = (int)p.parts;
    f.n = nc; f.n_pad = n_pad; f.zy = zy + c0;
    f.old_logp = old_logp ? old_logp + c0 : nullptr;
    f.adv = adv ? adv + c0 : nullptr; f.mask = mask + c0;
    f.eps_low = d->eps_low; f.eps_high = d->eps_high; f.inv_tv = d->inv_total_valid_tokens;
    f.gscale = gscale; f.sft = sft ? 1 : 0;
    f.logp = logp ? logp + c0 : nullptr; f.lse = lse ? lse + c0 : nullptr; f.ent = ent ? ent + c0 : nullptr;
    f.term = term + c0; f.g = bwd ? g : nullptr;
    f.ent_coef = d->entropy_coef; f.inv_ent_cnt = d->inv_entropy_count; f.eterm = eterm + c0;
    f.ge = bonus ? ge : nullptr; f.hent = bonus ? hent : nullptr;
    f.rs = bwd ? rs : nullptr; f.zt = zt; f.ld_z = p.ld_z; f.targets = targets + c0; f.V = V; f.cap = d->softcap;
    f.state = state; f.rescue = 0; f.dead = bwd ? (uint16_t*)dead : nullptr;

    mj::DzArgs z;
    z.zt = zt; z.ld_z = p.ld_z;
    z.lse = (mode == kBackwardOnly ? saved_lse : lse) + c0; z.g = g; z.targets = targets + c0;
    z.ge = bonus ? ge : nullptr; z.hent = bonus ? hent : nullptr; z.mask = mask + c0;
    z.V = V; z.n = nc; z.cap = d->softcap; z.n_live = n_live; z.c0 = (int)c0; z.state = state; z.rescue = 0;
    const unsigned dz_grid = (unsigned)(nc < 8192 ? nc : 8192);

    if (mode == kBackwardOnly) {
      {
        Timed t(MJ_GRPO_K_FINALIZE, st);
        mj::k_coeff_from_saved<<<(n_pad + 255) / 256, 256, 0, st>>>(
            saved_logp + c0, old_logp ? old_logp + c0 : nullptr, adv ? adv + c0 : nullptr, mask + c0, nc, n_pad,
            d->eps_low, d->eps_high, d->inv_total_valid_tokens, gscale * inv_t, sft ? 1 : 0, g, dead);
      }
      a.lse = saved_lse + c0;
      {
        Timed t(MJ_GRPO_K_LOGITS_STATS, st);
        k_grad<<<map.items(), mj::kThreads, lds, st>>>(a, map);
      }
      Timed t(MJ_GRPO_K_FINALIZE, st);
      mj::k_patch_grad<<<(nc + 255) / 256, 256, 0, st>>>(zt, p.ld_z, zy + c0, saved_lse + c0, g, targets + c0, nc, V,
                                                         d->softcap, state);
    } else if (exp_mode) {
      {
        Timed t(MJ_GRPO_K_LOGITS_STATS, st);
        k_exp<<<map.items(), mj::kThreads, lds, st>>>(a, map);
      }
      {
        Timed t(MJ_GRPO_K_FINALIZE, st);
        mj::k_finalize<mj::kStatsExp><<<n_pad / mj::kFinTokens, mj::kFinTokens * mj::kFinSlices, 0, st>>>(f);
      }
      // the rescue: the same chunk with a running maximum; every workgroup leaves at once unless the
      // range check in k_finalize failed
      Timed t(MJ_GRPO_K_RESCUE, st);
      f.rescue = 1; z.rescue = 1;
      k_max_rescue<<<kRescueGrid, mj::kThreads, lds, st>>>(a, map);
      mj::k_finalize<mj::kStatsMax><<<n_pad / mj::kFinTokens, mj::kFinTokens * mj::kFinSlices, 0, st>>>(f);
      if (bwd) mj::k_dz<<<dz_grid, 256, 0, st>>>(z);
    } else {
      {
        Timed t(MJ_GRPO_K_LOGITS_STATS, st);
        k_max<<<map.items(), mj::kThreads, lds, st>>>(a, map);
      }
      {
        Timed t(MJ_GRPO_K_FINALIZE, st);
        mj::k_finalize<mj::kStatsMax><<<n_pad / mj::kFinTokens, mj::kFinTokens * mj::kFinSlices, 0, st>>>(f);
      }
      if (bwd) {
        Timed t(MJ_GRPO_K_DZ, st);
        mj::k_dz<<<dz_grid, 256, 0, st>>>(z);
      }
    }
    if (bwd) {
      // the split count was planned for a full chunk; a shorter last chunk keeps it (the partial
      // buffer is sized for it) unless it has a single split anyway
      mj::DhArgs h;
      h.dzt = (const __bf16*)zt; h.w = (const __bf16*)lm_head; h.ld_z = p.ld_z; h.ld_w = d->ld_w;
      h.n = nc; h.n_pad = n_pad; h.H = H; h.V = V;
      h.splits = p.dh_splits; h.k_per_split = (int)p.dh_k_per_split;
      h.dh = (uint16_t*)d_hidden + c0 * ld_dh; h.ld_dh = ld_dh;
      h.part = part; h.n_live = n_live; h.c0 = (int)c0; h.rs = rs; h.state = state;
      h.dv = dv ? dv + c0 : nullptr; h.wv = pv ? pv->value_w : nullptr; h.dead = dead;
      const mj::TileMap mh = mj::TileMap::pick_shape((nc + BM - 1) / BM, (H + BN - 1) / BN, 0, h.splits);
      {
        Timed t(MJ_GRPO_K_DHIDDEN, st);
        mj::k_dhidden<BM, BN><<<mh.items(), mj::kThreads, lds, st>>>(h, mh);
      }
      if (h.splits > 1) {
        const int64_t work = (int64_t)nc * (H / 4);
        Timed t(MJ_GRPO_K_DHIDDEN_REDUCE, st);
        mj::k_dhidden_reduce<<<(unsigned)((work + 255) / 256), 256, 0, st>>>(part, h.splits, nc, n_pad, H, h.dh,
                                                                           h.ld_dh, rs, state, h.dv, h.wv);
      }

      // the token-side operand of the dW product, k-contiguous: (rs * hidden)^T while the 16-bit matrix
      // holds E, hidden^T once it holds dZ (the state word is final by now)
      {
        Timed t(MJ_GRPO_K_SCALE_HIDDEN, st);
        mj::k_scale_hidden<<<dim3((unsigned)(n_pad / 64), (unsigned)((H + 63) / 64)), 256, 0, st>>>(
            (const uint16_t*)hid_c, ld_hid, rs, state, nc, n_pad, H, hs);
      }
      mj::DwArgs w;
      w.dzt = (const __bf16*)zt; w.ht = (const __bf16*)hs; w.ld_z = p.ld_z;
      w.H = H; w.V = V; w.n = nc;
      w.dw = d_w; w.ld_dw = d->ld_w; w.n_live = n_live; w.c0 = (int)c0; w.dead = dead;
      w.accumulate = (c0 > 0 || (d->flags & MJ_GRPO_FLAG_DW_ACCUMULATE)) ? 1 : 0;
      const mj::TileMap mw = mj::TileMap::pick_shape((V + BM - 1) / BM, (H + BN - 1) / BN, 0, 1);
      {
        Timed t(MJ_GRPO_K_DW, st);
        if (dw_bf16) mj::k_dw<BM, BN, true><<<mw.items(), mj::kThreads, lds, st>>>(w, mw);
        else mj::k_dw<BM, BN, false><<<mw.items(), mj::kThreads, lds, st>>>(w, mw);
      }
    }
    if ((rc = check_launch("chunk kernels"))) return rc;
  }
  if (p.compact) {
    mj::ScatterArgs sc;
    sc.perm = perm; sc.n_live = n_live; sc.n = N; sc.H = H;
    float* slot[3] = {logp, lse, ent};
    for (int i = 0; i < 3; ++i) {
      const bool on = mode != kBackwardOnly && out_user[i] != nullptr;
      sc.f_in[i] = on ? slot[i] : nullptr;
      sc.f_out[i] = out_user[i];
    }
    sc.dh_p = bwd ? (const uint16_t*)d_hidden : nullptr; sc.dh = (uint16_t*)dh_user; sc.ld_dh = d->ld_hidden;
    mj::k_scatter_tokens<<<N, 256, 0, st>>>(sc);
    if ((rc = check_launch("k_scatter_tokens"))) return rc;
  }
  if (mode != kBackwardOnly) {
    {
      Timed t(MJ_GRPO_K_REDUCE_LOSS, st);
      mj::k_reduce_loss<<<1, 1024, 0, st>>>(term, eterm, N, d->entropy_coef, loss);
    }
    if ((rc = check_launch("k_reduce_loss"))) return rc;
  }
  return MJ_GRPO_OK;
}

}  // namespace

extern "C" {

int mj_grpo_version(void) { return 300; }   // 0.3.0: MJ_GRPO_FLAG_DW_BF16, d_lm_head as void*

const char* mj_grpo_last_error(void) { return mj::host::g_err; }

int mj_grpo_set_trace(MjGrpoTraceFn fn, void* user) {
  g_trace.fn = fn;
  g_trace.user = user;
  return MJ_GRPO_OK;
}

int mj_grpo_workspace_bytes(const MjGrpoDesc* desc, size_t* forward_bytes, size_t* forward_backward_bytes) {
  Plan p;
  int rc = make_plan(desc, &p);
  if (rc) return rc;
  if (forward_bytes) *forward_bytes = p.total_fwd;
  if (forward_backward_bytes) *forward_backward_bytes = p.total_bwd;
  return MJ_GRPO_OK;
}

int mj_grpo_forward(const MjGrpoDesc* desc, const void* hidden, const void* lm_head, const int32_t* targets,
                    const float* old_logp, const float* advantages, const float* mask, float* logp,
                    float* lse, float* token_entropy, float* loss, void* workspace, size_t workspace_bytes,
                    void* stream) {
  return run(kForward, desc, hidden, lm_head, targets, old_logp, advantages, mask, logp, lse, token_entropy,
             loss, nullptr, nullptr, nullptr, nullptr, workspace, workspace_bytes, stream);
}

int mj_grpo_forward_backward(const MjGrpoDesc* desc, const void* hidden, const void* lm_head,
                             const int32_t* targets, const float* old_logp, const float* advantages,
                             const float* mask, float* logp, float* lse, float* token_entropy, float* loss,
                             void* d_hidden, void* d_lm_head, void* workspace, size_t workspace_bytes,
                             void* stream) {
  return run(kForwardBackward, desc, hidden, lm_head, targets, old_logp, advantages, mask, logp, lse,
             token_entropy, loss, nullptr, nullptr, d_hidden, d_lm_head, workspace, workspace_bytes, stream);
}

int mj_grpo_sequence_entropy(const float* token_entropy, const float* mask, int64_t b, int64_t t, float* entropy,
                             float* entropy_loss, void* stream) {
  if (!token_entropy || !mask || !entropy || !entropy_loss) return fail(MJ_GRPO_ERR_NULL, "sequence_entropy: NULL pointer argument");
  if (b <= 0 || t <= 0 || b > (1 << 24) || t > (1 << 24)) return fail(MJ_GRPO_ERR_SHAPE, "sequence_entropy: bad shape b=%lld t=%lld", (long long)b, (long long)t);
  mj::k_sequence_entropy<<<(unsigned)((b + 3) / 4), 256, 0, (hipStream_t)stream>>>(token_entropy, mask, (int)b, (int)t, entropy, entropy_loss);
  return check_launch("k_sequence_entropy");
}

int mj_grpo_scale_gradients(void* d_hidden, int64_t n, int64_t h, int64_t ld_hidden, void* d_lm_head, int64_t hw,
                            int64_t v, int64_t ld_w, int d_lm_head_bf16, const float* scale, void* stream) {
  if (!scale) return fail(MJ_GRPO_ERR_NULL, "scale_gradients: scale is NULL");
  if (!d_hidden && !d_lm_head) return fail(MJ_GRPO_ERR_NULL, "scale_gradients: both gradients are NULL");
  hipStream_t st = (hipStream_t)stream;
  const unsigned grid = 2048;       // grid-stride: a launch whose workgroups all leave costs a few microseconds
  if (d_hidden) {
    if (n <= 0 || h <= 0 || ld_hidden < h || h % 8 || ld_hidden % 8)
      return fail(MJ_GRPO_ERR_SHAPE, "scale_gradients: bad d_hidden shape n=%lld h=%lld ld=%lld", (long long)n, (long long)h, (long long)ld_hidden);
    if (misaligned(d_hidden)) return fail(MJ_GRPO_ERR_ALIGN, "scale_gradients: d_hidden must be 16-byte aligned");
    mj::k_scale_inplace<true><<<grid, 256, 0, st>>>(d_hidden, n, h, ld_hidden, scale);
  }
  if (d_lm_head) {
    if (hw <= 0 || v <= 0 || ld_w < v || v % 8 || ld_w % 8)
      return fail(MJ_GRPO_ERR_SHAPE, "scale_gradients: bad d_lm_head shape h=%lld v=%lld ld=%lld", (long long)hw, (long long)v, (long long)ld_w);
    if (misaligned(d_lm_head)) return fail(MJ_GRPO_ERR_ALIGN, "scale_gradients: d_lm_head must be 16-byte aligned");
    if (d_lm_head_bf16) mj::k_scale_inplace<true><<<grid, 256, 0, st>>>(d_lm_head, hw, v, ld_w, scale);
    else mj::k_scale_inplace<false><<<grid, 256, 0, st>>>(d_lm_head, hw, v, ld_w, scale);
  }
  return check_launch("k_scale_inplace");
}

int mj_grpo_value_workspace_bytes(const MjGrpoDesc* desc, size_t* extra_bytes) {
  Plan p;
  int rc = make_plan(desc, &p);
  if (rc) return rc;
  if (extra_bytes) *extra_bytes = p.total_value - p.total_bwd;
  return MJ_GRPO_OK;
}

int mj_grpo_forward_backward_value(const MjGrpoDesc* desc, const MjPpoValue* value, const void* hidden,
                                   const void* lm_head, const int32_t* targets, const float* old_logp,
                                   const float* advantages, const float* mask, float* logp, float* lse,
                                   float* token_entropy, float* loss, void* d_hidden, void* d_lm_head,
                                   void* workspace, size_t workspace_bytes, void* stream) {
  if (value == nullptr) return fail(MJ_GRPO_ERR_NULL, "value is NULL (use mj_grpo_forward_backward)");
  return run(kForwardBackward, desc, hidden, lm_head, targets, old_logp, advantages, mask, logp, lse, token_entropy,
             loss, nullptr, nullptr, d_hidden, d_lm_head, workspace, workspace_bytes, stream, value);
}

int mj_value_head_forward(const void* hidden, int64_t ld_hidden, const float* value_w, const float* value_b,
                          float* values, int64_t n, int64_t h, void* stream) {
  if (!hidden || !value_w || !value_b || !values) return fail(MJ_GRPO_ERR_NULL, "value head: NULL pointer argument");
  if (n <= 0 || h <= 0 || n > (1ll << 30) || h > (1 << 20) || ld_hidden < h)
    return fail(MJ_GRPO_ERR_SHAPE, "value head: bad shape n=%lld h=%lld ld=%lld", (long long)n, (long long)h, (long long)ld_hidden);
  if (h % 8 || ld_hidden % 8 || misaligned(hidden) || misaligned(value_w))
    return fail(MJ_GRPO_ERR_ALIGN, "value head: h and ld_hidden must be multiples of 8, hidden and value_w 16-byte aligned");
  mj::k_value_head<<<(unsigned)((n + 3) / 4), 256, 0, (hipStream_t)stream>>>((const uint16_t*)hidden, ld_hidden, (int)n,
                                                                            (int)h, value_w, value_b, values);
  return check_launch("k_value_head");
}

int mj_grpo_backward(const MjGrpoDesc* desc, const void* hidden, const void* lm_head, const int32_t* targets,
                     const float* old_logp, const float* advantages, const float* mask, const float* lse,
                     const float* logp, void* d_hidden, void* d_lm_head, void* workspace,
                     size_t workspace_bytes, void* stream) {
  return run(kBackwardOnly, desc, hidden, lm_head, targets, old_logp, advantages, mask, nullptr, nullptr,
             nullptr, nullptr, lse, logp, d_hidden, d_lm_head, workspace, workspace_bytes, stream);
}

}  // extern "C"

// ---- forward without a caller workspace: the workspace is a static device array
namespace {
constexpr size_t kScratchBytes = (size_t)MJ_GRPO_NOALLOC_SCRATCH_BYTES;
}  // namespace
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
namespace {
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};   // device address of `scratch` on each device, once looked up

// The array's name is only a host-side handle; this returns the current device's copy of it.
int scratch_address(void** out) {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return fail(MJ_GRPO_ERR_HIP, "hipGetDevice: %s", hipGetErrorString(e));
  if (dev < 0 || dev >= kMaxDevices) return fail(MJ_GRPO_ERR_UNSUPPORTED, "device index %d out of range", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr)
      return fail(MJ_GRPO_ERR_HIP, "hipGetSymbolAddress(scratch): %s", hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return MJ_GRPO_OK;
}
}  // namespace

extern "C" {

int mj_grpo_forward_noalloc(const MjGrpoDesc* desc, const void* hidden, const void* lm_head, const int32_t* targets,
                            const float* old_logp, const float* advantages, const float* mask, float* logp,
                            float* lse, float* token_entropy, float* loss, void* stream) {
  if (desc == nullptr) return fail(MJ_GRPO_ERR_NULL, "desc is NULL");
  MjGrpoDesc d;
  Plan p;
  int rc;
  if ((rc = noalloc_plan(desc, kScratchBytes, &d, &p))) return rc;
  void* ws = nullptr;
  if ((rc = scratch_address(&ws))) return rc;
  return run(kForward, &d, hidden, lm_head, targets, old_logp, advantages, mask, logp, lse, token_entropy, loss,
             nullptr, nullptr, nullptr, nullptr, ws, kScratchBytes, stream);
}

}  // extern "C"

extern "C" {

int mj_grpo_advantages(int mode, const float* rewards, const int32_t* group_ids, float* advantages, int64_t b,
                       float eps, float alpha, int whiten, float clip_range, void* stream) {
  if (mode < mj::kAdvGrpo || mode > mj::kAdvDapo) return fail(MJ_GRPO_ERR_UNSUPPORTED, "unknown advantage mode %d", mode);
  if (!rewards || !advantages || (mode != mj::kAdvGlobal && !group_ids))
    return fail(MJ_GRPO_ERR_NULL, "rewards/group_ids/advantages is NULL");
  if (b <= 0 || b > (1 << 16)) return fail(MJ_GRPO_ERR_SHAPE, "batch must be in [1, 65536] (got %lld)", (long long)b);
  // the grouped estimators walk the batch once per sample (a batch is hundreds of sequences)
  if (mode != mj::kAdvGlobal && b > (1 << 13))
    return fail(MJ_GRPO_ERR_SHAPE, "grouped advantage estimators take at most 8192 sequences (got %lld)", (long long)b);
  if (!(eps > 0.f)) return fail(MJ_GRPO_ERR_UNSUPPORTED, "eps must be > 0");
  if (mode == mj::kAdvDapo && !(alpha >= 0.f)) return fail(MJ_GRPO_ERR_UNSUPPORTED, "alpha must be >= 0");
  mj::AdvArgs a;
  a.rewards = rewards; a.group_ids = group_ids; a.adv = advantages; a.b = (int)b; a.mode = mode; a.whiten = whiten;
  a.eps = eps; a.alpha = alpha; a.clip = clip_range;
  mj::k_advantages<<<1, 1024, 0, (hipStream_t)stream>>>(a);
  return check_launch("k_advantages");
}

int mj_grpo_group_advantages(const float* rewards, const int32_t* group_ids, float* advantages, int64_t b, float eps,
                             void* stream) {
  return mj_grpo_advantages(mj::kAdvGrpo, rewards, group_ids, advantages, b, eps, 0.f, 0, 0.f, stream);
}

int mj_grpo_gae(const float* rewards, const float* values, const float* completion_mask, float* advantages,
                float* returns, int64_t b, int64_t t, float gamma, float gae_lambda, int normalize, float eps,
                float clip_range, void* stream) {
  if (!rewards || !values || !completion_mask || !advantages || !returns) return fail(MJ_GRPO_ERR_NULL, "gae: NULL pointer argument");
  if (b <= 0 || t <= 0 || b > (1 << 24) || t > (1 << 24) || b * t > (1ll << 31))
    return fail(MJ_GRPO_ERR_SHAPE, "gae: bad shape b=%lld t=%lld", (long long)b, (long long)t);
  mj::GaeArgs a;
  a.rewards = rewards; a.values = values; a.mask = completion_mask; a.adv = advantages; a.ret = returns;
  a.b = (int)b; a.t = (int)t; a.gamma = gamma; a.lambda = gae_lambda;
  hipStream_t st = (hipStream_t)stream;
  mj::k_gae_scan<<<(unsigned)((b + 255) / 256), 256, 0, st>>>(a);
  if (normalize || clip_range > 0.f)
    mj::k_gae_normalize<<<1, 1024, 0, st>>>(advantages, completion_mask, b * t, normalize, eps, clip_range);
  return check_launch("gae kernels");
}

}  // extern "C"

// ----------------------------------------------------------------------------- sampler
extern "C" {

int mj_sample_logits(const void* hidden, int64_t ld_hidden, const void* lm_head, int64_t ld_w, float* logits,
                     int64_t ld_logits, int64_t b, int64_t h, int64_t vocab, float softcap, void* stream) {
  if (!hidden || !lm_head || !logits) return fail(MJ_GRPO_ERR_NULL, "hidden/lm_head/logits is NULL");
  if (b <= 0 || h <= 0 || vocab <= 0 || b > (1 << 24) || h > (1 << 20) || vocab > (1 << 21))
    return fail(MJ_GRPO_ERR_SHAPE, "sample_logits: bad shape b=%lld h=%lld vocab=%lld", (long long)b, (long long)h, (long long)vocab);
  if (ld_hidden < h || ld_w < vocab || ld_logits < vocab) return fail(MJ_GRPO_ERR_SHAPE, "sample_logits: leading dimension smaller than row length");
  if (h % 8 || vocab % 8 || ld_hidden % 8 || ld_w % 8 || ld_logits % 4)
    return fail(MJ_GRPO_ERR_ALIGN, "sample_logits: h, vocab, ld_hidden, ld_w must be multiples of 8 and ld_logits of 4");
  if (misaligned(hidden) || misaligned(lm_head) || misaligned(logits)) return fail(MJ_GRPO_ERR_ALIGN, "sample_logits: pointers must be 16-byte aligned");
  if (!(softcap >= 0.f) || !isfinite(softcap)) return fail(MJ_GRPO_ERR_UNSUPPORTED, "sample_logits: softcap must be >= 0");
  if (ld_w > (1 << 21) || ld_logits > (1 << 21) || ld_hidden > (1 << 20))
    return fail(MJ_GRPO_ERR_SHAPE, "sample_logits: leading dimensions too large (ld_hidden <= 2^20; ld_w, ld_logits <= 2^21)");
  int rc;
  mj::LogitsRowsArgs a;
  a.w = (const __bf16*)lm_head; a.hid = (const __bf16*)hidden; a.ld_w = ld_w; a.ld_hid = ld_hidden;
  a.V = (int)vocab; a.n = (int)b; a.H = (int)h; a.cap = softcap; a.out = logits; a.ld_out = ld_logits;
  // Batch-row tile and vocab columns per work item: the fewest rounds of resident workgroups (one
  // per CU) whose items are <= 256 columns wide.  Measured at 3584 x 152064: the 128-row tile beats
  // both a 64-row tile with two workgroups per CU (0.25 against 0.23 ms at 64 rows) and, past 128
  // rows, is beaten by the 256-row tile (two 128-row tiles: 0.35 against 0.32 ms at 192 rows).
  int bn;
  int64_t tiles_n, tile_rows;
  sample_tiles(b, vocab, &bn, &tiles_n, &tile_rows);
  a.tile_rows = (int)tile_rows;
  const mj::TileMap map = mj::TileMap::pick_shape((int)((vocab + tile_rows - 1) / tile_rows), (int)tiles_n, 1, 1);
  hipStream_t st = (hipStream_t)stream;
  if (bn == 128) {
    if ((rc = enable_lds(mj::k_logits_rows<BM, 128>))) return rc;
    mj::k_logits_rows<BM, 128><<<map.items(), mj::kThreads, mj::GemmTN<BM, 128>::kLdsBytes, st>>>(a, map);
  } else {
    if ((rc = enable_lds(mj::k_logits_rows<BM, BN>))) return rc;
    mj::k_logits_rows<BM, BN><<<map.items(), mj::kThreads, mj::GemmTN<BM, BN>::kLdsBytes, st>>>(a, map);
  }
  return check_launch("k_logits_rows");
}

int mj_sample_top_k(const float* logits, int64_t ld_logits, int64_t b, int64_t vocab, int k, float temperature,
                    const float* noise, int32_t* token, int32_t* top_idx, float* top_val, void* stream) {
  if (!logits || !token) return fail(MJ_GRPO_ERR_NULL, "sample_top_k: logits/token is NULL");
  if (b <= 0 || vocab <= 0 || b > (1 << 24) || vocab > (1 << 30) || ld_logits < vocab)
    return fail(MJ_GRPO_ERR_SHAPE, "sample_top_k: bad shape b=%lld vocab=%lld ld=%lld", (long long)b, (long long)vocab, (long long)ld_logits);
  if (k < 1 || k > mj::kTopKMax || k > vocab) return fail(MJ_GRPO_ERR_UNSUPPORTED, "sample_top_k: k must be in [1, min(%d, vocab)] (got %d)", mj::kTopKMax, k);
  if (!(temperature > 0.f) || !isfinite(temperature)) return fail(MJ_GRPO_ERR_UNSUPPORTED, "sample_top_k: temperature must be > 0");
  mj::TopKArgs a;
  a.logits = logits; a.ld = ld_logits; a.V = (int)vocab; a.k = k; a.t = temperature; a.noise = noise;
  a.token = token; a.top_idx = top_idx; a.top_val = top_val;
  mj::k_topk_sample<<<(unsigned)b, 1024, 0, (hipStream_t)stream>>>(a);
  return check_launch("k_topk_sample");
}

}  // extern "C"

// ----------------------------------------------------------------------------- RMSNorm
namespace {
constexpr int kNormMaxH = 8192;
int norm_grid(int64_t n) {   // workgroups of the backward (one row at a time each, rows with this stride): four per CU
  return (int)(n < 1024 ? n : 1024);
}
int norm_check(int64_t n, int64_t h, std::initializer_list<int64_t> lds, std::initializer_list<const void*> ptrs) {
  if (n <= 0 || h <= 0 || n > (1ll << 30)) return fail(MJ_GRPO_ERR_SHAPE, "rmsnorm: n and h must be positive (got %lld, %lld)", (long long)n, (long long)h);
  if (h % 8 || h > kNormMaxH) return fail(h % 8 ? MJ_GRPO_ERR_ALIGN : MJ_GRPO_ERR_UNSUPPORTED, "rmsnorm: h must be a multiple of 8 and <= %d (got %lld)", kNormMaxH, (long long)h);
  for (int64_t ld : lds) {
    if (ld < h) return fail(MJ_GRPO_ERR_SHAPE, "rmsnorm: leading dimension smaller than h");
    if (ld % 8) return fail(MJ_GRPO_ERR_ALIGN, "rmsnorm: leading dimensions must be multiples of 8");
  }
  for (const void* q : ptrs) {
    if (q == nullptr) return fail(MJ_GRPO_ERR_NULL, "rmsnorm: NULL pointer argument");
    if (misaligned(q)) return fail(MJ_GRPO_ERR_ALIGN, "rmsnorm: pointers must be 16-byte aligned");
  }
  return MJ_GRPO_OK;
}
}  // namespace

extern "C" {

int mj_rmsnorm_forward(const void* x, int64_t ld_x, const float* scale, void* y, int64_t ld_y, float* rstd,
                       int64_t n, int64_t h, float eps, void* stream) {
  int rc = norm_check(n, h, {ld_x, ld_y}, {x, scale, y});
  if (rc) return rc;
  mj::NormFwdArgs a;
  a.x = (const uint16_t*)x; a.scale = scale; a.y = (uint16_t*)y; a.rstd = rstd;
  a.ld_x = ld_x; a.ld_y = ld_y; a.n = (int)n; a.H = (int)h; a.eps = eps;
  const unsigned grid = (unsigned)((n + 3) / 4);
  if (h <= 4096) mj::k_rmsnorm_fwd<8><<<grid, 256, 0, (hipStream_t)stream>>>(a);
  else mj::k_rmsnorm_fwd<16><<<grid, 256, 0, (hipStream_t)stream>>>(a);
  return check_launch("k_rmsnorm_fwd");
}

int mj_rmsnorm_workspace_bytes(int64_t n, int64_t h, size_t* bytes) {
  int rc = norm_check(n, h, {}, {});
  if (rc) return rc;
  if (bytes) *bytes = (size_t)norm_grid(n) * (size_t)h * 4;
  return MJ_GRPO_OK;
}

int mj_rmsnorm_backward(const void* dy, int64_t ld_dy, const void* x, int64_t ld_x, const float* scale, void* dx,
                        int64_t ld_dx, float* dscale, int accumulate_dscale, int64_t n, int64_t h, float eps,
                        void* workspace, size_t workspace_bytes, void* stream) {
  int rc = norm_check(n, h, {ld_dy, ld_x, ld_dx}, {dy, x, scale, dx, workspace});
  if (rc) return rc;
  if (dscale == nullptr) return fail(MJ_GRPO_ERR_NULL, "rmsnorm: dscale is NULL");
  if (misaligned(dscale)) return fail(MJ_GRPO_ERR_ALIGN, "rmsnorm: pointers must be 16-byte aligned");
  const int grid = norm_grid(n);
  const size_t need = (size_t)grid * (size_t)h * 4;
  if (workspace_bytes < need) return fail(MJ_GRPO_ERR_WORKSPACE, "rmsnorm: workspace too small: %zu < %zu bytes", workspace_bytes, need);
  mj::NormBwdArgs a;
  a.dy = (const uint16_t*)dy; a.x = (const uint16_t*)x; a.scale = scale; a.dx = (uint16_t*)dx;
  a.part = (float*)workspace; a.ld_dy = ld_dy; a.ld_x = ld_x; a.ld_dx = ld_dx; a.n = (int)n; a.H = (int)h; a.eps = eps;
  hipStream_t st = (hipStream_t)stream;
  if (h <= 2048) mj::k_rmsnorm_bwd<1><<<grid, 256, 0, st>>>(a);
  else if (h <= 4096) mj::k_rmsnorm_bwd<2><<<grid, 256, 0, st>>>(a);
  else mj::k_rmsnorm_bwd<4><<<grid, 256, 0, st>>>(a);
  if ((rc = check_launch("k_rmsnorm_bwd"))) return rc;
  mj::k_rmsnorm_dscale<<<(unsigned)((h + 63) / 64), 256, 0, st>>>((const float*)workspace, grid, (int)h, dscale,
                                                                  accumulate_dscale);
  return check_launch("k_rmsnorm_dscale");
}

}  // extern "C"

// Explicit instantiations of the tile kernels used above.
template __global__ void mj::k_logits_stats<256, 256, mj::kStatsExp, false, false>(mj::LogitsArgs, mj::TileMap);
template __global__ void mj::k_logits_stats<256, 256, mj::kStatsExp, false, true>(mj::LogitsArgs, mj::TileMap);
template __global__ void mj::k_logits_stats<256, 256, mj::kStatsMax, false, false>(mj::LogitsArgs, mj::TileMap);
template __global__ void mj::k_logits_stats<256, 256, mj::kStatsMax, false, true>(mj::LogitsArgs, mj::TileMap);
template __global__ void mj::k_logits_stats<256, 256, mj::kStatsMax, true, false>(mj::LogitsArgs, mj::TileMap);
template __global__ void mj::k_logits_stats<256, 256, mj::kStatsMax, true, true>(mj::LogitsArgs, mj::TileMap);
template __global__ void mj::k_logits_stats<256, 256, mj::kStatsGrad, false, false>(mj::LogitsArgs, mj::TileMap);
template __global__ void mj::k_logits_stats<256, 256, mj::kStatsGrad, false, true>(mj::LogitsArgs, mj::TileMap);
template __global__ void mj::k_dhidden<256, 256>(mj::DhArgs, mj::TileMap);
template __global__ void mj::k_dw<256, 256, false>(mj::DwArgs, mj::TileMap);
template __global__ void mj::k_dw<256, 256, true>(mj::DwArgs, mj::TileMap);
template __global__ void mj::k_logits_rows<256, 256>(mj::LogitsRowsArgs, mj::TileMap);
template __global__ void mj::k_logits_rows<256, 128>(mj::LogitsRowsArgs, mj::TileMap);
