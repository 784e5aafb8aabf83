"""CPU oracle for the fused GRPO loss path.  TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg may import
this module; the product package never does.

It restates, on flattened tokens and in float64 NumPy, the arithmetic of the
reference's un-fused jnp loss:

  MLLM_JAX/train_modules/__init__.py:118-192   (logp, entropy, ratio/clip, loss)
  MLLM_JAX/language/qwen2/modular_qwen2.py:182 (logits = hidden @ lm_head[H,V])
  deprecated/MLLM_JAX/language/gemma/transformer.py:337-339 (final-logit softcap)
  plugins/training/update/train_step.py:15-24  (value_and_grad -> closed-form backward)
  plugins/training/advantage/grpo.py:28-52     (group-normalised advantages)
  plugins/training/advantage/estimators.py     (global / RLOO / DAPO / REINFORCE++ / GAE)
  plugins/training/ppo/module.py:59-150        (actor-critic twin: policy + value + entropy bonus)
  plugins/sft/jax/sft_module.py:22-45          (masked cross-entropy)
  MLLM_JAX/language/llama/llama.py:426-452     (RMSNorm producing `hidden`)
  MLLM_JAX/sample/sanple_utils.py:35-60        (top-k / categorical draw of the sampler)

The arithmetic itself lives in un-vendored JAX (jax.nn.log_softmax, jax.nn.softmax,
jnp.take_along_axis, jnp.clip, jnp.minimum, jax.value_and_grad; version unpinned in
the reference's requirements-tpu.txt:8-20, docs name jax 0.8.2).  JAX is not
installable here, and the reference holds no golden vector for this path, so the
restatement is pinned by what the mathematics fixes (tests/test_oracle_*.py):
scipy.special.log_softmax/logsumexp, closed forms (uniform logits, on-policy loss),
the six clip regions enumerated by hand, torch.autograd in float64 and central
finite differences for the backward, softcap limits, permutation invariance.

Parity unpinned (documented, accepted):
  * jax.random's threefry stream behind jax.random.categorical: the draw is restated as
    argmax(x + Gumbel noise) with the noise an input; which token a given JAX key yields is
    not reproduced.
  * XLA's bf16 rounding of logits under the Qwen dtype policy
    (modular_qwen2.py:143, llama.py:255-256) is deliberately not replicated: the
    oracle keeps float64 logits of bf16-valued inputs.
  * JAX's half-gradient tie rule exactly at ratio == 1-eps_low / 1+eps_high
    (lax.min / lax.clip JVP); the closed form here takes the full unclipped
    gradient on the closed interval.
  * How jax.lax.top_k orders -0 against +0 and where it puts NaNs: restated with the IEEE total
    order of XLA's sort comparators (-0 < +0, NaN largest); only an import could confirm it.
  * Target ids outside [0, V): jnp.take_along_axis wraps negative ids and yields NaN
    past V; the oracle is only ever called with ids in range (the kernels clamp such
    ids, and their tests compare against the oracle on the clamped ids).
"""
from __future__ import annotations

import numpy as np


# --------------------------------------------------------------------------- logits
def lm_head_logits(hidden, lm_head, softcap=None):
    """z = hidden[N,H] @ lm_head[H,V] (modular_qwen2.py:182), optional
    z = cap*tanh(z/cap) (gemma/transformer.py:337-339).  float64."""
    z = np.asarray(hidden, np.float64) @ np.asarray(lm_head, np.float64)
    if softcap:
        z = float(softcap) * np.tanh(z / float(softcap))
    return z


def _logsumexp(z):
    m = z.max(axis=-1, keepdims=True)
    return (m + np.log(np.exp(z - m).sum(axis=-1, keepdims=True)))[..., 0]


# --------------------------------------------------------------------------- forward
def token_logps_and_entropy(z, target_ids, temperature=1.0):
    """train_modules/__init__.py:124-126 and :136-138 on logits z[N,V].

    logp  = log_softmax(z)[t, y_t] / T        (division AFTER the log-softmax)
    probs = softmax(z / T);  H_t = -sum(probs * log(probs + 1e-9))
    Returns (logp[N], lse[N], token_entropy[N])."""
    z = np.asarray(z, np.float64)
    n = z.shape[0]
    y = np.asarray(target_ids).astype(np.int64)
    lse = _logsumexp(z)
    logp = (z[np.arange(n), y] - lse) / float(temperature)
    zt = z / float(temperature)
    p = np.exp(zt - _logsumexp(zt)[:, None])
    ent = -(p * np.log(p + 1e-9)).sum(axis=-1)
    return logp, lse, ent


def sequence_entropy_stats(token_entropy, mask, seq_shape):
    """train_modules/__init__.py:141-157: per-sample masked mean entropy and the
    'tokens 4..100 of the completion' truncated mean.  Empty rows give nan (the
    reference divides by zero there too)."""
    b, t = seq_shape
    ent = np.asarray(token_entropy, np.float64).reshape(b, t)
    m = np.asarray(mask).reshape(b, t)
    mf = m.astype(np.float64)
    with np.errstate(invalid="ignore", divide="ignore"):
        avg = (ent * mf).sum(-1) / mf.sum(-1)
        valid = (m == 1)
        cum = np.cumsum(valid, axis=-1)
        win = valid & (cum >= 4) & (cum <= 100)
        avg_trunc = (ent * win).sum(-1) / win.sum(-1)
    return avg, avg_trunc


def policy_loss_terms(logp, old_logp, advantages, mask, total_valid_token_count,
                      eps_low, eps_high):
    """train_modules/__init__.py:161-180.  Returns (loss, dloss/dlogp[N]).

    ratio = exp(logp-old); clipped = clip(ratio, 1-eps_low, 1+eps_high)
    loss  = sum(-min(ratio*adv, clipped*adv) * mask) / tvtc
    d/dlogp: -(mask/tvtc)*adv*ratio where the unclipped branch is the active min
    (inside the interval always; above it only for adv<0; below it only for adv>0)."""
    logp = np.asarray(logp, np.float64)
    old = logp if old_logp is None else np.asarray(old_logp, np.float64)
    adv = np.asarray(advantages, np.float64)
    m = np.asarray(mask, np.float64)
    lo, hi = 1.0 - float(eps_low), 1.0 + float(eps_high)
    ratio = np.exp(logp - old)
    clipped = np.clip(ratio, lo, hi)
    ptl = -np.minimum(ratio * adv, clipped * adv)
    tv = float(m.sum()) if total_valid_token_count is None else float(total_valid_token_count)
    loss = (ptl * m).sum() / tv
    active = ((ratio >= lo) & (ratio <= hi)) | ((ratio > hi) & (adv < 0)) | ((ratio < lo) & (adv > 0))
    g = -(m / tv) * adv * ratio * active
    return loss, g


def grpo_loss(hidden, lm_head, target_ids, old_logps, advantages, mask, *,
              total_valid_token_count=None, epsilon_low=0.2, epsilon_high=0.3,
              temperature=1.0, final_logit_softcap=None, seq_shape=None,
              with_grads=True):
    """Whole path, float64.  Mirrors TrainGRPOModule.__call__'s return dict
    (train_modules/__init__.py:185-192) plus token_entropy/lse and, when asked, the
    closed-form gradients d_hidden[N,H], d_lm_head[H,V] that jax.value_and_grad
    (update/train_step.py:24) yields for the loss."""
    h = np.asarray(hidden, np.float64)
    w = np.asarray(lm_head, np.float64)
    n = h.shape[0]
    y = np.asarray(target_ids).astype(np.int64)
    z_raw = h @ w
    cap = float(final_logit_softcap) if final_logit_softcap else None
    z = cap * np.tanh(z_raw / cap) if cap else z_raw
    logp, lse, ent = token_logps_and_entropy(z, y, temperature)
    adv = np.asarray(advantages, np.float64)
    if seq_shape is not None and adv.shape[0] == seq_shape[0] and adv.shape[0] != n:
        adv = np.repeat(adv, seq_shape[1])          # [B] -> [B,1] broadcast, :173
    loss, g = policy_loss_terms(logp, old_logps, adv, mask, total_valid_token_count,
                                epsilon_low, epsilon_high)
    out = {"loss": loss, "per_token_logps": logp, "lse": lse, "token_entropy": ent}
    if seq_shape is not None:
        out["entropy"], out["entropy_loss"] = sequence_entropy_stats(ent, mask, seq_shape)
    if with_grads:
        p = np.exp(z - lse[:, None])
        dz = -p
        dz[np.arange(n), y] += 1.0
        dz *= (g / float(temperature))[:, None]
        if cap:
            dz *= 1.0 - (z / cap) ** 2              # d tanh = 1 - tanh^2
        out["d_hidden"] = dz @ w.T
        out["d_lm_head"] = h.T @ dz
        out["dlogp"] = g
    return out


def ppo_actor_critic_loss(hidden, lm_head, value_w, value_b, target_ids, old_logps, advantages, mask, *,
                          returns=None, old_values=None, total_valid_token_count=None,
                          epsilon_low=0.2, epsilon_high=0.2, value_coef=0.5, value_clip_range=0.2,
                          entropy_coef=0.0, final_logit_softcap=None, with_grads=True):
    """PPOActorCriticModule.__call__ (plugins/training/ppo/module.py:59-150) on flattened,
    already shifted tokens, float64, with closed-form gradients.

      entropy     = sum(H_t * mask) / (sum(mask) + 1e-8)                       (:75-77)
      policy_loss = sum(-min(ratio*adv, clip(ratio)*adv) * mask) / tvtc        (:84-102)
      returns     = advantages + value_pred when absent (NOT detached, :107)
      old_values  = stop_gradient(value_pred) when absent                      (:118)
      value_loss  = sum(max((v-R)^2, (old + clip(v-old, +-c) - R)^2) * mask) / tvtc   (:131-138)
      loss        = policy_loss + value_coef*value_loss - entropy_coef*entropy (:140)

    value_pred = hidden @ value_w + value_b is the Dense(1) of :34-39, :52.  Where the two
    arguments of max() are equal each receives half the cotangent (lax.max's JVP)."""
    h = np.asarray(hidden, np.float64)
    w = np.asarray(lm_head, np.float64)
    wv = np.asarray(value_w, np.float64).reshape(-1)
    bv = float(np.asarray(value_b, np.float64).reshape(()))
    n = h.shape[0]
    y = np.asarray(target_ids).astype(np.int64)
    m = np.asarray(mask, np.float64)
    adv = np.asarray(advantages, np.float64)
    cap = float(final_logit_softcap) if final_logit_softcap else None
    z_raw = h @ w
    z = cap * np.tanh(z_raw / cap) if cap else z_raw
    logp, lse, ent = token_logps_and_entropy(z, y, 1.0)
    cnt = m.sum() + 1e-8
    entropy = (ent * m).sum() / cnt
    tv = float(m.sum()) if total_valid_token_count is None else float(total_valid_token_count)
    policy_loss, g = policy_loss_terms(logp, old_logps, adv, m, tv, epsilon_low, epsilon_high)

    vp = h @ wv + bv
    rt_free = returns is None
    rt = adv + vp if rt_free else np.asarray(returns, np.float64)
    ov = vp.copy() if old_values is None else np.asarray(old_values, np.float64)
    a = (vp - rt) ** 2
    da = 2.0 * (vp - rt) * (0.0 if rt_free else 1.0)
    if value_clip_range is not None:
        c = float(value_clip_range)
        delta = vp - ov
        clipped = ov + np.clip(delta, -c, c)
        inside = (np.abs(delta) <= c).astype(np.float64)
        b = (clipped - rt) ** 2
        db = 2.0 * (clipped - rt) * (inside - (1.0 if rt_free else 0.0))
        vl = np.maximum(a, b)
        dvl = np.where(a > b, da, np.where(a < b, db, 0.5 * (da + db)))
    else:
        vl, dvl = a, da
    value_loss = (vl * m).sum() / tv
    loss = policy_loss + float(value_coef) * value_loss - float(entropy_coef) * entropy
    out = {"loss": loss, "policy_loss": policy_loss, "value_loss": value_loss, "entropy": entropy,
           "value_pred_mean": vp.mean(), "return_mean": rt.mean(), "per_token_logps": logp,
           "token_entropy": ent, "value_pred": vp}
    if with_grads:
        p = np.exp(z - lse[:, None])
        dz = -p
        dz[np.arange(n), y] += 1.0
        dz *= g[:, None]
        # d(-coef*entropy)/dz_j = coef*mask/cnt * p_j * (a_j - sum_i p_i a_i) with
        # a_i = dH/dp_i negated = log(p_i + 1e-9) + p_i/(p_i + 1e-9)
        ai = np.log(p + 1e-9) + p / (p + 1e-9)
        dz += (float(entropy_coef) * m / cnt)[:, None] * p * (ai - (p * ai).sum(-1, keepdims=True))
        if cap:
            dz *= 1.0 - (z / cap) ** 2
        dv = float(value_coef) * dvl * m / tv
        out["d_hidden"] = dz @ w.T + dv[:, None] * wv[None, :]
        out["d_lm_head"] = h.T @ dz
        out["d_value_w"] = h.T @ dv
        out["d_value_b"] = dv.sum()
    return out


def rms_norm(x, scale, eps=1e-6, dy=None):
    """LlamaRMSNorm (MLLM_JAX/language/llama/llama.py:438-451), float64:
    y = x * rsqrt(mean(x^2, -1) + eps) * scale.  With dy, also the transpose
    (dx, dscale) that jax.value_and_grad yields:
      gs = dy*scale;  dx = r*gs - x*r^3*mean(gs*x);  dscale = sum_rows dy*x*r."""
    x = np.asarray(x, np.float64)
    s = np.asarray(scale, np.float64)
    r = 1.0 / np.sqrt((x * x).mean(-1, keepdims=True) + float(eps))
    y = x * r * s
    if dy is None:
        return y
    dy = np.asarray(dy, np.float64)
    gs = dy * s
    dx = r * gs - x * r ** 3 * (gs * x).mean(-1, keepdims=True)
    dscale = (dy * x * r).reshape(-1, x.shape[-1]).sum(0)
    return y, dx, dscale


def top_k_sample(logits, k=50, t=0.9, noise=None):
    """_top_k_sampling_batched (MLLM_JAX/sample/sanple_utils.py:35-53) with the categorical draw
    written as argmax(top_logits + Gumbel noise) (what jax.random.categorical evaluates).
    logits [B,V] float32; scaled = logits / float32(t) in float32 (the reference divides, :37); top-k in descending order,
    equal entries by ascending index (jax.lax.top_k); noise [B,k] or None (greedy).
    Returns (token[B], top_idx[B,k], top_val[B,k])."""
    x = np.asarray(logits, np.float32) / np.float32(t)
    b, v = x.shape
    # descending in the IEEE total order (-0 below +0, a NaN with the sign bit clear above +inf), the
    # order XLA's sort comparators give floats; equal keys by ascending index
    bits = x.view(np.uint32)
    key = np.where(bits & np.uint32(0x80000000), ~bits, bits | np.uint32(0x80000000)).astype(np.int64)
    order = np.lexsort((np.broadcast_to(np.arange(v), x.shape), -key), axis=-1)[:, :k]
    top_val = np.take_along_axis(x, order, axis=-1)
    if noise is None:
        pick = np.zeros(b, np.int64)
    else:
        pick = np.argmax(top_val + np.asarray(noise, np.float32), axis=-1)      # first maximum
    return order[np.arange(b), pick].astype(np.int32), order.astype(np.int32), top_val


# --------------------------------------------------------------------------- siblings
def grpo_advantages(rewards, group_ids, eps=1e-4):
    """plugins/training/advantage/grpo.py:28-52: (r - mean_g) / (std_g + eps),
    population std, float32 result."""
    r = np.asarray(rewards, np.float32)
    _, inv = np.unique(np.asarray(group_ids), return_inverse=True)
    ng = int(inv.max()) + 1
    cnt = np.maximum(np.bincount(inv, minlength=ng).astype(np.float32), 1.0)
    mean = np.bincount(inv, weights=r, minlength=ng).astype(np.float32) / cnt
    c = r - mean[inv]
    std = np.sqrt(np.bincount(inv, weights=c * c, minlength=ng).astype(np.float32) / cnt)
    return (c / (std[inv] + float(eps))).astype(np.float32)


def _group_index(group_ids):
    return np.unique(np.asarray(group_ids).reshape(-1), return_inverse=True)[1]


def global_normalized_advantages(rewards, eps=1e-4, clip_range=None):
    """advantage/estimators.py:37-55."""
    r = np.asarray(rewards, np.float32).reshape(-1)
    a = ((r - np.float32(r.mean())) / (np.float32(r.std()) + np.float32(eps))).astype(np.float32)
    return a if clip_range is None else np.clip(a, -clip_range, clip_range)


def rloo_advantages(rewards, group_ids, eps=1e-4, whiten=True, clip_range=None):
    """advantage/estimators.py:58-103: leave-one-out baseline inside each group (group mean for
    singletons), optional whitening over the batch."""
    r = np.asarray(rewards, np.float32).reshape(-1)
    inv = _group_index(group_ids)
    gsum = np.bincount(inv, weights=r).astype(np.float32)[inv]
    cnt = np.bincount(inv).astype(np.float32)[inv]
    base = np.where(cnt > 1, (gsum - r) / np.maximum(cnt - 1, 1), gsum / np.maximum(cnt, 1)).astype(np.float32)
    a = (r - base).astype(np.float32)
    if whiten:
        a = ((a - np.float32(a.mean())) / (np.float32(a.std()) + np.float32(eps))).astype(np.float32)
    return a if clip_range is None else np.clip(a, -clip_range, clip_range)


def dapo_advantages(rewards, group_ids, eps=1e-4, alpha=0.2, clip_range=None):
    """advantage/estimators.py:106-134."""
    a = (grpo_advantages(rewards, group_ids, eps) + np.float32(alpha) * global_normalized_advantages(rewards, eps)).astype(np.float32)
    return a if clip_range is None else np.clip(a, -clip_range, clip_range)


def gae_advantages(rewards, values, completion_mask, gamma=1.0, gae_lambda=0.95, normalize=True, eps=1e-4,
                   clip_range=None):
    """advantage/estimators.py:160-240: (advantages, returns), both [B,T] float32."""
    r = np.asarray(rewards, np.float32).reshape(-1)
    v = np.asarray(values, np.float32)
    m = np.asarray(completion_mask, np.float32)
    b, t = v.shape
    tok = np.zeros_like(m)
    for i in range(b):
        idx = np.nonzero(m[i] > 0)[0]
        if idx.size:
            tok[i, idx[-1]] = r[i]
    adv = np.zeros_like(v)
    gae = np.zeros(b, np.float32); nxt = np.zeros(b, np.float32)
    for k in range(t - 1, -1, -1):
        delta = tok[:, k] + np.float32(gamma) * nxt - v[:, k]
        gae = ((delta + np.float32(gamma) * np.float32(gae_lambda) * gae) * m[:, k]).astype(np.float32)
        adv[:, k] = gae
        nxt = v[:, k] * m[:, k]
    ret = (adv + v).astype(np.float32)
    if normalize and (m > 0).any():
        sel = adv[m > 0]
        adv = np.where(m > 0, (adv - np.float32(sel.mean())) / (np.float32(sel.std()) + np.float32(eps)), 0.0).astype(np.float32)
    if clip_range is not None:
        adv = np.clip(adv, -clip_range, clip_range).astype(np.float32)
    return adv, ret


def sft_cross_entropy(hidden, lm_head, labels, valid, *, with_grads=True):
    """plugins/sft/jax/sft_module.py:22-45 on flattened, already shifted tokens:
    loss = sum(-log_softmax(z)[t,label_t] * valid) / max(sum(valid), 1)."""
    h = np.asarray(hidden, np.float64)
    w = np.asarray(lm_head, np.float64)
    v = np.asarray(valid, np.float64)
    y = np.where(np.asarray(valid).astype(bool), np.asarray(labels), 0).astype(np.int64)
    n = h.shape[0]
    z = h @ w
    lse = _logsumexp(z)
    logp = z[np.arange(n), y] - lse
    denom = max(float(v.sum()), 1.0)
    out = {"loss": (-logp * v).sum() / denom, "token_count": int(v.sum()), "per_token_logps": logp}
    if with_grads:
        dz = np.exp(z - lse[:, None])
        dz[np.arange(n), y] -= 1.0
        dz *= (v / denom)[:, None]
        out["d_hidden"] = dz @ w.T
        out["d_lm_head"] = h.T @ dz
    return out


# ------------------------------------------------------------- large-shape oracle (torch)
def grpo_loss_chunked_torch(hidden, lm_head, target_ids, old_logps, advantages, mask, *,
                            total_valid_token_count=None, epsilon_low=0.2, epsilon_high=0.3,
                            final_logit_softcap=None, with_grads=True, chunk=1024,
                            dtype=None, rows=None, device="cpu", as_numpy=True):
    """Same arithmetic as grpo_loss (temperature 1) in torch, token-chunked so that
    BASELINE-sized shapes fit in memory.  float32 matmul by default (inputs are bf16-valued,
    so products are exact and only the accumulation rounds), float64 softmax statistics.
    `device` may name the GPU for the full-size configurations: the matmuls are then
    torch's own float32 GEMMs, still independent of the kernels under test.  `rows`
    restricts the work to a subset of token rows while the normaliser stays that of the
    whole batch; d_lm_head is then that subset's share."""
    import torch

    dt = dtype or torch.float32
    dev = torch.device(device)
    h = torch.as_tensor(hidden).to(dev).to(dt)
    w = torch.as_tensor(lm_head).to(dev).to(dt)
    y = torch.as_tensor(target_ids).to(dev).long()
    adv = torch.as_tensor(advantages).to(dev).double()
    m = torch.as_tensor(mask).to(dev).double()
    n = h.shape[0]
    tv = float(m.sum()) if total_valid_token_count is None else float(total_valid_token_count)
    old = None if old_logps is None else torch.as_tensor(old_logps).to(dev).double()
    idx = torch.arange(n, device=dev) if rows is None else torch.as_tensor(rows).to(dev).long()
    cap = float(final_logit_softcap) if final_logit_softcap else None
    lo, hi = 1.0 - float(epsilon_low), 1.0 + float(epsilon_high)
    logp = torch.zeros(n, dtype=torch.float64, device=dev)
    lse = torch.zeros(n, dtype=torch.float64, device=dev)
    ent = torch.zeros(n, dtype=torch.float64, device=dev)
    ptl = torch.zeros(n, dtype=torch.float64, device=dev)
    d_h = torch.zeros(h.shape, dtype=torch.float32, device=dev) if with_grads else None
    d_w = torch.zeros(w.shape, dtype=torch.float32, device=dev) if with_grads else None
    for s in range(0, idx.numel(), chunk):
        r = idx[s:s + chunk]
        z = (h[r] @ w).double()
        if cap:
            z = cap * torch.tanh(z / cap)
        l = torch.logsumexp(z, dim=-1)
        zy = z.gather(1, y[r, None])[:, 0]
        lp = zy - l
        p = torch.exp(z - l[:, None])
        e = -(p * torch.log(p + 1e-9)).sum(-1)
        o = lp if old is None else old[r]
        ratio = torch.exp(lp - o)
        clipped = ratio.clamp(lo, hi)
        a = adv[r]
        ptl[r] = -torch.minimum(ratio * a, clipped * a)
        logp[r], lse[r], ent[r] = lp, l, e
        if with_grads:
            active = ((ratio >= lo) & (ratio <= hi)) | ((ratio > hi) & (a < 0)) | ((ratio < lo) & (a > 0))
            g = -(m[r] / tv) * a * ratio * active
            dz = -p
            dz.scatter_add_(1, y[r, None], torch.ones(len(r), 1, dtype=torch.float64, device=dev))
            dz *= g[:, None]
            if cap:
                dz *= 1.0 - (z / cap) ** 2
            dzf = dz.to(dt)
            d_h[r] = (dzf @ w.T).float()
            d_w += (h[r].T @ dzf).float()
            del dz, dzf
        del z, p
    loss = float((ptl * m).sum() / tv)
    conv = (lambda t: t.cpu().numpy()) if as_numpy else (lambda t: t)
    out = {"loss": loss, "per_token_logps": conv(logp), "lse": conv(lse), "token_entropy": conv(ent)}
    if with_grads:
        out["d_hidden"] = conv(d_h)
        out["d_lm_head"] = conv(d_w)
    return out
