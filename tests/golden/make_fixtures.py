"""Writes the small golden fixtures of tests/golden/ from the float64 CPU oracle.

The reference repository holds no golden vector for the GRPO loss path (its tests never
touch TrainGRPOModule) and JAX cannot be imported in this environment, so these vectors
come from oracle/grpo_oracle.py, whose formulas tests/test_oracle_pins.py pins against
scipy, closed forms, float64 autograd and finite differences.  They freeze the oracle's
answers on fixed bf16-valued inputs so that a later change of the oracle or of the kernels
shows up as a diff against committed data.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import grpo_oracle as O  # noqa: E402


def bf16(x):
    return torch.from_numpy(np.asarray(x, np.float32)).to(torch.bfloat16).float().numpy()


CASES = {
    # name: (B, T, H, V, eps_low, eps_high, softcap, old_noise)
    "grpo_3x4_h8_v296": (3, 4, 8, 296, 0.2, 0.3, None, 0.05),
    "grpo_2x24_h64_v1000_clip": (2, 24, 64, 1000, 0.2, 0.28, None, 0.4),
    "grpo_4x8_h16_v520_softcap30": (4, 8, 16, 520, 0.2, 0.2, 30.0, 0.05),
    "grpo_onpolicy_2x16_h32_v776": (2, 16, 32, 776, 0.2, 0.3, None, None),
}


def make(name, b, t, h, v, el, eh, cap, noise):
    rng = np.random.default_rng(sum(map(ord, name)))
    n = b * t
    scale = 3.0 if cap else 1.0
    hid = bf16(rng.standard_normal((n, h)) * scale)
    w = bf16(rng.standard_normal((h, v)) * (0.3 * scale))
    y = rng.integers(0, v, n).astype(np.int32)
    adv = np.repeat(rng.standard_normal(b), t).astype(np.float32)
    lens = rng.integers(1, t + 1, b)
    mask = (np.arange(t)[None, :] < lens[:, None]).astype(np.float32).reshape(-1)
    old = None
    if noise is not None:
        base = O.grpo_loss(hid, w, y, None, adv, mask, final_logit_softcap=cap, with_grads=False)
        old = (base["per_token_logps"] + noise * rng.standard_normal(n)).astype(np.float32)
    tv = float(mask.sum()) + 3.0          # a global-batch normaliser, not this batch's own count
    out = O.grpo_loss(hid, w, y, old, adv, mask, total_valid_token_count=tv, epsilon_low=el,
                      epsilon_high=eh, final_logit_softcap=cap, seq_shape=(b, t))
    arrays = dict(hidden=hid, lm_head=w, target_ids=y, advantages=adv, mask=mask,
                  seq_shape=np.array([b, t]), total_valid_token_count=np.array(tv),
                  epsilon=np.array([el, eh]), softcap=np.array(cap or 0.0),
                  loss=np.array(out["loss"]), per_token_logps=out["per_token_logps"],
                  token_entropy=out["token_entropy"], entropy=out["entropy"],
                  entropy_loss=out["entropy_loss"], d_hidden=out["d_hidden"].astype(np.float32),
                  d_lm_head=out["d_lm_head"].astype(np.float32))
    if old is not None:
        arrays["old_logps"] = old
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **arrays)


def make_ext():
    """Fixtures of the rows next to the loss (tests/golden/ext/): PPO actor-critic, RMSNorm, top-k draw."""
    ext = os.path.join(HERE, "ext")
    os.makedirs(ext, exist_ok=True)
    rng = np.random.default_rng(777)
    # PPO actor-critic (plugins/training/ppo/module.py:59-150): given returns / old values, entropy bonus
    n, h, v = 40, 16, 296
    hid = bf16(rng.standard_normal((n, h))); w = bf16(rng.standard_normal((h, v)) * 0.3)
    wv = rng.standard_normal(h).astype(np.float32) * 0.2; bv = np.float32(0.1)
    y = rng.integers(0, v, n).astype(np.int32); adv = rng.standard_normal(n).astype(np.float32)
    mask = (rng.random(n) < 0.7).astype(np.float32)
    vp = hid.astype(np.float64) @ wv + bv
    returns = (vp + rng.standard_normal(n)).astype(np.float32)
    old_values = (vp + 0.3 * rng.standard_normal(n)).astype(np.float32)
    base = O.grpo_loss(hid, w, y, None, adv, mask, with_grads=False)
    old = (base["per_token_logps"] + 0.2 * rng.standard_normal(n)).astype(np.float32)
    hyper = dict(epsilon_low=0.2, epsilon_high=0.2, value_coef=0.5, value_clip_range=0.2, entropy_coef=0.05)
    out = O.ppo_actor_critic_loss(hid, w, wv, bv, y, old, adv, mask, returns=returns, old_values=old_values,
                                  total_valid_token_count=31.0, **hyper)
    np.savez_compressed(os.path.join(ext, "ppo_40_h16_v296.npz"), hidden=hid, lm_head=w, value_w=wv, value_b=bv,
                        target_ids=y, old_logps=old, advantages=adv, mask=mask, returns=returns,
                        old_values=old_values, total_valid_token_count=np.array(31.0),
                        hyper=np.array([hyper[k] for k in ("epsilon_low", "epsilon_high", "value_coef",
                                                           "value_clip_range", "entropy_coef")]),
                        **{k: np.asarray(out[k], np.float64) for k in ("loss", "policy_loss", "value_loss", "entropy",
                                                                       "per_token_logps", "d_hidden", "d_lm_head",
                                                                       "d_value_w", "d_value_b")})
    # RMSNorm (MLLM_JAX/language/llama/llama.py:438-451) and its transpose
    x = bf16(rng.standard_normal((9, 136)) * 1.7); sc = (1.0 + 0.3 * rng.standard_normal(136)).astype(np.float32)
    dy = bf16(rng.standard_normal((9, 136)))
    yy, dx, ds = O.rms_norm(x, sc, 1e-6, dy)
    np.savez_compressed(os.path.join(ext, "rmsnorm_9x136.npz"), x=x, scale=sc, dy=dy, eps=np.array(1e-6), y=yy, dx=dx,
                        dscale=ds)
    # top-k draw (MLLM_JAX/sample/sanple_utils.py:35-53) with ties and given Gumbel noise
    lg = np.round(rng.standard_normal((5, 1000)) * 4).astype(np.float32) / 2       # few distinct values: many ties
    noise = rng.gumbel(size=(5, 50)).astype(np.float32)
    tok, idx, val = O.top_k_sample(lg, k=50, t=0.9, noise=noise)
    np.savez_compressed(os.path.join(ext, "topk_5x1000_k50.npz"), logits=lg, noise=noise, k=np.array(50),
                        t=np.array(0.9), token=tok, top_idx=idx, top_val=val)


if __name__ == "__main__":
    for name, args in CASES.items():
        make(name, *args)
        print("wrote", name)
    make_ext()
    print("wrote ext/")
