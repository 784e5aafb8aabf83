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


if __name__ == "__main__":
    for name, args in CASES.items():
        make(name, *args)
        print("wrote", name)
