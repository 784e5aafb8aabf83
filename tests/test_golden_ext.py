"""Golden fixtures of the rows next to the loss (tests/golden/ext/*.npz): the oracle must reproduce
them on the CPU; the HIP paths must match them on the GPU (floating point within the task's
tolerances, token ids and top-k indices exactly)."""
import os

import numpy as np
import pytest

from oracle import grpo_oracle as O

EXT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "ext")
load = lambda name: dict(np.load(os.path.join(EXT, name), allow_pickle=False))
HYPER = ("epsilon_low", "epsilon_high", "value_coef", "value_clip_range", "entropy_coef")


def test_oracle_reproduces_ext_fixtures():
    d = load("ppo_40_h16_v296.npz")
    out = O.ppo_actor_critic_loss(d["hidden"], d["lm_head"], d["value_w"], d["value_b"], d["target_ids"], d["old_logps"],
                                  d["advantages"], d["mask"], returns=d["returns"], old_values=d["old_values"],
                                  total_valid_token_count=float(d["total_valid_token_count"]),
                                  **dict(zip(HYPER, map(float, d["hyper"]))))
    for k in ("loss", "policy_loss", "value_loss", "entropy", "per_token_logps", "d_hidden", "d_lm_head", "d_value_w"):
        np.testing.assert_allclose(out[k], d[k], rtol=1e-12, atol=1e-14, err_msg=k)
    r = load("rmsnorm_9x136.npz")
    y, dx, ds = O.rms_norm(r["x"], r["scale"], float(r["eps"]), r["dy"])
    np.testing.assert_allclose(y, r["y"], rtol=1e-13); np.testing.assert_allclose(dx, r["dx"], rtol=1e-12, atol=1e-15)
    np.testing.assert_allclose(ds, r["dscale"], rtol=1e-12)
    t = load("topk_5x1000_k50.npz")
    tok, idx, val = O.top_k_sample(t["logits"], k=int(t["k"]), t=float(t["t"]), noise=t["noise"])
    np.testing.assert_array_equal(tok, t["token"]); np.testing.assert_array_equal(idx, t["top_idx"])
    np.testing.assert_array_equal(val, t["top_val"])


@pytest.mark.gpu
def test_hip_paths_match_ext_fixtures():
    import torch
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    rel = lambda a, b: np.linalg.norm(np.asarray(a, np.float64) - b) / max(np.linalg.norm(b), 1e-30)
    # PPO: one sequence of 41 positions whose shifted tokens are the fixture's 40
    d = load("ppo_40_h16_v296.npz")
    n, h = d["hidden"].shape
    hid = torch.zeros(1, n + 1, h, dtype=torch.bfloat16); hid[0, :n] = torch.tensor(d["hidden"]).to(torch.bfloat16)
    ids = torch.zeros(1, n + 1, dtype=torch.long); ids[0, 1:] = torch.tensor(d["target_ids"]).long()
    labels = torch.zeros(1, n + 1); labels[0, 1:] = torch.tensor(d["mask"])
    hid_d = hid.to(dev).requires_grad_(); w_d = torch.tensor(d["lm_head"]).to(torch.bfloat16).to(dev).requires_grad_()
    wv_d = torch.tensor(d["value_w"]).to(dev).requires_grad_(); bv_d = torch.tensor(float(d["value_b"])).to(dev).requires_grad_()
    mod = M.PPOActorCriticModule(lambda input_ids, attention_mask: hid_d, w_d, (wv_d, bv_d),
                                 **dict(zip(HYPER, map(float, d["hyper"]))))
    out = mod({"input_ids": ids.to(dev), "attention_mask": torch.ones(1, n + 1, device=dev), "labels": labels.to(dev),
               "advantages": torch.tensor(d["advantages"])[None].to(dev), "old_per_token_logps": torch.tensor(d["old_logps"])[None].to(dev),
               "returns": torch.tensor(d["returns"])[None].to(dev), "old_values": torch.tensor(d["old_values"])[None].to(dev),
               "total_valid_token_count": float(d["total_valid_token_count"])})
    out["loss"].backward()
    torch.cuda.synchronize()
    for k in ("loss", "policy_loss", "value_loss", "entropy"):
        assert abs(float(out[k].detach()) - d[k]) <= 1e-3 * abs(d[k]) + 1e-6, k
    assert np.abs(out["per_token_logps"].cpu().numpy().reshape(-1) - d["per_token_logps"]).max() <= 1e-3
    assert rel(hid_d.grad[0, :n].float().cpu().numpy(), d["d_hidden"]) <= 2e-2
    assert rel(w_d.grad.float().cpu().numpy(), d["d_lm_head"]) <= 2e-2
    assert rel(wv_d.grad.cpu().numpy(), d["d_value_w"]) <= 2e-2
    # RMSNorm
    r = load("rmsnorm_9x136.npz")
    x = torch.tensor(r["x"]).to(torch.bfloat16).to(dev).requires_grad_(); s = torch.tensor(r["scale"]).to(dev).requires_grad_()
    y = M.rms_norm(x, s, float(r["eps"])); y.backward(torch.tensor(r["dy"]).to(torch.bfloat16).to(dev))
    torch.cuda.synchronize()
    np.testing.assert_allclose(y.detach().float().cpu().numpy(), r["y"], rtol=2 ** -8, atol=1e-6)
    assert rel(x.grad.float().cpu().numpy(), r["dx"]) <= 2e-2 and rel(s.grad.cpu().numpy(), r["dscale"]) <= 2e-3
    # top-k draw: exact
    t = load("topk_5x1000_k50.npz")
    tok, idx, val = M.top_k_sampling_batched(torch.tensor(t["noise"]), torch.tensor(t["logits"]).to(dev), k=int(t["k"]),
                                             t=float(t["t"]), return_top_k=True)
    np.testing.assert_array_equal(tok.cpu().numpy(), t["token"]); np.testing.assert_array_equal(idx.cpu().numpy(), t["top_idx"])
    np.testing.assert_array_equal(val.cpu().numpy(), t["top_val"])
