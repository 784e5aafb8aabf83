"""GPU parity with MJ_GRPO_FLAG_SKIP_MASKED: tokens without a gradient are left out of the backward
products; every output must still match the CPU oracle (and the dense pass) to the usual tolerances."""
import ctypes as C

import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O

pytestmark = pytest.mark.gpu

LOGP_ATOL, LOSS_RTOL, GRAD_RTOL, ENT_ATOL = 1e-3, 1e-3, 2e-2, 1e-3


def _rel(a, b):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def _inputs(seed, n, h, v, mask_kind):
    g = torch.Generator().manual_seed(seed)
    hid = torch.randn(n, h, generator=g).to(torch.bfloat16)
    w = (0.3 * torch.randn(h, v, generator=g)).to(torch.bfloat16)
    y = torch.randint(0, v, (n,), generator=g)
    adv = torch.randn(n, generator=g)
    if mask_kind == "interleaved":
        mask = (torch.rand(n, generator=g) < 0.4).float()
    elif mask_kind == "prefix":                     # completion spans: a run of ones per 64-token sequence
        lens = torch.randint(0, 65, (n // 64 + 1,), generator=g)
        mask = (torch.arange(64)[None] < lens[:, None]).float().reshape(-1)[:n]
        adv[: (n // 128) * 64] = 0.0                # whole sequences with advantage exactly 0
    elif mask_kind == "none":
        mask = torch.zeros(n)
    else:
        mask = torch.ones(n)
    ref_lp = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), None, np.zeros(n), np.ones(n),
                         with_grads=False)["per_token_logps"]
    old = torch.from_numpy(ref_lp).float() + 0.1 * torch.randn(n, generator=g)
    return hid, w, y, old, adv, mask


@pytest.mark.parametrize("n,h,v,mask_kind,chunk", [
    (300, 64, 1000, "interleaved", None), (1000, 136, 2008, "prefix", 256), (520, 72, 520, "all", None),
    (260, 64, 296, "none", None), (2048, 64, 1544, "prefix", 512), (64, 64, 512, "interleaved", None)])
def test_skip_masked_matches_oracle_and_dense(n, h, v, mask_kind, chunk):
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    hid, w, y, old, adv, mask = _inputs(n + h, n, h, v, mask_kind)
    to = lambda x: x.to(dev)
    kw = dict(epsilon_low=0.2, epsilon_high=0.28, chunk_tokens=chunk, return_token_entropy=True,
              total_valid_token_count=max(float(mask.sum()), 1.0))
    met_d, (dh_d, dw_d) = M.grpo_loss_value_and_grad(to(hid), to(w), to(y), to(old), to(adv), to(mask), **kw)
    met_s, (dh_s, dw_s) = M.grpo_loss_value_and_grad(to(hid), to(w), to(y), to(old), to(adv), to(mask),
                                                     skip_masked=True, **kw)
    torch.cuda.synchronize()
    ref = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), old.numpy(), adv.numpy(), mask.numpy(),
                      total_valid_token_count=kw["total_valid_token_count"], epsilon_low=0.2, epsilon_high=0.28)
    # the forward covers every token, bit for bit like the dense pass
    assert torch.equal(met_d["per_token_logps"], met_s["per_token_logps"])
    assert torch.equal(met_d["token_entropy"], met_s["token_entropy"])
    np.testing.assert_allclose(met_s["per_token_logps"].cpu().numpy(), ref["per_token_logps"], atol=LOGP_ATOL, rtol=0)
    np.testing.assert_allclose(met_s["token_entropy"].cpu().numpy(), ref["token_entropy"], atol=ENT_ATOL, rtol=0)
    assert abs(float(met_s["loss"]) - ref["loss"]) <= LOSS_RTOL * abs(ref["loss"]) + 1e-7
    dh_s_n, dw_s_n = dh_s.float().cpu().numpy(), dw_s.cpu().numpy()
    dead = (mask.numpy() == 0) | (adv.numpy() == 0)
    assert not dh_s_n[dead].any(), "tokens without a gradient must get exactly zero d_hidden rows"
    assert torch.equal(dh_d, dh_s), "d_hidden rows do not depend on which other tokens are present"
    if np.linalg.norm(ref["d_lm_head"]) > 0:
        assert _rel(dh_s_n, ref["d_hidden"]) <= GRAD_RTOL
        assert _rel(dw_s_n, ref["d_lm_head"]) <= GRAD_RTOL
        assert _rel(dw_s_n, dw_d.cpu().numpy()) <= 1e-3          # same products, other summation order
    else:
        assert not dw_s_n.any() and not dh_s_n.any()


def test_skip_masked_sft_ppo_bonus_and_separate_backward():
    import mllm_jax_amd as M
    from mllm_jax_amd import _lib
    from mllm_jax_amd.loss import _Prepared, _workspace, _ptr
    dev = torch.device("cuda:0")
    n, h, v = 777, 64, 1000
    hid, w, y, old, adv, mask = _inputs(5, n, h, v, "interleaved")
    to = lambda x: x.to(dev)
    # SFT: every unmasked token counts whatever the advantages hold
    out = M.sft_fused_loss(to(hid).requires_grad_(), to(w).requires_grad_(), to(y), to(mask), skip_masked=True)
    ref = O.sft_cross_entropy(hid.float().numpy(), w.float().numpy(), y.numpy(), mask.numpy())
    assert abs(float(out["loss"].detach()) - ref["loss"]) <= LOSS_RTOL * abs(ref["loss"])
    # entropy bonus: zero-advantage tokens still carry the bonus gradient, so only the mask decides
    adv0 = adv.clone(); adv0[:400] = 0.0
    met, (dh, dw) = M.grpo_loss_value_and_grad(to(hid), to(w), to(y), None, to(adv0), to(mask), entropy_coef=0.3,
                                               skip_masked=True)
    refp = O.ppo_actor_critic_loss(hid.float().numpy(), w.float().numpy(), np.zeros(h), 0.0, y.numpy(), None,
                                   adv0.numpy(), mask.numpy(), value_coef=0.0, entropy_coef=0.3, epsilon_high=0.3)
    assert abs(float(met["loss"]) - refp["loss"]) <= LOSS_RTOL * abs(refp["loss"])
    assert _rel(dh.float().cpu().numpy(), refp["d_hidden"]) <= GRAD_RTOL
    assert _rel(dw.cpu().numpy(), refp["d_lm_head"]) <= GRAD_RTOL
    # separate backward from a saved forward, compacted: the fused compacted pass up to the rounding of dZ
    kw = dict(total_valid_token_count=None, epsilon_low=0.2, epsilon_high=0.3, temperature=1.0,
              final_logit_softcap=None, seq_shape=None, chunk_tokens=256, skip_masked=True)
    p = _Prepared(to(hid), to(w), to(y), to(old), to(adv), to(mask), **kw)
    dh1, dw1 = p.forward_backward()
    _, both = _lib.workspace_bytes(p.desc)
    ws = _workspace(dev, both)
    dh2 = torch.empty_like(dh1); dw2 = torch.empty_like(dw1)
    _lib.check(_lib.load().mj_grpo_backward(
        C.byref(p.desc), _ptr(p.hidden), _ptr(p.w), _ptr(p.targets), _ptr(p.old), _ptr(p.adv), _ptr(p.mask),
        _ptr(p.lse), _ptr(p.logp), _ptr(dh2), _ptr(dw2), _ptr(ws), ws.numel(), p.stream()))
    torch.cuda.synchronize()
    assert _rel(dh2.float().cpu().numpy(), dh1.float().cpu().numpy()) <= 1e-2
    assert _rel(dw2.cpu().numpy(), dw1.cpu().numpy()) <= 1e-2
    assert torch.equal(dh1 == 0, dh2 == 0)
