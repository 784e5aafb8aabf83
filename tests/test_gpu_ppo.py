"""GPU parity of the actor-critic PPO loss (policy + value + entropy bonus): the HIP path
through the host mirror of plugins/training/ppo/module.py:59-150 against the CPU oracle on
identical seeded inputs.  Tolerances as for the GRPO loss: log-prob <= 1e-3 absolute,
scalars <= 1e-3 relative, gradients <= 2e-2 relative (Frobenius).
"""
import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O

pytestmark = pytest.mark.gpu

LOGP_ATOL, LOSS_RTOL, GRAD_RTOL = 1e-3, 1e-3, 2e-2


def _rel(a, b):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def _batch(seed, b, l, h, v, vocab_in=50):
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, vocab_in, (b, l), generator=g)
    emb = (torch.randn(vocab_in, h, generator=g)).to(torch.bfloat16)
    pos = (0.5 * torch.randn(l, h, generator=g)).to(torch.bfloat16)
    w = (0.3 * torch.randn(h, v, generator=g)).to(torch.bfloat16)
    wv = 0.2 * torch.randn(h, generator=g)
    bv = torch.tensor(0.1)
    lens = torch.randint(2, l + 1, (b,), generator=g)
    start = torch.randint(0, 2, (b,), generator=g)
    ar = torch.arange(l)[None, :]
    labels = ((ar >= start[:, None]) & (ar < lens[:, None])).long()
    adv = torch.randn(b, l - 1, generator=g)                   # per-token (GAE) advantages
    return ids, emb, pos, w, wv, bv, labels, adv


def _run_case(seed, b, l, h, v, *, old_noise=0.0, returns=False, old_values=False, adv_per_seq=False,
              tvtc=None, chunk_tokens=None, zero_adv_seqs=(), **hyper):
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    ids, emb, pos, w, wv, bv, labels, adv = _batch(seed, b, l, h, v)
    g = torch.Generator().manual_seed(seed + 1)
    t = l - 1
    for s_ in zero_adv_seqs:
        adv[s_] = 0.0                       # a group whose rewards are all equal: advantages exactly 0
    hidden_cpu = (emb[ids].float() + pos[None].float()).to(torch.bfloat16)        # [b,l,h]
    hid_flat = hidden_cpu[:, :-1].reshape(b * t, h).float().numpy()
    y = ids[:, 1:].reshape(-1).numpy()
    mask = labels[:, 1:].reshape(-1).float().numpy()
    if adv_per_seq:
        adv = adv[:, :1].contiguous()
    adv_flat = adv.expand(b, t).reshape(-1).numpy()
    vp_ref = hid_flat.astype(np.float64) @ wv.double().numpy() + float(bv)
    inputs = {"input_ids": ids.to(dev), "attention_mask": torch.ones(b, l, device=dev), "labels": labels.to(dev),
              "advantages": (adv[:, 0] if adv_per_seq else adv).to(dev)}
    okw = dict(returns=None, old_values=None)
    old = None
    if old_noise:
        lp = O.grpo_loss(hid_flat, w.float().numpy(), y, None, np.zeros(b * t), np.ones(b * t),
                         with_grads=False, final_logit_softcap=hyper.get("final_logit_softcap"))["per_token_logps"]
        old = (torch.from_numpy(lp).float() + old_noise * torch.randn(b * t, generator=g))
        inputs["old_per_token_logps"] = old.reshape(b, t).to(dev)
        old = old.numpy()
    if returns:
        r = torch.from_numpy(vp_ref).float() + torch.randn(b * t, generator=g)
        inputs["returns"] = r.reshape(b, t).to(dev); okw["returns"] = r.numpy()
    if old_values:
        ov = torch.from_numpy(vp_ref).float() + 0.3 * torch.randn(b * t, generator=g)
        inputs["old_values"] = ov.reshape(b, t).to(dev); okw["old_values"] = ov.numpy()
    if tvtc is not None:
        inputs["total_valid_token_count"] = tvtc

    hidden_dev = hidden_cpu.to(dev).requires_grad_()
    w_dev = w.to(dev).requires_grad_()
    wv_dev, bv_dev = wv.to(dev).requires_grad_(), bv.to(dev).requires_grad_()
    module = M.PPOActorCriticModule(lambda input_ids, attention_mask: hidden_dev, w_dev, (wv_dev, bv_dev),
                                    chunk_tokens=chunk_tokens, **hyper)
    out = module(inputs)
    out["loss"].backward()
    torch.cuda.synchronize()

    for k in ("skip_masked", "dhidden_splits"):
        hyper.pop(k, None)
    ohyper = {k: hyper[k] for k in ("epsilon_low", "epsilon_high", "value_coef", "value_clip_range",
                                    "entropy_coef", "final_logit_softcap") if k in hyper}
    ref = O.ppo_actor_critic_loss(hid_flat, w.float().numpy(), wv.numpy(), float(bv), y, old, adv_flat, mask,
                                  total_valid_token_count=tvtc, **okw, **ohyper)
    np.testing.assert_allclose(out["per_token_logps"].cpu().numpy().reshape(-1), ref["per_token_logps"],
                               atol=LOGP_ATOL, rtol=0)
    for k in ("loss", "policy_loss", "value_loss", "entropy", "value_pred_mean", "return_mean"):
        got = float(out[k].detach())
        assert abs(got - ref[k]) <= LOSS_RTOL * abs(ref[k]) + 2e-6, (k, got, ref[k])
    dh = hidden_dev.grad.float().cpu().numpy()
    assert not dh[:, -1].any(), "the last position feeds neither logits[:, :-1] nor values[:, :-1]"
    assert _rel(dh[:, :-1].reshape(b * t, h), ref["d_hidden"]) <= GRAD_RTOL
    assert _rel(w_dev.grad.float().cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
    if np.linalg.norm(ref["d_value_w"]) > 1e-12:
        assert _rel(wv_dev.grad.cpu().numpy(), ref["d_value_w"]) <= GRAD_RTOL
        assert abs(float(bv_dev.grad) - ref["d_value_b"]) <= GRAD_RTOL * abs(ref["d_value_b"]) + 1e-6
    else:
        assert float(wv_dev.grad.abs().max()) <= 1e-6
    return out, ref


def test_defaults_value_loss_is_masked_mean_squared_advantage():
    out, ref = _run_case(3, 3, 41, 64, 1000)
    # returns = adv + v, old_values = sg(v): the value head receives no gradient (module.py:107, :118)
    assert abs(float(out["value_loss"].detach()) - ref["value_loss"]) <= 1e-5 * ref["value_loss"]


@pytest.mark.parametrize("coef", [0.01, 0.5])
def test_entropy_bonus_with_given_returns_and_values(coef):
    _run_case(4, 4, 33, 72, 2008, returns=True, old_values=True, entropy_coef=coef, old_noise=0.05)


def test_off_policy_clipping_tvtc_and_asymmetric_eps():
    _run_case(5, 2, 65, 136, 520, old_noise=0.3, returns=True, old_values=True, tvtc=77.0,
              epsilon_low=0.1, epsilon_high=0.3, value_coef=1.3, entropy_coef=0.02)


def test_no_value_clip_and_per_sequence_advantages():
    _run_case(6, 3, 21, 64, 296, returns=True, value_clip_range=None, adv_per_seq=True, entropy_coef=0.03)


def test_softcap_with_entropy_bonus_across_chunks():
    _run_case(7, 5, 129, 64, 1544, returns=True, old_values=True, entropy_coef=0.05, final_logit_softcap=5.0,
              chunk_tokens=256, old_noise=0.1)


@pytest.mark.parametrize("splits", [1, 4])
def test_value_head_gradient_joins_d_hidden_in_the_product(splits):
    """entropy_coef = 0: the E-based backward; dv * value_w is added in the d_hidden product's own
    epilogue (one split) or in the fixed-order sum of the split partials."""
    _run_case(8, 4, 65, 136, 1000, returns=True, old_values=True, old_noise=0.1, value_coef=0.7,
              dhidden_splits=splits)


def test_value_head_with_skip_masked_and_chunks():
    _run_case(9, 6, 97, 64, 776, returns=True, old_values=True, old_noise=0.1, chunk_tokens=256, skip_masked=True)
    _run_case(10, 3, 41, 64, 520, skip_masked=True, entropy_coef=0.02, returns=True)


def test_skip_masked_keeps_the_critic_gradient_of_zero_advantage_tokens():
    """Advantage exactly 0 (every reward of a GRPO group equal) zeroes the policy gradient of a token
    but not the critic's: with returns given, d value_loss / d value_pred = 2 (v - R) reaches d_hidden
    through dv[t] * value_w, so such tokens must stay in the compacted batch."""
    out, ref = _run_case(11, 4, 65, 64, 776, returns=True, old_values=True, old_noise=0.1, skip_masked=True,
                         zero_adv_seqs=(1, 2))
    rows = np.abs(ref["d_hidden"].reshape(4, 64, 64)[1]).sum(-1)
    assert (rows > 0).any(), "the case must hold zero-advantage tokens with a critic gradient"
    _run_case(12, 4, 33, 64, 520, returns=True, skip_masked=True, zero_adv_seqs=(0, 1, 2, 3), chunk_tokens=256)


def test_value_method_and_no_grad_call_match_the_oracle():
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    b, l, h, v = 3, 33, 72, 520
    ids, emb, pos, w, wv, bv, labels, adv = _batch(12, b, l, h, v)
    hidden = (emb[ids].float() + pos[None].float()).to(torch.bfloat16)
    module = M.PPOActorCriticModule(lambda input_ids, attention_mask: hidden.to(dev), w.to(dev), (wv.to(dev), bv.to(dev)))
    vals = module.value(ids.to(dev), torch.ones(b, l, device=dev))
    ref_v = hidden.double().numpy() @ wv.double().numpy() + float(bv)
    assert tuple(vals.shape) == (b, l) and vals.dtype == torch.float32
    np.testing.assert_allclose(vals.cpu().numpy(), ref_v, atol=1e-4, rtol=1e-5)
    t = l - 1
    g = torch.Generator().manual_seed(13)
    r = torch.from_numpy(ref_v[:, :-1]).float() + torch.randn(b, t, generator=g)
    inputs = {"input_ids": ids.to(dev), "attention_mask": torch.ones(b, l, device=dev), "labels": labels.to(dev),
              "advantages": adv.to(dev), "returns": r.to(dev)}
    with torch.no_grad():
        out = module(inputs)
    ref = O.ppo_actor_critic_loss(hidden[:, :-1].reshape(b * t, h).float().numpy(), w.float().numpy(), wv.numpy(),
                                  float(bv), ids[:, 1:].reshape(-1).numpy(), None, adv.reshape(-1).numpy(),
                                  labels[:, 1:].reshape(-1).float().numpy(), returns=r.reshape(-1).numpy(),
                                  with_grads=False)
    for k in ("loss", "policy_loss", "value_loss", "entropy", "value_pred_mean", "return_mean"):
        assert abs(float(out[k]) - ref[k]) <= LOSS_RTOL * abs(ref[k]) + 2e-6, k
    assert not out["loss"].requires_grad


def test_entropy_only_gradient_through_value_and_grad():
    # zero advantages: the whole gradient is the entropy bonus; masked rows stay exactly zero
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(11)
    n, h, v = 300, 64, 1000
    hid = torch.randn(n, h, generator=g).to(torch.bfloat16)
    w = (0.4 * torch.randn(h, v, generator=g)).to(torch.bfloat16)
    y = torch.randint(0, v, (n,), generator=g)
    mask = (torch.rand(n, generator=g) < 0.7).float()
    metrics, (dh, dw) = M.grpo_loss_value_and_grad(hid.to(dev), w.to(dev), y.to(dev), None, torch.zeros(n, device=dev),
                                                   mask.to(dev), entropy_coef=1.0)
    ref = O.ppo_actor_critic_loss(hid.float().numpy(), w.float().numpy(), np.zeros(h), 0.0, y.numpy(), None,
                                  np.zeros(n), mask.numpy(), value_coef=0.0, entropy_coef=1.0)
    assert abs(float(metrics["loss"]) - ref["loss"]) <= LOSS_RTOL * abs(ref["loss"])
    assert abs(float(metrics["masked_mean_entropy"]) - ref["entropy"]) <= LOSS_RTOL * ref["entropy"]
    dh = dh.float().cpu().numpy()
    assert _rel(dh, ref["d_hidden"]) <= GRAD_RTOL
    assert _rel(dw.cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
    assert not dh[mask.numpy() == 0].any()


def test_separate_backward_refuses_entropy_bonus():
    import ctypes as C
    from mllm_jax_amd import _lib
    lib = _lib.load()
    d = _lib.MjGrpoDesc(n_tokens=64, hidden=64, vocab=512, ld_hidden=64, ld_w=512, eps_low=0.2, eps_high=0.2,
                        temperature=1.0, inv_total_valid_tokens=1.0, grad_loss_scale=1.0, entropy_coef=0.1,
                        inv_entropy_count=1.0 / 64)
    dev = torch.device("cuda:0")
    _, both = _lib.workspace_bytes(d)
    ws = torch.empty(both, dtype=torch.uint8, device=dev)
    buf = torch.zeros(64 * 512, dtype=torch.float32, device=dev)
    p = buf.data_ptr()
    st = lib.mj_grpo_backward(C.byref(d), p, p, p, p, p, p, p, p, p, p, ws.data_ptr(), both, None)
    assert st == 5      # MJ_GRPO_ERR_UNSUPPORTED
    assert b"entropy" in lib.mj_grpo_last_error()


def test_value_head_with_the_rescue_pass():
    """entropy_coef = 0 (E-based backward) with logits far outside the exp window: the running-maximum
    pass takes over on the device; dv * value_w still joins d_hidden."""
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    b, l, h, v = 4, 65, 64, 520
    ids, emb, pos, w, wv, bv, labels, adv = _batch(14, b, l, h, v)
    t = l - 1
    hidden = (emb[ids].float() + pos[None].float())
    w = w.float(); w[0, :] = 1.0
    hidden[..., 0] = 80.0                                    # every logit shifted by +80
    hidden, w = hidden.to(torch.bfloat16), w.to(torch.bfloat16)
    g = torch.Generator().manual_seed(15)
    hid_flat = hidden[:, :-1].reshape(b * t, h).float().numpy()
    vp_ref = hid_flat.astype(np.float64) @ wv.double().numpy() + float(bv)
    r = torch.from_numpy(vp_ref).float() + torch.randn(b * t, generator=g)
    hd, wd = hidden.to(dev).requires_grad_(), w.to(dev).requires_grad_()
    wvd, bvd = wv.to(dev).requires_grad_(), bv.to(dev).requires_grad_()
    module = M.PPOActorCriticModule(lambda input_ids, attention_mask: hd, wd, (wvd, bvd))
    out = module({"input_ids": ids.to(dev), "attention_mask": torch.ones(b, l, device=dev), "labels": labels.to(dev),
                  "advantages": adv.to(dev), "returns": r.reshape(b, t).to(dev)})
    out["loss"].backward()
    torch.cuda.synchronize()
    ref = O.ppo_actor_critic_loss(hid_flat, w.float().numpy(), wv.numpy(), float(bv), ids[:, 1:].reshape(-1).numpy(), None,
                                  adv.reshape(-1).numpy(), labels[:, 1:].reshape(-1).float().numpy(), returns=r.numpy())
    assert abs(ref["lse"].mean() - 80) < 15 if "lse" in ref else True
    assert abs(float(out["loss"].detach()) - ref["loss"]) <= LOSS_RTOL * abs(ref["loss"]) + 2e-6
    assert _rel(hd.grad[:, :-1].reshape(b * t, h).float().cpu().numpy(), ref["d_hidden"]) <= GRAD_RTOL
    assert _rel(wd.grad.float().cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
    assert _rel(wvd.grad.cpu().numpy(), ref["d_value_w"]) <= GRAD_RTOL
