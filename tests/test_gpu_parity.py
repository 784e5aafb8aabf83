"""GPU parity: the HIP path (through the C ABI) against the CPU oracle on identical seeded
inputs.  Tolerances are those of the task statement: per-token log-prob <= 1e-3 absolute,
loss <= 1e-3 relative, gradients <= 2e-2 relative (Frobenius; inputs and dZ are bf16),
entropy <= 1e-3 absolute.
"""
import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O

pytestmark = pytest.mark.gpu

LOGP_ATOL = 1e-3
LOSS_RTOL = 1e-3
GRAD_RTOL = 2e-2
ENT_ATOL = 1e-3


def _dev():
    assert torch.cuda.is_available(), "GPU tests need an MI355X"
    return torch.device("cuda:0")


def _rel(a, b):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def _case(seed, n, h, v, b, w_std=0.3, h_scale=1.0):
    g = torch.Generator().manual_seed(seed)
    hid = (torch.randn(n, h, generator=g) * h_scale).to(torch.bfloat16)
    w = (torch.randn(h, v, generator=g) * w_std).to(torch.bfloat16)
    y = torch.randint(0, v, (n,), generator=g)
    t = n // b
    adv = torch.randn(b, generator=g).repeat_interleave(t)
    lens = torch.randint(1, t + 1, (b,), generator=g)
    mask = (torch.arange(t)[None, :] < lens[:, None]).float().reshape(-1)
    return hid, w, y, adv, mask


def _run(hid, w, y, old, adv, mask, **kw):
    import mllm_jax_amd as M
    d = _dev()
    to = lambda x: None if x is None else torch.as_tensor(x).to(d)
    metrics, (dh, dw) = M.grpo_loss_value_and_grad(to(hid), to(w), to(y), to(old), to(adv), to(mask),
                                                   return_token_entropy=True, **kw)
    torch.cuda.synchronize()
    return ({k: v.detach().float().cpu().numpy() for k, v in metrics.items()},
            dh.float().cpu().numpy(), dw.float().cpu().numpy())


def _check(hid, w, y, old, adv, mask, *, seq_shape=None, chunk_tokens=None, **kw):
    okw = dict(kw)
    ref = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), None if old is None else old.numpy(),
                      adv.numpy(), mask.numpy(), seq_shape=seq_shape, **okw)
    met, dh, dw = _run(hid, w, y, old, adv, mask, seq_shape=seq_shape, chunk_tokens=chunk_tokens, **kw)
    np.testing.assert_allclose(met["per_token_logps"].reshape(-1), ref["per_token_logps"], atol=LOGP_ATOL, rtol=0)
    np.testing.assert_allclose(met["token_entropy"].reshape(-1), ref["token_entropy"], atol=ENT_ATOL, rtol=0)
    assert abs(met["loss"] - ref["loss"]) <= LOSS_RTOL * abs(ref["loss"]) + 1e-7
    if np.linalg.norm(ref["d_hidden"]) > 0:
        assert _rel(dh, ref["d_hidden"]) <= GRAD_RTOL
        assert _rel(dw, ref["d_lm_head"]) <= GRAD_RTOL
    else:
        assert not dh.any() and not dw.any()
    assert not dh[mask.numpy() == 0].any(), "masked tokens must have exactly zero d_hidden rows"
    if seq_shape is not None:
        ok = np.isfinite(ref["entropy"])
        np.testing.assert_allclose(met["entropy"][ok], ref["entropy"][ok], atol=ENT_ATOL)
        ok = np.isfinite(ref["entropy_loss"])
        np.testing.assert_allclose(met["entropy_loss"][ok], ref["entropy_loss"][ok], atol=ENT_ATOL)
    return met, dh, dw, ref


def _old_from(ref_logp, seed, scale=0.05):
    g = torch.Generator().manual_seed(seed)
    return torch.from_numpy(ref_logp).float() + scale * torch.randn(len(ref_logp), generator=g)


def _ref_logp(hid, w, y, **kw):
    return O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), None, np.zeros(len(y)),
                       np.ones(len(y)), with_grads=False, **kw)["per_token_logps"]


@pytest.mark.parametrize("n,h,v,b", [(12, 8, 296, 3), (64, 64, 1000, 4), (300, 136, 2008, 3), (520, 72, 520, 2)])
def test_small_ragged_shapes(n, h, v, b):
    hid, w, y, adv, mask = _case(1, n, h, v, b)
    old = _old_from(_ref_logp(hid, w, y), 2)
    _check(hid, w, y, old, adv, mask, seq_shape=(b, n // b), epsilon_low=0.2, epsilon_high=0.28)


def test_multiple_chunks_and_tvtc_override():
    hid, w, y, adv, mask = _case(3, 700, 64, 1536, 7)
    old = _old_from(_ref_logp(hid, w, y), 4)
    a = _check(hid, w, y, old, adv, mask, chunk_tokens=256, total_valid_token_count=1234.0)
    b = _check(hid, w, y, old, adv, mask, chunk_tokens=None, total_valid_token_count=1234.0)
    # chunking only changes the order of the token-sum in d_lm_head
    assert _rel(a[2], b[2]) < 1e-5
    np.testing.assert_array_equal(a[0]["per_token_logps"], b[0]["per_token_logps"])


def test_on_policy_closed_form():
    hid, w, y, adv, mask = _case(5, 256, 64, 1024, 4)
    met, dh, dw, ref = _check(hid, w, y, None, adv, mask)
    tv = mask.sum().item()
    assert abs(met["loss"] - (-(adv * mask).sum().item() / tv)) < 1e-5


def test_clip_regions():
    hid, w, y, _, _ = _case(6, 128, 64, 512, 2)
    lp = torch.from_numpy(_ref_logp(hid, w, y)).float()
    ratios = torch.tensor([0.5, 0.9, 1.0, 1.25, 1.29, 2.0]).repeat(22)[:128]
    adv = torch.tensor([-1.0, 1.0]).repeat_interleave(64)
    old = lp - torch.log(ratios)
    mask = torch.ones(128)
    for eps in [(0.2, 0.2), (0.2, 0.28), (0.2, 0.3)]:
        _check(hid, w, y, old, adv, mask, epsilon_low=eps[0], epsilon_high=eps[1])


def test_softcap_and_large_logits():
    hid, w, y, adv, mask = _case(7, 200, 64, 1000, 4, w_std=1.5, h_scale=2.0)   # |z| up to ~60: cap bites
    old = _old_from(_ref_logp(hid, w, y, final_logit_softcap=30.0), 8)
    _check(hid, w, y, old, adv, mask, final_logit_softcap=30.0)
    # +80 on one column: running max keeps exp finite
    w2 = w.clone().float()
    w2[:, 17] += 80.0 / hid.float().abs().sum(-1).mean()
    hid2 = hid.abs()
    w2 = w2.to(torch.bfloat16)
    old2 = _old_from(_ref_logp(hid2, w2, y), 9)
    _check(hid2, w2, y, old2, adv, mask)


def test_zero_advantage_and_empty_mask_row():
    hid, w, y, adv, mask = _case(10, 128, 64, 512, 4)
    mask = mask.clone(); mask[:32] = 0           # first sequence has no completion tokens
    met, dh, dw, _ = _check(hid, w, y, None, adv, mask, seq_shape=(4, 32))
    assert np.isnan(met["entropy"][0])            # reference divides by zero there as well
    met, dh, dw, _ = _check(hid, w, y, None, torch.zeros(128), mask)
    assert met["loss"] == 0 and not dw.any()


def test_targets_in_first_last_and_tail_tile():
    hid, w, y, adv, mask = _case(11, 64, 64, 776, 2)    # 776 = 3*256 + 8: last tile holds 8 columns
    y[:8] = 0; y[8:16] = 775; y[16:24] = 768; y[24:32] = 255; y[32:40] = 256
    mask[:] = 1
    _check(hid, w, y, _old_from(_ref_logp(hid, w, y), 12), adv, mask)


def test_column_permutation_invariance():
    hid, w, y, adv, mask = _case(13, 96, 64, 1288, 3)
    g = torch.Generator().manual_seed(14)
    perm = torch.randperm(1288, generator=g)
    inv = torch.argsort(perm)
    a = _run(hid, w, y, None, adv, mask)
    b = _run(hid, w[:, perm].contiguous(), inv[y], None, adv, mask)
    np.testing.assert_allclose(a[0]["per_token_logps"], b[0]["per_token_logps"], atol=2e-5)
    assert _rel(b[2], a[2][:, perm.numpy()]) < 2e-2


def test_forward_only_and_separate_backward_match_fused():
    import ctypes as C
    import mllm_jax_amd as M
    from mllm_jax_amd import _lib
    from mllm_jax_amd.loss import _Prepared, _workspace, _ptr
    d = _dev()
    hid, w, y, adv, mask = _case(15, 520, 64, 1032, 4)
    old = _old_from(_ref_logp(hid, w, y), 16)
    to = lambda x: x.to(d)
    kw = dict(total_valid_token_count=None, epsilon_low=0.2, epsilon_high=0.3, temperature=1.0,
              final_logit_softcap=None, seq_shape=None, chunk_tokens=256)
    p = _Prepared(to(hid), to(w), to(y), to(old), to(adv), to(mask), **kw)
    p.forward()
    torch.cuda.synchronize()
    fwd = (p.logp.clone(), p.lse.clone(), p.ent.clone(), p.loss.clone())
    dh, dw = p.forward_backward()
    torch.cuda.synchronize()
    for a, b in zip(fwd, (p.logp, p.lse, p.ent, p.loss)):
        assert torch.equal(a, b), "forward-only and fused passes must agree bit for bit"
    # separate backward from the saved lse/logp
    _, both = _lib.workspace_bytes(p.desc)
    ws = _workspace(d, both)
    dh2 = torch.empty_like(dh); dw2 = torch.empty_like(dw)
    _lib.check(_lib.load().mj_grpo_backward(
        C.byref(p.desc), _ptr(p.hidden), _ptr(p.w), _ptr(p.targets), _ptr(p.old), _ptr(p.adv), _ptr(p.mask),
        _ptr(p.lse), _ptr(p.logp), _ptr(dh2), _ptr(dw2), _ptr(ws), ws.numel(), p.stream()))
    torch.cuda.synchronize()
    # the fused pass forms dZ as rs * E (E = exp(z) in bf16), the separate backward rounds dZ itself
    # to bf16: same gradient, different roundings
    ref = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), old.numpy(), adv.numpy(), mask.numpy())
    for got_h, got_w in ((dh, dw), (dh2, dw2)):
        assert _rel(got_h.float().cpu().numpy(), ref["d_hidden"]) <= GRAD_RTOL
        assert _rel(got_w[:, :1032].cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
    assert _rel(dh2.float().cpu().numpy(), dh.float().cpu().numpy()) <= 1e-2
    assert _rel(dw2.cpu().numpy(), dw.cpu().numpy()) <= 1e-2


@pytest.mark.parametrize("shift", [100.0, -100.0])
def test_logits_outside_the_exp_window_take_the_rescue_pass(shift):
    """The fast statistics sum exp(z) without a running maximum and are valid while logsumexp stays
    within about +-60.  Here one chunk of three has every logit shifted by +-100 (a rank-one term in
    the hidden states): its range check fails on the device and the running-maximum pass redoes that
    chunk, the other chunks keep the fast results; all of it must match the oracle."""
    n, h, v, b = 768, 64, 1000, 3
    hid, w, y, adv, mask = _case(21, n, h, v, b)
    w = w.float()
    w[0, :] = 1.0                                  # hidden[:, 0] becomes a common offset of the logits
    hid = hid.float()
    hid[:, 0] = 0.0
    hid[256:512, 0] = shift                        # second chunk of 256 tokens only
    hid, w = hid.to(torch.bfloat16), w.to(torch.bfloat16)
    old = _old_from(_ref_logp(hid, w, y), 22)
    met, dh, dw, ref = _check(hid, w, y, old, adv, mask, seq_shape=(b, n // b), chunk_tokens=256,
                              epsilon_low=0.2, epsilon_high=0.28)
    assert abs(ref["lse"][300] - shift) < 15 and abs(ref["lse"][10]) < 15
    # forward-only takes the same decision per chunk: bit-identical outputs
    import mllm_jax_amd as M
    d = _dev()
    with torch.no_grad():
        fwd = M.grpo_fused_loss(hid.to(d), w.to(d), y.to(d), old.to(d), adv.to(d), mask.to(d), chunk_tokens=256,
                                epsilon_low=0.2, epsilon_high=0.28, return_token_entropy=True)
    np.testing.assert_array_equal(fwd["per_token_logps"].cpu().numpy().reshape(-1), met["per_token_logps"].reshape(-1))
    np.testing.assert_array_equal(fwd["token_entropy"].cpu().numpy().reshape(-1), met["token_entropy"].reshape(-1))


@pytest.mark.parametrize("shift,temperature", [(30.0, 0.3), (-30.0, 0.3), (40.0, 2.0)])
def test_tempered_sums_have_their_own_range_check(shift, temperature):
    """T != 1: the entropy's sums run over exp(z / T).  With T = 0.3 a logit offset of +-30 keeps
    sum exp(z) inside the window while exp(z / T) = exp(+-100) overflows or vanishes in float32, so the
    second check must send the chunk to the running-maximum pass; with T = 2 and +40 both sums stay
    inside.  Either way: the oracle."""
    n, h, v, b = 512, 64, 1000, 2
    hid, w, y, adv, mask = _case(23, n, h, v, b)
    w = w.float()
    w[0, :] = 1.0
    hid = hid.float()
    hid[:, 0] = 0.0
    hid[256:, 0] = shift
    hid, w = hid.to(torch.bfloat16), w.to(torch.bfloat16)
    old = _old_from(_ref_logp(hid, w, y, temperature=temperature), 24)
    _check(hid, w, y, old, adv, mask, seq_shape=(b, n // b), chunk_tokens=256, temperature=temperature)


def test_deterministic_and_accumulate():
    import mllm_jax_amd as M
    d = _dev()
    hid, w, y, adv, mask = _case(17, 300, 64, 1000, 3)
    args = [x.to(d) for x in (hid, w, y)] + [None, adv.to(d), mask.to(d)]
    m1, (dh1, dw1) = M.grpo_loss_value_and_grad(*args)
    m2, (dh2, dw2) = M.grpo_loss_value_and_grad(*args)
    assert torch.equal(dh1, dh2) and torch.equal(dw1, dw2) and torch.equal(m1["loss"], m2["loss"])
    acc = dw1.clone().contiguous()
    M.grpo_loss_value_and_grad(*args, accumulate_into=acc)
    assert _rel(acc.cpu().numpy(), 2 * dw1.cpu().numpy()) < 1e-6


def test_autograd_function_and_module_contract():
    import mllm_jax_amd as M
    d = _dev()
    b, l, h, v = 3, 33, 64, 1000
    g = torch.Generator().manual_seed(18)
    hidden = torch.randn(b, l, h, generator=g).to(torch.bfloat16).to(d).requires_grad_(True)
    w32 = (torch.randn(h, v, generator=g) * 0.3).to(torch.bfloat16).float().to(d).requires_grad_(True)
    ids = torch.randint(0, v, (b, l), generator=g).to(d)
    labels = torch.zeros(b, l, dtype=torch.int64); labels[:, 10:25] = 1
    inputs = {"input_ids": ids, "attention_mask": torch.ones(b, l, device=d), "labels": labels.to(d),
              "advantages": torch.tensor([1.0, -0.5, 0.25], device=d),
              "total_valid_token_count": float(labels[:, 1:].sum())}
    mod = M.TrainGRPOModule(model=lambda input_ids, attention_mask: hidden, lm_head=w32,
                            epsilon_low=0.2, epsilon_high=0.3)
    loss, metrics = M.loss_and_metrics(mod, inputs)
    (loss * 2.0).backward()
    assert set(metrics) == {"loss", "entropy", "entropy_loss", "per_token_logps"}
    assert metrics["per_token_logps"].shape == (b, l - 1)
    ref = O.grpo_loss(hidden.detach().float().cpu()[:, :-1].reshape(-1, h).numpy(), w32.detach().cpu().numpy(),
                      ids[:, 1:].reshape(-1).cpu().numpy(), None, inputs["advantages"].cpu().numpy(),
                      labels[:, 1:].reshape(-1).numpy(), seq_shape=(b, l - 1),
                      total_valid_token_count=inputs["total_valid_token_count"])
    assert abs(loss.item() - ref["loss"]) <= 1e-3 * abs(ref["loss"])
    assert w32.grad.dtype == torch.float32
    assert _rel(w32.grad.cpu().numpy(), 2 * ref["d_lm_head"]) <= GRAD_RTOL
    gh = hidden.grad.float().cpu().numpy()
    assert not gh[:, -1].any()
    assert _rel(gh[:, :-1].reshape(-1, h), 2 * ref["d_hidden"]) <= GRAD_RTOL
    # second PPO epoch: old_per_token_logps from the first call (update/ppo.py:39-44)
    inputs["old_per_token_logps"] = metrics["per_token_logps"]
    loss2, _ = M.loss_and_metrics(mod, inputs)
    assert abs(loss2.item() - loss.item()) < 1e-5


def test_sft_cross_entropy():
    import mllm_jax_amd as M
    d = _dev()
    hid, w, y, _, mask = _case(19, 260, 64, 1000, 4)
    ref = O.sft_cross_entropy(hid.float().numpy(), w.float().numpy(), y.numpy(), mask.numpy())
    hd = hid.to(d).requires_grad_(True); wd = w.to(d).requires_grad_(True)
    labels = torch.where(mask.bool(), y, torch.full_like(y, -100))
    out = M.sft_fused_loss(hd, wd, labels.to(d), mask.to(d))
    out["loss"].backward()
    assert abs(out["loss"].item() - ref["loss"]) <= 1e-3 * abs(ref["loss"])
    assert int(out["token_count"]) == ref["token_count"]
    assert _rel(wd.grad.float().cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
    assert _rel(hd.grad.float().cpu().numpy(), ref["d_hidden"]) <= GRAD_RTOL


def test_error_paths_on_device():
    import mllm_jax_amd as M
    from mllm_jax_amd._lib import MjGrpoError
    d = _dev()
    hid, w, y, adv, mask = _case(20, 16, 8, 296, 2)
    with pytest.raises(MjGrpoError):
        M.grpo_fused_loss(hid.to(d), w.to(d), y.to(d), None, adv.to(d), mask.to(d), temperature=0.0)
    with pytest.raises(MjGrpoError):    # vocab not a multiple of 8
        M.grpo_fused_loss(hid.to(d), w[:, :291].contiguous().to(d), y.to(d) % 291, None, adv.to(d), mask.to(d))
    with pytest.raises(RuntimeError):   # CPU tensors: no fallback
        M.grpo_fused_loss(hid, w, y, None, adv, mask)


def test_group_advantages_on_device():
    import mllm_jax_amd as M
    d = _dev()
    # the reference's own known answers for this estimator's siblings use this batch
    # (tests/test_advantage_estimators.py:33-34); the closed form is written out here
    r = np.asarray([1.0, 2.0, 3.0, 10.0, 20.0], np.float32); gid = np.asarray([0, 0, 0, 1, 1], np.int32)
    out = M.compute_grpo_advantages_by_group_id(rewards=torch.tensor(r, device=d), group_ids=torch.tensor(gid), eps=1e-4)
    s0, s1 = np.sqrt(2.0 / 3.0), 5.0
    expect = np.array([-1 / (s0 + 1e-4), 0.0, 1 / (s0 + 1e-4), -5 / (s1 + 1e-4), 5 / (s1 + 1e-4)])
    np.testing.assert_allclose(out.cpu().numpy(), expect, rtol=2e-7, atol=1e-7)
    # ragged groups, non-contiguous ids, a singleton group, against the oracle
    rng = np.random.default_rng(4)
    b = 777
    gid = rng.choice(np.array([-5, 3, 3000, 17, 42, 99999]), size=b).astype(np.int32)
    gid[0] = 123456                                      # singleton: advantage 0
    r = rng.standard_normal(b).astype(np.float32)
    out = M.compute_grpo_advantages_by_group_id(rewards=torch.tensor(r, device=d), group_ids=torch.tensor(gid, device=d))
    np.testing.assert_allclose(out.cpu().numpy(), O.grpo_advantages(r, gid), rtol=1e-6, atol=1e-6)
    assert out[0].item() == 0.0 and out.dtype == torch.float32
    with pytest.raises(ValueError):
        M.compute_grpo_advantages_by_group_id(rewards=torch.zeros(4, device=d), group_ids=torch.zeros(3))


@pytest.mark.parametrize("temp", [0.7, 2.0])
def test_temperature_divides_logp_and_tempers_the_entropy(temp):
    # logp = log_softmax(z)[y] / T, entropy of softmax(z / T) (train_modules/__init__.py:124-126, :136)
    hid, w, y, adv, mask = _case(31, 520, 72, 1544, 4)
    old = torch.from_numpy(_ref_logp(hid, w, y, temperature=temp)).float() + 0.1 * torch.randn(520, generator=torch.Generator().manual_seed(3))
    met, dh, dw, ref = _check(hid, w, y, old, adv, mask, seq_shape=(4, 130), chunk_tokens=256, temperature=temp,
                              epsilon_low=0.2, epsilon_high=0.3)
    plain = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), None, np.zeros(520), np.ones(520), with_grads=False)
    np.testing.assert_allclose(met["per_token_logps"].reshape(-1), plain["per_token_logps"] / temp, atol=1e-3)
    assert np.abs(met["token_entropy"].reshape(-1) - plain["token_entropy"]).max() > 0.05      # it is a different entropy


@pytest.mark.parametrize("b,t", [(3, 4), (5, 37), (4, 64), (7, 130), (2, 1000), (1, 7001)])
def test_sequence_entropy_kernel_against_oracle(b, t):
    """mj_grpo_sequence_entropy (train_modules/__init__.py:141-157) on masks that are not prefixes:
    interleaved zeros, rows with fewer than four valid tokens (window empty: nan), an empty row."""
    from mllm_jax_amd import _lib
    d = _dev()
    g = torch.Generator().manual_seed(100 * b + t)
    ent = torch.rand(b, t, generator=g) * 5
    mask = (torch.rand(b, t, generator=g) < 0.6).float()
    mask[0, :] = 0
    mask[0, : min(3, t)] = 1                      # three valid tokens: the 4..100 window is empty
    if b > 1:
        mask[1, :] = 0                            # empty row
    ref_e, ref_w = O.sequence_entropy_stats(ent.double().numpy().reshape(-1), mask.numpy().reshape(-1), (b, t))
    ent_d, mask_d = ent.to(d), mask.to(d)
    out = torch.empty(2, b, device=d)
    _lib.check(_lib.load().mj_grpo_sequence_entropy(ent_d.data_ptr(), mask_d.data_ptr(), b, t, out[0].data_ptr(),
                                                    out[1].data_ptr(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    got_e, got_w = out[0].cpu().numpy(), out[1].cpu().numpy()
    np.testing.assert_array_equal(np.isnan(got_e), np.isnan(ref_e))
    np.testing.assert_array_equal(np.isnan(got_w), np.isnan(ref_w))
    np.testing.assert_allclose(got_e[~np.isnan(ref_e)], ref_e[~np.isnan(ref_e)], rtol=1e-5)
    np.testing.assert_allclose(got_w[~np.isnan(ref_w)], ref_w[~np.isnan(ref_w)], rtol=1e-5)
    assert np.isnan(got_w[0])


def _shifted_case(seed, shift):
    n, h, v, b = 768, 64, 1000, 3
    hid, w, y, adv, mask = _case(seed, n, h, v, b)
    w = w.float(); w[0, :] = 1.0
    hid = hid.float(); hid[:, 0] = 0.0; hid[256:512, 0] = shift      # second 256-token chunk out of the exp window
    return hid.to(torch.bfloat16), w.to(torch.bfloat16), y, adv, mask, (n, h, v, b)


def test_rescue_pass_with_token_compaction_and_sft():
    """The on-device rescue (running-maximum pass for a chunk whose logsumexp leaves the exp window)
    together with the options that change what the chunk kernels see: compacted tokens, the SFT flag."""
    import mllm_jax_amd as M
    d = _dev()
    hid, w, y, adv, mask, (n, h, v, b) = _shifted_case(23, 90.0)
    old = _old_from(_ref_logp(hid, w, y), 24)
    ref = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), old.numpy(), adv.numpy(), mask.numpy())
    met, (dh, dw) = M.grpo_loss_value_and_grad(hid.to(d), w.to(d), y.to(d), old.to(d), adv.to(d), mask.to(d),
                                               chunk_tokens=256, skip_masked=True)
    torch.cuda.synchronize()
    np.testing.assert_allclose(met["per_token_logps"].cpu().numpy().reshape(-1), ref["per_token_logps"], atol=LOGP_ATOL, rtol=0)
    assert abs(met["loss"].item() - ref["loss"]) <= LOSS_RTOL * abs(ref["loss"])
    assert _rel(dh.float().cpu().numpy(), ref["d_hidden"]) <= GRAD_RTOL
    assert _rel(dw.cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
    sref = O.sft_cross_entropy(hid.float().numpy(), w.float().numpy(), y.numpy(), mask.numpy())
    hp, wp = hid.to(d).requires_grad_(), w.to(d).requires_grad_()
    out = M.sft_fused_loss(hp, wp, y.to(d), mask.to(d), chunk_tokens=256)
    out["loss"].backward()
    torch.cuda.synchronize()
    assert abs(out["loss"].item() - sref["loss"]) <= LOSS_RTOL * abs(sref["loss"])
    assert _rel(hp.grad.float().cpu().numpy(), sref["d_hidden"]) <= GRAD_RTOL
    assert _rel(wp.grad.float().cpu().numpy(), sref["d_lm_head"]) <= GRAD_RTOL


def test_rescue_pass_in_the_workspace_free_forward():
    import ctypes as C
    from mllm_jax_amd import _lib
    d = _dev()
    hid, w, y, adv, mask, (n, h, v, b) = _shifted_case(25, -95.0)
    ref = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), None, adv.numpy(), mask.numpy(), with_grads=False)
    desc = _lib.MjGrpoDesc()
    desc.n_tokens, desc.hidden, desc.vocab, desc.ld_hidden, desc.ld_w, desc.chunk_tokens = n, h, v, h, v, 256
    desc.eps_low, desc.eps_high, desc.temperature = 0.2, 0.3, 1.0
    desc.inv_total_valid_tokens, desc.grad_loss_scale = 1.0 / float(mask.sum()), 1.0
    t = lambda x, dt: x.to(d).to(dt).contiguous()
    hid_d, w_d, y_d, adv_d, mask_d = t(hid, torch.bfloat16), t(w, torch.bfloat16), t(y, torch.int32), t(adv, torch.float32), t(mask, torch.float32)
    logp, lse, ent = (torch.empty(n, device=d) for _ in range(3))
    loss = torch.empty(2, device=d)
    _lib.check(_lib.load().mj_grpo_forward_noalloc(C.byref(desc), hid_d.data_ptr(), w_d.data_ptr(), y_d.data_ptr(), None,
                                                   adv_d.data_ptr(), mask_d.data_ptr(), logp.data_ptr(), lse.data_ptr(),
                                                   ent.data_ptr(), loss.data_ptr(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    np.testing.assert_allclose(logp.cpu().numpy(), ref["per_token_logps"], atol=LOGP_ATOL, rtol=0)
    np.testing.assert_allclose(lse.cpu().numpy(), ref["lse"], atol=2e-3, rtol=0)
    assert abs(loss[0].item() - ref["loss"]) <= LOSS_RTOL * abs(ref["loss"]) + 1e-7
