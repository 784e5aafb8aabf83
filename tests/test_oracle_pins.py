"""Pins the CPU oracle (oracle/grpo_oracle.py) against what the mathematics fixes.

The reference holds no golden vector for this path (its tests never touch
TrainGRPOModule), so every check here is independent of the oracle's own formula:
scipy/torch library routines, closed forms, hand-enumerated clip regions, float64
autograd and central finite differences.
"""
import numpy as np
import pytest
import scipy.special as sps
import torch

from oracle import grpo_oracle as O


def _inputs(rng, n=12, h=8, v=37, b=3):
    hid = rng.standard_normal((n, h))
    w = rng.standard_normal((h, v)) * 0.5
    y = rng.integers(0, v, n)
    adv = np.repeat(rng.standard_normal(b), n // b)
    lens = rng.integers(1, n // b + 1, b)
    mask = (np.arange(n // b)[None, :] < lens[:, None]).astype(np.float64).reshape(-1)
    return hid, w, y, adv, mask


def test_logp_matches_scipy_log_softmax(rng):
    hid, w, y, *_ = _inputs(rng)
    z = hid @ w
    logp, lse, _ = O.token_logps_and_entropy(z, y)
    np.testing.assert_allclose(lse, sps.logsumexp(z, axis=-1), rtol=0, atol=1e-12)
    np.testing.assert_allclose(logp, sps.log_softmax(z, axis=-1)[np.arange(len(y)), y], atol=1e-12)


def test_temperature_divides_after_log_softmax(rng):
    # reference quirk: log_softmax(z)[y] / T, but entropy of softmax(z / T)
    hid, w, y, *_ = _inputs(rng)
    z = hid @ w
    lp1, _, _ = O.token_logps_and_entropy(z, y, 1.0)
    lp2, _, e2 = O.token_logps_and_entropy(z, y, 2.0)
    np.testing.assert_allclose(lp2, lp1 / 2.0, atol=1e-13)
    p = sps.softmax(z / 2.0, axis=-1)
    np.testing.assert_allclose(e2, -(p * np.log(p + 1e-9)).sum(-1), atol=1e-12)


def test_uniform_logits_closed_form():
    v = 151936
    z = np.zeros((3, v))
    logp, lse, ent = O.token_logps_and_entropy(z, np.array([0, 5, v - 1]))
    np.testing.assert_allclose(logp, -np.log(v), atol=1e-12)
    np.testing.assert_allclose(lse, np.log(v), atol=1e-12)
    # -sum p log(p+1e-9) with p = 1/V
    np.testing.assert_allclose(ent, -np.log(1.0 / v + 1e-9), atol=1e-9)
    assert abs(ent[0] - np.log(v)) <= v * 1e-9


def test_dominant_logit_limit():
    z = np.full((1, 50), -40.0)
    z[0, 7] = 40.0
    logp, _, ent = O.token_logps_and_entropy(z, np.array([7]))
    assert abs(logp[0]) < 1e-12 and abs(ent[0]) < 1e-6


def test_stream_entropy_bound(rng):
    # lse - sum p z differs from the reference's -sum p log(p+1e-9) by at most V*1e-9
    hid, w, y, *_ = _inputs(rng, v=296)
    z = hid @ w
    _, lse, ent = O.token_logps_and_entropy(z, y)
    p = sps.softmax(z, axis=-1)
    stream = lse - (p * z).sum(-1)
    assert np.all(stream - ent >= -1e-12) and np.all(stream - ent <= 296 * 1e-9)


@pytest.mark.parametrize("eps", [(0.2, 0.2), (0.2, 0.28), (0.2, 0.3)])
def test_clip_regions_by_hand(eps):
    lo, hi = 1 - eps[0], 1 + eps[1]
    ratios = np.array([0.5, 0.9, 1.0, 1.25, 1.29, 2.0])
    for adv in (-1.0, 1.0):
        logp = np.zeros(6)
        old = -np.log(ratios)
        loss, g = O.policy_loss_terms(logp, old, np.full(6, adv), np.ones(6), 6.0, *eps)
        exp_terms, exp_g = [], []
        for r in ratios:
            if adv > 0:       # A*min(r, clip(r)): capped above
                val = adv * min(r, hi)
                grad_on = r <= hi
            else:             # A*max(r, clip(r)): floored below
                val = adv * max(r, lo)
                grad_on = r >= lo
            exp_terms.append(-val)
            exp_g.append(-(adv * r) / 6.0 if grad_on else 0.0)
        np.testing.assert_allclose(loss, np.sum(exp_terms) / 6.0, atol=1e-12)
        np.testing.assert_allclose(g, exp_g, atol=1e-12)


def test_on_policy_closed_form(rng):
    hid, w, y, adv, mask = _inputs(rng)
    out = O.grpo_loss(hid, w, y, None, adv, mask, seq_shape=(3, 4))
    tv = mask.sum()
    np.testing.assert_allclose(out["loss"], -(adv * mask).sum() / tv, atol=1e-12)
    p = sps.softmax(hid @ w, axis=-1)
    onehot = np.eye(w.shape[1])[y]
    dz = (-(mask * adv) / tv)[:, None] * (onehot - p)
    np.testing.assert_allclose(out["d_hidden"], dz @ w.T, atol=1e-12)
    np.testing.assert_allclose(out["d_lm_head"], hid.T @ dz, atol=1e-12)


def test_mask_tvtc_and_zero_adv(rng):
    hid, w, y, adv, mask = _inputs(rng)
    old = O.grpo_loss(hid, w, y, None, adv, mask)["per_token_logps"] + 0.05 * rng.standard_normal(12)
    a = O.grpo_loss(hid, w, y, old, adv, mask, total_valid_token_count=7.0)
    b = O.grpo_loss(hid, w, y, old, adv, mask, total_valid_token_count=14.0)
    np.testing.assert_allclose(b["loss"], a["loss"] / 2, rtol=1e-13)
    np.testing.assert_allclose(b["d_lm_head"], a["d_lm_head"] / 2, rtol=1e-12, atol=1e-15)
    assert np.all(a["d_hidden"][mask == 0] == 0)
    z = O.grpo_loss(hid, w, y, old, np.zeros(12), mask)
    assert z["loss"] == 0 and not z["d_hidden"].any() and not z["d_lm_head"].any()


def _torch_twin(hid, w, y, old, adv, mask, tv, eps, cap, T=1.0):
    h = torch.tensor(hid, dtype=torch.float64, requires_grad=True)
    ww = torch.tensor(w, dtype=torch.float64, requires_grad=True)
    z = h @ ww
    if cap:
        z = torch.tanh(z / cap) * cap
    lp = torch.log_softmax(z, -1).gather(1, torch.tensor(y)[:, None])[:, 0] / T
    o = lp.detach() if old is None else torch.tensor(old)
    r = torch.exp(lp - o)
    a = torch.tensor(adv)
    ptl = -torch.minimum(r * a, r.clamp(1 - eps[0], 1 + eps[1]) * a)
    loss = (ptl * torch.tensor(mask)).sum() / tv
    loss.backward()
    return loss.item(), lp.detach().numpy(), h.grad.numpy(), ww.grad.numpy()


@pytest.mark.parametrize("cap", [None, 30.0, 2.0])
@pytest.mark.parametrize("T", [1.0, 0.7])
def test_backward_matches_float64_autograd(rng, cap, T):
    hid, w, y, adv, mask = _inputs(rng)
    hid *= 2.0
    base = O.grpo_loss(hid, w, y, None, adv, mask, final_logit_softcap=cap, temperature=T)
    old = base["per_token_logps"] + 0.3 * rng.standard_normal(12)   # wide: hits clip regions
    out = O.grpo_loss(hid, w, y, old, adv, mask, total_valid_token_count=9.0,
                      epsilon_low=0.2, epsilon_high=0.28, final_logit_softcap=cap, temperature=T)
    loss, lp, dh, dw = _torch_twin(hid, w, y, old, adv, mask, 9.0, (0.2, 0.28), cap, T)
    np.testing.assert_allclose(out["loss"], loss, rtol=1e-12)
    np.testing.assert_allclose(out["per_token_logps"], lp, atol=1e-12)
    np.testing.assert_allclose(out["d_hidden"], dh, atol=1e-12)
    np.testing.assert_allclose(out["d_lm_head"], dw, atol=1e-12)
    assert np.abs(out["d_hidden"]).max() > 0


def test_backward_matches_finite_differences(rng):
    hid, w, y, adv, mask = _inputs(rng, n=6, h=4, v=9, b=3)
    old = O.grpo_loss(hid, w, y, None, adv, mask)["per_token_logps"] + 0.05 * rng.standard_normal(6)
    f = lambda hh, ww: O.grpo_loss(hh, ww, y, old, adv, mask, final_logit_softcap=5.0,
                                   with_grads=False)["loss"]
    out = O.grpo_loss(hid, w, y, old, adv, mask, final_logit_softcap=5.0)
    d = 1e-6
    for (i, j) in [(0, 0), (3, 2), (5, 3)]:
        e = np.zeros_like(hid); e[i, j] = d
        np.testing.assert_allclose((f(hid + e, w) - f(hid - e, w)) / (2 * d), out["d_hidden"][i, j], atol=1e-8)
    for (i, j) in [(0, 0), (2, 8), (3, int(y[0]))]:
        e = np.zeros_like(w); e[i, j] = d
        np.testing.assert_allclose((f(hid, w + e) - f(hid, w - e)) / (2 * d), out["d_lm_head"][i, j], atol=1e-8)


def test_dz_rows_sum_to_zero_and_softcap_limit(rng):
    hid, w, y, adv, mask = _inputs(rng)
    a = O.grpo_loss(hid, w, y, None, adv, mask)
    b = O.grpo_loss(hid, w, y, None, adv, mask, final_logit_softcap=1e9)
    np.testing.assert_allclose(a["per_token_logps"], b["per_token_logps"], atol=1e-9)
    np.testing.assert_allclose(a["d_lm_head"], b["d_lm_head"], atol=1e-9)
    # d_lm_head = h^T dz and rows of dz sum to zero  =>  d_lm_head @ 1 = 0
    np.testing.assert_allclose(a["d_lm_head"].sum(-1), 0, atol=1e-12)


def test_column_permutation_invariance(rng):
    hid, w, y, adv, mask = _inputs(rng)
    perm = rng.permutation(w.shape[1])
    inv = np.argsort(perm)
    a = O.grpo_loss(hid, w, y, None, adv, mask)
    b = O.grpo_loss(hid, w[:, perm], inv[y], None, adv, mask)
    np.testing.assert_allclose(a["per_token_logps"], b["per_token_logps"], atol=1e-12)
    np.testing.assert_allclose(a["d_lm_head"][:, perm], b["d_lm_head"], atol=1e-12)


def test_sequence_entropy_stats_by_hand():
    ent = np.arange(1.0, 13.0).reshape(2, 6)
    mask = np.array([[0, 1, 1, 1, 1, 1], [1, 1, 0, 0, 0, 0]])
    avg, trunc = O.sequence_entropy_stats(ent.reshape(-1), mask.reshape(-1), (2, 6))
    np.testing.assert_allclose(avg, [(2 + 3 + 4 + 5 + 6) / 5, (7 + 8) / 2])
    # window = valid tokens whose running valid count is in [4, 100]
    np.testing.assert_allclose(trunc[0], (5 + 6) / 2)
    assert np.isnan(trunc[1])


def test_grpo_advantages_closed_form():
    # advantage/grpo.py:28-52: population std within group, eps 1e-4
    adv = O.grpo_advantages([1, 0, 0, 0, 1, 1], [7, 7, 7, 7, 9, 9])
    m, s = 0.25, np.sqrt(0.1875)
    np.testing.assert_allclose(adv[:4], [(1 - m) / (s + 1e-4)] + [(0 - m) / (s + 1e-4)] * 3, rtol=1e-6)
    np.testing.assert_allclose(adv[4:], 0.0, atol=1e-7)
    assert adv.dtype == np.float32


def test_sft_cross_entropy_vs_torch(rng):
    hid, w, y, _, mask = _inputs(rng)
    out = O.sft_cross_entropy(hid, w, y, mask)
    h = torch.tensor(hid, requires_grad=True); ww = torch.tensor(w, requires_grad=True)
    nll = torch.nn.functional.cross_entropy(h @ ww, torch.tensor(y), reduction="none")
    loss = (nll * torch.tensor(mask)).sum() / max(mask.sum(), 1.0)
    loss.backward()
    np.testing.assert_allclose(out["loss"], loss.item(), rtol=1e-12)
    np.testing.assert_allclose(out["d_lm_head"], ww.grad.numpy(), atol=1e-12)
    np.testing.assert_allclose(out["d_hidden"], h.grad.numpy(), atol=1e-12)


def test_chunked_torch_oracle_matches_float64(rng):
    hid, w, y, adv, mask = _inputs(rng, n=24, h=16, v=200, b=3)
    from conftest import bf16_round
    hid, w = bf16_round(hid), bf16_round(w)
    old = O.grpo_loss(hid, w, y, None, adv, mask)["per_token_logps"] + 0.05 * rng.standard_normal(24)
    a = O.grpo_loss(hid, w, y, old, adv, mask, final_logit_softcap=30.0, epsilon_high=0.2)
    b = O.grpo_loss_chunked_torch(hid, w, y, old, adv, mask, final_logit_softcap=30.0,
                                  epsilon_high=0.2, chunk=7)
    np.testing.assert_allclose(b["loss"], a["loss"], rtol=1e-6)
    np.testing.assert_allclose(b["per_token_logps"], a["per_token_logps"], atol=1e-5)
    np.testing.assert_allclose(b["token_entropy"], a["token_entropy"], atol=1e-5)
    np.testing.assert_allclose(b["d_hidden"], a["d_hidden"], atol=1e-6)
    np.testing.assert_allclose(b["d_lm_head"], a["d_lm_head"], atol=1e-6)


# --------------------------------------------------------------------------- PPO actor-critic
def _ppo_autograd(hid, w, wv, bv, y, old, adv, mask, returns, old_values, tv, el, eh, vc, clip, ec, cap):
    """Library-routine restatement (torch float64 autograd) of the actor-critic loss; written
    against plugins/training/ppo/module.py:66-140, not against the oracle."""
    t = lambda x: torch.tensor(np.asarray(x, np.float64))
    hid_t, w_t, wv_t = t(hid).requires_grad_(), t(w).requires_grad_(), t(wv).requires_grad_()
    bv_t = t(bv).requires_grad_()
    z = hid_t @ w_t
    if cap:
        z = cap * torch.tanh(z / cap)
    lsm = torch.log_softmax(z, -1)
    logp = lsm.gather(-1, torch.tensor(y)[:, None])[:, 0]
    probs = torch.softmax(z, -1)
    ent_t = -(probs * torch.log(probs + 1e-9)).sum(-1)
    m = t(mask)
    entropy = (ent_t * m).sum() / (m.sum() + 1e-8)
    oldt = logp.detach() if old is None else t(old)
    ratio = torch.exp(logp - oldt)
    a = t(adv)
    ppo = torch.minimum(ratio * a, torch.clamp(ratio, 1 - el, 1 + eh) * a)
    tvt = m.sum() if tv is None else tv
    policy = (-ppo * m).sum() / tvt
    vp = hid_t @ wv_t + bv_t
    rt = a + vp if returns is None else t(returns)
    ov = vp.detach() if old_values is None else t(old_values)
    if clip is not None:
        vclipped = ov + torch.clamp(vp - ov, -clip, clip)
        vl = torch.maximum((vp - rt) ** 2, (vclipped - rt) ** 2)
    else:
        vl = (vp - rt) ** 2
    vloss = (vl * m).sum() / tvt
    loss = policy + vc * vloss - ec * entropy
    loss.backward()
    return dict(loss=loss.item(), policy_loss=policy.item(), value_loss=vloss.item(), entropy=entropy.item(),
                d_hidden=hid_t.grad.numpy(), d_lm_head=w_t.grad.numpy(), d_value_w=wv_t.grad.numpy(),
                d_value_b=bv_t.grad.item())


@pytest.mark.parametrize("case", ["defaults", "given_returns_values", "no_clip", "entropy_softcap", "off_policy_tvtc"])
def test_ppo_actor_critic_matches_float64_autograd(rng, case):
    hid, w, y, adv_seq, mask = _inputs(rng)
    n, h = hid.shape
    wv, bv = rng.standard_normal(h) * 0.3, 0.17
    adv = rng.standard_normal(n)                     # per-token advantages (GAE), module.py:87-94
    kw = dict(returns=None, old_values=None, tv=None, el=0.2, eh=0.2, vc=0.5, clip=0.2, ec=0.0, cap=None)
    old = None
    if case == "given_returns_values":
        vp = hid @ wv + bv
        kw.update(returns=vp + rng.standard_normal(n), old_values=vp + 0.3 * rng.standard_normal(n), ec=0.01)
    elif case == "no_clip":
        kw.update(returns=rng.standard_normal(n), clip=None, vc=1.3)
    elif case == "entropy_softcap":
        kw.update(ec=0.05, cap=3.0, returns=rng.standard_normal(n))
    elif case == "off_policy_tvtc":
        z = hid @ w
        old = sps.log_softmax(z, -1)[np.arange(n), y] + 0.25 * rng.standard_normal(n)
        kw.update(tv=23.0, ec=0.02, el=0.1, eh=0.3, old_values=rng.standard_normal(n))
    ref = _ppo_autograd(hid, w, wv, bv, y, old, adv, mask, **kw)
    got = O.ppo_actor_critic_loss(hid, w, wv, bv, y, old, adv, mask, returns=kw["returns"],
                                  old_values=kw["old_values"], total_valid_token_count=kw["tv"],
                                  epsilon_low=kw["el"], epsilon_high=kw["eh"], value_coef=kw["vc"],
                                  value_clip_range=kw["clip"], entropy_coef=kw["ec"],
                                  final_logit_softcap=kw["cap"])
    for k in ("loss", "policy_loss", "value_loss", "entropy", "d_value_b"):
        np.testing.assert_allclose(got[k], ref[k], rtol=1e-10, atol=1e-12, err_msg=k)
    for k in ("d_hidden", "d_lm_head", "d_value_w"):
        np.testing.assert_allclose(got[k], ref[k], rtol=1e-9, atol=1e-12, err_msg=k)


def test_ppo_default_value_loss_is_mean_squared_advantage(rng):
    # returns = adv + v and old_values = sg(v): both branches equal adv^2, whatever the value head is,
    # and the value head receives no gradient (module.py:107, :118, :133-134)
    hid, w, y, _, mask = _inputs(rng)
    n, h = hid.shape
    adv = rng.standard_normal(n)
    out = O.ppo_actor_critic_loss(hid, w, rng.standard_normal(h), 0.4, y, None, adv, mask, value_coef=0.7)
    np.testing.assert_allclose(out["value_loss"], (adv ** 2 * mask).sum() / mask.sum(), rtol=1e-12)
    np.testing.assert_allclose(out["d_value_w"], 0.0, atol=1e-12)
    np.testing.assert_allclose(out["policy_loss"], -(adv * mask).sum() / mask.sum(), rtol=1e-12)   # ratio == 1


def test_ppo_entropy_gradient_finite_differences(rng):
    # only the entropy bonus active: advantages zero, value_coef zero
    hid, w, y, _, mask = _inputs(rng, n=6, h=5, v=11, b=3)
    n, h = hid.shape
    wv = np.zeros(h)
    f = lambda hh, ww: O.ppo_actor_critic_loss(hh, ww, wv, 0.0, y, None, np.zeros(n), mask, value_coef=0.0,
                                               entropy_coef=1.0, with_grads=False)["loss"]
    out = O.ppo_actor_critic_loss(hid, w, wv, 0.0, y, None, np.zeros(n), mask, value_coef=0.0, entropy_coef=1.0)
    np.testing.assert_allclose(out["loss"], -out["entropy"], rtol=1e-12)
    e = 1e-6
    for (i, j) in [(0, 0), (2, 3), (5, 4)]:
        d = np.zeros_like(hid); d[i, j] = e
        np.testing.assert_allclose(out["d_hidden"][i, j], (f(hid + d, w) - f(hid - d, w)) / (2 * e), rtol=1e-5, atol=1e-9)
    for (i, j) in [(0, 0), (3, 7), (4, 10)]:
        d = np.zeros_like(w); d[i, j] = e
        np.testing.assert_allclose(out["d_lm_head"][i, j], (f(hid, w + d) - f(hid, w - d)) / (2 * e), rtol=1e-5, atol=1e-9)


def test_ppo_uniform_policy_has_maximal_entropy_and_no_entropy_gradient():
    v, n, h = 64, 4, 3
    hid = np.ones((n, h)); w = np.zeros((h, v))
    out = O.ppo_actor_critic_loss(hid, w, np.zeros(h), 0.0, np.arange(n), None, np.zeros(n), np.ones(n),
                                  entropy_coef=0.5, value_coef=0.0)
    np.testing.assert_allclose(out["entropy"], np.log(v), atol=1e-6)       # 1e-9 inside the log, module.py:76
    np.testing.assert_allclose(out["d_lm_head"], 0.0, atol=1e-15)


# --------------------------------------------------------------------------- RMSNorm
def test_rms_norm_matches_torch_and_autograd(rng):
    x = rng.standard_normal((5, 24)); s = rng.standard_normal(24); dy = rng.standard_normal((5, 24))
    xt = torch.tensor(x, requires_grad=True); st = torch.tensor(s, requires_grad=True)
    yt = torch.nn.functional.rms_norm(xt, (24,), st, eps=1e-6)
    yt.backward(torch.tensor(dy))
    y, dx, ds = O.rms_norm(x, s, 1e-6, dy)
    np.testing.assert_allclose(y, yt.detach().numpy(), rtol=1e-12, atol=1e-14)
    np.testing.assert_allclose(dx, xt.grad.numpy(), rtol=1e-10, atol=1e-13)
    np.testing.assert_allclose(ds, st.grad.numpy(), rtol=1e-10, atol=1e-13)


def test_rms_norm_closed_forms():
    # a constant row c: y = sign(c) * scale / sqrt(1 + eps / c^2); rescaling x leaves y unchanged as eps -> 0
    s = np.array([1.0, -2.0, 0.5, 3.0])
    y = O.rms_norm(np.full((1, 4), -3.0), s, 1e-6)
    np.testing.assert_allclose(y[0], -s / np.sqrt(1 + 1e-6 / 9.0), rtol=1e-14)
    x = np.array([[1.0, 2.0, -2.0, 4.0]])
    np.testing.assert_allclose(O.rms_norm(x, s, 0.0), O.rms_norm(7.0 * x, s, 0.0), rtol=1e-14)
    np.testing.assert_allclose(O.rms_norm(x, s, 0.0)[0], x[0] / 2.5 * s, rtol=1e-14)   # rms = sqrt(25/4)
    # dx is orthogonal to x when eps = 0 (the norm is scale invariant)
    _, dx, _ = O.rms_norm(x, s, 0.0, np.array([[0.3, -1.0, 2.0, 0.7]]))
    assert abs((dx * x).sum()) < 1e-13


# --------------------------------------------------------------------------- sampler
def test_top_k_sample_against_torch_topk_and_by_hand(rng):
    x = rng.standard_normal((6, 500)).astype(np.float32)
    tok, idx, val = O.top_k_sample(x, k=7, t=0.5, noise=None)
    tv, ti = torch.topk(torch.tensor(x) * np.float32(2.0), 7, dim=-1)            # distinct values: order is unique
    np.testing.assert_array_equal(idx, ti.numpy())
    np.testing.assert_array_equal(val, tv.numpy())
    np.testing.assert_array_equal(tok, x.argmax(-1))                             # greedy = the largest
    # ties go to the lower index; the noise decides among the k
    y = np.array([[1.0, 3.0, 3.0, 0.0, 3.0, 2.0]], np.float32)
    tok, idx, val = O.top_k_sample(y, k=4, t=1.0, noise=np.array([[0.0, 0.0, 5.0, 0.0]], np.float32))
    np.testing.assert_array_equal(idx, [[1, 2, 4, 5]])
    np.testing.assert_array_equal(val, [[3.0, 3.0, 3.0, 2.0]])
    assert tok[0] == 4
    # signed zeros and NaN by hand, in the IEEE total order: -0 below +0, a NaN (sign bit clear) above +inf
    w = np.array([[0.0, -0.0, 1.0, -0.0, 0.0, -1.0]], np.float32)
    _, idx, val = O.top_k_sample(w, k=5, t=1.0, noise=None)
    np.testing.assert_array_equal(idx, [[2, 0, 4, 1, 3]])
    np.testing.assert_array_equal(np.signbit(val), [[False, False, False, True, True]])
    w = np.array([[2.0, np.nan, np.inf, -np.inf, 3.0]], np.float32)
    tok, idx, _ = O.top_k_sample(w, k=3, t=1.0, noise=None)
    np.testing.assert_array_equal(idx, [[1, 2, 4]])
    assert tok[0] == 1
    # Gumbel-max over the top k follows softmax(top_logits): frequencies of a 3-way draw
    z = np.array([[np.log(0.6), np.log(0.3), np.log(0.1), -50.0]], np.float32)
    u = rng.random((20000, 3)); g = -np.log(-np.log(u))
    draws = np.array([O.top_k_sample(z, k=3, t=1.0, noise=g[i:i + 1])[0][0] for i in range(0, 20000, 10)])
    freq = np.bincount(draws, minlength=3) / len(draws)
    np.testing.assert_allclose(freq, [0.6, 0.3, 0.1], atol=0.04)


# --------------------------------------------------------------------------- advantage estimators
# The known answers below are the ones the reference's own tests hold
# (tests/test_advantage_estimators.py:19-106): same inputs, same expected values.
R5 = np.asarray([1.0, 2.0, 3.0, 10.0, 20.0], np.float32)
G5 = np.asarray([0, 0, 0, 1, 1], np.int32)


def test_advantage_estimators_reference_known_answers():
    r4 = np.asarray([0.0, 1.0, 2.0, 3.0], np.float32)
    np.testing.assert_allclose(O.global_normalized_advantages(r4, 1e-4), (r4 - r4.mean()) / (r4.std() + 1e-4), atol=1e-6)
    out = O.global_normalized_advantages(np.asarray([-100.0, 0.0, 100.0], np.float32), 1e-6, clip_range=0.5)
    assert (out <= 0.5).all() and (out >= -0.5).all()
    np.testing.assert_allclose(O.rloo_advantages(R5, G5, eps=1e-6, whiten=False), [-1.5, 0.0, 1.5, -10.0, 10.0], atol=1e-6)
    w = O.rloo_advantages(R5, G5, eps=1e-6, whiten=True)
    assert abs(float(w.mean())) < 1e-5 and float(w.std()) > 0.5
    np.testing.assert_allclose(O.dapo_advantages(R5, G5, 1e-4, 0.5),
                               O.grpo_advantages(R5, G5, 1e-4) + 0.5 * O.global_normalized_advantages(R5, 1e-4), atol=1e-6)
    one = np.ones((1, 3), np.float32)
    adv, ret = O.gae_advantages([1.0], np.zeros((1, 3), np.float32), one, 1.0, 1.0, normalize=False, eps=1e-6)
    np.testing.assert_allclose(adv, one, atol=1e-6); np.testing.assert_allclose(ret, one, atol=1e-6)
    adv, _ = O.gae_advantages([1.0], np.zeros((1, 3), np.float32), np.asarray([[0.0, 1.0, 1.0]], np.float32), 1.0, 1.0,
                              normalize=False, eps=1e-6)
    np.testing.assert_allclose(adv, [[0.0, 1.0, 1.0]], atol=1e-6)


def test_gae_by_hand_with_discount_and_values():
    # one sequence, completion tokens 1..2, reward 2 on the last: delta_2 = 2 - v2, delta_1 = g*v2 - v1
    v = np.asarray([[0.5, 0.2, -0.1, 0.9]], np.float32); m = np.asarray([[0, 1, 1, 0]], np.float32)
    g, lam = 0.9, 0.8
    adv, ret = O.gae_advantages([2.0], v, m, g, lam, normalize=False)
    d2 = 2.0 - (-0.1); d1 = g * (-0.1) - 0.2
    np.testing.assert_allclose(adv, [[0.0, d1 + g * lam * d2, d2, 0.0]], atol=1e-6)
    np.testing.assert_allclose(ret, adv + v, atol=1e-7)


def test_lm_head_logits_against_brute_force_and_tanh_identity(rng):
    """lm_head_logits is hidden @ lm_head with the [in, out] kernel layout (a transposed operand or a
    [V,H] layout fails the brute-force sum), and the softcap is cap*tanh(z/cap): odd, bounded by the
    cap, the identity for |z| << cap."""
    hid = rng.standard_normal((5, 7))
    w = rng.standard_normal((7, 11))
    z = O.lm_head_logits(hid, w)
    brute = np.array([[sum(hid[t, k] * w[k, v] for k in range(7)) for v in range(11)] for t in range(5)])
    np.testing.assert_allclose(z, brute, atol=1e-12)
    np.testing.assert_allclose(z, torch.from_numpy(hid) @ torch.from_numpy(w), atol=1e-12)
    zc = O.lm_head_logits(hid * 20, w, softcap=30.0)
    raw = O.lm_head_logits(hid * 20, w)
    assert np.abs(zc).max() < 30.0 and np.abs(raw).max() > 30.0
    np.testing.assert_allclose(zc, -O.lm_head_logits(-hid * 20, w, softcap=30.0), atol=1e-12)
    np.testing.assert_allclose(O.lm_head_logits(hid * 1e-3, w, softcap=30.0), raw * (1e-3 / 20), rtol=1e-6)
    # inverse: atanh(zc/cap)*cap recovers the raw logits
    np.testing.assert_allclose(np.arctanh(zc / 30.0) * 30.0, raw, rtol=1e-9)


def test_top_k_divides_by_temperature_like_the_reference():
    """sanple_utils.py:37 computes logits / t.  In float32 that differs from logits * (1/t) by an ulp
    for some values, which can reorder near-ties; the oracle must divide."""
    x = np.array([[1.0000001, 1.0, 3.3, 0.7, 2.9000001, 2.9]], np.float32)
    t = np.float32(0.9)
    _, idx, val = O.top_k_sample(x, k=6, t=float(t), noise=None)
    np.testing.assert_array_equal(val[0], np.sort((x / t)[0])[::-1])
    assert val.dtype == np.float32
    # a value where the two formulations differ in the last bit
    xs = np.arange(1, 4097, dtype=np.float32) / np.float32(7.0)
    assert np.any(xs / t != xs * np.float32(1.0 / float(t)))
    _, _, v2 = O.top_k_sample(xs[None, :], k=8, t=float(t), noise=None)
    np.testing.assert_array_equal(v2[0], np.sort(xs / t)[::-1][:8])
