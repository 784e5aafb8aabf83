"""GPU: seeded sweep over combinations of the options of the fused loss (shape, chunking, softcap,
temperature, clip range, on-/off-policy, token compaction, bf16 or float32 lm_head gradient, padded
row pitches, gradient accumulation), each case checked against the CPU oracle to the path's
tolerances.  The single-feature tests elsewhere pin each option; this one looks for interactions."""
import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O
from test_gpu_parity import ENT_ATOL, GRAD_RTOL, LOGP_ATOL, LOSS_RTOL, _case, _old_from, _ref_logp, _rel

pytestmark = pytest.mark.gpu


def _draw(seed):
    r = np.random.default_rng(seed)
    b = int(r.integers(1, 6))
    t = int(r.integers(1, 140))
    h = 8 * int(r.integers(1, 24))
    v = 8 * int(r.integers(8, 300))
    opts = dict(
        chunk_tokens=[None, 256, 512][int(r.integers(0, 3))],
        final_logit_softcap=[None, None, 30.0, 5.0][int(r.integers(0, 4))],
        temperature=[1.0, 1.0, 0.7, 1.6][int(r.integers(0, 4))],
        epsilon_low=[0.2, 0.1][int(r.integers(0, 2))],
        epsilon_high=[0.3, 0.2, 0.28][int(r.integers(0, 3))],
        skip_masked=bool(r.integers(0, 2)),
    )
    extra = dict(off_policy=bool(r.integers(0, 2)), bf16_grad=bool(r.integers(0, 2)),
                 pad_h=8 * int(r.integers(0, 3)), pad_v=8 * int(r.integers(0, 3)),
                 accumulate=bool(r.integers(0, 2)), w_std=[0.3, 1.0][int(r.integers(0, 2))])
    return b, t, h, v, opts, extra


def _wide(x, pad, fill):
    if pad == 0:
        return x
    wide = torch.full((x.shape[0], x.shape[1] + pad), fill, dtype=x.dtype, device=x.device)
    wide[:, : x.shape[1]] = x
    return wide[:, : x.shape[1]]


def _draw_tiny(seed):
    """The same options on shapes far below one tile: 1..3 sequences of 1..8 tokens, hidden 8 or 16, vocab 8..64."""
    _, _, _, _, opts, extra = _draw(seed)
    r = np.random.default_rng(seed + 7)
    return int(r.integers(1, 4)), int(r.integers(1, 9)), 8 * int(r.integers(1, 3)), 8 * int(r.integers(1, 9)), opts, extra


@pytest.mark.parametrize("seed", list(range(100, 124)) + [-s for s in range(3000, 3012)])
def test_option_combinations_against_the_oracle(seed):
    import mllm_jax_amd as M
    b, t, h, v, opts, extra = _draw(seed) if seed >= 0 else _draw_tiny(-seed)
    seed = abs(seed)
    n = b * t
    hid, w, y, adv, mask = _case(seed, n, h, v, b, w_std=extra["w_std"])
    okw = {k: opts[k] for k in ("final_logit_softcap", "temperature", "epsilon_low", "epsilon_high")}
    old = _old_from(_ref_logp(hid, w, y, final_logit_softcap=opts["final_logit_softcap"],
                              temperature=opts["temperature"]), seed + 1) if extra["off_policy"] else None
    ref = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), None if old is None else old.numpy(),
                      adv.numpy(), mask.numpy(), seq_shape=(b, t), **okw)
    dev = torch.device("cuda:0")
    hid_d, w_d = _wide(hid.to(dev), extra["pad_h"], 3.0), _wide(w.to(dev), extra["pad_v"], -2.0)
    gdt = torch.bfloat16 if extra["bf16_grad"] else torch.float32
    acc = start = None
    if extra["accumulate"]:
        g = torch.Generator().manual_seed(seed + 2)
        start = (0.01 * torch.randn(h, v, generator=g)).to(gdt).to(dev)
        acc = _wide(start.clone(), extra["pad_v"], 9.0)
        if extra["pad_v"] == 0:
            acc = acc.contiguous()
    met, (dh, dw) = M.grpo_loss_value_and_grad(
        hid_d, w_d, y.to(dev), None if old is None else old.to(dev), adv.to(dev), mask.to(dev), seq_shape=(b, t),
        return_token_entropy=True, accumulate_into=acc, lm_head_grad_dtype=gdt, **opts)
    torch.cuda.synchronize()
    what = f"seed {seed}: b={b} t={t} h={h} v={v} {opts} {extra}"
    np.testing.assert_allclose(met["per_token_logps"].float().cpu().numpy().reshape(-1), ref["per_token_logps"],
                               atol=LOGP_ATOL, rtol=0, err_msg=what)
    np.testing.assert_allclose(met["token_entropy"].float().cpu().numpy().reshape(-1), ref["token_entropy"],
                               atol=ENT_ATOL, rtol=0, err_msg=what)
    assert abs(met["loss"].item() - ref["loss"]) <= LOSS_RTOL * abs(ref["loss"]) + 1e-7, what
    dwn = dw.float().cpu().numpy() - (start.float().cpu().numpy() if start is not None else 0.0)
    dhn = dh.float().cpu().numpy().reshape(n, h)
    if np.linalg.norm(ref["d_hidden"]) > 0:
        assert _rel(dhn, ref["d_hidden"]) <= GRAD_RTOL, what
        # an accumulator in bf16 rounds start + gradient to 8 bits: its own share of the error
        tol = GRAD_RTOL + (2.0 ** -8 * np.linalg.norm(start.float().cpu().numpy()) / np.linalg.norm(ref["d_lm_head"])
                           if (start is not None and extra["bf16_grad"]) else 0.0)
        assert _rel(dwn, ref["d_lm_head"]) <= tol, what
    else:
        assert not dhn.any() and not np.abs(dwn).max() > 1e-6, what
    assert not dhn[mask.numpy() == 0].any(), what
