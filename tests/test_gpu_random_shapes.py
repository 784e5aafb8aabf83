"""GPU parity over seeded random shapes and option combinations (ragged everything): each case
runs the fused pass through the C ABI and is compared with the CPU oracle at the usual tolerances."""
import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O

pytestmark = pytest.mark.gpu


def _rel(a, b):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def _cases(count=36, seed=1234):
    rng = np.random.default_rng(seed)
    for i in range(count):
        n = int(rng.integers(1, 900))
        h = int(rng.integers(1, 40)) * 8
        v = int(rng.integers(1, 400)) * 8
        yield dict(i=i, n=n, h=h, v=v, chunk=int(rng.choice([0, 256, 512])), cap=float(rng.choice([0.0, 0.0, 5.0, 30.0])),
                   old=bool(rng.integers(0, 2)), skip=bool(rng.integers(0, 2)), coef=float(rng.choice([0.0, 0.0, 0.2])),
                   mask_p=float(rng.choice([0.0, 0.3, 0.9, 1.0])), tv=bool(rng.integers(0, 2)), seed=int(rng.integers(1 << 30)))


@pytest.mark.parametrize("c", list(_cases()), ids=lambda c: f"{c['i']}-n{c['n']}h{c['h']}v{c['v']}")
def test_random_case(c):
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(c["seed"])
    n, h, v = c["n"], c["h"], c["v"]
    hid = torch.randn(n, h, generator=g).to(torch.bfloat16)
    w = (torch.randn(h, v, generator=g) * (1.5 / np.sqrt(h))).to(torch.bfloat16)
    y = torch.randint(0, v, (n,), generator=g)
    adv = torch.randn(n, generator=g)
    mask = (torch.rand(n, generator=g) < c["mask_p"]).float()
    cap = c["cap"] or None
    old = None
    if c["old"]:
        lp = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), None, np.zeros(n), np.ones(n),
                         with_grads=False, final_logit_softcap=cap)["per_token_logps"]
        old = torch.from_numpy(lp).float() + 0.2 * torch.randn(n, generator=g)
    tv = float(mask.sum()) + 3.0 if c["tv"] else max(float(mask.sum()), 1.0)
    to = lambda x: None if x is None else x.to(dev)
    met, (dh, dw) = M.grpo_loss_value_and_grad(
        to(hid), to(w), to(y), to(old), to(adv), to(mask), total_valid_token_count=tv, epsilon_low=0.2,
        epsilon_high=0.3, final_logit_softcap=cap, chunk_tokens=c["chunk"] or None, return_token_entropy=True,
        entropy_coef=c["coef"], skip_masked=c["skip"])
    torch.cuda.synchronize()
    ref = O.ppo_actor_critic_loss(hid.float().numpy(), w.float().numpy(), np.zeros(h), 0.0, y.numpy(),
                                  None if old is None else old.numpy(), adv.numpy(), mask.numpy(),
                                  total_valid_token_count=tv, epsilon_low=0.2, epsilon_high=0.3, value_coef=0.0,
                                  entropy_coef=c["coef"], final_logit_softcap=cap)
    np.testing.assert_allclose(met["per_token_logps"].cpu().numpy(), ref["per_token_logps"], atol=1e-3, rtol=0)
    np.testing.assert_allclose(met["token_entropy"].cpu().numpy(), ref["token_entropy"], atol=1e-3, rtol=0)
    assert abs(float(met["loss"]) - ref["loss"]) <= 1e-3 * abs(ref["loss"]) + 1e-6
    dh_n, dw_n = dh.float().cpu().numpy(), dw.cpu().numpy()
    assert np.isfinite(dh_n).all() and np.isfinite(dw_n).all()
    if np.linalg.norm(ref["d_lm_head"]) > 1e-12:
        assert _rel(dh_n, ref["d_hidden"]) <= 2e-2
        assert _rel(dw_n, ref["d_lm_head"]) <= 2e-2
    else:
        assert not dh_n.any() and not dw_n.any()
    assert not dh_n[mask.numpy() == 0].any()
