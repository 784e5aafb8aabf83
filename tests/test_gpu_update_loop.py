"""GPU: the whole update loop (ppo_update over training_step over TrainGRPOModule, all on the
HIP kernels) against a float64 simulation of the same loop built from the CPU oracle:
plugins/training/update/ppo.py:31-44 + update/train_step.py:24-43 with plain SGD as the optimizer."""
import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O
from conftest import bf16_round

pytestmark = pytest.mark.gpu

B, L, H, V, VIN = 8, 33, 64, 1000, 40
LR, ACC, EPOCHS = 2.0, 2, 2


def _data(seed=5):
    g = torch.Generator().manual_seed(seed)
    ids = torch.randint(0, VIN, (B, L), generator=g)
    lens = torch.randint(4, L + 1, (B,), generator=g)
    labels = ((torch.arange(L)[None] >= 2) & (torch.arange(L)[None] < lens[:, None])).long()
    adv = torch.randn(B, generator=g)
    emb = torch.randn(VIN, H, generator=g).to(torch.bfloat16).float()
    w = (0.3 * torch.randn(H, V, generator=g)).to(torch.bfloat16).float()
    return ids, labels, adv, emb, w


def _simulate(ids, labels, adv, emb, w):
    """float64 SGD over the oracle's gradients, same micro-batching, same bf16 view of the parameters."""
    emb, w = emb.double().numpy().copy(), w.double().numpy().copy()
    ids_n, mask_all = ids.numpy(), labels[:, 1:].numpy().astype(np.float64)
    tv = mask_all.sum()
    mb = B // ACC
    old_all, losses = None, []
    for epoch in range(EPOCHS):
        acc_e, acc_w, logps = np.zeros_like(emb), np.zeros_like(w), []
        for i in range(ACC):
            rows = slice(i * mb, (i + 1) * mb)
            x = ids_n[rows]
            hid = bf16_round(emb)[x[:, :-1].reshape(-1)].astype(np.float64)
            old = None if old_all is None else old_all[rows].reshape(-1)
            out = O.grpo_loss(hid, bf16_round(w), x[:, 1:].reshape(-1), old, np.repeat(adv.numpy()[rows], L - 1),
                              mask_all[rows].reshape(-1), total_valid_token_count=tv, epsilon_low=0.2, epsilon_high=0.3)
            np.add.at(acc_e, x[:, :-1].reshape(-1), out["d_hidden"])
            acc_w += out["d_lm_head"]
            logps.append(out["per_token_logps"].reshape(mb, L - 1))
            losses.append(out["loss"])
        emb -= LR * acc_e / ACC
        w -= LR * acc_w / ACC
        if epoch == 0:
            old_all = np.concatenate(logps)
    return emb, w, old_all, losses


@pytest.mark.parametrize("direct", [False, True])
def test_two_epochs_two_micro_batches_match_float64_simulation(direct):
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    ids, labels, adv, emb, w = _data()
    params = {"embed": emb.to(dev).requires_grad_(), "lm_head": w.to(dev).requires_grad_()}

    def apply_fn(p, inputs):
        module = M.TrainGRPOModule(model=lambda input_ids, attention_mask: p["embed"].to(torch.bfloat16)[input_ids],
                                   lm_head=p["lm_head"], epsilon_low=0.2, epsilon_high=0.3)
        return module(inputs)

    state = M.LossTrainState.create(apply_fn=apply_fn, params=params, tx=lambda p, g: {k: p[k] - LR * g[k] for k in p},
                                    grad_accum_steps=ACC, lm_head_key="lm_head" if direct else None)
    datas = {"input_ids": ids.to(dev), "attention_mask": torch.ones(B, L, device=dev), "labels": labels.to(dev),
             "advantages": adv.to(dev)}
    tv = datas["labels"][:, 1:].sum()                                          # runner/grpo_gsm8k.py:770
    losses = []

    def step(st, local):
        st, meta = M.training_step(st, local)
        losses.append(float(meta["loss"]))
        return st, meta

    res = M.PolicyGradientUpdateModule().update(state=state, batch=datas, total_valid_token_count=tv, train_step=step,
                                                grad_accum_steps=ACC, ppo_steps=EPOCHS)
    torch.cuda.synchronize()
    emb_ref, w_ref, old_ref, loss_ref = _simulate(ids, labels, adv, emb, w)
    assert res.state.step == EPOCHS and res.state.micro_step == 0
    np.testing.assert_allclose(res.batch["old_per_token_logps"].cpu().numpy(), old_ref, atol=1e-3, rtol=0)
    np.testing.assert_allclose(losses, loss_ref, rtol=2e-3, atol=1e-6)
    rel = lambda a, b, base: np.linalg.norm(a - b) / np.linalg.norm(b - base)
    d_w = rel(res.state.params["lm_head"].detach().double().cpu().numpy(), w_ref, w.double().numpy())
    d_e = rel(res.state.params["embed"].detach().double().cpu().numpy(), emb_ref, emb.double().numpy())
    assert d_w <= 2e-2 and d_e <= 2e-2, (d_w, d_e)
    # the second epoch is off-policy: its ratios differ from 1, so its losses differ from the first epoch's
    assert abs(losses[2] - losses[0]) > 1e-4
    assert set(res.last_meta) >= {"loss", "entropy", "entropy_loss", "per_token_logps"}
