"""Host logic of the update loop (mllm-jax_amd/update.py) on the CPU: the contract of
plugins/training/update/ppo.py:6-46 and update/train_step.py:6-44, exercised with stand-in
modules the way the reference's own tests use dummies (tests/test_rollout_backend_factory.py:15-23).
No fused kernel runs here."""
import numpy as np
import pytest
import torch

import mllm_jax_amd as M


def test_slice_data_matches_dynamic_slice_semantics():
    x = torch.arange(10 * 3).reshape(10, 3)
    parts = [M.slice_data(x, 4, i) for i in range(4)]          # 10 // 4 = 2 rows each, 2 rows dropped
    assert [p.shape[0] for p in parts] == [2, 2, 2, 2]
    assert torch.equal(torch.cat(parts), x[:8])
    assert parts[1].data_ptr() == x[2:].data_ptr()              # a view, not a copy


def test_ppo_update_contract_with_recording_step():
    b, t = 8, 5
    datas = {"input_ids": torch.arange(b * (t + 1)).reshape(b, t + 1), "labels": torch.ones(b, t + 1),
             "advantages": torch.arange(b).float()}
    calls = []

    def step(state, local):
        calls.append({k: (v.clone() if isinstance(v, torch.Tensor) else v) for k, v in local.items()})
        logps = local["input_ids"][:, 1:].float() * 0.5 + state        # recognisable, state-dependent
        return state + 1, {"per_token_logps": logps, "entropy": torch.tensor(float(state)), "loss": torch.tensor(0.)}

    state, out, last_meta, entropy = M.ppo_update(state=0, datas=datas, total_valid_token_count=123.0,
                                                  train_step=step, grad_accum_steps=4, ppo_steps=3)
    assert state == 12 and len(calls) == 12
    # every micro-batch sees the GLOBAL count (ppo.py:37) and its own rows
    assert all(c["total_valid_token_count"] == 123.0 for c in calls)
    for e in range(3):
        for i in range(4):
            c = calls[e * 4 + i]
            assert torch.equal(c["input_ids"], datas["input_ids"][2 * i:2 * i + 2])
            assert ("old_per_token_logps" in c) == (e > 0)
    # epoch 0's logps, concatenated in micro-batch order, are the old logps of later epochs (ppo.py:39-43)
    expect = torch.cat([datas["input_ids"][2 * i:2 * i + 2, 1:].float() * 0.5 + i for i in range(4)])
    assert torch.equal(out["old_per_token_logps"], expect)
    assert torch.equal(calls[5]["old_per_token_logps"], expect[2:4])
    assert float(entropy) == 3.0                                 # last micro-batch of epoch 0 (ppo.py:44)
    assert "old_per_token_logps" not in datas                    # the caller's mapping is not mutated
    assert float(last_meta["entropy"]) == 11.0
    res = M.PPOUpdateModule().update(state=0, batch=datas, total_valid_token_count=1.0, train_step=step,
                                     grad_accum_steps=2, ppo_steps=1)
    assert isinstance(res, M.UpdateResult) and res.state == 2 and res.batch["old_per_token_logps"].shape == (8, 5)


def _quadratic_state(grad_accum_steps, lr=0.1):
    w0 = torch.tensor([1.0, -2.0, 0.5], requires_grad=True)
    frozen = torch.tensor([3.0])

    def apply_fn(params, inputs):
        r = inputs["x"] @ params["w"] - inputs["y"]
        return {"loss": (r ** 2).sum() / inputs["total"], "per_token_logps": r.detach(), "aux": r.detach().abs()}

    return M.LossTrainState.create(apply_fn=apply_fn, params={"w": w0, "frozen": frozen},
                                   tx=lambda p, g: {k: (p[k] - lr * g[k] if k in g else p[k]) for k in p},
                                   grad_accum_steps=grad_accum_steps)


def test_training_step_without_accumulation_applies_every_step():
    st = _quadratic_state(1)
    x = torch.tensor([[1.0, 0.0, 2.0], [0.5, 1.0, -1.0]]); y = torch.tensor([0.3, -0.7])
    st2, m = M.training_step(st, {"x": x, "y": y, "total": 2.0})
    w = st.params["w"].detach()
    g = 2 * x.T @ (x @ w - y) / 2.0
    assert st2.step == 1 and st.step == 0 and st2.grad_accum is None
    torch.testing.assert_close(st2.params["w"].detach(), w - 0.1 * g)
    assert st2.params["w"].requires_grad and not st2.params["frozen"].requires_grad
    assert m["per_token_logps"].shape == (2,) and m["aux"].dim() == 0          # aux entries are mean-reduced (:21)


def test_training_step_accumulates_then_updates_with_the_mean():
    st = _quadratic_state(3)
    g_ = torch.Generator().manual_seed(0)
    xs = [torch.randn(2, 3, generator=g_) for _ in range(3)]; ys = [torch.randn(2, generator=g_) for _ in range(3)]
    w = st.params["w"].detach().clone()
    grads = [2 * x.T @ (x @ w - y) / 6.0 for x, y in zip(xs, ys)]
    for i in range(3):
        st, _ = M.training_step(st, {"x": xs[i], "y": ys[i], "total": 6.0})
        if i < 2:
            assert st.step == 0 and st.micro_step == i + 1
            torch.testing.assert_close(st.params["w"].detach(), w)              # no update yet (:43)
            torch.testing.assert_close(st.grad_accum["w"], sum(grads[:i + 1]))
    assert st.step == 1 and st.micro_step == 0
    torch.testing.assert_close(st.params["w"].detach(), w - 0.1 * sum(grads) / 3)   # grads / micro_in_mini (:36)
    assert not st.grad_accum["w"].any()                                          # zeroed (:39)


def test_direct_accumulation_requires_the_fused_call():
    st = _quadratic_state(2).replace(lm_head_key="w")
    with pytest.raises(RuntimeError, match="differentiable fused-loss calls"):
        M.training_step(st, {"x": torch.ones(1, 3), "y": torch.zeros(1), "total": 1.0})
