"""GPU: the terminal-loss path of the autograd function.  Inside terminal_loss() the backward hands
autograd the [H,V] gradient tensor the kernel wrote (no multiply, no copy); a broken promise
(upstream gradient != 1) shows up as NaN in element [0,0] of the lm_head gradient."""
import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O
from test_gpu_parity import GRAD_RTOL, _case, _rel

pytestmark = pytest.mark.gpu


def _setup(seed):
    hid, w, y, adv, mask = _case(seed, 256, 64, 1000, 2)
    ref = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), None, adv.numpy(), mask.numpy())
    dev = torch.device("cuda:0")
    hp = hid.to(dev).requires_grad_()
    wp = w.float().to(dev).requires_grad_()          # float32 master weights, as in the reference
    args = (y.to(dev), None, adv.to(dev), mask.to(dev))
    return ref, hp, wp, args


def test_terminal_backward_returns_the_kernel_output_itself():
    import mllm_jax_amd as M
    from mllm_jax_amd import loss as L
    ref, hp, wp, args = _setup(51)
    seen = {}
    orig = L._Prepared.forward_backward

    def spy(self, *a, **k):
        d_h, d_wv = orig(self, *a, **k)
        seen["ptr"] = d_wv.data_ptr()
        return d_h, d_wv

    L._Prepared.forward_backward = spy
    try:
        with M.terminal_loss():
            out = M.grpo_fused_loss(hp, wp, *args)
            out["loss"].backward()
    finally:
        L._Prepared.forward_backward = orig
    torch.cuda.synchronize()
    assert wp.grad.data_ptr() == seen["ptr"], "the [H,V] gradient was copied or rescaled on the way to autograd"
    assert _rel(wp.grad.cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
    assert _rel(hp.grad.float().cpu().numpy(), ref["d_hidden"]) <= GRAD_RTOL


def test_broken_promise_poisons_the_lm_head_gradient():
    import mllm_jax_amd as M
    ref, hp, wp, args = _setup(52)
    with M.terminal_loss():
        out = M.grpo_fused_loss(hp, wp, *args)
        (out["loss"] * 0.5).backward()
    torch.cuda.synchronize()
    assert torch.isnan(wp.grad[0, 0]) and torch.isfinite(wp.grad[0, 1:]).all() and torch.isfinite(wp.grad[1:]).all()
    # outside the context the general path scales correctly
    hp.grad = None
    wp.grad = None
    out = M.grpo_fused_loss(hp, wp, *args)
    (out["loss"] * 0.5).backward()
    torch.cuda.synchronize()
    assert _rel(wp.grad.cpu().numpy(), 0.5 * ref["d_lm_head"]) <= GRAD_RTOL


def test_accumulating_with_a_scaled_loss_poisons_the_accumulator():
    import mllm_jax_amd as M
    ref, hp, wp, args = _setup(53)
    acc = torch.zeros_like(wp)
    with M.accumulate_lm_head_grad_into(acc):
        out = M.grpo_fused_loss(hp, wp, *args)
        (out["loss"] / 2).backward()
    torch.cuda.synchronize()
    assert torch.isnan(acc[0, 0]) and torch.isfinite(acc[0, 1:]).all()
    acc.zero_()
    with M.accumulate_lm_head_grad_into(acc):
        out = M.grpo_fused_loss(hp, wp, *args)
        out["loss"].backward()
    torch.cuda.synchronize()
    assert _rel(acc.cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL


def test_bf16_copy_of_float32_weights_is_reused_until_they_change():
    import mllm_jax_amd as M
    from mllm_jax_amd import loss as L
    ref, hp, wp, args = _setup(54)
    assert L._bf16_weights(wp) is not L._bf16_weights(wp)                     # outside the context: a cast per call
    with M.cache_bf16_lm_head():
        a = L._bf16_weights(wp)
        assert a.dtype == torch.bfloat16 and L._bf16_weights(wp) is a        # same tensor, same version: reused
        out1 = M.grpo_fused_loss(hp, wp, *args)["loss"].item()
        with torch.no_grad():
            wp.mul_(1.5)                                                      # an optimizer step writes in place
        b = L._bf16_weights(wp)
        assert b is not a and torch.equal(b, wp.detach().to(torch.bfloat16))
        out2 = M.grpo_fused_loss(hp, wp, *args)["loss"].item()
        assert out1 == out2 == pytest.approx(ref["loss"], rel=1e-3)           # on-policy: the loss does not depend on W
        lp1 = M.grpo_fused_loss(hp, wp, *args)["per_token_logps"]
        with torch.no_grad():
            wp.mul_(0.5)
        lp2 = M.grpo_fused_loss(hp, wp, *args)["per_token_logps"]
        assert not torch.equal(lp1, lp2)                                      # the stale copy is not used
        # a write through .data does not bump the version counter: the documented hazard and its remedy
        c = L._bf16_weights(wp)
        wp.data.mul_(2.0)
        assert L._bf16_weights(wp) is c                                       # stale: the cache cannot see this write
        M.invalidate_bf16_lm_head()
        d = L._bf16_weights(wp)
        assert d is not c and torch.equal(d, wp.detach().to(torch.bfloat16))
    assert not L._bf16_copies                                                 # leaving the context drops the copies
    # outside the context a .data write is seen at once (no cache)
    lp3 = M.grpo_fused_loss(hp, wp, *args)["per_token_logps"]
    wp.data.mul_(0.5)
    lp4 = M.grpo_fused_loss(hp, wp, *args)["per_token_logps"]
    assert not torch.equal(lp3, lp4)


def test_upstream_gradient_is_applied_on_the_device_and_costs_nothing_when_it_is_one():
    """Outside terminal_loss(): backward multiplies d_hidden and d_lm_head in place by the upstream
    gradient through mj_grpo_scale_gradients (a launch that leaves at once when it is 1)."""
    import mllm_jax_amd as M
    ref, hp, wp, args = _setup(55)
    out = M.grpo_fused_loss(hp, wp, *args)
    out["loss"].backward()
    g1h, g1w = hp.grad.clone(), wp.grad.clone()
    assert _rel(g1w.float().cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
    hp.grad = wp.grad = None
    out = M.grpo_fused_loss(hp, wp, *args)
    (out["loss"] * 0.25).backward()
    torch.cuda.synchronize()
    assert torch.equal(wp.grad, g1w * 0.25)                                   # a power of two: exact in any dtype
    assert torch.equal(hp.grad, g1h * 0.25)
    hp.grad = wp.grad = None
    # the same constant known before the call: the kernels write the scaled gradients, the loss comes back scaled
    out2 = M.grpo_fused_loss(hp, wp, *args, loss_scale=0.25)
    assert out2["loss"].item() == pytest.approx(0.25 * out["loss"].item(), rel=1e-6)
    out2["loss"].backward()
    torch.cuda.synchronize()
    assert _rel(wp.grad.float().cpu().numpy(), 0.25 * ref["d_lm_head"]) <= GRAD_RTOL
    assert _rel(hp.grad.float().cpu().numpy(), 0.25 * g1h.float().cpu().numpy()) <= 1e-2
    # the gradients of a call are handed out once
    out3 = M.grpo_fused_loss(hp, wp, *args)
    out3["loss"].backward(retain_graph=True)
    with pytest.raises(RuntimeError, match="once"):
        out3["loss"].backward()
