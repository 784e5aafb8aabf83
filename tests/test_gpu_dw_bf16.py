"""GPU: the lm_head gradient as a bf16 matrix (MJ_GRPO_FLAG_DW_BF16), for callers whose lm_head
parameter is bf16.  The reference's parameter gradients are float32 (llama/llama.py:251-256), so
the yardstick is the float32 output of the same pass: with one chunk the bf16 matrix must be its
round-to-nearest-even image bit for bit (same accumulators, one rounding), and with several chunks
or an accumulator it must stay within the gradient tolerance of the CPU oracle."""
import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O
from test_gpu_parity import GRAD_RTOL, _case, _old_from, _ref_logp, _rel

pytestmark = pytest.mark.gpu

N, H, V, B = 520, 72, 1000, 4       # V: three full 256-row tiles and a ragged one


def _inputs(seed):
    hid, w, y, adv, mask = _case(seed, N, H, V, B)
    old = _old_from(_ref_logp(hid, w, y), seed + 1)
    ref = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), old.numpy(), adv.numpy(), mask.numpy())
    dev = torch.device("cuda:0")
    return [t.to(dev) for t in (hid, w, y, old, adv, mask)], ref


@pytest.mark.parametrize("skip_masked", [False, True])
def test_one_chunk_is_the_rounded_float32_gradient(skip_masked):
    import mllm_jax_amd as M
    args, ref = _inputs(51)
    _, (dh32, dw32) = M.grpo_loss_value_and_grad(*args, chunk_tokens=1024, skip_masked=skip_masked)
    _, (dh16, dw16) = M.grpo_loss_value_and_grad(*args, chunk_tokens=1024, skip_masked=skip_masked,
                                                 lm_head_grad_dtype=torch.bfloat16)
    torch.cuda.synchronize()
    assert dw16.dtype == torch.bfloat16 and tuple(dw16.shape) == (H, V)
    assert torch.equal(dw16, dw32.to(torch.bfloat16))
    assert torch.equal(dh16, dh32)
    assert _rel(dw16.float().cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL


def test_several_chunks_round_once_per_chunk():
    import mllm_jax_amd as M
    args, ref = _inputs(53)
    _, (_, dw16) = M.grpo_loss_value_and_grad(*args, chunk_tokens=256, lm_head_grad_dtype=torch.bfloat16)
    torch.cuda.synchronize()
    assert _rel(dw16.float().cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL


def test_padded_bf16_accumulator():
    """Adds into a bf16 buffer that is a column slice of a wider one: fp32 sum of the value in memory
    and the new gradient, one rounding, padding columns untouched."""
    import mllm_jax_amd as M
    args, ref = _inputs(55)
    hid, w = args[0], args[1]
    pad = 40
    w_w = torch.full((H, V + pad), 1.0, dtype=torch.bfloat16, device=w.device)
    w_w[:, :V] = w
    acc_w = torch.full((H, V + pad), 5.0, dtype=torch.bfloat16, device=w.device)
    acc = acc_w[:, :V]
    g = torch.Generator().manual_seed(56)
    start = (0.01 * torch.randn(H, V, generator=g)).to(torch.bfloat16).to(w.device)
    acc.copy_(start)
    _, (_, dw32) = M.grpo_loss_value_and_grad(hid, w_w[:, :V], *args[2:], chunk_tokens=1024)
    M.grpo_loss_value_and_grad(hid, w_w[:, :V], *args[2:], chunk_tokens=1024, accumulate_into=acc)
    torch.cuda.synchronize()
    assert (acc_w[:, V:] == 5.0).all(), "padding columns of the accumulator were written"
    assert torch.equal(acc, (start.float() + dw32).to(torch.bfloat16))
    assert _rel(acc.float().cpu().numpy() - start.float().cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL


def test_autograd_hands_a_bf16_parameter_a_bf16_gradient():
    import mllm_jax_amd as M
    args, ref = _inputs(57)
    hid, w = args[0].clone().requires_grad_(), args[1].clone().requires_grad_()
    calls = []
    real = M.loss._Prepared.forward_backward

    def spy(self, d_w=None, value=None, dw_dtype=torch.float32):
        calls.append(dw_dtype)
        return real(self, d_w, value, dw_dtype)

    M.loss._Prepared.forward_backward = spy
    try:
        out = M.grpo_fused_loss(hid, w, *args[2:])
        out["loss"].backward()
    finally:
        M.loss._Prepared.forward_backward = real
    torch.cuda.synchronize()
    assert calls == [torch.bfloat16]
    assert w.grad.dtype == torch.bfloat16
    assert _rel(w.grad.float().cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
    assert _rel(hid.grad.float().cpu().numpy(), ref["d_hidden"]) <= GRAD_RTOL
    # float32 master weights keep the reference's float32 gradient
    w32 = args[1].float().requires_grad_()
    M.grpo_fused_loss(args[0], w32, *args[2:])["loss"].backward()
    torch.cuda.synchronize()
    assert w32.grad.dtype == torch.float32
    assert _rel(w32.grad.cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL


def test_other_gradient_dtypes_are_refused():
    import mllm_jax_amd as M
    args, _ = _inputs(59)
    with pytest.raises(ValueError, match="float32 or bfloat16"):
        M.grpo_loss_value_and_grad(*args, lm_head_grad_dtype=torch.float16)


def test_separate_backward_writes_the_rounded_float32_gradient():
    """mj_grpo_backward (the transpose pass alone, from saved lse / logp) with the flag set."""
    import ctypes as C
    from mllm_jax_amd import _lib
    from mllm_jax_amd.loss import _Prepared, _workspace, _ptr
    args, ref = _inputs(61)
    kw = dict(total_valid_token_count=None, epsilon_low=0.2, epsilon_high=0.3, temperature=1.0,
              final_logit_softcap=None, seq_shape=None, chunk_tokens=1024)
    p = _Prepared(*args, **kw)
    p.forward()
    _, both = _lib.workspace_bytes(p.desc)
    ws = _workspace(args[0].device, both)
    out = {}
    for name, dtype, flag in (("f32", torch.float32, 0), ("bf16", torch.bfloat16, _lib.FLAG_DW_BF16)):
        dh = torch.empty((N, H), dtype=torch.bfloat16, device=ws.device)
        dw = torch.empty((H, V), dtype=dtype, device=ws.device)
        p.desc.flags = flag
        _lib.check(_lib.load().mj_grpo_backward(
            C.byref(p.desc), _ptr(p.hidden), _ptr(p.w), _ptr(p.targets), _ptr(p.old), _ptr(p.adv), _ptr(p.mask),
            _ptr(p.lse), _ptr(p.logp), _ptr(dh), _ptr(dw), _ptr(ws), ws.numel(), p.stream()))
        torch.cuda.synchronize()
        out[name] = (dh, dw)
    assert torch.equal(out["bf16"][1], out["f32"][1].to(torch.bfloat16))
    assert torch.equal(out["bf16"][0], out["f32"][0])
    assert _rel(out["bf16"][1].float().cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
