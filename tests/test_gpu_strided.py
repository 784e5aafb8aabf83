"""GPU: operands that are column slices of wider buffers (ld_hidden > H, ld_w > V), the layout a
caller gets from `x[:, :H]` or a padded parameter.  Checked against the CPU oracle, dense and with
the skip-masked option, with a padded gradient accumulator, and for untouched padding columns."""
import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O
from test_gpu_parity import GRAD_RTOL, LOGP_ATOL, LOSS_RTOL, _case, _old_from, _ref_logp, _rel

pytestmark = pytest.mark.gpu

N, H, V, B = 520, 72, 1000, 4
PAD_H, PAD_V = 24, 40        # pitches 96 and 1040: multiples of 8, larger than the rows


def _wide(t, pad, fill):
    wide = torch.full((t.shape[0], t.shape[1] + pad), fill, dtype=t.dtype, device="cuda:0")
    wide[:, : t.shape[1]] = t.to("cuda:0")
    return wide


@pytest.mark.parametrize("skip_masked", [False, True])
def test_column_slices_of_wider_buffers(skip_masked):
    import mllm_jax_amd as M
    hid, w, y, adv, mask = _case(31, N, H, V, B)
    old = _old_from(_ref_logp(hid, w, y), 32)
    ref = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), old.numpy(), adv.numpy(), mask.numpy())
    hid_w, w_w = _wide(hid, PAD_H, 7.0), _wide(w, PAD_V, -3.0)
    hv, wv = hid_w[:, :H], w_w[:, :V]
    assert hv.stride(0) == H + PAD_H and wv.stride(0) == V + PAD_V
    dev = hv.device
    met, (dh, dw) = M.grpo_loss_value_and_grad(hv, wv, y.to(dev), old.to(dev), adv.to(dev), mask.to(dev),
                                               chunk_tokens=256, skip_masked=skip_masked)
    torch.cuda.synchronize()
    assert tuple(dh.shape) == (N, H) and tuple(dw.shape) == (H, V)
    np.testing.assert_allclose(met["per_token_logps"].cpu().numpy().reshape(-1), ref["per_token_logps"],
                               atol=LOGP_ATOL, rtol=0)
    assert abs(met["loss"].item() - ref["loss"]) <= LOSS_RTOL * abs(ref["loss"])
    assert _rel(dh.float().cpu().numpy(), ref["d_hidden"]) <= GRAD_RTOL
    assert _rel(dw.cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
    # the inputs' padding columns are read by nobody and still hold their fill
    assert (hid_w[:, H:] == 7.0).all() and (w_w[:, V:] == -3.0).all()


def test_padded_accumulator_keeps_its_padding():
    import mllm_jax_amd as M
    hid, w, y, adv, mask = _case(33, N, H, V, B)
    ref = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), None, adv.numpy(), mask.numpy())
    hid_w, w_w = _wide(hid, PAD_H, 1.0), _wide(w, PAD_V, 1.0)
    dev = hid_w.device
    acc_w = torch.full((H, V + PAD_V), 5.0, dtype=torch.float32, device=dev)
    acc = acc_w[:, :V]
    acc.fill_(0.25)
    for _ in range(2):
        M.grpo_loss_value_and_grad(hid_w[:, :H], w_w[:, :V], y.to(dev), None, adv.to(dev), mask.to(dev),
                                   chunk_tokens=256, accumulate_into=acc)
    torch.cuda.synchronize()
    assert (acc_w[:, V:] == 5.0).all(), "padding columns of the accumulator were written"
    assert _rel((acc.cpu().numpy() - 0.25) / 2.0, ref["d_lm_head"]) <= GRAD_RTOL


def test_autograd_gradient_of_a_strided_hidden_view():
    """hidden[:, :H] of a wider activation through the autograd function: the gradient reaches the
    wide tensor with zeros in the columns that were sliced away."""
    import mllm_jax_amd as M
    hid, w, y, adv, mask = _case(34, 256, H, V, 2)
    ref = O.grpo_loss(hid.float().numpy(), w.float().numpy(), y.numpy(), None, adv.numpy(), mask.numpy())
    wide = _wide(hid, PAD_H, 2.0).requires_grad_()
    wp = w.to("cuda:0").requires_grad_()
    dev = wide.device
    out = M.grpo_fused_loss(wide[:, :H], wp, y.to(dev), None, adv.to(dev), mask.to(dev))
    out["loss"].backward()
    torch.cuda.synchronize()
    assert _rel(wide.grad[:, :H].float().cpu().numpy(), ref["d_hidden"]) <= GRAD_RTOL
    assert not wide.grad[:, H:].any()
    assert _rel(wp.grad.float().cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
