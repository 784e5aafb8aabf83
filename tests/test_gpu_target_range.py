"""GPU: target ids outside [0, V).  The rule of the C ABI: such ids are clamped to the nearest valid
id, the same way in the forward and the backward, so the result is that of the oracle on the clamped
ids (-100, the usual ignore label, acts as id 0; V+5 as V-1) -- for masked and unmasked tokens."""
import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O
from test_gpu_parity import GRAD_RTOL, LOGP_ATOL, LOSS_RTOL, _case, _old_from, _ref_logp, _rel

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("skip_masked", [False, True])
def test_out_of_range_targets_are_clamped_in_both_passes(skip_masked):
    import mllm_jax_amd as M
    n, h, v, b = 384, 64, 1000, 3
    hid, w, y, adv, mask = _case(41, n, h, v, b)
    y = y.clone()
    bad = {3: -100, 10: -1, 57: v, 130: v + 5, 200: 2 ** 31 - 1, 383: -(2 ** 31)}
    for t, val in bad.items():
        y[t] = val
    mask = mask.clone()
    mask[[3, 57, 200]] = 1.0          # some of them carry a gradient ...
    mask[[10, 130, 383]] = 0.0        # ... and some are masked
    yc = y.clamp(0, v - 1)
    old = _old_from(_ref_logp(hid, w, yc), 42)
    ref = O.grpo_loss(hid.float().numpy(), w.float().numpy(), yc.numpy(), old.numpy(), adv.numpy(), mask.numpy())
    dev = torch.device("cuda:0")
    met, (dh, dw) = M.grpo_loss_value_and_grad(hid.to(dev), w.to(dev), y.to(dev), old.to(dev), adv.to(dev),
                                               mask.to(dev), chunk_tokens=256, skip_masked=skip_masked)
    torch.cuda.synchronize()
    logp = met["per_token_logps"].cpu().numpy().reshape(-1)
    assert np.isfinite(logp).all()
    np.testing.assert_allclose(logp, ref["per_token_logps"], atol=LOGP_ATOL, rtol=0)
    assert abs(met["loss"].item() - ref["loss"]) <= LOSS_RTOL * abs(ref["loss"])
    assert _rel(dh.float().cpu().numpy(), ref["d_hidden"]) <= GRAD_RTOL
    assert _rel(dw.cpu().numpy(), ref["d_lm_head"]) <= GRAD_RTOL
    # the separate backward applies the same rule
    lib_dh, lib_dw = _separate_backward(M, hid, w, y, old, adv, mask, met)
    assert _rel(lib_dh, ref["d_hidden"]) <= GRAD_RTOL and _rel(lib_dw, ref["d_lm_head"]) <= GRAD_RTOL


def _separate_backward(M, hid, w, y, old, adv, mask, met):
    import ctypes as C
    from mllm_jax_amd import _lib
    dev = torch.device("cuda:0")
    n, h = hid.shape
    v = w.shape[1]
    d = _lib.MjGrpoDesc()
    d.n_tokens, d.hidden, d.vocab, d.ld_hidden, d.ld_w = n, h, v, h, v
    d.eps_low, d.eps_high, d.temperature = 0.2, 0.3, 1.0
    d.inv_total_valid_tokens, d.grad_loss_scale = 1.0 / float(mask.sum()), 1.0
    _, both = _lib.workspace_bytes(d)
    ws = torch.empty(both, dtype=torch.uint8, device=dev)
    t = lambda x, dt: x.to(dev).to(dt).contiguous()
    hid_d, w_d, y_d = t(hid, torch.bfloat16), t(w, torch.bfloat16), t(y, torch.int32)
    old_d, adv_d, mask_d = t(old, torch.float32), t(adv, torch.float32), t(mask, torch.float32)
    logp, lse = torch.empty(n, device=dev), torch.empty(n, device=dev)
    loss = torch.empty(2, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    lib = _lib.load()
    _lib.check(lib.mj_grpo_forward(C.byref(d), hid_d.data_ptr(), w_d.data_ptr(), y_d.data_ptr(), old_d.data_ptr(),
                                   adv_d.data_ptr(), mask_d.data_ptr(), logp.data_ptr(), lse.data_ptr(), None,
                                   loss.data_ptr(), ws.data_ptr(), ws.numel(), st))
    dh = torch.empty(n, h, dtype=torch.bfloat16, device=dev)
    dw = torch.empty(h, v, dtype=torch.float32, device=dev)
    _lib.check(lib.mj_grpo_backward(C.byref(d), hid_d.data_ptr(), w_d.data_ptr(), y_d.data_ptr(), old_d.data_ptr(),
                                    adv_d.data_ptr(), mask_d.data_ptr(), lse.data_ptr(), logp.data_ptr(),
                                    dh.data_ptr(), dw.data_ptr(), ws.data_ptr(), ws.numel(), st))
    torch.cuda.synchronize()
    return dh.float().cpu().numpy(), dw.cpu().numpy()
