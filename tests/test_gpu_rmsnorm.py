"""GPU parity of the RMSNorm kernels (forward and backward) against the CPU oracle.
Outputs are bf16: forward within one bf16 rounding of the float64 result, gradients <= 2e-2
relative (Frobenius), dscale (float32 sums) <= 2e-3 relative."""
import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O

pytestmark = pytest.mark.gpu


def _rel(a, b):
    a = np.asarray(a, np.float64); b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


@pytest.mark.parametrize("n,h", [(1, 8), (7, 64), (300, 896), (1027, 3584), (64, 4096), (33, 4104), (16, 8192),
                                 (2100, 2048), (5, 2056), (3000, 1536)])
def test_forward_backward_match_oracle(n, h):
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(n * 131 + h)
    x = (torch.randn(n, h, generator=g) * 1.7).to(torch.bfloat16)
    s = 1.0 + 0.3 * torch.randn(h, generator=g)
    dy = torch.randn(n, h, generator=g).to(torch.bfloat16)
    xd = x.to(dev).requires_grad_(); sd = s.to(dev).requires_grad_()
    y = M.rms_norm(xd, sd, 1e-6)
    y.backward(dy.to(dev))
    torch.cuda.synchronize()
    yr, dxr, dsr = O.rms_norm(x.float().numpy(), s.numpy(), 1e-6, dy.float().numpy())
    assert y.dtype == torch.bfloat16 and y.shape == (n, h)
    np.testing.assert_allclose(y.detach().float().cpu().numpy(), yr, rtol=2 ** -8, atol=1e-6)   # one bf16 rounding
    assert _rel(xd.grad.float().cpu().numpy(), dxr) <= 2e-2
    np.testing.assert_allclose(xd.grad.float().cpu().numpy(), dxr, rtol=2 ** -7, atol=2e-2 * np.abs(dxr).max())
    assert _rel(sd.grad.cpu().numpy(), dsr) <= 2e-3
    assert sd.grad.dtype == torch.float32


def test_batched_shape_strided_rows_and_accumulate():
    import ctypes as C
    import mllm_jax_amd as M
    from mllm_jax_amd import _lib
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(3)
    b, l, h = 3, 17, 136
    big = torch.randn(b, l, h + 8, generator=g).to(torch.bfloat16).to(dev)
    x = big[..., :h]                                            # row stride h + 8
    s = torch.randn(h, generator=g).to(dev)
    y = M.rms_norm(x, s, 1e-5)
    yr = O.rms_norm(x.float().cpu().numpy(), s.cpu().numpy(), 1e-5)
    np.testing.assert_allclose(y.float().cpu().numpy(), yr, rtol=2 ** -8, atol=1e-6)
    # accumulate_dscale adds to what the buffer holds; two calls are bit-identical (fixed order)
    lib = _lib.load()
    n = b * l
    x2 = x.reshape(n, h).contiguous(); dy = torch.randn(n, h, generator=g).to(torch.bfloat16).to(dev)
    need = C.c_size_t(); _lib.check(lib.mj_rmsnorm_workspace_bytes(n, h, C.byref(need)))
    ws = torch.empty(need.value, dtype=torch.uint8, device=dev)
    dx = torch.empty_like(x2); ds = torch.full((h,), 2.0, device=dev); ds2 = torch.empty(h, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    for out, acc in ((ds, 1), (ds2, 0)):
        _lib.check(lib.mj_rmsnorm_backward(dy.data_ptr(), h, x2.data_ptr(), h, s.data_ptr(), dx.data_ptr(), h,
                                           out.data_ptr(), acc, n, h, 1e-5, ws.data_ptr(), ws.numel(), st))
    torch.cuda.synchronize()
    assert torch.equal(ds, ds2 + 2.0) or torch.allclose(ds, ds2 + 2.0, rtol=1e-6, atol=1e-6)
    ds3 = torch.empty(h, device=dev)
    _lib.check(lib.mj_rmsnorm_backward(dy.data_ptr(), h, x2.data_ptr(), h, s.data_ptr(), dx.data_ptr(), h,
                                       ds3.data_ptr(), 0, n, h, 1e-5, ws.data_ptr(), ws.numel(), st))
    torch.cuda.synchronize()
    assert torch.equal(ds2, ds3)


def test_norm_feeds_the_fused_loss_end_to_end():
    # x -> RMSNorm -> fused GRPO loss; gradients w.r.t. x and scale against the chained oracle
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(9)
    n, h, v = 192, 64, 1000
    x = torch.randn(n, h, generator=g).to(torch.bfloat16)
    s = 1.0 + 0.2 * torch.randn(h, generator=g)
    w = (0.3 * torch.randn(h, v, generator=g)).to(torch.bfloat16)
    yid = torch.randint(0, v, (n,), generator=g); adv = torch.randn(n, generator=g)
    mask = (torch.rand(n, generator=g) < 0.8).float()
    xd = x.to(dev).requires_grad_(); sd = s.to(dev).requires_grad_(); wd = w.to(dev).requires_grad_()
    hid = M.rms_norm(xd, sd)
    out = M.grpo_fused_loss(hid, wd, yid.to(dev), None, adv.to(dev), mask.to(dev))
    out["loss"].backward()
    torch.cuda.synchronize()
    hid_ref = hid.detach().float().cpu().numpy()                # the bf16 hidden the loss kernel saw
    ref = O.grpo_loss(hid_ref, w.float().numpy(), yid.numpy(), None, adv.numpy(), mask.numpy())
    _, dxr, dsr = O.rms_norm(x.float().numpy(), s.numpy(), 1e-6, ref["d_hidden"])
    assert abs(float(out["loss"].detach()) - ref["loss"]) <= 1e-3 * abs(ref["loss"])
    assert _rel(xd.grad.float().cpu().numpy(), dxr) <= 3e-2      # two bf16 roundings in the chain
    assert _rel(sd.grad.cpu().numpy(), dsr) <= 2e-2
    assert _rel(wd.grad.float().cpu().numpy(), ref["d_lm_head"]) <= 2e-2
