"""GPU: mj_grpo_forward_noalloc (the forward whose workspace is a static device array) against
mj_grpo_forward with a caller workspace, through the C ABI: bit-identical outputs on two calls in a
row, the second on a smaller input, and a clean refusal of a shape that cannot fit."""
import ctypes as C

import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(seed, n, h, v):
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(seed)
    hid = torch.randn(n, h, generator=g).to(torch.bfloat16).to(dev)
    w = (0.2 * torch.randn(h, v, generator=g)).to(torch.bfloat16).to(dev)
    y = torch.randint(0, v, (n,), generator=g).to(torch.int32).to(dev)
    old = (-7.0 + 0.3 * torch.randn(n, generator=g)).to(dev)
    adv = torch.randn(n, generator=g).to(dev)
    mask = (torch.rand(n, generator=g) < 0.7).float().to(dev)
    return hid, w, y, old, adv, mask


def _desc(n, h, v, mask, chunk=0):
    from mllm_jax_amd import _lib
    d = _lib.MjGrpoDesc()
    d.n_tokens, d.hidden, d.vocab, d.ld_hidden, d.ld_w, d.chunk_tokens = n, h, v, h, v, chunk
    d.eps_low, d.eps_high, d.temperature = 0.2, 0.28, 1.0
    d.inv_total_valid_tokens, d.grad_loss_scale = 1.0 / float(mask.sum().item()), 1.0
    return d


def _both(seed, n, h, v):
    from mllm_jax_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    hid, w, y, old, adv, mask = _inputs(seed, n, h, v)
    st = torch.cuda.current_stream().cuda_stream
    outs = []
    for static in (False, True):
        d = _desc(n, h, v, mask)
        logp, lse, ent = (torch.full((n,), float("nan"), device=dev) for _ in range(3))
        loss = torch.full((2,), float("nan"), device=dev)
        common = (C.byref(d), hid.data_ptr(), w.data_ptr(), y.data_ptr(), old.data_ptr(), adv.data_ptr(),
                  mask.data_ptr(), logp.data_ptr(), lse.data_ptr(), ent.data_ptr(), loss.data_ptr())
        if static:
            _lib.check(lib.mj_grpo_forward_noalloc(*common, st))
        else:
            fwd, _ = _lib.workspace_bytes(d)
            ws = torch.empty(fwd, dtype=torch.uint8, device=dev)
            _lib.check(lib.mj_grpo_forward(*common, ws.data_ptr(), ws.numel(), st))
        torch.cuda.synchronize()
        outs.append((logp, lse, ent, loss))
    for a, b in zip(*outs):
        assert torch.isfinite(a).all()
        assert torch.equal(a, b)


def test_static_scratch_forward_matches_workspace_forward_twice():
    print("no-alloc forward: 2100 x 128 x 152064", flush=True)
    _both(61, 2100, 128, 152064)     # 14.3 KB of statistics per chunk token: two internal chunks of <= 2048 tokens
    print("no-alloc forward: 300 x 64 x 1000 (smaller, same static array)", flush=True)
    _both(62, 300, 64, 1000)


def test_shape_that_cannot_fit_is_refused():
    from mllm_jax_amd import _lib
    lib = _lib.load()
    dev = torch.device("cuda:0")
    n, h, v = 4096, 64, 1000
    hid, w, y, old, adv, mask = _inputs(63, n, h, v)
    d = _desc(n, h, v, mask)
    d.n_tokens = 1 << 24                       # 12 bytes per token alone exceed the static array
    out = torch.empty(n, device=dev)
    loss = torch.empty(2, device=dev)
    rc = lib.mj_grpo_forward_noalloc(C.byref(d), hid.data_ptr(), w.data_ptr(), y.data_ptr(), old.data_ptr(),
                                     adv.data_ptr(), mask.data_ptr(), out.data_ptr(), out.data_ptr(), None,
                                     loss.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 4 and b"static array" in lib.mj_grpo_last_error()
    d = _desc(n, h, v, mask, chunk=1 << 20)    # an explicit chunk that does not fit is refused, not shrunk
    d.vocab, d.ld_w = 1 << 21, 1 << 21
    rc = lib.mj_grpo_forward_noalloc(C.byref(d), hid.data_ptr(), w.data_ptr(), y.data_ptr(), old.data_ptr(),
                                     adv.data_ptr(), mask.data_ptr(), out.data_ptr(), out.data_ptr(), None,
                                     loss.data_ptr(), torch.cuda.current_stream().cuda_stream)
    assert rc == 4
