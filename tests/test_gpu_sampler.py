"""GPU parity of the sampler step: last-position logits against a float64 product, the top-k /
categorical draw bit-exactly against the CPU oracle on the SAME float32 logits and noise."""
import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O

pytestmark = pytest.mark.gpu


def test_last_position_logits_match_float64_product():
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(1)
    # batch sizes either side of the 128-row tile, vocabularies that give work items of
    # 8 .. 256 columns, one full-size vocabulary
    for b, h, v, cap in [(5, 64, 1000, None), (128, 896, 5000, None), (300, 136, 2008, 30.0), (1, 8, 8, None),
                         (64, 72, 3000, None), (65, 72, 3000, None), (129, 64, 1000, 10.0), (16, 128, 152064, None),
                         (100, 64, 66000, None)]:
        hid = torch.randn(b, h, generator=g).to(torch.bfloat16)
        w = (0.2 * torch.randn(h, v, generator=g)).to(torch.bfloat16)
        out = M.last_position_logits(hid.to(dev), w.to(dev), cap)
        ref = O.lm_head_logits(hid.float().numpy(), w.float().numpy(), cap)
        assert out.dtype == torch.float32 and tuple(out.shape) == (b, v)
        np.testing.assert_allclose(out.cpu().numpy(), ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("b,v,k,t", [(3, 1000, 50, 0.9), (64, 152064, 50, 1.0), (7, 129, 64, 0.7), (2, 50, 50, 1.0),
                                     (5, 4097, 1, 1.0)])
def test_top_k_draw_is_bit_exact(b, v, k, t):
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(b * 1000 + k)
    logits = (3.0 * torch.randn(b, v, generator=g)).float()
    u = torch.rand(b, k, generator=g)
    noise = -torch.log(-torch.log(u))
    tok, idx, val = M.top_k_sampling_batched(noise.to(dev), logits.to(dev), k=k, t=t, return_top_k=True)
    rt, ri, rv = O.top_k_sample(logits.numpy(), k=k, t=t, noise=noise.numpy())
    np.testing.assert_array_equal(idx.cpu().numpy(), ri)
    np.testing.assert_array_equal(val.cpu().numpy(), rv)
    np.testing.assert_array_equal(tok.cpu().numpy(), rt)


@pytest.mark.parametrize("t", [3.0, 1.7, 0.6])
def test_neighbouring_floats_that_divide_to_the_same_quotient(t):
    """A cluster of adjacent float32 values around the k-th largest: after the division by t > 1
    neighbours collapse into equal quotients and the lower index must win, also for elements that
    sit a few ulps below the kernel's raw-value threshold."""
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(7)
    b, v, k = 4, 70000, 50
    x = rng.normal(-5.0, 0.5, size=(b, v)).astype(np.float32)
    for r in range(b):
        pos = rng.choice(v, size=300, replace=False)
        steps = rng.integers(0, 40, size=300)
        base = np.float32([2.0, -1.5, 1e-3, 300.0][r])
        vals = base.copy()
        cluster = np.array([np.nextafter(base, np.float32(np.inf), dtype=np.float32)] * 300, np.float32)
        for j, s_ in enumerate(steps):
            c = base
            for _ in range(int(s_)):
                c = np.nextafter(c, np.float32(np.inf), dtype=np.float32)
            cluster[j] = c
        x[r, pos] = cluster
    noise = rng.gumbel(size=(b, k)).astype(np.float32)
    tok, idx, val = M.top_k_sampling_batched(torch.tensor(noise), torch.tensor(x, device=dev), k=k, t=t, return_top_k=True)
    rt, ri, rv = O.top_k_sample(x, k=k, t=t, noise=noise)
    np.testing.assert_array_equal(idx.cpu().numpy(), ri)
    np.testing.assert_array_equal(val.cpu().numpy(), rv)
    np.testing.assert_array_equal(tok.cpu().numpy(), rt)


def test_signed_zeros_and_nans_follow_the_total_order():
    """Rows of +0 / -0 / tiny values (the k-th place falls among zeros of both signs) and rows with
    NaN and infinities: selection and order are those of the IEEE total order, as in the oracle."""
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(11)
    for v, k in ((50, 34), (129, 64), (5000, 50), (70000, 50)):
        x = rng.normal(0, 1e-3, size=(6, v)).astype(np.float32)
        x[:, ::7] = 0.0
        x[:, 3::11] = -0.0
        x[3] = np.where(rng.random(v) < 0.5, 0.0, -0.0).astype(np.float32)      # nothing but zeros
        x[4, rng.integers(0, v, size=5)] = np.nan
        x[5, rng.integers(0, v, size=3)] = np.inf
        x[5, rng.integers(0, v, size=3)] = -np.inf
        tok, idx, val = M.top_k_sampling_batched(None, torch.tensor(x, device=dev), k=k, t=1.3, return_top_k=True)
        rt, ri, rv = O.top_k_sample(x, k=k, t=1.3, noise=None)
        np.testing.assert_array_equal(idx.cpu().numpy(), ri)
        np.testing.assert_array_equal(val.cpu().numpy().view(np.uint32), rv.view(np.uint32))
        np.testing.assert_array_equal(tok.cpu().numpy(), rt)


def test_ties_duplicates_and_negative_values():
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(0)
    # few distinct values: the k-th largest is shared by many entries, lower indices must win
    x = rng.integers(-3, 4, size=(9, 3000)).astype(np.float32)
    x[4] = -7.0                                             # a constant row: indices 0..k-1
    x[5, 100:] = -np.inf
    noise = rng.gumbel(size=(9, 50)).astype(np.float32)
    tok, idx, val = M.top_k_sampling_batched(torch.tensor(noise), torch.tensor(x, device=dev), k=50, t=1.0, return_top_k=True)
    rt, ri, rv = O.top_k_sample(x, k=50, t=1.0, noise=noise)
    np.testing.assert_array_equal(idx.cpu().numpy(), ri)
    np.testing.assert_array_equal(val.cpu().numpy(), rv)
    np.testing.assert_array_equal(tok.cpu().numpy(), rt)
    np.testing.assert_array_equal(idx[4].cpu().numpy(), np.arange(50))


def test_greedy_generator_draws_and_fused_step():
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(5)
    b, h, v = 32, 64, 4000
    hid = torch.randn(b, h, generator=g).to(torch.bfloat16).to(dev)
    w = (0.5 * torch.randn(h, v, generator=g)).to(torch.bfloat16).to(dev)
    logits = M.last_position_logits(hid, w)
    np.testing.assert_array_equal(M.greedy_sampling(None, logits).cpu().numpy(), logits.argmax(-1).cpu().numpy())
    gen = torch.Generator(device=dev).manual_seed(7)
    a = M.sample_next_tokens(gen, hid, w, k=50, t=1.0)
    gen.manual_seed(7)
    b2 = M.sample_next_tokens(gen, hid, w, k=50, t=1.0)
    assert torch.equal(a, b2) and a.dtype == torch.int32               # same generator state, same draw
    top = torch.topk(logits, 50, dim=-1).indices
    assert bool((top == a[:, None]).any(-1).all())                      # every draw lies inside its row's top 50
    # draws follow softmax over the top k: a sharply peaked row is (almost) always its argmax
    peaked = torch.zeros(1, v, device=dev); peaked[0, 123] = 40.0
    assert int(M.top_k_sampling_batched(gen, peaked, k=50, t=1.0)[0]) == 123
    with pytest.raises(M._lib.MjGrpoError):
        M.top_k_sampling_batched(None, logits, k=65)


def test_near_equal_logits_overflow_the_pool_and_take_the_slow_path():
    # more than 4096 logits share the 12 leading key bits of the k-th largest: the byte-wise select runs
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(2)
    x = np.full((4, 30000), 1.5, np.float32)
    x[1] += (rng.random(30000) * 1e-3).astype(np.float32)       # all inside one 12-bit bin, distinct low bits
    x[2, ::7] = 9.0                                             # 4286 equal maxima: ties beyond k
    x[3] = rng.integers(0, 3, 30000).astype(np.float32)         # three values
    noise = rng.gumbel(size=(4, 50)).astype(np.float32)
    tok, idx, val = M.top_k_sampling_batched(torch.tensor(noise), torch.tensor(x, device=dev), k=50, t=1.0, return_top_k=True)
    rt, ri, rv = O.top_k_sample(x, k=50, t=1.0, noise=noise)
    np.testing.assert_array_equal(idx.cpu().numpy(), ri)
    np.testing.assert_array_equal(val.cpu().numpy(), rv)
    np.testing.assert_array_equal(tok.cpu().numpy(), rt)
