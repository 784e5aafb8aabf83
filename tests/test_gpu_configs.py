"""GPU parity at the BASELINE.json configuration shapes (configs[0..4]).

The CPU oracle's float64 NumPy form is too slow at these sizes, so the checker here is the
oracle's chunked torch form (oracle.grpo_oracle.grpo_loss_chunked_torch): float32 torch matmuls
(independent of the kernels under test) with float64 softmax statistics.  configs[0] is checked
on the CPU (the reference's own CPU-runnable case); configs[1..4] are checked with the oracle's
torch form running on the GPU, at full hidden/vocab size; configs[3] (32768 tokens) is checked on
its first 16384 tokens with the normaliser of the whole batch.  Size-independent properties
(dZ rows sum to zero => d_lm_head rows sum to zero; masked rows have zero d_hidden) are checked
at full size too.
"""
import dataclasses

import numpy as np
import pytest
import torch

from oracle import grpo_oracle as O

pytestmark = pytest.mark.gpu

LOGP_ATOL, LOSS_RTOL, GRAD_RTOL, ENT_ATOL = 1e-3, 1e-3, 2e-2, 1e-3


def _rel(a, b):
    return float((a.double() - b.double()).norm() / b.double().norm().clamp_min(1e-30))


def _make(idx, seqs=None):
    import mllm_jax_amd as M
    dev = torch.device("cuda:0")
    cfg = M.CONFIGS[idx]
    kw = dict(epsilon_low=cfg.eps_low, epsilon_high=cfg.eps_high, final_logit_softcap=cfg.softcap)

    def logp_fn(wl):
        with torch.no_grad():
            return M.grpo_fused_loss(wl["hidden"], wl["lm_head"], wl["target_ids"], None, wl["advantages"],
                                     wl["mask"], total_valid_token_count=wl["total_valid_token_count"],
                                     **kw)["per_token_logps"]

    from mllm_jax_amd.workloads import gumbel_max_targets as sample_fn

    wl = M.make_workload(cfg, dev, 20250 + idx, logp_fn=logp_fn, sample_fn=sample_fn, seqs=seqs)
    return M, cfg, kw, wl


def _check_against(ref, met, dh, dw, rows=None):
    sel = slice(None) if rows is None else rows
    logp = met["per_token_logps"].reshape(-1)[sel].double().cpu()
    ent = met["token_entropy"].reshape(-1)[sel].double().cpu()
    r_logp = torch.as_tensor(ref["per_token_logps"])[sel].cpu()
    r_ent = torch.as_tensor(ref["token_entropy"])[sel].cpu()
    assert (logp - r_logp).abs().max().item() <= LOGP_ATOL
    assert (ent - r_ent).abs().max().item() <= ENT_ATOL
    return logp, ent


def test_config0_qwen05b_against_cpu_oracle():
    M, cfg, kw, wl = _make(0)
    met, (dh, dw) = M.grpo_loss_value_and_grad(
        wl["hidden"], wl["lm_head"], wl["target_ids"], wl["old_logps"], wl["advantages"], wl["mask"],
        total_valid_token_count=wl["total_valid_token_count"], seq_shape=wl["seq_shape"],
        return_token_entropy=True, **kw)
    torch.cuda.synchronize()
    ref = O.grpo_loss_chunked_torch(
        wl["hidden"].cpu(), wl["lm_head"].cpu(), wl["target_ids"].cpu(), wl["old_logps"].cpu(),
        wl["advantages"].cpu(), wl["mask"].cpu(), total_valid_token_count=wl["total_valid_token_count"],
        epsilon_low=cfg.eps_low, epsilon_high=cfg.eps_high, chunk=256, device="cpu", as_numpy=False)
    _check_against(ref, met, dh, dw)
    assert abs(met["loss"].item() - ref["loss"]) <= LOSS_RTOL * abs(ref["loss"])
    assert _rel(dh.float().cpu(), ref["d_hidden"]) <= GRAD_RTOL
    assert _rel(dw.cpu(), ref["d_lm_head"]) <= GRAD_RTOL
    assert wl["old_logps"] is not None and wl["advantages"].abs().max() > 0


@pytest.mark.parametrize("idx,seqs", [(1, None), (2, None), (4, None), (3, 64)])
def test_config_shapes_against_torch_form_of_oracle(idx, seqs):
    M, cfg, kw, wl = _make(idx, seqs=seqs)
    n = wl["hidden"].shape[0]
    met, (dh, dw) = M.grpo_loss_value_and_grad(
        wl["hidden"], wl["lm_head"], wl["target_ids"], wl["old_logps"], wl["advantages"], wl["mask"],
        total_valid_token_count=wl["total_valid_token_count"], seq_shape=wl["seq_shape"],
        return_token_entropy=True, **kw)
    torch.cuda.synchronize()
    ref = O.grpo_loss_chunked_torch(
        wl["hidden"], wl["lm_head"], wl["target_ids"], wl["old_logps"], wl["advantages"], wl["mask"],
        total_valid_token_count=wl["total_valid_token_count"], epsilon_low=cfg.eps_low,
        epsilon_high=cfg.eps_high, final_logit_softcap=cfg.softcap, chunk=1024, device="cuda:0",
        as_numpy=False)
    _check_against(ref, met, dh, dw)
    assert abs(met["loss"].item() - ref["loss"]) <= LOSS_RTOL * abs(ref["loss"])
    assert _rel(dh.float(), ref["d_hidden"]) <= GRAD_RTOL
    assert _rel(dw, ref["d_lm_head"]) <= GRAD_RTOL
    # per-row check on unmasked rows, and exact zeros on masked ones
    valid = wl["mask"] > 0
    num = (dh.float() - ref["d_hidden"])[valid].norm(dim=-1)
    den = ref["d_hidden"][valid].norm(dim=-1)
    nz = den > 1e-12
    assert (num[nz] / den[nz]).max().item() <= 5e-2
    assert not dh[~valid].any()
    # rows of dZ sum to zero (no softcap)  =>  rows of d_lm_head sum to ~0 relative to their size
    if cfg.softcap is None:
        rs = dw.double().sum(-1).abs().max().item()
        assert rs <= 1e-3 * dw.double().abs().sum(-1).max().item()
    # the per-sample entropy metrics of the reference's return dict
    b, t = wl["seq_shape"]
    ent_ref = (torch.as_tensor(ref["token_entropy"]).reshape(b, t) * wl["mask"].reshape(b, t).double()).sum(-1) \
        / wl["mask"].reshape(b, t).double().sum(-1)
    assert (met["entropy"].double() - ent_ref).abs().max().item() <= ENT_ATOL
    del ref, dh, dw
    M.release_workspaces()
    torch.cuda.empty_cache()


def test_config3_full_size_runs_and_is_consistent():
    """Llama-3-8B shape at its full 32768 tokens: the fused pass must agree with the forward-only
    pass bit for bit and keep the size-independent gradient properties."""
    M, cfg, kw, wl = _make(3)
    with torch.no_grad():
        fwd = M.grpo_fused_loss(wl["hidden"], wl["lm_head"], wl["target_ids"], wl["old_logps"],
                                wl["advantages"], wl["mask"], return_token_entropy=True,
                                total_valid_token_count=wl["total_valid_token_count"], **kw)
    met, (dh, dw) = M.grpo_loss_value_and_grad(
        wl["hidden"], wl["lm_head"], wl["target_ids"], wl["old_logps"], wl["advantages"], wl["mask"],
        total_valid_token_count=wl["total_valid_token_count"], seq_shape=wl["seq_shape"],
        return_token_entropy=True, **kw)
    torch.cuda.synchronize()
    assert torch.equal(fwd["per_token_logps"].reshape(-1), met["per_token_logps"].reshape(-1))
    assert torch.equal(fwd["token_entropy"].reshape(-1), met["token_entropy"].reshape(-1))
    assert torch.equal(fwd["loss"], met["loss"])
    assert met["token_entropy"].shape == wl["seq_shape"]
    assert not dh[wl["mask"] == 0].any() and dh[wl["mask"] > 0].float().abs().sum() > 0
    rs = dw.double().sum(-1).abs().max().item()
    assert rs <= 1e-3 * dw.double().abs().sum(-1).max().item()
    # all 32768 tokens against the oracle, in two halves of rows (the second half is the chunk the
    # kernels reach with a non-zero chunk origin and an accumulating dW); the halves' d_lm_head
    # shares add up to the whole gradient
    n = wl["hidden"].shape[0]
    ref_dw = None
    for half in (torch.arange(0, n // 2), torch.arange(n // 2, n)):
        ref = O.grpo_loss_chunked_torch(
            wl["hidden"], wl["lm_head"], wl["target_ids"], wl["old_logps"], wl["advantages"], wl["mask"],
            total_valid_token_count=wl["total_valid_token_count"], epsilon_low=cfg.eps_low,
            epsilon_high=cfg.eps_high, final_logit_softcap=cfg.softcap, chunk=1024, rows=half, device="cuda:0",
            as_numpy=False)
        rows = half.to(dh.device)
        _check_against(ref, met, dh, dw, rows=rows)
        assert _rel(dh[rows].float(), ref["d_hidden"][rows]) <= GRAD_RTOL
        ref_dw = ref["d_lm_head"] if ref_dw is None else ref_dw.add_(ref["d_lm_head"])
        del ref
    assert _rel(dw, ref_dw) <= GRAD_RTOL
    del ref_dw
    M.release_workspaces()
    torch.cuda.empty_cache()


def test_config3_full_size_skip_masked_equals_dense():
    """Same full-size shape (two chunks of 16384 tokens): leaving the masked tokens out of the backward
    products changes neither the forward outputs nor d_hidden (bit for bit) and d_lm_head only by
    summation order."""
    M, cfg, kw, wl = _make(3)
    args = (wl["hidden"], wl["lm_head"], wl["target_ids"], wl["old_logps"], wl["advantages"], wl["mask"])
    opts = dict(total_valid_token_count=wl["total_valid_token_count"], seq_shape=wl["seq_shape"],
                return_token_entropy=True, **kw)
    met_d, (dh_d, dw_d) = M.grpo_loss_value_and_grad(*args, **opts)
    dh_d, dw_d = dh_d.clone(), dw_d.clone()
    met_s, (dh_s, dw_s) = M.grpo_loss_value_and_grad(*args, skip_masked=True, **opts)
    torch.cuda.synchronize()
    assert torch.equal(met_d["per_token_logps"], met_s["per_token_logps"])
    assert torch.equal(met_d["token_entropy"], met_s["token_entropy"])
    assert abs(float(met_d["loss"]) - float(met_s["loss"])) <= 1e-5 * abs(float(met_d["loss"]))
    assert torch.equal(dh_d, dh_s)
    assert _rel(dw_s, dw_d) <= 1e-3
    M.release_workspaces()
    torch.cuda.empty_cache()
