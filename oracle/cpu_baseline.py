"""CPU baseline for the bench's `cpu_baseline` leg.  TEST/BENCH INFRASTRUCTURE ONLY.

The reference's path is un-fused jnp on XLA (MLLM_JAX/train_modules/__init__.py:118-180
under jax.value_and_grad, plugins/training/update/train_step.py:24).  JAX is not
installed on the build or GPU box, so this is a port ("kind": "port") of the same
un-fused arithmetic to torch on the host cores: materialised float32 [n,V] logits,
log_softmax, gather, softmax entropy, ratio/clip/min, masked sum / tvtc, and
torch.autograd for the backward to d_hidden and d_lm_head.
"""
from __future__ import annotations

import os
import time


def unfused_loss_fwd_bwd(hidden_bf16, lm_head_bf16, target_ids, old_logps, advantages, mask,
                         total_valid_token_count, epsilon_low, epsilon_high, softcap=None):
    """One fwd+bwd of the un-fused loss on CPU tensors.  Returns (loss, logp, d_h, d_w)."""
    import torch

    h = hidden_bf16.float().requires_grad_(True)
    w = lm_head_bf16.float().requires_grad_(True)
    z = h @ w                                                   # modular_qwen2.py:182
    if softcap:
        z = torch.tanh(z / softcap) * softcap                   # gemma/transformer.py:337-339
    logp_all = torch.log_softmax(z, dim=-1)                     # :125
    logp = logp_all.gather(1, target_ids.long()[:, None])[:, 0]  # :124-126
    p = torch.softmax(z, dim=-1)                                # :136
    ent = -(p * torch.log(p + 1e-9)).sum(-1)                    # :138
    old = logp.detach() if old_logps is None else old_logps
    ratio = torch.exp(logp - old)                               # :169
    clipped = ratio.clamp(1.0 - epsilon_low, 1.0 + epsilon_high)  # :170
    ptl = -torch.minimum(ratio * advantages, clipped * advantages)  # :174-178
    loss = (ptl * mask).sum() / total_valid_token_count         # :180
    loss.backward()
    return loss.detach(), logp.detach(), ent.detach(), h.grad, w.grad


def time_cpu_baseline(workload, sample_tokens, repeats=1, threads=None):
    """Times the port on the first `sample_tokens` tokens of a workload dict of CPU
    tensors (keys as produced by the package's workload generator).  Returns
    {"tokens_per_s", "seconds", "cores", "sample_tokens"}."""
    import torch

    cores = threads or os.cpu_count() or 1
    torch.set_num_threads(cores)
    n = min(int(sample_tokens), workload["hidden"].shape[0])
    sl = slice(0, n)
    args = (workload["hidden"][sl].cpu(), workload["lm_head"].cpu(), workload["target_ids"][sl].cpu(),
            None if workload.get("old_logps") is None else workload["old_logps"][sl].cpu().float(),
            workload["advantages"][sl].cpu().float(), workload["mask"][sl].cpu().float(),
            float(workload["total_valid_token_count"]), float(workload["epsilon_low"]),
            float(workload["epsilon_high"]), workload.get("softcap"))
    best = float("inf")
    for _ in range(max(1, repeats)):
        t0 = time.perf_counter()
        unfused_loss_fwd_bwd(*args)
        best = min(best, time.perf_counter() - t0)
    return {"tokens_per_s": n / best, "seconds": best, "cores": cores, "sample_tokens": n}
