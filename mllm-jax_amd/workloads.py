"""Synthetic inputs of the five benchmark configurations (BASELINE.json `configs`).

Seeded torch generators on the requested device; the same tensors feed the kernels, the
parity tests' CPU oracle and the bench's CPU baseline.  The advantage generator restates
plugins/training/advantage/grpo.py:28-52 and the mask follows the rollout's contiguous
completion span (plugins/training/rollout/sampling.py:98-108).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Callable, Optional

import torch


@dataclass(frozen=True)
class LossConfig:
    name: str
    seqs: int            # B = prompts x group size
    seq_len: int         # T
    hidden: int
    vocab: int
    group: int           # G
    w_std: float
    own_softmax_targets: bool
    reward_p: float      # Bernoulli parameter of the {0,1} rewards
    len_lo: int
    len_hi: int
    eps_low: float = 0.2
    eps_high: float = 0.2
    softcap: Optional[float] = None
    token_entropy: bool = False

    @property
    def tokens(self) -> int:
        return self.seqs * self.seq_len


CONFIGS = (
    LossConfig("qwen2.5-0.5b", 2, 256, 896, 151936, 2, 0.02, False, 0.5, 64, 256),
    LossConfig("qwen2.5-1.5b", 32, 128, 1536, 151936, 8, 0.02, True, 0.5, 64, 128),
    LossConfig("qwen2.5-7b", 128, 128, 3584, 152064, 8, 0.015, False, 0.3, 32, 128),
    LossConfig("llama-3-8b", 128, 256, 4096, 128256, 16, 0.02, True, 0.5, 64, 256,
               eps_high=0.28, token_entropy=True),
    LossConfig("gemma-2-2b", 128, 128, 2304, 256000, 8, 0.02, False, 0.5, 32, 128, softcap=30.0),
)


def group_advantages(rewards: torch.Tensor, group: int, eps: float = 1e-4) -> torch.Tensor:
    """(r - mean_g) / (std_g + eps) with the population std of each group of `group`
    consecutive sequences (advantage/grpo.py:41-51), float32."""
    r = rewards.float().reshape(-1, group)
    c = r - r.mean(-1, keepdim=True)
    std = (c * c).mean(-1, keepdim=True).sqrt()
    return (c / (std + eps)).reshape(-1)


def make_workload(cfg: LossConfig, device, seed: int,
                  logp_fn: Optional[Callable[[dict], torch.Tensor]] = None,
                  sample_fn: Optional[Callable[[dict, torch.Generator], torch.Tensor]] = None,
                  tokens_per_seq: Optional[int] = None, seqs: Optional[int] = None) -> dict:
    """Builds one batch.  `logp_fn(workload) -> logp[N]` supplies the current log-probs that
    old_logps = logp + 0.05*randn are derived from (None leaves old_logps = None: on-policy).
    `sample_fn(workload, generator) -> ids[N]` draws targets from the model's own softmax for the
    configurations that ask for it (falls back to uniform ids when None).
    `tokens_per_seq` / `seqs` shrink the batch (tests); hidden and vocab stay at full size."""
    b = seqs or cfg.seqs
    t = tokens_per_seq or cfg.seq_len
    n = b * t
    g = torch.Generator(device="cpu").manual_seed(seed)
    gd = torch.Generator(device=device).manual_seed(seed)
    hidden = torch.randn(n, cfg.hidden, generator=gd, device=device, dtype=torch.float32).to(torch.bfloat16)
    w = (torch.randn(cfg.hidden, cfg.vocab, generator=gd, device=device, dtype=torch.float32)
         * cfg.w_std).to(torch.bfloat16)
    targets = torch.randint(0, cfg.vocab, (n,), generator=g).to(torch.int32)
    grp = min(cfg.group, b)
    rewards = (torch.rand(b, generator=g) < cfg.reward_p).float()
    if b == 2:
        rewards = torch.tensor([1.0, 0.0])          # two identical rewards would zero every advantage
    adv_seq = group_advantages(rewards, grp)
    lo, hi = min(cfg.len_lo, t), min(cfg.len_hi, t)
    lens = torch.randint(lo, hi + 1, (b,), generator=g)
    mask = (torch.arange(t)[None, :] < lens[:, None]).float().reshape(-1)
    wl = {
        "config": cfg, "seq_shape": (b, t), "hidden": hidden, "lm_head": w,
        "target_ids": targets.to(device), "advantages": adv_seq.repeat_interleave(t).to(device),
        "mask": mask.to(device), "old_logps": None,
        "total_valid_token_count": float(mask.sum().item()),
        "epsilon_low": cfg.eps_low, "epsilon_high": cfg.eps_high, "softcap": cfg.softcap,
    }
    if cfg.own_softmax_targets and sample_fn is not None:
        wl["target_ids"] = sample_fn(wl, g).to(torch.int32).to(device)
    if logp_fn is not None:
        logp = logp_fn(wl).detach().float().reshape(-1).cpu()
        wl["old_logps"] = (logp + 0.05 * torch.randn(n, generator=g)).to(device)
    return wl


def gumbel_max_targets(wl: dict, gen: torch.Generator) -> torch.Tensor:
    """`sample_fn` for make_workload: one Gumbel-max draw per token from softmax(hidden @ lm_head) at
    temperature 1 ("targets sampled from the model's own softmax"), 1024 tokens at a time.  Input
    generation only: plain torch on the workload's device, not the loss path."""
    h, w = wl["hidden"].float(), wl["lm_head"].float()
    out = torch.empty(h.shape[0], dtype=torch.int64, device=h.device)
    g = torch.Generator(device=h.device).manual_seed(int(gen.initial_seed()) + 1)
    for s in range(0, h.shape[0], 1024):
        z = h[s:s + 1024] @ w
        u = torch.rand(z.shape, generator=g, device=h.device).clamp_min(1e-20)
        out[s:s + 1024] = (z - torch.log(-torch.log(u))).argmax(-1)
    return out


def flops(cfg_or_shape) -> float:
    """Algorithmic flop of one fwd+bwd: 6*N*H*V (logits, dHidden, dW)."""
    if isinstance(cfg_or_shape, LossConfig):
        n, h, v = cfg_or_shape.tokens, cfg_or_shape.hidden, cfg_or_shape.vocab
    else:
        n, h, v = cfg_or_shape
    return 6.0 * n * h * v
