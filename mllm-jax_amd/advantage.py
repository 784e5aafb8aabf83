"""Advantage estimators on the device: host mirrors of plugins/training/advantage/grpo.py and
plugins/training/advantage/estimators.py (same names, keyword arguments and error behaviour),
evaluated by the HIP kernels in libmj_grpo.so on GPU tensors.  Each returns float32 GPU tensors.
No CPU fallback exists.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib

_MODES = {"grpo": 0, "global": 1, "rloo": 2, "dapo": 3}


def _rewards(rewards, name="rewards") -> torch.Tensor:
    r = torch.as_tensor(rewards)
    if r.device.type != "cuda":
        raise RuntimeError(f"{name} must be a GPU tensor; the advantage estimators have no CPU path")
    r = r.reshape(-1).to(torch.float32).contiguous()       # estimators.py:10-16 flattens
    if r.numel() <= 0:
        raise ValueError(f"{name} must be non-empty")
    return r


def _group_ids(group_ids, r: torch.Tensor) -> torch.Tensor:
    g = torch.as_tensor(group_ids, device=r.device).reshape(-1)
    if g.numel() != r.numel():
        raise ValueError(f"group_ids must have shape [B] with B={r.numel()}, got size={g.numel()}")
    return g.to(torch.int32).contiguous()


def _clip(clip_range: Optional[float]) -> float:
    if clip_range is None:
        return 0.0
    if float(clip_range) <= 0:
        raise ValueError("clip_range must be > 0 when set")
    return float(clip_range)


def _run(mode: str, r: torch.Tensor, g: Optional[torch.Tensor], eps: float, alpha: float, whiten: bool,
         clip: float) -> torch.Tensor:
    if float(eps) <= 0:
        raise ValueError("eps must be > 0")
    out = torch.empty_like(r)
    with torch.cuda.device(r.device):
        _lib.check(_lib.load().mj_grpo_advantages(
            _MODES[mode], r.data_ptr(), None if g is None else g.data_ptr(), out.data_ptr(), r.numel(), float(eps),
            float(alpha), int(bool(whiten)), clip, torch.cuda.current_stream(r.device).cuda_stream))
    return out


def compute_global_normalized_advantages(*, rewards, eps: float = 1e-4, clip_range: Optional[float] = None):
    """estimators.py:37-55: (r - mean) / (std + eps) over the batch, optional clip."""
    r = _rewards(rewards)
    return _run("global", r, None, eps, 0.0, False, _clip(clip_range))


def compute_rloo_advantages_by_group_id(*, rewards, group_ids, eps: float = 1e-4, whiten: bool = True,
                                        clip_range: Optional[float] = None):
    """estimators.py:58-103: reward minus the mean of the other samples of its group (0 for singleton
    groups), optionally centred and scaled over the batch."""
    r = _rewards(rewards)
    return _run("rloo", r, _group_ids(group_ids, r), eps, 0.0, whiten, _clip(clip_range))


def compute_dapo_advantages_by_group_id(*, rewards, group_ids, eps: float = 1e-4, alpha: float = 0.2,
                                        clip_range: Optional[float] = None):
    """estimators.py:106-134: group-normalised advantages + alpha * globally normalised ones."""
    if float(alpha) < 0:
        raise ValueError("alpha must be >= 0")
    r = _rewards(rewards)
    return _run("dapo", r, _group_ids(group_ids, r), eps, alpha, False, _clip(clip_range))


def compute_reinforce_plus_plus_advantages_by_group_id(*, rewards, group_ids, eps: float = 1e-4,
                                                       clip_range: Optional[float] = None):
    """estimators.py:137-157: the leave-one-out baseline with whitening."""
    return compute_rloo_advantages_by_group_id(rewards=rewards, group_ids=group_ids, eps=eps, whiten=True,
                                               clip_range=clip_range)


def _mask_2d(completion_mask, r: torch.Tensor) -> torch.Tensor:
    m = torch.as_tensor(completion_mask, device=r.device).to(torch.float32)
    if m.dim() != 2:
        raise ValueError(f"completion_mask must be rank-2 [B, T], got shape={tuple(m.shape)}")
    if m.shape[0] != r.numel():
        raise ValueError(f"completion_mask batch must match rewards (B={r.numel()}), got {m.shape[0]}")
    return m.contiguous()


def compute_gae_advantages(*, rewards, values, completion_mask, gamma: float = 1.0, gae_lambda: float = 0.95,
                           normalize: bool = True, eps: float = 1e-4,
                           clip_range: Optional[float] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """estimators.py:180-240: token-level GAE advantages and returns [B, T] from a sequence-level
    reward placed on the last completion token; returns = un-normalised advantages + values."""
    r = _rewards(rewards)
    v = torch.as_tensor(values, device=r.device).to(torch.float32)
    if v.dim() != 2:
        raise ValueError(f"values must be rank-2 [B, T], got shape={tuple(v.shape)}")
    if v.shape[0] != r.numel():
        raise ValueError(f"values batch must match rewards (B={r.numel()}), got {v.shape[0]}")
    m = torch.as_tensor(completion_mask, device=r.device).to(torch.float32)
    if m.dim() != 2:
        raise ValueError(f"completion_mask must be rank-2 [B, T], got shape={tuple(m.shape)}")
    if v.shape != m.shape:
        raise ValueError(f"values and completion_mask must match shape, got {tuple(v.shape)} vs {tuple(m.shape)}")
    v, m = v.contiguous(), m.contiguous()
    adv, ret = torch.empty_like(v), torch.empty_like(v)
    with torch.cuda.device(r.device):
        _lib.check(_lib.load().mj_grpo_gae(
            r.data_ptr(), v.data_ptr(), m.data_ptr(), adv.data_ptr(), ret.data_ptr(), v.shape[0], v.shape[1],
            float(gamma), float(gae_lambda), int(bool(normalize)), float(eps), _clip(clip_range),
            torch.cuda.current_stream(r.device).cuda_stream))
    return adv, ret


def build_token_rewards_from_final(*, rewards, completion_mask) -> torch.Tensor:
    """estimators.py:160-177: [B, T] rewards with the sequence reward on the last completion token
    (the GAE kernel with zero values, gamma = 1, lambda = 0 yields exactly these per-token deltas)."""
    r = _rewards(rewards)
    m = _mask_2d(completion_mask, r)
    adv, _ = compute_gae_advantages(rewards=r, values=torch.zeros_like(m), completion_mask=m, gamma=1.0,
                                    gae_lambda=0.0, normalize=False)
    return adv
