"""Host side of the sampler's last-position step: logits of the newest position and the
top-k / categorical draw over them, on the HIP kernels in libmj_grpo.so.

Mirrors MLLM_JAX/sample/sanple_utils.py:35-60 (_top_k_sampling_batched, _temperature_sampling,
_greedy_sampling) as used by the decode step (sample_state_right_padding2.py:219-234).
jax.random.categorical(key, x) is argmax(x + Gumbel noise); here the Gumbel noise comes from a
torch.Generator (or from the caller), so draws are reproducible but do not replay JAX's
threefry stream.  No CPU fallback exists.
"""
from __future__ import annotations

from typing import Optional, Union

import torch

from . import _lib


def _gumbel(shape, device, generator: Optional[torch.Generator]) -> torch.Tensor:
    u = torch.rand(shape, device=device, dtype=torch.float32, generator=generator)
    tiny = torch.finfo(torch.float32).tiny
    return -torch.log(-torch.log(u.clamp_min(tiny)).clamp_min(tiny))


def last_position_logits(hidden_last: torch.Tensor, lm_head: torch.Tensor,
                         final_logit_softcap: Optional[float] = None) -> torch.Tensor:
    """float32 logits [B, V] = hidden_last [B, H] @ lm_head [H, V] (qwen2/modular_qwen2.py:182 for
    the newest position, `logits[:, -1]` of sample_state_right_padding2.py:230)."""
    if hidden_last.device.type != "cuda":
        raise RuntimeError("last_position_logits needs GPU tensors; there is no CPU path")
    if hidden_last.dim() != 2 or lm_head.dim() != 2 or hidden_last.shape[1] != lm_head.shape[0]:
        raise ValueError(f"hidden {tuple(hidden_last.shape)} and lm_head {tuple(lm_head.shape)} do not form [B,H] x [H,V]")
    hid = hidden_last.detach().to(torch.bfloat16)
    if hid.stride(1) != 1 or hid.stride(0) % 8 or hid.data_ptr() % 16:
        hid = hid.contiguous()
    w = lm_head.detach().to(torch.bfloat16)
    if w.stride(1) != 1 or w.stride(0) % 8 or w.data_ptr() % 16:
        w = w.contiguous()
    b, h = hid.shape
    v = w.shape[1]
    out = torch.empty((b, v), dtype=torch.float32, device=hid.device)
    with torch.cuda.device(hid.device):
        _lib.check(_lib.load().mj_sample_logits(
            hid.data_ptr(), hid.stride(0), w.data_ptr(), w.stride(0), out.data_ptr(), v, b, h, v,
            float(final_logit_softcap or 0.0), torch.cuda.current_stream(hid.device).cuda_stream))
    return out


def top_k_sampling_batched(rng: Union[torch.Generator, torch.Tensor, None], logits: torch.Tensor, k: int = 50,
                           t: float = 0.9, return_top_k: bool = False):
    """_top_k_sampling_batched (sanple_utils.py:35-53): per row, the k largest of logits / t, a
    categorical draw among them, the drawn entry's vocabulary index (int32 [B]).

    rng: a torch.Generator on the logits' device, or a float32 [B, k] tensor of Gumbel noise
    (slot j belongs to the j-th largest logit), or None for the greedy choice."""
    if logits.device.type != "cuda":
        raise RuntimeError("top_k_sampling_batched needs GPU tensors; there is no CPU path")
    if logits.dim() != 2:
        raise ValueError(f"logits must be [B, V], got {tuple(logits.shape)}")
    lg = logits.detach().to(torch.float32)
    if lg.stride(1) != 1:
        lg = lg.contiguous()
    b, v = lg.shape
    if isinstance(rng, torch.Tensor):
        noise = rng.to(device=lg.device, dtype=torch.float32).contiguous()
        if tuple(noise.shape) != (b, k):
            raise ValueError(f"noise must be [B, k] = {(b, k)}, got {tuple(noise.shape)}")
    elif rng is None:
        noise = None
    else:
        noise = _gumbel((b, k), lg.device, rng)
    token = torch.empty(b, dtype=torch.int32, device=lg.device)
    idx = torch.empty((b, k), dtype=torch.int32, device=lg.device) if return_top_k else None
    val = torch.empty((b, k), dtype=torch.float32, device=lg.device) if return_top_k else None
    with torch.cuda.device(lg.device):
        _lib.check(_lib.load().mj_sample_top_k(
            lg.data_ptr(), lg.stride(0), b, v, int(k), float(t), None if noise is None else noise.data_ptr(),
            token.data_ptr(), None if idx is None else idx.data_ptr(), None if val is None else val.data_ptr(),
            torch.cuda.current_stream(lg.device).cuda_stream))
    return (token, idx, val) if return_top_k else token


def greedy_sampling(rng, logits: torch.Tensor) -> torch.Tensor:
    """_greedy_sampling (sanple_utils.py:58-60): argmax over the vocabulary (first maximum)."""
    del rng
    return top_k_sampling_batched(None, logits, k=1, t=1.0)


def sample_next_tokens(rng, hidden_last: torch.Tensor, lm_head: torch.Tensor, k: int = 50, t: float = 1.0,
                       final_logit_softcap: Optional[float] = None) -> torch.Tensor:
    """The decode step's `self.sample_fn(key2, logits[:, -1])` (sample_state_right_padding2.py:229-230)
    from the final hidden state of the newest position: product and draw, nothing in between."""
    return top_k_sampling_batched(rng, last_position_logits(hidden_last, lm_head, final_logit_softcap), k=k, t=t)
