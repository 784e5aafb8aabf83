"""Host side of the RMSNorm kernels: the final norm that produces the loss path's `hidden`.

Mirrors LlamaRMSNorm (MLLM_JAX/language/llama/llama.py:426-452; the backbone's `self.norm`,
qwen2/modular_qwen2.py:76, :128) as a differentiable torch function over the HIP kernels in
libmj_grpo.so.  No CPU fallback exists.
"""
from __future__ import annotations

import torch

from . import _lib

_parts: dict = {}


def _check(x: torch.Tensor, scale: torch.Tensor):
    if x.device.type != "cuda":
        raise RuntimeError(f"rms_norm needs tensors on an MI355X device (got {x.device}); there is no CPU path")
    if x.shape[-1] != scale.numel():
        raise ValueError(f"scale has {scale.numel()} elements, x has {x.shape[-1]} features")


def _rows(t: torch.Tensor) -> torch.Tensor:
    t2 = t.reshape(-1, t.shape[-1])
    if t2.dtype != torch.bfloat16:
        t2 = t2.to(torch.bfloat16)
    if t2.stride(1) != 1 or t2.stride(0) % 8 or t2.data_ptr() % 16:
        t2 = t2.contiguous()
    return t2


class _RmsNormFn(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, scale, eps):
        x2 = _rows(x)
        s32 = scale.detach().reshape(-1).to(torch.float32).contiguous()
        n, h = x2.shape
        y = torch.empty((n, h), dtype=torch.bfloat16, device=x.device)
        with torch.cuda.device(x.device):
            _lib.check(_lib.load().mj_rmsnorm_forward(
                x2.data_ptr(), x2.stride(0), s32.data_ptr(), y.data_ptr(), h, None, n, h, float(eps),
                torch.cuda.current_stream(x.device).cuda_stream))
        ctx.save_for_backward(x2, s32)
        ctx.meta = (x.shape, x.dtype, scale.shape, scale.dtype, float(eps))
        return y.reshape(x.shape).to(x.dtype)                    # cast back to the input dtype (llama.py:451)

    @staticmethod
    def backward(ctx, dy):
        x2, s32 = ctx.saved_tensors
        shape, x_dtype, s_shape, s_dtype, eps = ctx.meta
        n, h = x2.shape
        dy2 = _rows(dy)
        dx = torch.empty((n, h), dtype=torch.bfloat16, device=x2.device)
        ds = torch.empty(h, dtype=torch.float32, device=x2.device)
        lib = _lib.load()
        import ctypes as C
        need = C.c_size_t()
        _lib.check(lib.mj_rmsnorm_workspace_bytes(n, h, C.byref(need)))
        key = (x2.device.index, need.value)
        ws = _parts.get(key)
        if ws is None:
            _parts.clear()
            ws = _parts[key] = torch.empty(need.value, dtype=torch.uint8, device=x2.device)
        with torch.cuda.device(x2.device):
            _lib.check(lib.mj_rmsnorm_backward(
                dy2.data_ptr(), dy2.stride(0), x2.data_ptr(), x2.stride(0), s32.data_ptr(), dx.data_ptr(), h,
                ds.data_ptr(), 0, n, h, eps, ws.data_ptr(), ws.numel(),
                torch.cuda.current_stream(x2.device).cuda_stream))
        return dx.reshape(shape).to(x_dtype), ds.reshape(s_shape).to(s_dtype), None


def rms_norm(x: torch.Tensor, scale: torch.Tensor, eps: float = 1e-6) -> torch.Tensor:
    """y = x * rsqrt(mean(x^2, -1) + eps) * scale in float32, returned in x's dtype
    (llama.py:438-451).  x: [..., H] bf16 on the GPU (other float dtypes are cast), scale: [H].
    Differentiable with respect to x and scale."""
    _check(x, scale)
    return _RmsNormFn.apply(x, scale, eps)


class LlamaRMSNorm:
    """Call-compatible stand-in for the reference module (llama.py:426-452): holds `scale`."""

    def __init__(self, scale: torch.Tensor, eps: float = 1e-6):
        self.scale, self.eps = scale, eps

    def __call__(self, x: torch.Tensor) -> torch.Tensor:
        return rms_norm(x, self.scale, self.eps)
