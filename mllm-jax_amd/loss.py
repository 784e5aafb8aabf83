"""Host side of the fused GRPO loss: the reference's loss-function contract on top of
the HIP kernels in libmj_grpo.so.

Mirrors, for the lm_head + loss part only:
  MLLM_JAX/train_modules/__init__.py:84-192   TrainGRPOModule (inputs / outputs, hyper-parameters)
  plugins/training/update/train_step.py:15-24 loss_fn + jax.value_and_grad(has_aux=True)
  plugins/sft/jax/sft_module.py:22-45         TrainSftModule (masked cross-entropy)
  plugins/training/ppo/module.py:59-150       PPOActorCriticModule (policy + value + entropy bonus)

torch is used for device memory, streams and autograd plumbing only; all arithmetic on
[tokens, vocab]-sized data happens in the HIP kernels.  No CPU fallback exists.
"""
from __future__ import annotations

import contextlib
import ctypes as C
import threading
import weakref
from typing import Any, Callable, Mapping, Optional

import torch

from . import _lib

class _DeviceWorkspace:
    """The cached workspace of one device and the stream that used it last."""
    __slots__ = ("tensor", "stream")

    def __init__(self, tensor: torch.Tensor, stream: torch.cuda.Stream):
        self.tensor, self.stream = tensor, stream


_workspaces: dict[Any, _DeviceWorkspace] = {}


def _workspace(device: torch.device, nbytes: int) -> torch.Tensor:
    """One workspace per device, grown on demand.  The library's rule is "two calls may overlap only
    if they use distinct workspaces": a call on another stream than the previous one first waits for
    everything that stream had enqueued, so calls from several streams share the buffer one after
    the other instead of each stream keeping ~6 GB of its own.  Under stream capture the buffer is a
    fresh allocation from the graph's own pool and is not cached: a captured address must never be
    handed to eager code."""
    stream = torch.cuda.current_stream(device)
    if torch.cuda.is_current_stream_capturing():
        return torch.empty(nbytes, dtype=torch.uint8, device=device)
    key = (device.type, device.index)
    ent = _workspaces.get(key)
    if ent is not None and ent.stream != stream:
        stream.wait_event(ent.stream.record_event())
        ent.tensor.record_stream(stream)      # the caching allocator must not recycle it under this stream
        ent.stream = stream
    if ent is None or ent.tensor.numel() < nbytes:
        _workspaces.pop(key, None)
        ent = None                            # free the old buffer before asking for the larger one
        ent = _DeviceWorkspace(torch.empty(nbytes, dtype=torch.uint8, device=device), stream)
        _workspaces[key] = ent
    return ent.tensor


def release_workspaces() -> None:
    """Drops the cached workspaces (one per device) and any cached bf16 copy of float32 weights."""
    _workspaces.clear()
    _bf16_copies.clear()


_bf16_copies: dict = {}      # id(tensor) -> (weak reference to it, state key, bf16 copy)


class _Bf16Cache(threading.local):
    depth: int = 0


_bf16_cache = _Bf16Cache()


@contextlib.contextmanager
def cache_bf16_lm_head():
    """Within this context the bf16 copy that the kernels read of a FLOAT32 lm_head is kept between
    calls for as long as the same tensor object is unchanged (same object, same autograd version
    counter, same storage and layout) and dropped on leaving.  The cast of [H,V] is a 3.3 GB pass at
    the Qwen2.5-7B shape; the micro-batches and PPO epochs between two optimizer steps all read the
    same weights (ppo_update opens this context around each of those spans).

    Opt-in because the version counter does not see every write: `w.data.add_(...)`, the
    torch._foreach_* updates of some optimizers and some checkpoint loaders change the values
    without bumping it.  Open the context only around code that does not write the weights that
    way, or call invalidate_bf16_lm_head() after such a write.  Outside the context every call
    casts anew (what the reference does: param_dtype f32, dtype bf16,
    MLLM_JAX/language/llama/llama.py:251-256)."""
    _bf16_cache.depth += 1
    try:
        yield
    finally:
        _bf16_cache.depth -= 1
        if _bf16_cache.depth == 0:
            _bf16_copies.clear()


def invalidate_bf16_lm_head() -> None:
    """Forgets every cached bf16 copy (see cache_bf16_lm_head): call after writing float32 weights
    through `.data` or any other route that does not bump the tensor's version counter."""
    _bf16_copies.clear()


def _bf16_weights(w: torch.Tensor) -> torch.Tensor:
    """bf16 matrix for the kernels: the tensor itself when it is bf16, else a cast -- per call, or kept
    under cache_bf16_lm_head()."""
    if w.dtype == torch.bfloat16:
        return w.detach()
    if _bf16_cache.depth == 0:
        return w.detach().to(torch.bfloat16)
    ident = id(w)                        # the caller's tensor object (detach() makes a new one per call)
    key = (w._version, w.data_ptr(), tuple(w.shape), tuple(w.stride()))
    hit = _bf16_copies.get(ident)
    if hit is not None and hit[0]() is w and hit[1] == key:
        return hit[2]
    copy = w.detach().to(torch.bfloat16)
    try:
        _bf16_copies[ident] = (weakref.ref(w, lambda _r, i=ident: _bf16_copies.pop(i, None)), key, copy)
    except TypeError:                    # objects that cannot be weakly referenced: no cache
        pass
    return copy


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _as_f32(x, n: int, device, name: str) -> torch.Tensor:
    t = torch.as_tensor(x, device=device)
    if t.numel() != n:
        raise ValueError(f"{name} has {t.numel()} elements, expected {n}")
    return t.reshape(n).to(torch.float32).contiguous()


class _Prepared:
    """Validated, flattened device arguments of one call."""

    def __init__(self, hidden, lm_head, target_ids, old_logps, advantages, mask, *,
                 total_valid_token_count, epsilon_low, epsilon_high, temperature,
                 final_logit_softcap, seq_shape, chunk_tokens, sft=False, accumulate=False,
                 entropy_coef=0.0, entropy_token_count=None, skip_masked=False, dhidden_splits=0, loss_scale=1.0):
        if hidden.device.type != "cuda":
            raise RuntimeError("grpo_fused_loss needs tensors on an MI355X device (got "
                               f"{hidden.device}); there is no CPU path")
        if hidden.dim() == 3:
            if seq_shape is None:
                seq_shape = (hidden.shape[0], hidden.shape[1])
            hidden = hidden.reshape(-1, hidden.shape[-1])
        if hidden.dim() != 2 or lm_head.dim() != 2 or hidden.shape[1] != lm_head.shape[0]:
            raise ValueError(f"hidden {tuple(hidden.shape)} and lm_head {tuple(lm_head.shape)} do not "
                             "form [N,H] x [H,V]")
        n, h = hidden.shape
        v = lm_head.shape[1]
        if seq_shape is not None and seq_shape[0] * seq_shape[1] != n:
            raise ValueError(f"seq_shape {seq_shape} does not match {n} tokens")
        dev = hidden.device
        self.n, self.h, self.v, self.seq_shape, self.device = n, h, v, seq_shape, dev
        self.hidden = self._operand(hidden.to(torch.bfloat16))
        self.w = self._operand(_bf16_weights(lm_head))
        self.targets = torch.as_tensor(target_ids, device=dev).reshape(-1).to(torch.int32).contiguous()
        if self.targets.numel() != n:
            raise ValueError(f"target_ids has {self.targets.numel()} elements, expected {n}")
        self.mask = _as_f32(mask, n, dev, "mask")
        self.old = None if old_logps is None else _as_f32(old_logps, n, dev, "old_logps")
        if sft:
            self.adv = None
        else:
            adv = torch.as_tensor(advantages, device=dev).to(torch.float32)
            if adv.numel() != n:
                # the reference passes [B] and broadcasts over the sequence (train_modules/__init__.py:173)
                if seq_shape is None or adv.numel() != seq_shape[0]:
                    raise ValueError(f"advantages has {adv.numel()} elements; expected {n} tokens or "
                                     "one per sequence with seq_shape given")
                adv = adv.reshape(-1, 1).expand(seq_shape[0], seq_shape[1])
            self.adv = adv.reshape(n).contiguous()
        if total_valid_token_count is None:
            tv = float(self.mask.sum().item())       # reference default: mask.sum() (:179)
            if sft:
                tv = max(tv, 1.0)                    # sft_module.py:14
        else:
            tv = float(total_valid_token_count)
        self.tv = tv
        d = _lib.MjGrpoDesc()
        d.n_tokens, d.hidden, d.vocab = n, h, v
        d.ld_hidden, d.ld_w = self.hidden.stride(0), self.w.stride(0)
        d.chunk_tokens = int(chunk_tokens or 0)
        d.eps_low, d.eps_high = float(epsilon_low), float(epsilon_high)
        d.temperature = float(temperature)
        d.softcap = float(final_logit_softcap or 0.0)
        d.inv_total_valid_tokens = (1.0 / tv) if tv != 0 else float("inf")
        self.loss_scale = float(loss_scale)
        d.grad_loss_scale = self.loss_scale      # the kernels write gradients of loss_scale * loss
        d.dhidden_splits = int(dhidden_splits or 0)
        d.entropy_coef = float(entropy_coef)
        if entropy_coef != 0.0 or entropy_token_count is not None:
            cnt = float(self.mask.sum().item()) if entropy_token_count is None else float(entropy_token_count)
            d.inv_entropy_count = 1.0 / (cnt + 1e-8)             # ppo/module.py:77
        d.flags = (_lib.FLAG_SFT if sft else 0) | (_lib.FLAG_DW_ACCUMULATE if accumulate else 0) \
            | (_lib.FLAG_SKIP_MASKED if skip_masked else 0)
        self.desc = d
        self.logp = torch.empty(n, dtype=torch.float32, device=dev)
        self.lse = torch.empty(n, dtype=torch.float32, device=dev)
        self.ent = torch.empty(n, dtype=torch.float32, device=dev)
        self.loss = torch.empty(2, dtype=torch.float32, device=dev)   # [loss, masked-mean entropy]

    @staticmethod
    def _operand(t: torch.Tensor) -> torch.Tensor:
        """A row-major bf16 matrix the kernels can read in place: unit column stride, row pitch a
        multiple of 8 elements and at least the row length, 16-byte aligned base; anything else is
        copied into a dense tensor."""
        ok = t.stride(1) == 1 and t.stride(0) % 8 == 0 and t.stride(0) >= t.shape[1] and t.data_ptr() % 16 == 0
        return t if ok else t.contiguous()

    def stream(self) -> int:
        return torch.cuda.current_stream(self.device).cuda_stream

    def forward(self) -> None:
        fwd, _ = _lib.workspace_bytes(self.desc)
        ws = _workspace(self.device, fwd)
        with torch.cuda.device(self.device):
            _lib.check(_lib.load().mj_grpo_forward(
                C.byref(self.desc), _ptr(self.hidden), _ptr(self.w), _ptr(self.targets), _ptr(self.old),
                _ptr(self.adv), _ptr(self.mask), _ptr(self.logp), _ptr(self.lse), _ptr(self.ent),
                _ptr(self.loss), _ptr(ws), ws.numel(), self.stream()))

    def forward_backward(self, d_w: Optional[torch.Tensor] = None, value: Optional["_ValueHead"] = None,
                         dw_dtype: torch.dtype = torch.float32):
        """One fused pass.  The lm_head gradient goes into `d_w` (float32 or bf16, laid out like
        lm_head; added to when the descriptor says accumulate) or into a new tensor of `dw_dtype`."""
        _, both = _lib.workspace_bytes(self.desc)
        if value is not None:
            both += _lib.value_workspace_bytes(self.desc)
        ws = _workspace(self.device, both)
        # d_hidden is written with the row pitch of hidden (the descriptor has one ld_hidden for both)
        ld = self.hidden.stride(0)
        d_h = torch.empty((self.n, ld), dtype=torch.bfloat16, device=self.device)[:, : self.h]
        if d_w is None:
            d_w = torch.empty((self.h, self.w.stride(0)), dtype=dw_dtype, device=self.device)
        if d_w.dtype not in (torch.float32, torch.bfloat16):
            raise ValueError(f"the lm_head gradient is float32 or bfloat16 (got {d_w.dtype})")
        if d_w.dtype == torch.bfloat16:
            self.desc.flags |= _lib.FLAG_DW_BF16
        else:
            self.desc.flags &= ~_lib.FLAG_DW_BF16
        with torch.cuda.device(self.device):
            if value is None:
                _lib.check(_lib.load().mj_grpo_forward_backward(
                    C.byref(self.desc), _ptr(self.hidden), _ptr(self.w), _ptr(self.targets), _ptr(self.old),
                    _ptr(self.adv), _ptr(self.mask), _ptr(self.logp), _ptr(self.lse), _ptr(self.ent),
                    _ptr(self.loss), _ptr(d_h), _ptr(d_w), _ptr(ws), ws.numel(), self.stream()))
            else:
                _lib.check(_lib.load().mj_grpo_forward_backward_value(
                    C.byref(self.desc), C.byref(value.struct(self.n, self.h, self.device)), _ptr(self.hidden),
                    _ptr(self.w), _ptr(self.targets), _ptr(self.old), _ptr(self.adv), _ptr(self.mask),
                    _ptr(self.logp), _ptr(self.lse), _ptr(self.ent), _ptr(self.loss), _ptr(d_h), _ptr(d_w),
                    _ptr(ws), ws.numel(), self.stream()))
        return d_h, d_w[:, : self.v]

    def metrics(self, return_token_entropy: bool, sft: bool = False) -> dict:
        """The reference's return dict (train_modules/__init__.py:185-192)."""
        out = {"loss": self.loss[0]}
        shape = self.seq_shape if self.seq_shape is not None else (self.n,)
        out["per_token_logps"] = self.logp.reshape(shape)
        if sft:
            out["token_count"] = self.mask.sum().to(torch.int32)
            return out
        if self.seq_shape is not None:
            # per-sample masked mean entropy (:141-143) and its tokens-4..100 window (:148-157): one kernel
            b, t = self.seq_shape
            stats = torch.empty((2, b), dtype=torch.float32, device=self.device)
            with torch.cuda.device(self.device):
                _lib.check(_lib.load().mj_grpo_sequence_entropy(
                    _ptr(self.ent), _ptr(self.mask), b, t, stats[0].data_ptr(), stats[1].data_ptr(), self.stream()))
            out["entropy"], out["entropy_loss"] = stats[0], stats[1]
        if return_token_entropy:
            out["token_entropy"] = self.ent.reshape(shape)
        if self.desc.inv_entropy_count != 0.0:
            out["masked_mean_entropy"] = self.loss[1]
        return out


class _ValueHead:
    """Device arguments and outputs of the critic's value head for one fused call
    (include/mj_grpo.h: MjPpoValue; plugins/training/ppo/module.py:34-39, :104-138)."""

    def __init__(self, weight, bias, returns, old_values, value_coef, value_clip_range):
        self.w = weight.detach().reshape(-1).to(torch.float32).contiguous()
        self.b = bias.detach().reshape(-1)[:1].to(torch.float32).contiguous()
        self.returns, self.old_values = returns, old_values
        self.coef, self.clip = float(value_coef), value_clip_range
        self.values = self.value_loss = self.d_w = self.d_b = None

    def struct(self, n: int, h: int, device) -> "_lib.MjPpoValue":
        if self.w.numel() != h:
            raise ValueError(f"value head weight has {self.w.numel()} elements, expected hidden size {h}")
        f32 = lambda x, name: None if x is None else _as_f32(x, n, device, name)
        self.returns, self.old_values = f32(self.returns, "returns"), f32(self.old_values, "old_values")
        self.values = torch.empty(n, dtype=torch.float32, device=device)
        self.value_loss = torch.empty(1, dtype=torch.float32, device=device)
        self.d_w = torch.empty(h, dtype=torch.float32, device=device)
        self.d_b = torch.empty(1, dtype=torch.float32, device=device)
        v = _lib.MjPpoValue()
        v.value_w, v.value_b = self.w.data_ptr(), self.b.data_ptr()
        v.returns, v.old_values = _ptr(self.returns), _ptr(self.old_values)
        v.value_coef = self.coef
        v.use_clip = 0 if self.clip is None else 1
        v.value_clip = 0.0 if self.clip is None else float(self.clip)
        v.values, v.value_loss = self.values.data_ptr(), self.value_loss.data_ptr()
        v.d_value_w, v.d_value_b = self.d_w.data_ptr(), self.d_b.data_ptr()
        return v


_DEFAULTS = dict(total_valid_token_count=None, epsilon_low=0.2, epsilon_high=0.3, temperature=1.0,
                 final_logit_softcap=None, seq_shape=None, chunk_tokens=None, entropy_coef=0.0,
                 entropy_token_count=None, skip_masked=False, dhidden_splits=0, loss_scale=1.0)


def grpo_loss_value_and_grad(hidden, lm_head, target_ids, old_logps, advantages, mask, *,
                             return_token_entropy=False, accumulate_into=None,
                             lm_head_grad_dtype=torch.float32, **kw):
    """value_and_grad form of the loss, the call shape of the reference's train step
    (plugins/training/update/train_step.py:24): returns (metrics, (d_hidden, d_lm_head)).

    d_hidden is bf16 [N,H]; d_lm_head is float32 [H,V] (the reference's parameter gradients
    are float32) unless `lm_head_grad_dtype=torch.bfloat16` asks the dW kernel for a bf16 matrix.
    `accumulate_into` (a float32 or bf16 [H,V] tensor) makes the kernel add into an existing
    gradient buffer instead of overwriting (grad accumulation, train_step.py:30-33).
    One fused pass: 6*N*H*V flop, 16-bit logits of at most `chunk_tokens` tokens in the workspace.
    `entropy_coef` != 0 subtracts entropy_coef * sum(H_t*mask)/(sum(mask)+1e-8) from the loss
    (the entropy bonus of plugins/training/ppo/module.py:75-77, :140), gradient included; that
    entropy is returned as metrics["masked_mean_entropy"].
    `skip_masked=True` leaves tokens that cannot carry a gradient (mask 0; advantage 0) out of the
    backward products: same results, less work when the batch holds prompt / padding positions."""
    opts = {**_DEFAULTS, **kw}
    p = _Prepared(hidden, lm_head, target_ids, old_logps, advantages, mask,
                  accumulate=accumulate_into is not None, **opts)
    if accumulate_into is not None:
        _check_accumulator(accumulate_into, p)
    d_h, d_w = p.forward_backward(accumulate_into, dw_dtype=lm_head_grad_dtype)
    return p.metrics(return_token_entropy), (d_h.reshape(hidden.shape), d_w)


def _check_accumulator(buf: torch.Tensor, p: "_Prepared") -> None:
    if buf.dtype not in (torch.float32, torch.bfloat16) or tuple(buf.shape) != (p.h, p.v) \
            or buf.stride(1) != 1 or buf.stride(0) != p.w.stride(0) or buf.device != p.device:
        raise ValueError("the lm_head gradient accumulator must be a float32 or bfloat16 [H,V] device tensor "
                         "laid out like lm_head")


class _CallMode(threading.local):
    buffer: Optional[torch.Tensor] = None   # lm_head gradient accumulator of accumulate_lm_head_grad_into
    uses: int = 0
    terminal: bool = False                  # inside terminal_loss()


_accumulate_target = _CallMode()


@contextlib.contextmanager
def accumulate_lm_head_grad_into(buffer: torch.Tensor):
    """Within this context every differentiable fused-loss call ADDS its lm_head gradient into
    `buffer` (float32 or bf16 [H,V]) inside the dW kernel and hands autograd no lm_head gradient: the
    grad-accumulation `ga + g` of plugins/training/update/train_step.py:30-33 without a
    separate [H,V] gradient tensor or a pass over it.  The loss must be terminal (it is
    differentiated with upstream gradient 1, as training_step does; any other upstream gradient
    turns buffer[0, 0] into NaN, see terminal_loss); yields a counter object whose `.uses` says
    how many calls accumulated."""
    prev, prev_uses = _accumulate_target.buffer, _accumulate_target.uses
    _accumulate_target.buffer, _accumulate_target.uses = buffer, 0
    try:
        yield _accumulate_target
    finally:
        _accumulate_target.buffer, _accumulate_target.uses = prev, prev_uses


@contextlib.contextmanager
def terminal_loss():
    """Within this context the caller promises that every fused loss is differentiated with
    upstream gradient exactly 1 -- what jax.value_and_grad of the reference's loss_fn does
    (plugins/training/update/train_step.py:15-24).  The backward then hands autograd the [H,V]
    gradient the kernel wrote as it is: no `d_w * grad` pass over 2 GB and no second copy.  The
    promise is checked on the device without a host synchronisation: an upstream gradient other
    than 1 adds NaN to element [0, 0] of the lm_head gradient, so a broken promise cannot go
    unnoticed downstream."""
    prev = _accumulate_target.terminal
    _accumulate_target.terminal = True
    try:
        yield
    finally:
        _accumulate_target.terminal = prev


def _poison_unless_one(grad_loss: torch.Tensor) -> torch.Tensor:
    g = grad_loss.reshape(-1)[:1].to(torch.float32)
    return torch.where(g == 1, torch.zeros_like(g), torch.full_like(g, float("nan")))


def _apply_upstream(grad_loss: torch.Tensor, d_h: torch.Tensor, d_w: Optional[torch.Tensor]) -> None:
    """Multiplies the gradients the kernels wrote by the upstream gradient, in place and on the
    device: when it is 1 -- the loss itself is what gets differentiated -- the launches leave at once
    (no pass over [N,H] or [H,V], no host synchronisation)."""
    g = grad_loss.detach().reshape(-1)[:1].to(torch.float32).contiguous()
    with torch.cuda.device(d_h.device):
        _lib.check(_lib.load().mj_grpo_scale_gradients(
            d_h.data_ptr(), d_h.shape[0], d_h.shape[1], d_h.stride(0),
            None if d_w is None else d_w.data_ptr(), 0 if d_w is None else d_w.shape[0],
            0 if d_w is None else d_w.shape[1], 0 if d_w is None else d_w.stride(0),
            int(d_w is not None and d_w.dtype == torch.bfloat16), g.data_ptr(),
            torch.cuda.current_stream(d_h.device).cuda_stream))


class _FusedLossFn(torch.autograd.Function):
    """loss = loss_scale * (policy loss - entropy_coef * entropy [+ value_coef * value_loss]) with the
    gradients the kernels wrote in the same pass.  value_w / value_b / value are None without a value
    head.  The gradients are handed out once: a second backward through the same call raises."""

    @staticmethod
    def forward(ctx, hidden, lm_head, prepared: _Prepared, want_grad: bool, value_w=None, value_b=None,
                value: Optional[_ValueHead] = None):
        ctx.direct = ctx.terminal = False
        ctx.d_h = ctx.d_w = ctx.buf = ctx.value = None
        if want_grad:
            # a bf16 parameter takes a bf16 gradient: the dW kernel writes it, no conversion pass
            dw_dtype = torch.bfloat16 if lm_head.dtype == torch.bfloat16 else torch.float32
            buf = _accumulate_target.buffer if lm_head.requires_grad else None
            if buf is not None:
                _check_accumulator(buf, prepared)
                prepared.desc.flags |= _lib.FLAG_DW_ACCUMULATE
                ctx.d_h, _ = prepared.forward_backward(buf, value)
                _accumulate_target.uses += 1
                ctx.direct, ctx.buf = True, buf
            else:
                ctx.d_h, ctx.d_w = prepared.forward_backward(None, value, dw_dtype)
                ctx.terminal = _accumulate_target.terminal
            ctx.shapes = (hidden.shape, hidden.dtype, lm_head.dtype)
            if value is not None:
                ctx.value = (value.d_w, value.d_b, value_w.shape, value_w.dtype, value_b.shape, value_b.dtype)
        else:
            prepared.forward()
        loss = prepared.loss[0].clone()
        if value is not None and value.value_loss is not None:
            loss = loss + value.coef * value.value_loss[0]
        if prepared.loss_scale != 1.0:
            loss = loss * prepared.loss_scale
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        if ctx.d_h is None:
            raise RuntimeError("the fused loss hands out the gradients of a call once (they are scaled in place); "
                               "evaluate the loss again instead of a second backward through the same call")
        shape, h_dtype, w_dtype = ctx.shapes
        d_h, ctx.d_h = ctx.d_h, None
        d_w, ctx.d_w = ctx.d_w, None
        if ctx.direct:
            gw = None                      # already added into the accumulator by the dW kernel ...
            ctx.buf[0, :1].add_(_poison_unless_one(grad_loss))   # ... with upstream gradient 1
            _apply_upstream(grad_loss, d_h, None)
        elif ctx.terminal:
            d_w[0, :1].add_(_poison_unless_one(grad_loss))
            _apply_upstream(grad_loss, d_h, None)
            gw = d_w
        else:
            _apply_upstream(grad_loss, d_h, d_w)
            gw = d_w
        if gw is not None and gw.dtype != w_dtype:
            gw = gw.to(w_dtype)
        gh = d_h.reshape(shape).to(h_dtype)
        gwv = gbv = None
        if ctx.value is not None:
            d_wv, d_bv, wv_shape, wv_dtype, bv_shape, bv_dtype = ctx.value
            gwv = (d_wv * grad_loss).reshape(wv_shape).to(wv_dtype)
            gbv = (d_bv * grad_loss).reshape(bv_shape).to(bv_dtype)
        return gh, gw, None, None, gwv, gbv, None


def grpo_fused_loss(hidden, lm_head, target_ids, old_logps, advantages, mask, *,
                    return_token_entropy=False, **kw) -> dict:
    """The reference's loss contract on flattened tokens.

    hidden [N,H] or [B,T,H] bf16, lm_head [H,V] bf16 (or float32 master weights),
    target_ids [N] int, old_logps [N] float32 or None (None = on-policy, ratio 1,
    train_modules/__init__.py:161-165), advantages [N] (or [B] with seq_shape=(B,T)),
    mask [N] in {0,1}.  Returns {"loss", "per_token_logps", "entropy", "entropy_loss"
    [, "token_entropy"]} like train_modules/__init__.py:185-192; "loss" is differentiable
    with respect to hidden and lm_head, everything else carries no gradient.
    `loss_scale=c` returns c * loss with the kernels writing the gradients of c * loss directly
    (a constant known before the call, e.g. 1 / gradient-accumulation steps: multiplying the
    returned loss afterwards gives the same result through an in-place pass over both gradients)."""
    opts = {**_DEFAULTS, **kw}
    p = _Prepared(hidden, lm_head, target_ids, old_logps, advantages, mask, **opts)
    want = torch.is_grad_enabled() and (hidden.requires_grad or lm_head.requires_grad)
    loss = _FusedLossFn.apply(hidden, lm_head, p, want, None, None, None)
    out = p.metrics(return_token_entropy)
    out["loss"] = loss
    return out


def sft_fused_loss(hidden, lm_head, labels, valid, **kw) -> dict:
    """Masked next-token cross-entropy of plugins/sft/jax/sft_module.py:22-45 on already
    shifted, flattened tokens: loss = sum(-logp * valid) / max(sum(valid), 1).  Positions with
    valid == 0 may hold any label (the reference maps them to 0, :35)."""
    opts = {**_DEFAULTS, **kw}
    labels = torch.as_tensor(labels, device=hidden.device)
    validb = torch.as_tensor(valid, device=hidden.device).reshape(-1).bool()
    safe = torch.where(validb, labels.reshape(-1), torch.zeros_like(labels.reshape(-1)))
    p = _Prepared(hidden, lm_head, safe, None, None, validb.to(torch.float32), sft=True, **opts)
    want = torch.is_grad_enabled() and (hidden.requires_grad or lm_head.requires_grad)
    loss = _FusedLossFn.apply(hidden, lm_head, p, want, None, None, None)
    out = p.metrics(False, sft=True)
    out["loss"] = loss
    return out


class TrainGRPOModule:
    """Drop-in for the reference's TrainGRPOModule (MLLM_JAX/train_modules/__init__.py:84-192)
    with the lm_head product fused into the loss.

    `model(input_ids=..., attention_mask=...)` returns the FINAL HIDDEN STATES [B,L,H] (what
    Qwen2Model returns before lm_head, qwen2/modular_qwen2.py:161) and `lm_head` is the
    [H,V] kernel (or a zero-argument callable returning it).  `__call__(inputs)` takes the
    reference's batch dict (input_ids, attention_mask, labels, advantages and optionally
    old_per_token_logps, total_valid_token_count) and returns its metrics dict.

    `ref_model` and `beta` are accepted and, as in the reference, have no effect on the loss: the
    reference evaluates the reference model's log-probs (:129-132) but no KL term enters `loss`
    (:176-180).  `pad_token_id`, `num_pre_Q`, `max_lengths`, `entropy_threshold` are unused there too."""

    def __init__(self, model: Callable, lm_head, pad_token_id: float = 0, num_pre_Q: int = 1,
                 ref_model: Any = None, beta: float = 0.04, temperature: float = 1.0,
                 max_lengths: float = 2048, epsilon_low: float = 0.2, epsilon_high: float = 0.3,
                 entropy_threshold: float = 0.3, final_logit_softcap: Optional[float] = None,
                 chunk_tokens: Optional[int] = None, skip_masked: bool = False, dhidden_splits: int = 0):
        self.dhidden_splits = dhidden_splits
        self.model, self.lm_head = model, lm_head
        self.pad_token_id, self.num_pre_Q, self.ref_model, self.beta = pad_token_id, num_pre_Q, ref_model, beta
        self.temperature, self.max_lengths = temperature, max_lengths
        self.epsilon_low, self.epsilon_high = epsilon_low, epsilon_high
        self.entropy_threshold = entropy_threshold
        self.final_logit_softcap, self.chunk_tokens = final_logit_softcap, chunk_tokens
        self.skip_masked = skip_masked

    def __call__(self, inputs: Mapping[str, Any]) -> dict:
        input_ids, labels = inputs["input_ids"], inputs["labels"]
        hidden = self.model(input_ids=input_ids, attention_mask=inputs["attention_mask"])
        w = self.lm_head() if callable(self.lm_head) else self.lm_head
        b, l = input_ids.shape
        hid = hidden[:, :-1, :]                       # logits[..., :-1, :]   (:124)
        chosen = input_ids[:, 1:]                     # :118
        mask = labels[:, 1:]                          # :120
        return grpo_fused_loss(
            hid.reshape(b * (l - 1), -1), w, chosen.reshape(-1), inputs.get("old_per_token_logps"),
            inputs["advantages"], mask.reshape(-1),
            total_valid_token_count=inputs.get("total_valid_token_count"),
            epsilon_low=self.epsilon_low, epsilon_high=self.epsilon_high, temperature=self.temperature,
            final_logit_softcap=self.final_logit_softcap, seq_shape=(b, l - 1),
            chunk_tokens=self.chunk_tokens, skip_masked=self.skip_masked, dhidden_splits=self.dhidden_splits)


class PPOActorCriticModule:
    """Drop-in for the reference's PPOActorCriticModule.__call__ (plugins/training/ppo/module.py:59-150)
    with the lm_head product, the policy term and the entropy bonus (value and gradient) fused
    into the HIP kernels.

    `model(input_ids=..., attention_mask=...)` returns the final hidden states [B,L,H];
    `lm_head` is the [H,V] kernel; `value_head` is (weight [H] or [H,1], bias scalar tensor),
    the Dense(1, use_bias=True) of module.py:34-39 (each may be a zero-argument callable).
    The value head is a [B*L,H] x [H] product and a handful of element-wise operations on
    [B,L] tensors; those run as torch device ops."""

    def __init__(self, model: Callable, lm_head, value_head, temperature: float = 1.0,
                 epsilon_low: float = 0.2, epsilon_high: float = 0.2, value_coef: float = 0.5,
                 value_clip_range: Optional[float] = 0.2, entropy_coef: float = 0.0,
                 final_logit_softcap: Optional[float] = None, chunk_tokens: Optional[int] = None,
                 skip_masked: bool = False, dhidden_splits: int = 0):
        self.skip_masked, self.dhidden_splits = skip_masked, dhidden_splits
        self.model, self.lm_head, self.value_head = model, lm_head, value_head
        self.temperature, self.epsilon_low, self.epsilon_high = temperature, epsilon_low, epsilon_high
        self.value_coef, self.value_clip_range, self.entropy_coef = value_coef, value_clip_range, entropy_coef
        self.final_logit_softcap, self.chunk_tokens = final_logit_softcap, chunk_tokens

    def _head(self):
        return self.value_head() if callable(self.value_head) else self.value_head

    def _values(self, hidden: torch.Tensor) -> torch.Tensor:
        """Dense(1), squeezed (module.py:52): one wavefront per token row, float32 accumulation and
        result (the reference rounds the result to the activation dtype before casting it back to
        float32 at :127)."""
        wv, bv = self._head()
        if hidden.device.type != "cuda":
            raise RuntimeError("the value head needs tensors on an MI355X device; there is no CPU path")
        shape = hidden.shape[:-1]
        h2 = _Prepared._operand(hidden.detach().reshape(-1, hidden.shape[-1]).to(torch.bfloat16))
        w = wv.detach().reshape(-1).to(torch.float32).contiguous()
        b = bv.detach().reshape(-1)[:1].to(torch.float32).contiguous()
        out = torch.empty(h2.shape[0], dtype=torch.float32, device=hidden.device)
        with torch.cuda.device(hidden.device):
            _lib.check(_lib.load().mj_value_head_forward(
                h2.data_ptr(), h2.stride(0), w.data_ptr(), b.data_ptr(), out.data_ptr(), h2.shape[0], h2.shape[1],
                torch.cuda.current_stream(hidden.device).cuda_stream))
        return out.reshape(shape)

    def value(self, input_ids, attention_mask) -> torch.Tensor:
        """module.py:55-57 (no gradient: use __call__ for training)."""
        return self._values(self.model(input_ids=input_ids, attention_mask=attention_mask))

    @staticmethod
    def _like(x, ref: torch.Tensor, name: str) -> torch.Tensor:
        # the [B] / [B,1] / [B,T] broadcasting of module.py:88-94, :108-114, :119-125
        x = torch.as_tensor(x, device=ref.device)
        if x.dim() == 1:
            x = x[:, None]
        if x.shape != ref.shape:
            if x.shape[1] == 1:
                x = x.expand(ref.shape)
            else:
                raise ValueError(f"{name} shape {tuple(x.shape)} does not match {tuple(ref.shape)}")
        return x

    def __call__(self, inputs: Mapping[str, Any]) -> dict:
        input_ids, labels = inputs["input_ids"], inputs["labels"]
        hidden = self.model(input_ids=input_ids, attention_mask=inputs["attention_mask"])
        w = self.lm_head() if callable(self.lm_head) else self.lm_head
        wv, bv = self._head()
        b, l = input_ids.shape
        t = l - 1
        mask = labels[:, 1:].to(torch.float32)                                   # :67
        advantages = self._like(inputs["advantages"], mask, "advantages")        # :87-94
        msum = mask.sum()
        tv = inputs.get("total_valid_token_count")
        hid = hidden[:, :-1, :].reshape(b * t, -1)
        p = _Prepared(hid, w, input_ids[:, 1:].reshape(-1),
                      inputs.get("old_per_token_logps"), advantages.reshape(-1), mask.reshape(-1),
                      total_valid_token_count=float(tv) if tv is not None else float(msum.item()),
                      epsilon_low=self.epsilon_low, epsilon_high=self.epsilon_high,
                      temperature=self.temperature, final_logit_softcap=self.final_logit_softcap,
                      seq_shape=(b, t), chunk_tokens=self.chunk_tokens, skip_masked=self.skip_masked,
                      dhidden_splits=self.dhidden_splits, entropy_coef=self.entropy_coef,
                      entropy_token_count=float(msum.item()) if self.entropy_coef != 0.0 or tv is None else None)
        returns = inputs.get("returns")                                          # :105-114
        if returns is not None:
            returns = self._like(returns, mask, "returns").to(torch.float32)
        old_values = inputs.get("old_values", inputs.get("values"))              # :116-125
        if old_values is not None:
            old_values = self._like(old_values, mask, "old_values").to(torch.float32)
        want = torch.is_grad_enabled() and (hidden.requires_grad or w.requires_grad or wv.requires_grad
                                            or bv.requires_grad)
        if want:
            # value head, clipped value loss and their gradients inside the fused pass
            head = _ValueHead(wv, bv, None if returns is None else returns.reshape(-1),
                              None if old_values is None else old_values.reshape(-1), self.value_coef,
                              self.value_clip_range)
            loss = _FusedLossFn.apply(hid, w, p, True, wv, bv, head)             # :140
            value_pred = head.values.reshape(b, t)
            value_loss = head.value_loss[0]
        else:
            fused = _FusedLossFn.apply(hid, w, p, False, None, None, None)
            value_pred = self._values(hidden)[:, :-1]                            # :104
            rt = advantages + value_pred if returns is None else returns
            ov = value_pred if old_values is None else old_values
            if self.value_clip_range is not None:
                c = float(self.value_clip_range)
                clipped = ov + torch.clamp(value_pred - ov, -c, c)
                vl = torch.maximum((value_pred - rt) ** 2, (clipped - rt) ** 2)  # :133-134
            else:
                vl = (value_pred - rt) ** 2
            value_loss = (vl * mask).sum() / p.tv                                # :138
            loss = fused + float(self.value_coef) * value_loss
        entropy = p.loss[1] if p.desc.inv_entropy_count != 0.0 else (p.ent.reshape(b, t) * mask).sum() / (msum + 1e-8)  # :77
        policy_loss = (p.loss[0] + self.entropy_coef * entropy).detach()
        rt_mean = (advantages + value_pred).mean() if returns is None else returns.mean()
        return {"loss": loss, "policy_loss": policy_loss, "value_loss": value_loss.detach(), "entropy": entropy,
                "value_pred_mean": value_pred.mean(), "return_mean": rt_mean,
                "per_token_logps": p.logp.reshape(b, t)}


def compute_grpo_advantages_by_group_id(*, rewards, group_ids, eps: float = 1e-4) -> torch.Tensor:
    """Device counterpart of plugins/training/advantage/grpo.py:8-52: float32 advantages [B],
    (r - mean_g) / (std_g + eps) within each group id (population std, variable group sizes).
    `rewards` must be a GPU tensor; `group_ids` is moved beside it."""
    rewards = torch.as_tensor(rewards)
    if rewards.device.type != "cuda":
        raise RuntimeError("compute_grpo_advantages_by_group_id needs GPU tensors; there is no CPU path")
    if rewards.dim() != 1:
        raise ValueError(f"rewards must be rank-1 [B], got shape={tuple(rewards.shape)}")
    group_ids = torch.as_tensor(group_ids, device=rewards.device)
    if group_ids.shape != rewards.shape:
        raise ValueError(f"group_ids must have same shape as rewards, got {tuple(group_ids.shape)} vs "
                         f"{tuple(rewards.shape)}")
    if rewards.numel() == 0:
        raise ValueError("No groups found (empty batch?)")
    r = rewards.to(torch.float32).contiguous()
    g = group_ids.to(torch.int32).contiguous()
    out = torch.empty_like(r)
    with torch.cuda.device(r.device):
        _lib.check(_lib.load().mj_grpo_group_advantages(r.data_ptr(), g.data_ptr(), out.data_ptr(), r.numel(),
                                                        float(eps), torch.cuda.current_stream(r.device).cuda_stream))
    return out


def loss_and_metrics(module: Callable[[Mapping[str, Any]], dict], inputs: Mapping[str, Any]):
    """loss_fn of plugins/training/update/train_step.py:15-22: pops per_token_logps, means
    the other metrics, returns (loss, metrics | {"per_token_logps": ...})."""
    metrics = dict(module(inputs))
    per_token_logps = metrics.pop("per_token_logps", None)
    metrics = {k: torch.mean(v.float()) for k, v in metrics.items()}
    return metrics["loss"], {**metrics, "per_token_logps": per_token_logps}
