"""Host side of the update loop around the fused loss: the reference's micro-batch /
PPO-epoch contract on torch device tensors.

Mirrors
  plugins/training/update/ppo.py:6-46          ppo_update (epochs x micro-batches, global
                                               total_valid_token_count, epoch-0 per_token_logps
                                               cached as old_per_token_logps)
  plugins/training/update/train_step.py:6-44   training_step (value_and_grad with aux, gradient
                                               accumulation, update when micro_step == micro_in_mini)
  plugins/training/ppo/train_step.py:8-45      ppo_training_step (same step for the actor-critic module)
  plugins/training/runner/grpo_gsm8k.py:185-190  slice_data (leading-axis micro-batch slice)
  plugins/training/update/modules.py:10-60     PPOUpdateModule / PolicyGradientUpdateModule

The reference's state is a functional flax TrainState; here it is a small mutable-free
dataclass whose `replace` returns a new object, so callers written against the reference
(`state, meta = train_step(state, batch)`) read the same.  What is MI355X-specific: when the
state names its lm_head parameter (`lm_head_key`) and accumulates gradients, the dW kernel adds
straight into the accumulator (no per-micro-batch [H,V] gradient tensor, no `ga + g` pass).
"""
from __future__ import annotations

import dataclasses
from typing import Any, Callable, Dict, Mapping, Optional

import torch

from .loss import accumulate_lm_head_grad_into, cache_bf16_lm_head, terminal_loss

Params = Dict[str, torch.Tensor]


@dataclasses.dataclass(frozen=True)
class UpdateResult:
    """plugins/training/api (UpdateResult): what an update module hands back to the runner."""
    state: Any
    batch: Mapping[str, Any]
    last_meta: Mapping[str, Any]
    entropy: Any


@dataclasses.dataclass(frozen=True)
class LossTrainState:
    """The fields of the reference's TrainState that training_step touches.

    apply_fn(params, inputs) -> metrics dict whose "loss" is differentiable with respect to the
    tensors in `params` (e.g. a TrainGRPOModule / PPOActorCriticModule built over them).
    tx(params, grads) -> new params: the optimizer update (optax in the reference; any callable
    here).  grad_accum None = apply every step (train_step.py:26-28); otherwise a dict of
    float32 accumulators, one per parameter, and micro_in_mini micro-steps per update."""
    apply_fn: Callable[[Params, Mapping[str, Any]], Dict[str, Any]]
    params: Params
    tx: Callable[[Params, Params], Params]
    step: int = 0
    grad_accum: Optional[Params] = None
    micro_step: int = 0
    micro_in_mini: int = 1
    lm_head_key: Optional[str] = None      # parameter whose gradient the dW kernel accumulates in place

    def replace(self, **kw) -> "LossTrainState":
        return dataclasses.replace(self, **kw)

    def apply_gradients(self, *, grads: Params, **kw) -> "LossTrainState":
        with torch.no_grad():
            new = self.tx(self.params, grads)
        new = {k: v.detach().requires_grad_(self.params[k].requires_grad) for k, v in new.items()}
        return self.replace(params=new, step=self.step + 1, **kw)

    @staticmethod
    def create(*, apply_fn, params: Params, tx, grad_accum_steps: int = 1,
               lm_head_key: Optional[str] = None) -> "LossTrainState":
        """training2.py:94-118: accumulators exist only when grad_accum_steps > 1."""
        ga = None
        if grad_accum_steps > 1:
            ga = {k: torch.zeros(v.shape, dtype=torch.float32, device=v.device) for k, v in params.items()}
        return LossTrainState(apply_fn=apply_fn, params=params, tx=tx, grad_accum=ga,
                              micro_in_mini=int(grad_accum_steps), lm_head_key=lm_head_key)


def slice_data(x, accumulate_steps: int, i: int):
    """runner/grpo_gsm8k.py:185-188: micro-batch i of accumulate_steps along the leading axis
    (a view; remainder rows beyond accumulate_steps * (B // accumulate_steps) are dropped)."""
    micro = int(x.shape[0]) // int(accumulate_steps)
    start = int(i) * micro
    return x[start:start + micro]


def _loss_and_aux(state: LossTrainState, inputs: Mapping[str, Any]):
    # loss_fn of train_step.py:15-22
    metrics = dict(state.apply_fn(state.params, inputs))
    per_token_logps = metrics.pop("per_token_logps", None)
    metrics = {k: torch.mean(torch.as_tensor(v).float()) for k, v in metrics.items()}
    return metrics["loss"], {**metrics, "per_token_logps": per_token_logps}


def training_step(state: LossTrainState, inputs: Mapping[str, Any]):
    """train_step.py:6-44 (and ppo/train_step.py:8-45): returns (new_state, metrics).

    metrics holds the mean of every entry of the module's dict (detached) plus
    "per_token_logps" as the module returned it."""
    keys = [k for k, v in state.params.items() if v.requires_grad]
    direct = state.grad_accum is not None and state.lm_head_key is not None \
        and state.params[state.lm_head_key].requires_grad
    # the loss is differentiated right here with upstream gradient 1 (value_and_grad, train_step.py:24),
    # so the fused loss may hand autograd the kernel's [H,V] gradient as it is
    if direct:
        with terminal_loss(), accumulate_lm_head_grad_into(state.grad_accum[state.lm_head_key]) as target:
            loss, metrics = _loss_and_aux(state, inputs)
            if target.uses != 1:
                raise RuntimeError(f"apply_fn made {target.uses} differentiable fused-loss calls; exactly one "
                                   "may add into the lm_head accumulator per micro-step")
        keys = [k for k in keys if k != state.lm_head_key]
    else:
        with terminal_loss():
            loss, metrics = _loss_and_aux(state, inputs)
    got = torch.autograd.grad(loss, [state.params[k] for k in keys], allow_unused=True) if keys else ()
    grads = {k: (g if g is not None else torch.zeros_like(state.params[k])) for k, g in zip(keys, got)}
    metrics = {k: (v.detach() if isinstance(v, torch.Tensor) else v) for k, v in metrics.items()}

    if state.grad_accum is None:                                             # :26-28
        return state.apply_gradients(grads=grads), metrics

    with torch.no_grad():                                                    # :30-33
        for k, g in grads.items():
            state.grad_accum[k].add_(g.to(torch.float32))
    state = state.replace(micro_step=state.micro_step + 1)
    if state.micro_step == state.micro_in_mini:                              # :35-43
        with torch.no_grad():
            mean = {k: (ga / state.micro_in_mini).to(state.params[k].dtype) for k, ga in state.grad_accum.items()
                    if state.params[k].requires_grad}
        state = state.apply_gradients(grads=mean, micro_step=state.micro_step % state.micro_in_mini)
        with torch.no_grad():
            for ga in state.grad_accum.values():
                ga.zero_()
    return state, metrics


ppo_training_step = training_step


def ppo_update(*, state: Any, datas: Mapping[str, Any], total_valid_token_count: Any,
               train_step: Callable[[Any, Any], Any] = training_step,
               slice_data: Callable[[Any, int, int], Any] = slice_data,
               grad_accum_steps: int, ppo_steps: int):
    """update/ppo.py:6-46, the same loop (a caller contract, not a redesign: the
    runner and the update modules call it with exactly these keywords): ppo_steps passes over the
    global batch in grad_accum_steps micro-batches.  Every micro-batch is normalised by the GLOBAL total_valid_token_count
    (:37); the first pass collects per_token_logps, which become old_per_token_logps for the
    later passes (:39-43).  Returns (state, datas with old_per_token_logps, last_meta, entropy)."""
    datas_dict = dict(datas)
    last_meta: Mapping[str, Any] = {}
    entropy = None
    per_token_logps = []
    # float32 master weights are cast to bf16 once per optimizer step, not once per micro-batch: an
    # update replaces the parameter tensors (LossTrainState.apply_gradients), which ends a cached copy
    with cache_bf16_lm_head():
        for ppo_step_idx in range(int(ppo_steps)):
            for micro_idx in range(int(grad_accum_steps)):
                local = {k: slice_data(v, int(grad_accum_steps), int(micro_idx)) for k, v in datas_dict.items()}
                local["total_valid_token_count"] = total_valid_token_count
                state, last_meta = train_step(state, local)
                if ppo_step_idx == 0:
                    per_token_logps.append(last_meta["per_token_logps"])
            if ppo_step_idx == 0:
                datas_dict["old_per_token_logps"] = torch.cat(per_token_logps, dim=0)
                entropy = last_meta.get("entropy")
    return state, datas_dict, last_meta, entropy


@dataclasses.dataclass(frozen=True)
class PPOUpdateModule:
    """update/modules.py:10-34."""

    def update(self, *, state, batch, total_valid_token_count, train_step=training_step,
               slice_data=slice_data, grad_accum_steps: int, ppo_steps: int) -> UpdateResult:
        state, batch_out, last_meta, entropy = ppo_update(
            state=state, datas=batch, total_valid_token_count=total_valid_token_count, train_step=train_step,
            slice_data=slice_data, grad_accum_steps=int(grad_accum_steps), ppo_steps=int(ppo_steps))
        return UpdateResult(state=state, batch=batch_out, last_meta=last_meta, entropy=entropy)


class PolicyGradientUpdateModule(PPOUpdateModule):
    """update/modules.py:37-60 (same loop; no value head requirement)."""


__all__ = ["LossTrainState", "UpdateResult", "slice_data", "training_step", "ppo_training_step", "ppo_update",
           "PPOUpdateModule", "PolicyGradientUpdateModule"]
