"""Structural checks of the batch dict that flows into the loss path.

Host-side mirror of validate_grpo_batch / BatchSchemaError
(plugins/training/api/batch_schema.py:7-146): same stages, same required keys per stage, same
rank / leading-dimension / T-1 rules, ValueError subclass on violation.  Works on anything with
.shape and .dtype (torch tensors on the GPU included; nothing is copied or synchronised).
"""
from __future__ import annotations

from typing import Any, Mapping, Optional, Tuple

STAGES = ("rollout", "rewarded", "advantaged", "train_step", "train_ready")


class BatchSchemaError(ValueError):
    """A rollout / train batch does not have the expected structure."""


def _shape(name: str, value: Any) -> Tuple[int, ...]:
    if not (hasattr(value, "shape") and hasattr(value, "dtype")):
        raise BatchSchemaError(f"{name} must be array-like (has .shape/.dtype), got: {type(value).__name__}")
    return tuple(int(s) for s in value.shape)


def _need(batch: Mapping[str, Any], *names: str) -> None:
    absent = [k for k in names if k not in batch]
    if absent:
        raise BatchSchemaError(f"Missing required keys: {absent}. Present keys: {sorted(batch.keys())}")


def _per_sequence(batch: Mapping[str, Any], name: str, rank: int, bsz: int) -> Tuple[int, ...]:
    shp = _shape(name, batch[name])
    if len(shp) != rank:
        raise BatchSchemaError(f"{name} must be rank-{rank} but got shape={shp} dtype={batch[name].dtype}")
    if shp[0] != bsz:
        raise BatchSchemaError(f"{name} first dim must be {bsz} to match batch size, got shape={shp}")
    return shp


def validate_grpo_batch(batch: Mapping[str, Any], *, stage: str) -> None:
    """Raises BatchSchemaError unless `batch` has the structure the given pipeline stage promises:
    rollout -> input_ids / attention_mask / labels [B, T] (T > 1); rewarded -> + rewards [B];
    advantaged -> + advantages [B]; train_step -> + scalar total_valid_token_count (and a well-formed
    old_per_token_logps [B, T-1] if present); train_ready -> old_per_token_logps required.
    group_ids, when present, must be [B].  Dtypes are not checked (batch_schema.py:59-146)."""
    stage = str(stage).strip().lower()
    if stage not in STAGES:
        raise ValueError(f"Unknown stage={stage!r}")
    level = STAGES.index(stage)

    _need(batch, "input_ids", "attention_mask", "labels")
    ids = _shape("input_ids", batch["input_ids"])
    for name in ("input_ids", "attention_mask", "labels"):
        shp = _shape(name, batch[name])
        if len(shp) != 2:
            raise BatchSchemaError(f"{name} must be rank-2 but got shape={shp} dtype={batch[name].dtype}")
        if shp != ids:
            raise BatchSchemaError(f"input_ids and {name} must have the same shape; got input_ids={ids} {name}={shp}")
    bsz, seq_len = ids
    if bsz <= 0:
        raise BatchSchemaError(f"Batch size must be > 0, got {bsz}")
    if seq_len <= 1:
        raise BatchSchemaError(f"Sequence length must be > 1 (needs T-1), got {seq_len}")

    if level >= 1:
        _need(batch, "rewards")
        _per_sequence(batch, "rewards", 1, bsz)
    if "group_ids" in batch:
        _per_sequence(batch, "group_ids", 1, bsz)
    if level >= 2:
        _need(batch, "advantages")
        _per_sequence(batch, "advantages", 1, bsz)
    if level >= 3:
        _need(batch, "total_valid_token_count")
        tv = batch["total_valid_token_count"]
        if hasattr(tv, "shape") and hasattr(tv, "dtype"):
            if _shape("total_valid_token_count", tv) != ():
                raise BatchSchemaError(f"total_valid_token_count must be scalar (shape=()), got {tuple(tv.shape)}")
        elif not isinstance(tv, (int, float)):
            raise BatchSchemaError("total_valid_token_count must be a scalar array or Python number, "
                                   f"got {type(tv).__name__}")
        if level >= 4:
            _need(batch, "old_per_token_logps")
        if "old_per_token_logps" in batch:
            old = _per_sequence(batch, "old_per_token_logps", 2, bsz)
            if old[1] != seq_len - 1:
                raise BatchSchemaError("old_per_token_logps second dim must be T-1 to match input_ids[:,1:]; "
                                       f"got old_per_token_logps={old} input_ids={ids}")


__all__ = ["BatchSchemaError", "validate_grpo_batch", "STAGES"]
