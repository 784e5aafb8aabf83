"""validate_grpo_batch: the cases of the reference's own test (tests/test_jit8_schema_and_cli.py:16-97
-- five stages on a 4 x 8 batch, a mismatched attention_mask) restated, plus the remaining rules."""
import numpy as np
import pytest
import torch

import mllm_jax_amd as M


def _batch(b=4, t=8, xp=np):
    labels = np.zeros((b, t), np.int32); labels[:, t // 2:] = 1
    d = {"input_ids": np.zeros((b, t), np.int32), "attention_mask": np.ones((b, t), np.int32), "labels": labels,
         "group_ids": np.arange(b, dtype=np.int32), "rewards": np.zeros(b, np.float32),
         "advantages": np.ones(b, np.float32), "old_per_token_logps": np.zeros((b, t - 1), np.float32),
         "total_valid_token_count": int(labels[:, 1:].sum())}
    return d if xp is np else {k: (torch.as_tensor(v) if hasattr(v, "shape") else v) for k, v in d.items()}


STAGE_KEYS = {"rollout": ["input_ids", "attention_mask", "labels", "group_ids"],
              "rewarded": ["input_ids", "attention_mask", "labels", "group_ids", "rewards"],
              "advantaged": ["input_ids", "attention_mask", "labels", "group_ids", "rewards", "advantages"],
              "train_step": ["input_ids", "attention_mask", "labels", "group_ids", "rewards", "advantages",
                             "total_valid_token_count"],
              "train_ready": ["input_ids", "attention_mask", "labels", "group_ids", "rewards", "advantages",
                              "total_valid_token_count", "old_per_token_logps"]}


@pytest.mark.parametrize("xp", [np, torch])
@pytest.mark.parametrize("stage", list(STAGE_KEYS))
def test_happy_path_per_stage(stage, xp):
    full = _batch(xp=xp)
    M.validate_grpo_batch({k: full[k] for k in STAGE_KEYS[stage]}, stage=stage)
    M.validate_grpo_batch(full, stage=stage.upper() + " ")          # case and blanks are normalised


def test_rejects_mismatched_shapes():
    with pytest.raises(M.BatchSchemaError):
        M.validate_grpo_batch({"input_ids": np.zeros((2, 4), np.int32), "attention_mask": np.ones((2, 5), np.int32),
                               "labels": np.zeros((2, 4), np.int32)}, stage="rollout")


@pytest.mark.parametrize("stage,change", [
    ("rollout", lambda d: d.pop("labels")),
    ("rollout", lambda d: d.update(input_ids=np.zeros(4, np.int32))),
    ("rollout", lambda d: d.update(input_ids=np.zeros((4, 1), np.int32), attention_mask=np.zeros((4, 1)), labels=np.zeros((4, 1)))),
    ("rollout", lambda d: d.update(group_ids=np.zeros(3, np.int32))),
    ("rollout", lambda d: d.update(labels=[[0] * 8] * 4)),
    ("rewarded", lambda d: d.pop("rewards")),
    ("rewarded", lambda d: d.update(rewards=np.zeros((4, 1), np.float32))),
    ("advantaged", lambda d: d.update(advantages=np.zeros(5, np.float32))),
    ("train_step", lambda d: d.pop("total_valid_token_count")),
    ("train_step", lambda d: d.update(total_valid_token_count=np.zeros(2))),
    ("train_step", lambda d: d.update(total_valid_token_count="12")),
    ("train_step", lambda d: d.update(old_per_token_logps=np.zeros((4, 8), np.float32))),
    ("train_ready", lambda d: d.pop("old_per_token_logps")),
])
def test_each_rule_is_enforced(stage, change):
    d = _batch()
    change(d)
    with pytest.raises(M.BatchSchemaError):
        M.validate_grpo_batch(d, stage=stage)


def test_unknown_stage_and_scalar_forms():
    with pytest.raises(ValueError):
        M.validate_grpo_batch(_batch(), stage="sampled")
    d = _batch()
    for tv in (17, 17.0, np.array(17), torch.tensor(17)):
        d["total_valid_token_count"] = tv
        M.validate_grpo_batch(d, stage="train_ready")
    assert issubclass(M.BatchSchemaError, ValueError)
