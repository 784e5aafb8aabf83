"""MI355X-native fused GRPO loss (lm_head product + streaming log-softmax + clipped
policy-ratio loss, forward and backward) behind the reference's loss-function contract."""
from .advantage import (build_token_rewards_from_final, compute_dapo_advantages_by_group_id,
                        compute_gae_advantages, compute_global_normalized_advantages,
                        compute_reinforce_plus_plus_advantages_by_group_id, compute_rloo_advantages_by_group_id)
from .batch_schema import BatchSchemaError, validate_grpo_batch
from .loss import (PPOActorCriticModule, compute_grpo_advantages_by_group_id, TrainGRPOModule, grpo_fused_loss, grpo_loss_value_and_grad, loss_and_metrics,
                   release_workspaces, sft_fused_loss)
from .loss import accumulate_lm_head_grad_into, cache_bf16_lm_head, invalidate_bf16_lm_head, terminal_loss
from .norm import LlamaRMSNorm, rms_norm
from .sample import greedy_sampling, last_position_logits, sample_next_tokens, top_k_sampling_batched
from .update import (LossTrainState, PolicyGradientUpdateModule, PPOUpdateModule, UpdateResult, ppo_training_step,
                     ppo_update, slice_data, training_step)
from .workloads import CONFIGS, LossConfig, gumbel_max_targets, make_workload

__all__ = ["TrainGRPOModule", "PPOActorCriticModule", "grpo_fused_loss", "grpo_loss_value_and_grad", "loss_and_metrics",
           "sft_fused_loss", "release_workspaces", "accumulate_lm_head_grad_into", "terminal_loss", "cache_bf16_lm_head", "invalidate_bf16_lm_head", "LossTrainState",
           "PolicyGradientUpdateModule", "PPOUpdateModule", "UpdateResult", "ppo_training_step", "ppo_update",
           "slice_data", "training_step", "LlamaRMSNorm", "rms_norm", "build_token_rewards_from_final", "compute_dapo_advantages_by_group_id", "compute_gae_advantages",
           "compute_global_normalized_advantages", "compute_reinforce_plus_plus_advantages_by_group_id",
           "compute_rloo_advantages_by_group_id", "BatchSchemaError", "validate_grpo_batch", "greedy_sampling", "last_position_logits", "sample_next_tokens", "top_k_sampling_batched", "compute_grpo_advantages_by_group_id", "CONFIGS", "LossConfig", "make_workload", "gumbel_max_targets"]
