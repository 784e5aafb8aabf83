/* mj_grpo.h -- C ABI of the MI355X (gfx950) fused GRPO loss library, libmj_grpo.so.
 *
 * The reference (demon2036/MLLM-JAX) has no FFI for this path: the boundary there is
 * the Python callable TrainGRPOModule.__call__ (MLLM_JAX/train_modules/__init__.py:96-192)
 * differentiated by jax.value_and_grad (plugins/training/update/train_step.py:15-24).
 * The entry points below are what a binding for that callable would call; each one
 * names the reference statements it replaces.
 *
 * Conventions: plain pointers to DEVICE memory and sizes, no allocation inside the
 * library, every kernel is enqueued on the caller's hipStream_t (passed as void*),
 * calls return immediately (asynchronous), status is an int (0 = ok) and
 * mj_grpo_last_error() gives the message of the calling thread's last failure.
 * Two calls may overlap only if they use distinct workspaces.
 *
 * Shapes: tokens are flattened, N = B*(L-1) after the reference's shift
 * (train_modules/__init__.py:118-125).  hidden[N, ld_hidden] bf16 row-major,
 * lm_head[H, ld_w] bf16 row-major (Flax Dense kernel layout [in, out],
 * MLLM_JAX/language/llama/llama.py:889), targets[N] int32 in [0, V),
 * (ids outside are clamped to the nearest valid id, the same way in both passes, without a
 * host check; the reference's jnp.take_along_axis wraps negative ids and yields NaN past V),
 * old_logp[N] f32 or NULL (NULL = on-policy, ratio == 1, train_modules/__init__.py:161-165),
 * advantages[N] f32 (the reference's [B] broadcast per token, :173), mask[N] f32 in {0,1}.
 * Requirements: H % 8 == 0, V % 8 == 0, ld_hidden % 8 == 0, ld_w % 8 == 0,
 * bf16 pointers, d_lm_head and the workspace 16-byte aligned, temperature > 0.
 */
#ifndef MJ_GRPO_H
#define MJ_GRPO_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  MJ_GRPO_OK = 0,
  MJ_GRPO_ERR_NULL = 1,        /* required pointer is NULL */
  MJ_GRPO_ERR_SHAPE = 2,       /* N/H/V/ld out of range */
  MJ_GRPO_ERR_ALIGN = 3,       /* pointer or leading dimension not 16-byte aligned */
  MJ_GRPO_ERR_WORKSPACE = 4,   /* workspace missing or too small */
  MJ_GRPO_ERR_UNSUPPORTED = 5, /* e.g. temperature <= 0, unknown flag, entropy bonus with temperature != 1 */
  MJ_GRPO_ERR_HIP = 6          /* a HIP call or kernel launch failed */
};

enum {
  MJ_GRPO_FLAG_DW_ACCUMULATE = 1u << 0, /* d_lm_head += (grad accumulation, train_step.py:30-33) */
  MJ_GRPO_FLAG_SFT = 1u << 1,           /* masked cross-entropy instead of the clipped surrogate
                                           (plugins/sft/jax/sft_module.py:22-45): per-token loss
                                           -logp, advantages/old_logp ignored */
  MJ_GRPO_FLAG_SKIP_MASKED = 1u << 2,   /* tokens whose gradient is zero by construction (mask 0: prompt
                                           and padding positions, labels of train_modules/__init__.py:120;
                                           advantage 0 when nothing else feeds the gradient, i.e. no entropy
                                           bonus and no value head) are moved
                                           behind the others and left out of the backward products.
                                           Same outputs (d_lm_head up to summation order); the forward
                                           still covers every token.  No counterpart in the reference,
                                           which multiplies the zeros.  Needs a larger workspace. */
  MJ_GRPO_FLAG_DW_BF16 = 1u << 3        /* d_lm_head is a bf16 [H, ld_w] matrix instead of a float one (for
                                           callers whose lm_head parameter, and so its gradient, is bf16;
                                           the reference's parameter gradients are float32,
                                           llama/llama.py:251-256).  Each entry is summed in fp32 and rounded
                                           once per call and per chunk of chunk_tokens; with
                                           MJ_GRPO_FLAG_DW_ACCUMULATE the value in memory is added in fp32
                                           before that rounding. */
};

typedef struct MjGrpoDesc {
  int64_t n_tokens;      /* N */
  int64_t hidden;        /* H */
  int64_t vocab;         /* V */
  int64_t ld_hidden;     /* elements between rows of hidden (>= H) */
  int64_t ld_w;          /* elements between rows of lm_head (>= V) */
  int64_t chunk_tokens;  /* tokens whose 16-bit logits live in the workspace at once; 0 = default */
  float eps_low;         /* TrainGRPOModule.epsilon_low  (train_modules/__init__.py:92) */
  float eps_high;        /* TrainGRPOModule.epsilon_high (:93) */
  float temperature;     /* T > 0 (:91).  As in the reference, logp = log_softmax(z)[y] / T (:124-126) while the
                            entropy is that of softmax(z / T) (:136); lse[] is always logsumexp(z) */
  float softcap;         /* final-logit softcap, 0 = off (gemma/transformer.py:337-339) */
  float inv_total_valid_tokens; /* 1 / total_valid_token_count (:179-180) */
  float grad_loss_scale; /* upstream d(loss); 1 for a terminal loss */
  uint32_t flags;
  uint32_t dhidden_splits; /* pieces the vocab sum of the d_hidden product is cut into (fp32 partial sums,
                            added in fixed order); 0 = chosen by the library, at most 32 */
  float entropy_coef;    /* PPOActorCriticModule.entropy_coef (plugins/training/ppo/module.py:140):
                            the loss becomes policy_loss - entropy_coef * entropy; 0 = GRPO */
  float inv_entropy_count; /* 1 / (sum(mask) + 1e-8), the normaliser of that entropy (:79); 0 = unused */
} MjGrpoDesc;

/* Library version, MAJOR*10000 + MINOR*100 + PATCH. */
int mj_grpo_version(void);

/* Message of the calling thread's last non-zero status ("" if none). */
const char* mj_grpo_last_error(void);

/* Workspace sizes in bytes for the three entry points below. */
int mj_grpo_workspace_bytes(const MjGrpoDesc* desc, size_t* forward_bytes,
                            size_t* forward_backward_bytes);

/* Forward only (no gradient).  Replaces train_modules/__init__.py:124-126 (log-softmax +
 * gather), :136-138 (per-token entropy), :161-180 (ratio, clip, min, masked normalised sum)
 * on top of the lm_head product (qwen2/modular_qwen2.py:182), streaming over vocab tiles:
 * no [N,V] tensor is written.  Outputs: logp[N], lse[N], token_entropy[N] (may be NULL),
 * loss[2]: loss[0] = policy loss - entropy_coef * entropy, loss[1] = entropy =
 * sum(token_entropy * mask) * inv_entropy_count (plugins/training/ppo/module.py:77-79; 0 when
 * inv_entropy_count is 0).  */
int mj_grpo_forward(const MjGrpoDesc* desc, const void* hidden, const void* lm_head,
                    const int32_t* targets, const float* old_logp, const float* advantages,
                    const float* mask, float* logp, float* lse, float* token_entropy,
                    float* loss, void* workspace, size_t workspace_bytes, void* stream);

/* mj_grpo_forward without a workspace argument, for callers that cannot allocate device memory
 * (code under HIP graph capture, tight serving loops that score log-probs, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  The statistics that mj_grpo_forward keeps in the
 * caller's workspace live in a static device array of MJ_GRPO_NOALLOC_SCRATCH_BYTES that every device
 * the library runs on holds until the process ends; the call allocates and frees nothing.
 * chunk_tokens == 0 picks the largest chunk that fits (at most 16384 tokens).  Shapes whose workspace
 * does not fit even with 256-token chunks (12 bytes per token plus 6 * ceil(V/256) * 4 bytes per
 * token of a chunk) are refused with MJ_GRPO_ERR_WORKSPACE.  All calls on one device share the
 * array: calls that overlap on a device (two streams, two threads) race; serialise them.  Outputs
 * are those of mj_grpo_forward bit for bit.  The first call on a device (from any thread) looks the
 * array's address up (hipGetSymbolAddress) and raises the kernels' LDS limit (hipFuncSetAttribute):
 * make one call per device outside stream capture before capturing others. */
#define MJ_GRPO_NOALLOC_SCRATCH_BYTES (32u << 20)
int mj_grpo_forward_noalloc(const MjGrpoDesc* desc, const void* hidden, const void* lm_head,
                            const int32_t* targets, const float* old_logp, const float* advantages,
                            const float* mask, float* logp, float* lse, float* token_entropy,
                            float* loss, void* stream);

/* Forward and backward in one pass (executes 6*N*H*V flop).  Replaces
 * jax.value_and_grad(loss_fn) of plugins/training/update/train_step.py:15-24 restricted to
 * the lm_head + loss part: besides the forward outputs it writes
 * d_hidden[N, ld_hidden] bf16 and d_lm_head[H, ld_w] f32 (bf16 with MJ_GRPO_FLAG_DW_BF16), both already multiplied by
 * grad_loss_scale.  The workspace holds 16-bit (half) logits for chunk_tokens tokens at a time.
 * With entropy_coef != 0 the gradient includes the entropy bonus,
 * d(-coef*entropy)/dz = coef * mask * inv_entropy_count * p * (log p + H_t). */
int mj_grpo_forward_backward(const MjGrpoDesc* desc, const void* hidden, const void* lm_head,
                             const int32_t* targets, const float* old_logp,
                             const float* advantages, const float* mask, float* logp,
                             float* lse, float* token_entropy, float* loss, void* d_hidden,
                             void* d_lm_head, void* workspace, size_t workspace_bytes,
                             void* stream);

/* Upstream gradient that is only known on the device.  The reference differentiates the loss itself
 * (jax.value_and_grad, plugins/training/update/train_step.py:15-24: upstream gradient 1, which is what
 * grad_loss_scale = 1 gives); a caller whose autodiff hands it d(total)/d(loss) as a device scalar
 * after the fused pass has run (torch.autograd) applies it here: d_hidden[n, ld_hidden] bf16 and
 * d_lm_head[h, ld_w] (float32, or bf16 when d_lm_head_bf16 != 0) are multiplied in place by *scale.
 * When *scale == 1 every workgroup leaves at once: no pass over either matrix, no host
 * synchronisation.  Either pointer may be NULL (skipped).  Padding columns past h / v are untouched. */
int mj_grpo_scale_gradients(void* d_hidden, int64_t n, int64_t h, int64_t ld_hidden, void* d_lm_head,
                            int64_t lm_head_rows, int64_t v, int64_t ld_w, int d_lm_head_bf16,
                            const float* scale, void* stream);

/* The two per-sequence entropy entries of the reference's return dict
 * (MLLM_JAX/train_modules/__init__.py:141-157) from the per-token entropies of a forward:
 * token_entropy, mask: float32 [b, t] row-major; entropy[b] = sum(H * mask) / sum(mask) (nan for an
 * empty row, as in the reference); entropy_loss[b] = the mean of H over the tokens with mask == 1
 * whose running count of such tokens lies in [4, 100]. */
int mj_grpo_sequence_entropy(const float* token_entropy, const float* mask, int64_t b, int64_t t,
                             float* entropy, float* entropy_loss, void* stream);

/* PPO actor-critic: the critic's value head and clipped value loss ride the same call
 * (plugins/training/ppo/module.py:34-39, :52, :104-140).  All pointers are device pointers.
 *   value_pred[t] = hidden[t, :] . value_w + value_b[0]                          (Dense(1), float32)
 *   returns      NULL: advantages + value_pred, NOT detached (:107);   old_values NULL: stop_gradient(value_pred) (:118)
 *   vl_t = use_clip ? max((v - R)^2, (old + clip(v - old, +-value_clip) - R)^2) : (v - R)^2       (:131-136)
 *   value_loss[0] = sum(vl * mask) * inv_total_valid_tokens                                       (:138)
 * The gradient of value_coef * value_loss reaches d_hidden inside the d_hidden product's epilogue
 * (d_hidden[t, :] += dv_t * value_w), d_value_w[H] and d_value_b[1] are written in float32, all scaled by
 * grad_loss_scale.  loss[0] stays policy loss - entropy_coef * entropy; the caller adds
 * value_coef * value_loss[0] (:140).  value_w and d_value_w must be 16-byte aligned. */
typedef struct MjPpoValue {
  const float* value_w;      /* [H] */
  const float* value_b;      /* [1] */
  const float* returns;      /* [N] or NULL */
  const float* old_values;   /* [N] or NULL */
  float value_coef;          /* PPOActorCriticModule.value_coef */
  float value_clip;          /* PPOActorCriticModule.value_clip_range when use_clip != 0 */
  int32_t use_clip;          /* value_clip_range is not None */
  int32_t reserved;
  float* values;             /* out [N]: value_pred */
  float* value_loss;         /* out [1] */
  float* d_value_w;          /* out [H] */
  float* d_value_b;          /* out [1] */
} MjPpoValue;

/* mj_grpo_forward_backward with the value head (value != NULL required).  The workspace size is
 * that of mj_grpo_workspace_bytes plus mj_grpo_value_workspace_bytes, the extra part at the end. */
int mj_grpo_value_workspace_bytes(const MjGrpoDesc* desc, size_t* extra_bytes);
int mj_grpo_forward_backward_value(const MjGrpoDesc* desc, const MjPpoValue* value, const void* hidden,
                                   const void* lm_head, const int32_t* targets, const float* old_logp,
                                   const float* advantages, const float* mask, float* logp, float* lse,
                                   float* token_entropy, float* loss, void* d_hidden, void* d_lm_head,
                                   void* workspace, size_t workspace_bytes, void* stream);

/* The value head alone (PPOActorCriticModule.value, module.py:55-57): values[n] = hidden . value_w + value_b. */
int mj_value_head_forward(const void* hidden, int64_t ld_hidden, const float* value_w, const float* value_b,
                          float* values, int64_t n, int64_t h, void* stream);

/* Backward from a saved forward (lse[N], logp[N]): recomputes the logits chunk by chunk
 * (8*N*H*V flop with the forward).  Same outputs as the backward half above.  For callers
 * that must separate the two passes (e.g. a forward under no-grad followed later by a
 * backward with a non-unit upstream gradient).  entropy_coef must be 0 here. */
int mj_grpo_backward(const MjGrpoDesc* desc, const void* hidden, const void* lm_head,
                     const int32_t* targets, const float* old_logp, const float* advantages,
                     const float* mask, const float* lse, const float* logp, void* d_hidden,
                     void* d_lm_head, void* workspace, size_t workspace_bytes, void* stream);

/* Sequence-level advantage estimators on the device (host NumPy in the reference, evaluated by the
 * runner at runner/grpo_gsm8k.py:680).  rewards, advantages: float32 [b]; group_ids: int32 [b] (any
 * ids, any group sizes; unused by MJ_GRPO_ADV_GLOBAL).  b <= 65536 (MJ_GRPO_ADV_GLOBAL), b <= 8192 for the
 * grouped estimators, which walk the batch once per sample.
 *   MJ_GRPO_ADV_GRPO    (r - mean_g) / (std_g + eps), population std     advantage/grpo.py:8-52
 *   MJ_GRPO_ADV_GLOBAL  (r - mean) / (std + eps)                          advantage/estimators.py:37-55
 *   MJ_GRPO_ADV_RLOO    r - mean of the others in the group (group mean for singletons); whiten != 0
 *                       then centres and scales over the batch            estimators.py:58-103, :137-157
 *   MJ_GRPO_ADV_DAPO    GRPO + alpha * GLOBAL                             estimators.py:106-134
 * clip_range > 0 clips the result to [-clip_range, clip_range] (estimators.py:28-34). */
enum { MJ_GRPO_ADV_GRPO = 0, MJ_GRPO_ADV_GLOBAL = 1, MJ_GRPO_ADV_RLOO = 2, MJ_GRPO_ADV_DAPO = 3 };
int mj_grpo_advantages(int mode, const float* rewards, const int32_t* group_ids, float* advantages,
                       int64_t b, float eps, float alpha, int whiten, float clip_range, void* stream);

/* mj_grpo_advantages(MJ_GRPO_ADV_GRPO, ...): compute_grpo_advantages_by_group_id. */
int mj_grpo_group_advantages(const float* rewards, const int32_t* group_ids, float* advantages,
                             int64_t b, float eps, void* stream);

/* Token-level GAE (compute_gae_advantages, advantage/estimators.py:180-240; the sequence reward is
 * placed on the last completion token, build_token_rewards_from_final, :160-177).  rewards [b];
 * values, completion_mask, advantages, returns: float32 [b, t] row-major.  normalize != 0 centres and
 * scales the advantages over the completion tokens and zeroes the others; clip_range > 0 clips. */
int mj_grpo_gae(const float* rewards, const float* values, const float* completion_mask,
                float* advantages, float* returns, int64_t b, int64_t t, float gamma, float gae_lambda,
                int normalize, float eps, float clip_range, void* stream);

/* Launch tracing.  The reference's observability of this path is a set of wall-clock phase timers
 * around the update (plugins/training/runner/grpo_gsm8k.py:615-792, printed under
 * PRINT_TRAIN_TIME_BREAKDOWN); here a caller can watch the individual kernels.  While a callback is
 * set, every kernel launch of the entry points above is bracketed by two calls of it on the calling
 * thread: phase 0 just before the launch is enqueued on `stream`, phase 1 just after (the three
 * launches of the running-maximum rescue pass count as one, MJ_GRPO_K_RESCUE).  The callback may
 * record events on `stream`; it must not synchronise or enqueue work that the kernels depend on.
 * fn == NULL switches tracing off.  Process-wide and not thread-safe: set it while no call runs. */
enum {
  MJ_GRPO_K_LOGITS_STATS = 0,
  MJ_GRPO_K_FINALIZE = 1,
  MJ_GRPO_K_DZ = 2,
  MJ_GRPO_K_DHIDDEN = 3,
  MJ_GRPO_K_DHIDDEN_REDUCE = 4,
  MJ_GRPO_K_DW = 5,
  MJ_GRPO_K_REDUCE_LOSS = 6,
  MJ_GRPO_K_SCALE_HIDDEN = 7,
  MJ_GRPO_K_RESCUE = 8,
  MJ_GRPO_K_COUNT = 9
};
typedef void (*MjGrpoTraceFn)(void* user, int kernel_id, int phase, void* stream);
int mj_grpo_set_trace(MjGrpoTraceFn fn, void* user);

#ifdef __cplusplus
}
#endif
#endif /* MJ_GRPO_H */
