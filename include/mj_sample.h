/* mj_sample.h -- C ABI of the sampler's last-position step on MI355X (gfx950): logits of the
 * newest position and the top-k / categorical draw over them.
 *
 * Replaces, in the reference's decode loop (MLLM_JAX/sample/sample_state_right_padding2.py:219-234):
 *   logits[:, -1] = hidden_last @ lm_head                     (qwen2/modular_qwen2.py:182)
 *   _top_k_sampling_batched(rng, logits, k=50, t)             (MLLM_JAX/sample/sanple_utils.py:35-53)
 *   _greedy_sampling                                          (sanple_utils.py:58-60)
 * Conventions are those of mj_grpo.h (device pointers, caller-owned buffers, caller's stream,
 * no allocation, MjGrpoStatus codes, mj_grpo_last_error()).
 *
 * Random numbers stay with the caller: jax.random.categorical(key, x) is argmax(x + Gumbel
 * noise), so the draw takes the noise as an input ([b, k] float32, one value per sorted top-k
 * slot) and is a deterministic function of it.
 */
#ifndef MJ_SAMPLE_H_
#define MJ_SAMPLE_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* logits[b, ld_logits] (float32) = hidden[b, ld_hidden] (bf16) @ lm_head[h, ld_w] (bf16), with the
 * optional final-logit softcap (0 = off).  h, vocab, ld_hidden, ld_w multiples of 8, ld_logits a
 * multiple of 4, 16-byte aligned bases. */
int mj_sample_logits(const void* hidden, int64_t ld_hidden, const void* lm_head, int64_t ld_w,
                     float* logits, int64_t ld_logits, int64_t b, int64_t h, int64_t vocab,
                     float softcap, void* stream);

/* Per row: the k (<= 64) largest of logits / t (a division, as the reference's `logits / t`,
 * MLLM_JAX/sample/sanple_utils.py:37) in descending order (equal values: lower index
 * first, as jax.lax.top_k), then token = top_idx[argmax_j(top_val[j] + noise[j])] (first maximum
 * on ties, as jnp.argmax).  noise == NULL draws greedily (the largest logit).  top_idx / top_val
 * ([b, k]) may be NULL. */
int mj_sample_top_k(const float* logits, int64_t ld_logits, int64_t b, int64_t vocab, int k,
                    float temperature, const float* noise, int32_t* token, int32_t* top_idx,
                    float* top_val, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MJ_SAMPLE_H_ */
