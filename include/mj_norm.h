/* mj_norm.h -- C ABI of the RMSNorm that produces the fused loss path's `hidden` on MI355X (gfx950).
 *
 * Replaces LlamaRMSNorm (MLLM_JAX/language/llama/llama.py:426-452) as instantiated for the final
 * norm of the backbone (MLLM_JAX/language/qwen2/modular_qwen2.py:76, applied at :128; Llama:
 * llama.py:752) and its transpose under jax.value_and_grad
 * (plugins/training/update/train_step.py:24):
 *     y = x * rsqrt(mean(x^2, axis=-1) + eps) * scale,   computed in float32, stored as bf16.
 *
 * Conventions are those of mj_grpo.h: device pointers, caller-owned buffers, kernels enqueued on
 * the caller's hipStream_t, no allocation, no synchronisation, status codes MjGrpoStatus with
 * the message in mj_grpo_last_error().  x, y, dy, dx are bf16 [n, ld_*] with h and every ld_* a
 * multiple of 8 and 16-byte aligned bases; scale, dscale, rstd are float32.  h <= 8192.
 */
#ifndef MJ_NORM_H_
#define MJ_NORM_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* y[n,h] = rmsnorm(x) * scale (llama.py:438-451); rstd[n] = rsqrt(mean(x^2) + eps) is written
 * when rstd is not NULL. */
int mj_rmsnorm_forward(const void* x, int64_t ld_x, const float* scale, void* y, int64_t ld_y,
                       float* rstd, int64_t n, int64_t h, float eps, void* stream);

/* Bytes of workspace mj_rmsnorm_backward needs (per-workgroup partial sums of dscale). */
int mj_rmsnorm_workspace_bytes(int64_t n, int64_t h, size_t* bytes);

/* Transpose of the forward: dx[n,h] (bf16) and dscale[h] (float32; added to the existing
 * contents when accumulate_dscale != 0, the grad-accumulation of update/train_step.py:30-33).
 * Deterministic: fixed summation order, no atomics. */
int mj_rmsnorm_backward(const void* dy, int64_t ld_dy, const void* x, int64_t ld_x, const float* scale,
                        void* dx, int64_t ld_dx, float* dscale, int accumulate_dscale, int64_t n,
                        int64_t h, float eps, void* workspace, size_t workspace_bytes, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MJ_NORM_H_ */
