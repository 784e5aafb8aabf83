/* mj_grpo_bench.h -- measurement support for bench.py, built into libmj_grpo_bench.so: NOT part of
 * the product ABI (include/mj_grpo.h) and not linked by a trainer.  No counterpart in the reference,
 * whose only timers are wall-clock phase timers (plugins/training/runner/grpo_gsm8k.py:615-792).
 *
 * Per-kernel timing: mj_bench_trace is a launch-trace callback for mj_grpo_set_trace
 * (include/mj_grpo.h).  Between mj_bench_profile_begin and mj_bench_profile_end it brackets every
 * kernel launch of the product library with a pair of HIP events recorded on the stream the
 * kernel is launched on; mj_bench_profile_end waits for them and returns, per kernel id
 * (MJ_GRPO_K_*), the summed duration in milliseconds and the number of launches.  Process-wide and
 * not thread-safe: use from one thread.
 */
#ifndef MJ_GRPO_BENCH_H
#define MJ_GRPO_BENCH_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

int mj_bench_profile_begin(int max_launches);
int mj_bench_profile_end(double* total_ms /* [n_ids] */, int* launches /* [n_ids] */, int n_ids);
void mj_bench_trace(void* user, int kernel_id, int phase, void* stream);

/* An MFMA-only loop with the register tile of the product kernels (4 wavefronts x 16 blocks of
 * v_mfma_f32_32x32x16_bf16 per workgroup, no memory traffic while it runs).  operands: 1 MiB of
 * bf16 data on the device (what the multipliers see: random values or zeros); out: workgroups * 256
 * floats; *flop receives the flop executed.  Timed by the caller with events on `stream`; shows what
 * the matrix cores sustain under the GPU's power cap for a given operand data pattern.
 * shape 0: 4 x 4 blocks of v_mfma_f32_32x32x16_bf16 per wavefront, shape 1: 8 x 8 blocks of
 * v_mfma_f32_16x16x32_bf16 (twice the flop per iteration; *flop accounts for it), both with the
 * accumulators in rotation; shape 2: as 1 with the two k-steps of a block issued back to back on its
 * accumulator (the order of the GemmTN16 tile engine). */
int mj_bench_probe_mfma(const void* operands, float* out, int workgroups, int iters, int shape, double* flop,
                        void* stream);

/* Message of the calling thread's last non-zero status from the functions above. */
const char* mj_bench_last_error(void);

#ifdef __cplusplus
}
#endif
#endif /* MJ_GRPO_BENCH_H */
