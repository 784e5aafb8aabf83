// mj_bench.hip -- measurement support of bench.py (include/mj_grpo_bench.h): per-kernel HIP-event
// timing behind the product library's launch-trace hook, and an MFMA-only probe kernel.  Built into
// libmj_grpo_bench.so; the product library does not depend on it.
#include "../../include/mj_grpo_bench.h"

#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include <new>

#include "gemm_tn.hpp"

namespace {

thread_local char g_err[256] = "";
int fail(const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return 1;
}

struct Profiler {
  bool on = false;
  hipEvent_t* ev = nullptr;
  int* kid = nullptr;
  int cap = 0, used = 0;   // event pairs
  bool open = false;       // a phase-0 call is waiting for its phase-1 call
} g_prof;

}  // namespace

namespace mj {

// One workgroup = 4 wavefronts, each with the register tile of the product kernels: 4 x 4 blocks of
// v_mfma_f32_32x32x16_bf16 (SHAPE 0) or 8 x 8 blocks of v_mfma_f32_16x16x32_bf16 (SHAPE 1, 2), 256
// accumulators either way.  Two operand sets alternate so that consecutive instructions never see
// the same inputs.  SHAPE 0, 1: the accumulators in rotation (k-step outer, blocks inner); SHAPE 2:
// the two k-steps of a block back to back on its accumulator (the order of GemmTN16).  Per wavefront
// and iteration: 2 * 16 * 32768 flop (SHAPE 0), 2 * 64 * 16384 (SHAPE 1, 2).
template <int SHAPE>
__global__ __launch_bounds__(256) void k_probe_mfma(const bf16x8* src, float* out, int iters) {
  constexpr int F = SHAPE == 0 ? 4 : 8;      // fragments per operand and k-step
  bf16x8 a[2][F], b[2][F];
  const int t = threadIdx.x + blockIdx.x * 256;
#pragma unroll
  for (int s = 0; s < 2; ++s)
#pragma unroll
    for (int i = 0; i < F; ++i) {
      a[s][i] = src[(t * 32 + s * F + i) & 65535];
      b[s][i] = src[(t * 32 + 16 + s * F + i) & 65535];
    }
  float sum = 0.f;
  if (SHAPE == 0) {
    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
          for (int j = 0; j < 4; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a[s][i], b[s][j], acc[i][j], 0, 0, 0);
    }
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) sum += acc[i][j][r];
  } else {
    f32x4 acc[8][8];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;
    // one k-step of 32 over the 8 x 8 blocks = the flop of two k-steps of 16 over 4 x 4 blocks of 32 x 32
    for (int it = 0; it < iters; ++it) {
      if (SHAPE == 1) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
          for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[s][i], b[s][j], acc[i][j], 0, 0, 0);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
          for (int j = 0; j < 8; ++j) {
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[0][i], b[0][j], acc[i][j], 0, 0, 0);
            acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[1][i], b[1][j], acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);     // keeps the pair together
          }
      }
    }
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
      for (int j = 0; j < 8; ++j)
#pragma unroll
        for (int r = 0; r < 4; ++r) sum += acc[i][j][r];
  }
  out[t] = sum;
}

}  // namespace mj

extern "C" {

const char* mj_bench_last_error(void) { return g_err; }

int mj_bench_profile_begin(int max_launches) {
  if (g_prof.on) return fail("profiling already on");
  if (max_launches <= 0 || max_launches > (1 << 16)) return fail("max_launches out of range");
  g_prof.ev = new (std::nothrow) hipEvent_t[2 * (size_t)max_launches];
  g_prof.kid = new (std::nothrow) int[max_launches];
  hipError_t e = (g_prof.ev && g_prof.kid) ? hipSuccess : hipErrorOutOfMemory;
  int made = 0;
  for (; e == hipSuccess && made < 2 * max_launches; ++made) e = hipEventCreate(&g_prof.ev[made]);
  if (e != hipSuccess) {   // undo the partial set-up: nothing stays allocated after a failure
    for (int i = 0; i + 1 < made; ++i) (void)hipEventDestroy(g_prof.ev[i]);
    delete[] g_prof.ev;
    delete[] g_prof.kid;
    g_prof = Profiler();
    return fail("profile set-up: %s", hipGetErrorString(e));
  }
  g_prof.cap = max_launches;
  g_prof.used = 0;
  g_prof.open = false;
  g_prof.on = true;
  return 0;
}

void mj_bench_trace(void* /*user*/, int kernel_id, int phase, void* stream) {
  if (!g_prof.on) return;
  hipStream_t st = (hipStream_t)stream;
  if (phase == 0) {
    if (g_prof.used >= g_prof.cap) return;
    g_prof.kid[g_prof.used] = kernel_id;
    (void)hipEventRecord(g_prof.ev[2 * g_prof.used], st);
    g_prof.open = true;
  } else if (g_prof.open) {
    (void)hipEventRecord(g_prof.ev[2 * g_prof.used + 1], st);
    ++g_prof.used;
    g_prof.open = false;
  }
}

int mj_bench_profile_end(double* total_ms, int* launches, int n_ids) {
  if (!g_prof.on) return fail("profiling is not on");
  if (!total_ms || !launches || n_ids <= 0) return fail("total_ms/launches is NULL");
  for (int k = 0; k < n_ids; ++k) { total_ms[k] = 0.0; launches[k] = 0; }
  int rc = 0;
  for (int i = 0; i < g_prof.used; ++i) {
    float ms = 0.f;
    hipError_t e = hipEventSynchronize(g_prof.ev[2 * i + 1]);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, g_prof.ev[2 * i], g_prof.ev[2 * i + 1]);
    if (e != hipSuccess) { rc = fail("profile event: %s", hipGetErrorString(e)); break; }
    if (g_prof.kid[i] >= 0 && g_prof.kid[i] < n_ids) {
      total_ms[g_prof.kid[i]] += ms;
      launches[g_prof.kid[i]] += 1;
    }
  }
  for (int i = 0; i < 2 * g_prof.cap; ++i) (void)hipEventDestroy(g_prof.ev[i]);
  delete[] g_prof.ev;
  delete[] g_prof.kid;
  g_prof = Profiler();
  return rc;
}

int mj_bench_probe_mfma(const void* operands, float* out, int workgroups, int iters, int shape, double* flop,
                        void* stream) {
  if (!operands || !out) return fail("probe: operands/out is NULL");
  if (workgroups <= 0 || workgroups > (1 << 16) || iters <= 0) return fail("probe: bad workgroups/iters");
  if (((uintptr_t)operands & 15u) != 0) return fail("probe: operands must be 16-byte aligned");
  if (shape == 0) mj::k_probe_mfma<0><<<workgroups, 256, 0, (hipStream_t)stream>>>((const mj::bf16x8*)operands, out, iters);
  else if (shape == 1) mj::k_probe_mfma<1><<<workgroups, 256, 0, (hipStream_t)stream>>>((const mj::bf16x8*)operands, out, iters);
  else if (shape == 2) mj::k_probe_mfma<2><<<workgroups, 256, 0, (hipStream_t)stream>>>((const mj::bf16x8*)operands, out, iters);
  else return fail("probe: shape must be 0, 1 or 2");
  const double per_iter = shape == 0 ? 2.0 * 16.0 * 32768.0 : 2.0 * 64.0 * 16384.0;   // shapes 1 and 2 alike
  if (flop) *flop = (double)workgroups * 4.0 * iters * per_iter;
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? 0 : fail("k_probe_mfma: %s", hipGetErrorString(e));
}

}  // extern "C"
