"""Benchmark of the fused GRPO loss (forward + backward) on one MI355X.

`python bench.py [--gpus 1] [--steps K] [--warmup W] [--config 2]` prints ONE JSON line.
A step is one fwd+bwd pass of the loss over one synthetic batch of the chosen configuration
(default: BASELINE.json configs[2], the Qwen2.5-7B shape 16384 x 3584 x 152064 the metric is
quoted on), inputs resident in HBM, through the host API that wraps the C ABI.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA, published
PEAK_HBM_GBS = 8000.0

# Bytes per launch that crossed the L2 <-> fabric boundary (Infinity Cache or HBM behind it), from
# two rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE), each scaled by what the same counter reads for
# a plain 1 GiB device copy (x2.00 fetch, x1.00 write); summary in profiles/.  Keyed by
# (config index, kernel); None for workloads that were not counted.
MEASURED_TRAFFIC_BYTES = {          # default chunk (one launch of each kernel per step at configs 0-2 and 4)
    (0, "k_logits_stats"): 0.40e9, (0, "k_dhidden"): 0.42e9, (0, "k_dw"): 0.71e9,
    (2, "k_logits_stats"): 29.82e9, (2, "k_dhidden"): 26.12e9, (2, "k_dw"): 27.59e9,
}
TRAFFIC_SOURCE = {0: "profiles/cfg0_qwen05b_fused_fwd_bwd.txt", 2: "profiles/cfg2_qwen7b_fused_fwd_bwd.txt"}


class BenchLib:
    """libmj_grpo_bench.so (include/mj_grpo_bench.h): per-kernel HIP-event timing behind the product
    library's launch-trace hook, and the MFMA-only probe.  Bench-only code: the product does not load it."""

    KERNELS = ("k_logits_stats", "k_finalize", "k_dz", "k_dhidden", "k_dhidden_reduce", "k_dw",
               "k_reduce_loss", "k_scale_hidden", "k_rescue")

    def __init__(self, product):
        import ctypes as C
        self.C = C
        path = os.path.join(ROOT, "mllm_jax_amd", "libmj_grpo_bench.so")
        if not os.path.exists(path):
            raise RuntimeError(f"{path} is missing: run `python -m mllm_jax_amd.build`")
        self.lib = C.CDLL(path)
        self.lib.mj_bench_last_error.restype = C.c_char_p
        self.lib.mj_bench_profile_end.argtypes = [C.POINTER(C.c_double), C.POINTER(C.c_int), C.c_int]
        self.lib.mj_bench_probe_mfma.argtypes = [C.c_void_p, C.c_void_p, C.c_int, C.c_int, C.c_int,
                                                 C.POINTER(C.c_double), C.c_void_p]
        self.product = product

    def _check(self, status):
        if status != 0:
            raise RuntimeError("bench library: " + self.lib.mj_bench_last_error().decode())

    def profile_begin(self, max_launches):
        self._check(self.lib.mj_bench_profile_begin(int(max_launches)))
        self.product.mj_grpo_set_trace(self.C.cast(self.lib.mj_bench_trace, self.C.c_void_p), None)

    def profile_end(self) -> dict:
        """{kernel name: (total_ms, launches)} since profile_begin."""
        self.product.mj_grpo_set_trace(None, None)
        n = len(self.KERNELS)
        ms, cnt = (self.C.c_double * n)(), (self.C.c_int * n)()
        self._check(self.lib.mj_bench_profile_end(ms, cnt, n))
        return {self.KERNELS[i]: (ms[i], cnt[i]) for i in range(n)}

    def probe_mfma(self, operands, out, workgroups, iters, shape, stream) -> float:
        flop = self.C.c_double(0.0)
        self._check(self.lib.mj_bench_probe_mfma(operands, out, workgroups, iters, shape, self.C.byref(flop), stream))
        return flop.value


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--config", type=int, default=2, help="index into BASELINE.json configs (default 2)")
    ap.add_argument("--chunk-tokens", type=int, default=0)
    ap.add_argument("--dhidden-splits", type=int, default=0, help="vocab splits of the d_hidden product (0 = library's choice)")
    ap.add_argument("--pad-w", type=int, default=0, help="extra elements in the row pitch of lm_head (ld_w = vocab + this)")
    ap.add_argument("--smi", action="store_true",
                    help="sample power / shader clock / temperature with rocm-smi during the timed loop (use >= 50 steps)")
    ap.add_argument("--zero-operands", action="store_true",
                    help="time the same launches with all-zero hidden and lm_head (MFMA power depends on the operand "
                         "data; the loss value is then meaningless)")
    ap.add_argument("--mfma-probe", action="store_true",
                    help="instead of the loss: run the library's MFMA-only loop (no memory traffic) for ~3 s each with "
                         "random and with all-zero bf16 operands and print what the matrix cores sustain under the "
                         "power cap, with amd-smi power / clock samples")
    ap.add_argument("--entropy-coef", type=float, default=0.0,
                    help="add PPO's entropy bonus (plugins/training/ppo/module.py:140): times the running-maximum "
                         "kernels + the in-place dZ pass instead of the default path")
    ap.add_argument("--dw-dtype", choices=("f32", "bf16"), default="f32",
                    help="dtype of the lm_head gradient the dW kernel writes (the reference's is float32: the default)")
    ap.add_argument("--graph", action="store_true",
                    help="capture one step in a HIP graph and time its replays (small shapes are launch-bound; implies "
                         "--no-kernel-events: the per-kernel timers then run in a separate eager loop)")
    ap.add_argument("--neighbours", action="store_true",
                    help="instead of the loss step, time the steps either side of it (RMSNorm, sampler, value head, "
                         "group advantages) at the config's shape against the HBM roofline")
    ap.add_argument("--no-kernel-events", action="store_true",
                    help="time the steps without the per-kernel HIP events (each event pair leaves ~10 us between "
                         "two kernels: nothing at the headline shape, 10 %% of a step at the smallest); the per-kernel "
                         "figures and the roofline object then come from a second, short, instrumented loop")
    ap.add_argument("--cpu-sample-tokens", type=int, default=8192)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--skip-masked", action="store_true",
                    help="time the main loop with MJ_GRPO_FLAG_SKIP_MASKED (tokens without a gradient left out of "
                         "the backward products); off by default: the headline executes all 6*N*H*V flop")
    ap.add_argument("--no-extras", "--no-skip-masked-extra", dest="no_extras", action="store_true",
                    help="do not add the two short side timings to the JSON line: the skip-masked step and the "
                         "step in 8192-token chunks")
    ap.add_argument("--no-vendor-gemm", action="store_true",
                    help="skip timing the three bare bf16 products with the vendor GEMM (torch.matmul = hipBLASLt)")
    ap.add_argument("--copy-calibration-mib", type=int, default=0,
                    help="also run one plain device copy of this many MiB (a kernel of known traffic, to scale "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs the loss path on ONE GPU (no collectives, no sharding); "
              "run it with --gpus 1", file=sys.stderr)
        return 2

    import torch

    import mllm_jax_amd as M
    from mllm_jax_amd import _lib

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible; the fused loss has no CPU path", file=sys.stderr)
        return 3
    dev = torch.device("cuda:0")
    blib = BenchLib(_lib.load())
    if args.mfma_probe:
        from bench_probes import mfma_probe
        print(json.dumps(mfma_probe(torch, blib, dev)), flush=True)
        return 0
    cfg = M.CONFIGS[args.config]
    kw = dict(epsilon_low=cfg.eps_low, epsilon_high=cfg.eps_high, final_logit_softcap=cfg.softcap,
              chunk_tokens=args.chunk_tokens or None, dhidden_splits=args.dhidden_splits)
    step_kw = dict(entropy_coef=args.entropy_coef) if args.entropy_coef else {}
    if args.dw_dtype == "bf16":
        step_kw["lm_head_grad_dtype"] = torch.bfloat16

    def logp_fn(wl):
        with torch.no_grad():
            out = M.grpo_fused_loss(wl["hidden"], wl["lm_head"], wl["target_ids"], None, wl["advantages"],
                                    wl["mask"], total_valid_token_count=wl["total_valid_token_count"], **kw)
        return out["per_token_logps"]

    # configs[1] and [3] draw their targets from the model's own softmax
    wl = M.make_workload(cfg, dev, 20250 + args.config, logp_fn=logp_fn, sample_fn=M.gumbel_max_targets)
    n, h, v = cfg.tokens, cfg.hidden, cfg.vocab
    if args.pad_w:
        wide = torch.zeros(h, v + args.pad_w, dtype=torch.bfloat16, device=dev)
        wide[:, :v] = wl["lm_head"]
        wl["lm_head"] = wide[:, :v]

    def step(skip_masked=args.skip_masked):
        return M.grpo_loss_value_and_grad(
            wl["hidden"], wl["lm_head"], wl["target_ids"], wl["old_logps"], wl["advantages"], wl["mask"],
            total_valid_token_count=wl["total_valid_token_count"], seq_shape=wl["seq_shape"],
            return_token_entropy=cfg.token_entropy, skip_masked=skip_masked, **step_kw, **kw)

    if args.neighbours:
        from bench_probes import neighbours
        print(json.dumps(neighbours(torch, M, _lib, cfg, wl, dev)), flush=True)
        return 0
    if args.zero_operands:
        wl["hidden"].zero_()
        wl["lm_head"].zero_()
    if args.copy_calibration_mib:
        src = torch.empty(args.copy_calibration_mib << 20, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    if 64 * args.steps > 60000:          # more event pairs than the library's profiler takes (65536)
        args.no_kernel_events = True
    eager_step = step
    if args.graph:
        # the library's calls record into a capturing stream as they are (no allocation, no host
        # synchronisation; the first calls above ran outside the capture)
        args.no_kernel_events = True
        # warm-up and capture run on the same side stream; inside the capture the workspace is a fresh
        # allocation from the graph's own pool (the host API never caches a captured buffer)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                eager_step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            captured = eager_step()

        def step():
            graph.replay()
            return captured
        for _ in range(2):
            step()
        torch.cuda.synchronize()
    if not args.no_kernel_events:
        blib.profile_begin(64 * max(args.steps, 1))
    sampler = None
    if args.smi:
        from bench_probes import SmiSampler
        sampler = SmiSampler()
    if sampler:
        sampler.__enter__()
        time.sleep(1.0)                 # a few idle samples first
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        metrics, grads = step()
    torch.cuda.synchronize()
    t_end = time.perf_counter()
    dt = t_end - t0
    if sampler:
        sampler.__exit__()
    prof_steps = args.steps
    if args.no_kernel_events:
        prof_steps = min(args.steps, 5)
        blib.profile_begin(64 * prof_steps)
        for _ in range(prof_steps):
            eager_step()
        torch.cuda.synchronize()
    prof = blib.profile_end()

    ms_per_step = dt / args.steps * 1e3
    tokens_per_s = n * args.steps / dt
    flop_step = 6.0 * n * h * v
    mfu = flop_step / (ms_per_step * 1e-3) / (PEAK_BF16_TFLOPS * 1e12)

    gemms = {k: prof[k] for k in ("k_logits_stats", "k_dhidden", "k_dw")}
    dom = max(gemms, key=lambda k: gemms[k][0])
    dom_ms, dom_launches = gemms[dom]
    flop_per_launch = 2.0 * n * h * v * prof_steps / max(dom_launches, 1)   # algorithmic 2*n_chunk*H*V
    avg_launch_ms = dom_ms / max(dom_launches, 1)
    achieved = flop_per_launch / (avg_launch_ms * 1e-3) / 1e12
    roofline = {"bound": "mfma", "kernel": dom, "achieved": round(achieved, 1), "peak": PEAK_BF16_TFLOPS,
                "unit": "TFLOP/s", "frac": round(achieved / PEAK_BF16_TFLOPS, 4),
                "avg_launch_ms": round(avg_launch_ms, 3), "launches": dom_launches,
                "flop_per_launch": flop_per_launch,
                "traffic": None if args.chunk_tokens else MEASURED_TRAFFIC_BYTES.get((args.config, dom)),
                "traffic_source": None if args.chunk_tokens or args.config not in TRAFFIC_SOURCE else
                "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this bench at this config, summary in "
                + TRAFFIC_SOURCE[args.config] + " (not re-measured in this run)"}

    line = {
        "metric": "grpo_fused_loss_fwd_bwd_tokens_per_s", "value": round(tokens_per_s, 1), "unit": "tokens/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 3),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "bf16",
        "data": "synthetic",
        "config": {"workload": f"BASELINE configs[{args.config}] {cfg.name}: fused GRPO loss fwd+bwd, "
                               f"{n} tokens x hidden {h} x vocab {v}", "tokens": n, "hidden": h, "vocab": v,
                   "chunk_tokens": args.chunk_tokens or min(16384, n), "softcap": cfg.softcap,
                   "ld_w": v + args.pad_w, "dhidden_splits": args.dhidden_splits or "auto", "dw_dtype": args.dw_dtype,
                   "eps": [cfg.eps_low, cfg.eps_high]},
        "pct_bf16_mfma_peak": round(100.0 * mfu, 2),
        "algorithmic_tflops": round(flop_step / (ms_per_step * 1e-3) / 1e12, 1),
        "loss": float(metrics["loss"].item()),
        "roofline": roofline,
        "kernel_ms_per_step": {k: round(v_[0] / prof_steps, 3) for k, v_ in prof.items()},
    }

    if sampler:
        line["smi"] = sampler.summary(t0, t_end)
    if args.zero_operands:
        line["config"]["operands"] = "all-zero hidden and lm_head"
    if args.no_kernel_events:
        line["config"]["kernel_events"] = "separate loop of %d steps after the timed one" % prof_steps
    if args.entropy_coef:
        line["config"]["entropy_coef"] = args.entropy_coef
    if args.graph:
        line["config"]["launch"] = "replays of one HIP graph of the step"
    line["config"]["skip_masked"] = bool(args.skip_masked)
    if not args.skip_masked and not args.no_extras:
        # Not the headline: the same step with tokens that cannot carry a gradient (mask 0, advantage 0)
        # left out of the backward products.  Same outputs; fewer than 6*N*H*V flop executed.
        for _ in range(2):
            eager_step(True)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(5):
            eager_step(True)
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t1) / 5 * 1e3
        live = float(((wl["mask"] != 0) & (wl["advantages"].reshape(wl["mask"].shape) != 0)).float().mean().item())
        line["skip_masked_extra"] = {"ms_per_step": round(ms, 3), "tokens_per_s": round(n / ms * 1e3, 1),
                                     "live_token_fraction": round(live, 4),
                                     "note": "MJ_GRPO_FLAG_SKIP_MASKED; executes 2NHV + 4*live*NHV flop"}

    if not args.no_extras and not args.chunk_tokens and n > 8192:
        # Not the headline either: the same dense step with the 16-bit matrix E held for 8192 tokens at a
        # time (the default holds min(N, 16384) tokens' rows), i.e. with the workspace at half the size.
        ckw = dict(kw, chunk_tokens=8192)

        def chunked_step():
            return M.grpo_loss_value_and_grad(
                wl["hidden"], wl["lm_head"], wl["target_ids"], wl["old_logps"], wl["advantages"], wl["mask"],
                total_valid_token_count=wl["total_valid_token_count"], seq_shape=wl["seq_shape"],
                return_token_entropy=cfg.token_entropy, **step_kw, **ckw)
        for _ in range(2):
            chunked_step()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(5):
            chunked_step()
        torch.cuda.synchronize()
        ms = (time.perf_counter() - t1) / 5 * 1e3
        line["chunked_extra"] = {"chunk_tokens": 8192, "ms_per_step": round(ms, 3), "tokens_per_s": round(n / ms * 1e3, 1),
                                 "pct_bf16_mfma_peak": round(100.0 * flop_step / (ms * 1e-3) / (PEAK_BF16_TFLOPS * 1e12), 2),
                                 "note": "the matrix E = exp(z) of 8192 tokens at a time: two launches of each product "
                                         "at this shape, the second d_lm_head launch adds to the first"}

    if not args.no_vendor_gemm:
        # Context for the roofline fraction: what the vendor's tuned GEMM reaches on this very
        # GPU for the three bare products (no softmax statistics, no loss, bf16 outputs).
        del metrics, grads
        M.release_workspaces()
        torch.cuda.empty_cache()
        from bench_probes import vendor_gemm
        line["vendor_gemm"] = vendor_gemm(torch, wl["hidden"], wl["lm_head"], wl["mask"], n, h, v)

    if not args.no_cpu_baseline:
        from oracle.cpu_baseline import time_cpu_baseline
        cpu_wl = {k: (t.cpu() if hasattr(t, "cpu") else t) for k, t in wl.items()}
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1)))
        res = time_cpu_baseline(cpu_wl, min(args.cpu_sample_tokens, n), repeats=1, threads=cores)
        line["cpu_baseline"] = {
            "value": round(res["tokens_per_s"], 2), "unit": "tokens/s", "cores": res["cores"], "kind": "port",
            "sample": f"first {res['sample_tokens']} tokens of the same batch at full hidden/vocab, un-fused "
                      f"float32 torch-CPU fwd+bwd, {res['seconds']:.1f} s (JAX is not installed)"}
    print(json.dumps(line), flush=True)
    return 0


if __name__ == "__main__":
    sys.exit(main())
