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
MEASURED_TRAFFIC_BYTES = {          # default chunk (16384 tokens: one launch of each kernel per step)
    (2, "k_logits_stats"): 31.38e9,
    (2, "k_dhidden"): 34.44e9,
    (2, "k_dw"): 37.51e9,
}


def _vendor_gemm(torch, hidden, w, mask, n, h, v, reps=5):
    dev = hidden.device
    out = {}
    # a stand-in dZ with the zero rows the real one has (tokens outside the loss): MFMA throughput on
    # this GPU depends on the operand data (zeros draw less power), so the comparison keeps the pattern
    dz = torch.empty(n, v, dtype=torch.bfloat16, device=dev).normal_(0, 0.01)
    dz.mul_(mask.reshape(n, 1).to(torch.bfloat16))
    cases = {"logits": (lambda o: torch.matmul(hidden, w, out=o), (n, v)),
             "dhidden": (lambda o: torch.matmul(dz, w.t(), out=o), (n, h)),
             "dw": (lambda o: torch.matmul(hidden.t(), dz, out=o), (h, v))}
    total = 0.0
    for name, (fn, shape) in cases.items():
        o = torch.empty(shape, dtype=torch.bfloat16, device=dev)
        for _ in range(2):
            fn(o)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn(o)
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        total += ms
        out[name] = {"ms": round(ms, 3), "tflops": round(2.0 * n * h * v / ms / 1e9, 1)}
        del o
    out["sum_ms"] = round(total, 3)
    out["note"] = ("torch.matmul (hipBLASLt) bf16 in, bf16 out, same shapes, same GPU, dZ with the same zero rows; "
                   "products only")
    return out


class _SmiSampler:
    """Polls `amd-smi metric -p -c -t --json` in a thread while the timed loop runs (socket power, the
    shader clock of every XCD and the hotspot temperature as the driver reports them); the GPU work is
    not touched."""

    def __init__(self, period_s=0.15):
        import threading
        self.period, self.samples, self._stop = period_s, [], threading.Event()
        self._thread = threading.Thread(target=self._run, daemon=True)

    @staticmethod
    def _num(x):
        if isinstance(x, dict):
            x = x.get("value")
        return float(x) if isinstance(x, (int, float)) else None

    def _run(self):
        import subprocess
        while not self._stop.is_set():
            try:
                out = subprocess.run(["amd-smi", "metric", "-p", "-c", "-t", "--json"], capture_output=True,
                                     text=True, timeout=10).stdout
                doc = json.loads(out)
                gpu = (doc.get("gpu_data") if isinstance(doc, dict) else doc)[0]
                rec = {}
                pw = self._num(gpu.get("power", {}).get("socket_power"))
                if pw is not None:
                    rec["power_w"] = pw
                clks = [self._num(v.get("clk")) for k, v in gpu.get("clock", {}).items()
                        if k.startswith("gfx_") and isinstance(v, dict)]
                clks = [c for c in clks if c is not None]
                if clks:
                    rec["sclk_mhz"] = round(sum(clks) / len(clks), 1)
                temp = gpu.get("temperature", {})
                hot = self._num(temp.get("hotspot")) if isinstance(temp, dict) else None
                if hot is not None:
                    rec["junction_c"] = hot
                if rec:
                    rec["t"] = round(time.perf_counter(), 3)
                    self.samples.append(rec)
            except Exception as e:      # the sampler must never break the benchmark
                self.samples.append({"error": repr(e)[:80]})
                break
            self._stop.wait(self.period)

    def __enter__(self):
        self._thread.start()
        return self

    def __exit__(self, *exc):
        self._stop.set()
        self._thread.join(timeout=15)

    def summary(self, t0, t1):
        inside = [r for r in self.samples if "t" in r and t0 + 0.3 <= r["t"] <= t1]
        out = {"samples_in_timed_loop": len(inside), "samples_total": len(self.samples)}
        for key in ("power_w", "sclk_mhz", "junction_c"):
            vals = sorted(r[key] for r in inside if key in r)
            if vals:
                out[key] = {"min": vals[0], "median": vals[len(vals) // 2], "max": vals[-1]}
        idle = [r for r in self.samples if "t" in r and r["t"] < t0 - 0.05]
        if idle and "power_w" in idle[0]:
            out["before_loop"] = {k: idle[-1].get(k) for k in ("power_w", "sclk_mhz", "junction_c")}
        errs = [r["error"] for r in self.samples if "error" in r]
        if errs:
            out["error"] = errs[0]
        return out


def _mfma_probe(torch, _lib, dev):
    import ctypes as C
    lib = _lib.load()
    out = torch.empty(1024 * 256, dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    res = {"metric": "mfma_only_bf16_tflops", "unit": "TFLOP/s", "peak": PEAK_BF16_TFLOPS,
           "kernel": "k_probe_mfma: 1024 workgroups x 4 wavefronts x (4x4 blocks of v_mfma_f32_32x32x16_bf16), "
                     "operands in registers, two operand sets alternating"}
    for name in ("random", "zero"):
        ops = torch.randn(512 * 1024, device=dev).to(torch.bfloat16) if name == "random" \
            else torch.zeros(512 * 1024, dtype=torch.bfloat16, device=dev)
        flop = C.c_double(0.0)
        launch = lambda: _lib.check(lib.mj_grpo_probe_mfma(ops.data_ptr(), out.data_ptr(), 1024, 20000, C.byref(flop), st))
        launch()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        with _SmiSampler() as smi:
            time.sleep(0.6)
            t0 = time.perf_counter()
            e0.record()
            reps = 60                      # ~50 ms per launch: about 3 s of sustained MFMA work
            for _ in range(reps):
                launch()
            e1.record()
            torch.cuda.synchronize()
            t1 = time.perf_counter()
        ms = e0.elapsed_time(e1) / reps
        res[name] = {"ms_per_launch": round(ms, 3), "tflops": round(flop.value / ms / 1e9, 1),
                     "frac_of_peak": round(flop.value / ms / 1e9 / PEAK_BF16_TFLOPS, 4), "smi": smi.summary(t0, t1)}
    return res


def _neighbours(torch, M, _lib, cfg, wl, dev, iters=20) -> dict:
    """The steps either side of the loss at this config's shape, each called through the C ABI and
    timed with events on the stream it is launched on: final RMSNorm forward / backward
    (llama/llama.py:426-452), the sampler's last-position logits and top-k draw
    (sample_state_right_padding2.py:229-230, sanple_utils.py:35-53), the critic's value head
    (plugins/training/ppo/module.py:34-52) and group advantages (advantage/grpo.py:28-52).  All but
    the last are bound by HBM; `bytes` is the algorithmic traffic of one call."""
    lib = _lib.load()
    st = torch.cuda.current_stream(dev).cuda_stream
    n, h, v = cfg.tokens, cfg.hidden, cfg.vocab
    b_seq = wl["seq_shape"][0]
    x, w = wl["hidden"], wl["lm_head"]
    f32 = dict(dtype=torch.float32, device=dev)
    scale = torch.ones(h, **f32)
    y, dx = torch.empty_like(x), torch.empty_like(x)
    rstd, dscale = torch.empty(n, **f32), torch.empty(h, **f32)
    need = _lib.C.c_size_t(0)
    _lib.check(lib.mj_rmsnorm_workspace_bytes(n, h, _lib.C.byref(need)))
    nws = torch.empty(max(need.value, 16), dtype=torch.uint8, device=dev)
    last = x[:: n // b_seq][:b_seq].contiguous()
    logits = torch.empty((b_seq, v), **f32)
    noise = torch.zeros((b_seq, 50), **f32)
    token = torch.empty(b_seq, dtype=torch.int32, device=dev)
    wv, bv, values = torch.full((h,), 0.01, **f32), torch.zeros(1, **f32), torch.empty(n, **f32)
    rewards = torch.rand(b_seq, **f32)
    gid = (torch.arange(b_seq, device=dev) // max(cfg.group, 1)).to(torch.int32)
    adv = torch.empty(b_seq, **f32)
    calls = {
        "rmsnorm_forward": (lambda: lib.mj_rmsnorm_forward(x.data_ptr(), x.stride(0), scale.data_ptr(), y.data_ptr(), h,
                                                          rstd.data_ptr(), n, h, 1e-6, st), 2 * n * h * 2 + n * 4),
        "rmsnorm_backward": (lambda: lib.mj_rmsnorm_backward(y.data_ptr(), h, x.data_ptr(), x.stride(0), scale.data_ptr(),
                                                            dx.data_ptr(), h, dscale.data_ptr(), 0, n, h, 1e-6,
                                                            nws.data_ptr(), nws.numel(), st), 3 * n * h * 2),
        "sample_logits": (lambda: lib.mj_sample_logits(last.data_ptr(), h, w.data_ptr(), w.stride(0), logits.data_ptr(), v,
                                                      b_seq, h, v, float(cfg.softcap or 0.0), st),
                          h * v * 2 + b_seq * h * 2 + b_seq * v * 4),
        "sample_top_k": (lambda: lib.mj_sample_top_k(logits.data_ptr(), v, b_seq, v, 50, 1.0, noise.data_ptr(),
                                                    token.data_ptr(), None, None, st), b_seq * v * 4),
        "value_head_forward": (lambda: lib.mj_value_head_forward(x.data_ptr(), x.stride(0), wv.data_ptr(), bv.data_ptr(),
                                                                values.data_ptr(), n, h, st), n * h * 2 + n * 4),
        "group_advantages": (lambda: lib.mj_grpo_group_advantages(rewards.data_ptr(), gid.data_ptr(), adv.data_ptr(), b_seq,
                                                                 1e-4, st), b_seq * 12),
    }
    def vendor_product():       # the same product through torch.matmul (hipBLASLt), bf16 result: a yardstick only
        torch.matmul(last, w)
        return 0
    calls["vendor_matmul_for_sample_logits"] = (vendor_product, h * v * 2 + b_seq * h * 2 + b_seq * v * 2)
    # what plain streaming reaches on this GPU beyond the 256 MB Infinity Cache: the value head (read
    # only) and the RMSNorm forward (read + write) on a 1.07 GB matrix, and torch's own sum and copy
    # over 1 GiB -- yardsticks for the fractions of the nominal 8 TB/s above
    bn_, bh_ = 131072, 4096
    bigx = torch.empty((bn_, bh_), dtype=torch.bfloat16, device=dev).normal_()
    bigy = torch.empty_like(bigx)
    bigw, bigs, bigv = torch.full((bh_,), 0.01, **f32), torch.ones(bh_, **f32), torch.empty(bn_, **f32)
    calls["stream_read_1GB_value_head_yardstick"] = (
        lambda: lib.mj_value_head_forward(bigx.data_ptr(), bh_, bigw.data_ptr(), bv.data_ptr(), bigv.data_ptr(), bn_, bh_, st),
        bn_ * bh_ * 2)
    calls["stream_read_write_1GB_rmsnorm_yardstick"] = (
        lambda: lib.mj_rmsnorm_forward(bigx.data_ptr(), bh_, bigs.data_ptr(), bigy.data_ptr(), bh_, None, bn_, bh_, 1e-6, st),
        2 * bn_ * bh_ * 2)
    bigf = bigx.view(torch.float32)

    def torch_read():
        torch.sum(bigf)
        return 0

    def torch_copy():
        bigy.copy_(bigx)
        return 0
    calls["torch_sum_1GB_read_yardstick"] = (torch_read, bn_ * bh_ * 2)
    calls["torch_copy_1GB_read_plus_write_yardstick"] = (torch_copy, 2 * bn_ * bh_ * 2)
    rows = {}
    for name, (fn, nbytes) in calls.items():
        for _ in range(3):
            _lib.check(fn())
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record()
        for _ in range(iters):
            _lib.check(fn())
        e1.record()
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / iters
        gbs = nbytes / (ms * 1e-3) / 1e9
        rows[name] = {"ms": round(ms, 4), "bytes": nbytes, "GB_per_s": round(gbs, 1), "frac_of_hbm_peak": round(gbs / 8000.0, 4)}
    return {"metric": "neighbour_steps", "config": {"workload": f"BASELINE configs shape {n} tokens x hidden {h} x vocab {v}",
                                                    "sequences": b_seq}, "iters": iters,
            "hbm_peak_GB_per_s": 8000.0, "rows": rows}


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
    ap.add_argument("--no-skip-masked-extra", action="store_true",
                    help="do not add the short skip-masked timing to the JSON line")
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
    if args.mfma_probe:
        print(json.dumps(_mfma_probe(torch, _lib, dev)), flush=True)
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

    wl = M.make_workload(cfg, dev, 20250 + args.config, logp_fn=logp_fn)
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
        print(json.dumps(_neighbours(torch, M, _lib, cfg, wl, dev)), flush=True)
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
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(2):
                eager_step()
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            captured = eager_step()

        def step():
            graph.replay()
            return captured
        for _ in range(2):
            step()
        torch.cuda.synchronize()
    if not args.no_kernel_events:
        _lib.profile_begin(64 * max(args.steps, 1))
    sampler = _SmiSampler() if args.smi else None
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
        _lib.profile_begin(64 * prof_steps)
        for _ in range(prof_steps):
            eager_step()
        torch.cuda.synchronize()
    prof = _lib.profile_end()

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
                "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this bench, summary in "
                                  "profiles/cfg2_qwen7b_fused_fwd_bwd.txt (not re-measured in this run)"}

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
    if not args.skip_masked and not args.no_skip_masked_extra:
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

    if not args.no_vendor_gemm:
        # Context for the roofline fraction: what the vendor's tuned GEMM reaches on this very
        # GPU for the three bare products (no softmax statistics, no loss, bf16 outputs).
        del metrics, grads
        M.release_workspaces()
        torch.cuda.empty_cache()
        line["vendor_gemm"] = _vendor_gemm(torch, wl["hidden"], wl["lm_head"], wl["mask"], n, h, v)

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
