"""Side measurements of bench.py (none of them is the benchmark's `value`): the vendor GEMM on the
three bare products, amd-smi power / clock sampling, the MFMA-only probe loop, and the steps
either side of the loss (RMSNorm, sampler, value head, group advantages).  bench.py imports what
a flag asks for."""
from __future__ import annotations

import json
import time

PEAK_BF16_TFLOPS = 2500.0      # MI355X dense bf16 MFMA, published


def vendor_gemm(torch, hidden, w, mask, n, h, v, reps=5):
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


class SmiSampler:
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


def mfma_probe(torch, blib, dev):
    """What the matrix cores sustain under the power cap with no memory traffic: the bench library's
    MFMA-only loop with random and with all-zero bf16 operands, for both instruction shapes."""
    out = torch.empty(1024 * 256, dtype=torch.float32, device=dev)
    st = torch.cuda.current_stream().cuda_stream
    res = {"metric": "mfma_only_bf16_tflops", "unit": "TFLOP/s", "peak": PEAK_BF16_TFLOPS,
           "kernel": "k_probe_mfma: 1024 workgroups x 4 wavefronts x 256 accumulators (4x4 blocks of "
                     "v_mfma_f32_32x32x16_bf16, or 8x8 blocks of v_mfma_f32_16x16x32_bf16), operands in registers, "
                     "two operand sets alternating; 'chained': the two k-steps of a block back to back on "
                     "its accumulator (the order of the GemmTN16 engine), otherwise the accumulators in rotation"}
    for shape, sname in ((0, "32x32x16"), (1, "16x16x32"), (2, "16x16x32_chained")):
        for name in ("random", "zero"):
            ops = torch.randn(512 * 1024, device=dev).to(torch.bfloat16) if name == "random" \
                else torch.zeros(512 * 1024, dtype=torch.bfloat16, device=dev)
            iters = 20000 if shape == 0 else 10000          # the same flop per launch for both shapes
            launch = lambda: blib.probe_mfma(ops.data_ptr(), out.data_ptr(), 1024, iters, shape, st)
            flop = launch()
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            with SmiSampler() as smi:
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
            res[f"{sname}_{name}"] = {"ms_per_launch": round(ms, 3), "tflops": round(flop / ms / 1e9, 1),
                                      "frac_of_peak": round(flop / ms / 1e9 / PEAK_BF16_TFLOPS, 4),
                                      "smi": smi.summary(t0, t1)}
    return res


def neighbours(torch, M, _lib, cfg, wl, dev, iters=20) -> dict:
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
