"""CPU-side checks of the C ABI: the library loads, exports every symbol that
include/mj_grpo.h declares, and rejects bad descriptors / pointers with a status and a
message before touching any device (no compute call is made here)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from mllm_jax_amd import _lib, build
    if not os.path.exists(_lib.LIB_PATH) or not os.path.exists(build.BENCH_LIB):
        build.build(verbose=False)
    return _lib


def _desc(lib, **kw):
    d = lib.MjGrpoDesc()
    d.n_tokens, d.hidden, d.vocab, d.ld_hidden, d.ld_w = 64, 64, 512, 64, 512
    d.temperature, d.inv_total_valid_tokens, d.grad_loss_scale = 1.0, 1.0 / 64, 1.0
    d.eps_low, d.eps_high = 0.2, 0.3
    for k, v in kw.items():
        setattr(d, k, v)
    return d


def test_header_symbols_are_exported(lib):
    header = open(os.path.join(ROOT, "include", "mj_grpo.h")).read() + open(os.path.join(ROOT, "include", "mj_norm.h")).read() \
        + open(os.path.join(ROOT, "include", "mj_sample.h")).read()
    declared = set(re.findall(r"\b(mj_(?:grpo|rmsnorm|sample|value)_[a-z_]+)\s*\(", header))
    assert declared == set(lib.EXPORTS)
    handle = lib.load()
    for name in declared:
        assert hasattr(handle, name)
    assert handle.mj_grpo_version() >= 100


def test_bench_library_exports_its_header_and_the_product_does_not(lib):
    """Measurement support (event timing behind the launch-trace hook, the MFMA-only probe) lives in
    libmj_grpo_bench.so / include/mj_grpo_bench.h; the product library exports none of it."""
    header = open(os.path.join(ROOT, "include", "mj_grpo_bench.h")).read()
    declared = set(re.findall(r"\b(mj_bench_[a-z_]+)\s*\(", header))
    assert declared == {"mj_bench_profile_begin", "mj_bench_profile_end", "mj_bench_trace", "mj_bench_probe_mfma",
                        "mj_bench_last_error"}
    bench = C.CDLL(os.path.join(os.path.dirname(lib.LIB_PATH), "libmj_grpo_bench.so"))
    product = lib.load()
    for name in declared:
        assert hasattr(bench, name)
        assert not hasattr(product, name)
    for name in ("mj_grpo_profile_begin", "mj_grpo_profile_end", "mj_grpo_probe_mfma"):
        assert not hasattr(product, name)
    # switching the trace hook on and off needs no device
    assert product.mj_grpo_set_trace(C.cast(bench.mj_bench_trace, C.c_void_p), None) == 0
    assert product.mj_grpo_set_trace(None, None) == 0


def test_desc_layout_matches_header(lib):
    # 6 x int64 + 6 x float + 2 x uint32 + 2 x float
    assert C.sizeof(lib.MjGrpoDesc) == 6 * 8 + 6 * 4 + 2 * 4 + 2 * 4


def test_workspace_sizes_scale_with_chunk(lib):
    big = _desc(lib, n_tokens=16384, hidden=3584, vocab=152064, ld_hidden=3584, ld_w=152064)
    f, b = lib.workspace_bytes(big)
    small = _desc(lib, n_tokens=16384, hidden=3584, vocab=152064, ld_hidden=3584, ld_w=152064, chunk_tokens=2048)
    f2, b2 = lib.workspace_bytes(small)
    assert f2 < f and b2 < b
    # the workspace never holds N x V logits: two 16-bit chunk buffers + transposed operands
    assert b2 < 16384 * 152064 * 2


@pytest.mark.parametrize("kw,code", [
    (dict(n_tokens=0), 2), (dict(vocab=-8), 2), (dict(ld_w=256), 2),
    (dict(vocab=508, ld_w=508), 3), (dict(hidden=60, ld_hidden=60), 3), (dict(ld_hidden=68), 3),
    (dict(temperature=0.0), 5), (dict(temperature=0.7, entropy_coef=0.1, inv_entropy_count=0.1), 5), (dict(softcap=-1.0), 5), (dict(chunk_tokens=-5), 2),
    (dict(inv_total_valid_tokens=float("inf")), 2),
    (dict(entropy_coef=float("nan")), 2), (dict(inv_entropy_count=-1.0), 2), (dict(flags=1 << 7), 5),
    (dict(vocab=1 << 22, ld_w=1 << 22), 2), (dict(chunk_tokens=1 << 21), 2),
])
def test_bad_descriptors(lib, kw, code):
    with pytest.raises(lib.MjGrpoError) as e:
        lib.workspace_bytes(_desc(lib, **kw))
    assert e.value.code == code and len(str(e.value)) > 20


def test_every_documented_flag_is_accepted(lib):
    assert (lib.FLAG_DW_ACCUMULATE, lib.FLAG_SFT, lib.FLAG_SKIP_MASKED, lib.FLAG_DW_BF16) == (1, 2, 4, 8)
    base = lib.workspace_bytes(_desc(lib))
    for flags in (lib.FLAG_DW_ACCUMULATE, lib.FLAG_SFT, lib.FLAG_DW_BF16, lib.FLAG_DW_ACCUMULATE | lib.FLAG_DW_BF16):
        assert lib.workspace_bytes(_desc(lib, flags=flags)) == base      # none of these needs workspace
    assert lib.workspace_bytes(_desc(lib, flags=lib.FLAG_SKIP_MASKED | lib.FLAG_DW_BF16))[1] > base[1]


def test_null_and_workspace_errors_before_any_launch(lib):
    h = lib.load()
    d = _desc(lib)
    fake = 0x1000   # never dereferenced: argument checks fail first
    st = h.mj_grpo_forward(C.byref(d), None, fake, fake, None, fake, fake, fake, fake, None, fake, fake, 1 << 30, None)
    assert st == 1 and b"NULL" in h.mj_grpo_last_error()
    st = h.mj_grpo_forward(C.byref(d), fake, fake, fake, None, fake, fake, fake, fake, None, fake, None, 0, None)
    assert st == 4
    st = h.mj_grpo_forward(C.byref(d), fake, fake, fake, None, fake, fake, fake, fake, None, fake, fake, 16, None)
    assert st == 4 and b"too small" in h.mj_grpo_last_error()
    st = h.mj_grpo_forward(C.byref(d), fake + 2, fake, fake, None, fake, fake, fake, fake, None, fake, fake, 1 << 30, None)
    assert st == 3
    st = h.mj_grpo_forward_backward(C.byref(d), fake, fake, fake, None, fake, fake, fake, fake, None, fake, None,
                                    fake, fake, 1 << 30, None)
    assert st == 1
    st = h.mj_grpo_backward(C.byref(d), fake, fake, fake, None, fake, fake, None, fake, fake, fake, fake, 1 << 30, None)
    assert st == 1
    st = h.mj_grpo_forward(None, fake, fake, fake, None, fake, fake, fake, fake, None, fake, fake, 1 << 30, None)
    assert st == 1


def test_host_api_refuses_cpu_tensors(lib):
    import torch
    import mllm_jax_amd as M
    with pytest.raises(RuntimeError, match="no CPU path"):
        M.grpo_fused_loss(torch.zeros(8, 8, dtype=torch.bfloat16), torch.zeros(8, 16, dtype=torch.bfloat16),
                          torch.zeros(8, dtype=torch.long), None, torch.zeros(8), torch.ones(8))


def test_workload_generator_shapes_and_advantages():
    import numpy as np
    import torch
    from mllm_jax_amd import CONFIGS, make_workload
    from mllm_jax_amd.workloads import group_advantages
    from oracle.grpo_oracle import grpo_advantages
    r = torch.tensor([1.0, 0, 0, 1, 1, 1, 0, 0])
    np.testing.assert_allclose(group_advantages(r, 4).numpy(), grpo_advantages(r.numpy(), [0] * 4 + [1] * 4), rtol=1e-6)
    assert [c.tokens for c in CONFIGS] == [512, 4096, 16384, 32768, 16384]
    import dataclasses
    tiny = dataclasses.replace(CONFIGS[0], hidden=16, vocab=64)
    wl = make_workload(tiny, "cpu", 1)
    assert wl["hidden"].shape == (512, 16) and wl["lm_head"].shape == (16, 64)
    assert wl["advantages"].abs().max() > 0 and wl["total_valid_token_count"] == wl["mask"].sum().item()


def test_rmsnorm_argument_checks_before_any_launch(lib):
    h = lib.load()
    fake = 0x1000   # never dereferenced: argument checks fail first
    sz = C.c_size_t()
    assert h.mj_rmsnorm_workspace_bytes(4096, 3584, C.byref(sz)) == 0 and sz.value == 1024 * 3584 * 4
    assert h.mj_rmsnorm_workspace_bytes(10, 64, C.byref(sz)) == 0 and sz.value == 10 * 64 * 4     # one partial row per workgroup, one workgroup per row up to 1024
    assert h.mj_rmsnorm_workspace_bytes(0, 64, C.byref(sz)) == 2
    assert h.mj_rmsnorm_workspace_bytes(8, 60, C.byref(sz)) == 3
    assert h.mj_rmsnorm_workspace_bytes(8, 16384, C.byref(sz)) == 5 and b"8192" in h.mj_grpo_last_error()
    assert h.mj_rmsnorm_forward(None, 64, fake, fake, 64, None, 8, 64, 1e-6, None) == 1
    assert h.mj_rmsnorm_forward(fake, 56, fake, fake, 64, None, 8, 64, 1e-6, None) == 2      # ld < h
    assert h.mj_rmsnorm_forward(fake + 4, 64, fake, fake, 64, None, 8, 64, 1e-6, None) == 3  # alignment
    assert h.mj_rmsnorm_backward(fake, 64, fake, 64, fake, fake, 64, fake, 0, 8, 64, 1e-6, fake, 16, None) == 4
    assert b"workspace too small" in h.mj_grpo_last_error()


def test_sampler_argument_checks_before_any_launch(lib):
    h = lib.load()
    fake = 0x1000
    assert h.mj_sample_logits(None, 64, fake, 512, fake, 512, 4, 64, 512, 0.0, None) == 1
    assert h.mj_sample_logits(fake, 64, fake, 512, fake, 500, 4, 64, 512, 0.0, None) == 2
    assert h.mj_sample_logits(fake, 64, fake, 516, fake, 520, 4, 64, 516, 0.0, None) == 3
    assert h.mj_sample_logits(fake, 64, fake, 512, fake, 512, 4, 64, 512, -1.0, None) == 5
    assert h.mj_sample_top_k(fake, 512, 4, 512, 65, 1.0, None, fake, None, None, None) == 5
    assert h.mj_sample_top_k(fake, 512, 4, 40, 50, 1.0, None, fake, None, None, None) == 5      # k > vocab
    assert h.mj_sample_top_k(fake, 512, 4, 512, 50, 0.0, None, fake, None, None, None) == 5
    assert h.mj_sample_top_k(fake, 512, 4, 512, 50, 1.0, None, None, None, None, None) == 1


def test_skip_masked_flag_enlarges_the_workspace(lib):
    d = _desc(lib)
    fwd0, both0 = lib.workspace_bytes(d)
    d.flags = lib.FLAG_SKIP_MASKED
    fwd1, both1 = lib.workspace_bytes(d)
    n, h = d.n_tokens, d.hidden
    assert fwd1 >= fwd0 + n * h * 2 + n * 4 * 10          # slot-order hidden copy, permutation, per-token copies
    assert both1 - fwd1 >= both0 - fwd0 + n * h * 2       # slot-order d_hidden


def test_headers_are_plain_c_and_the_library_links_from_c(lib, tmp_path):
    """include/*.h must compile as C99 (no C++-isms, no torch types) and a C program must be able to
    call the library through them: version, a rejected descriptor, the error text."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("gcc not available")
    src = tmp_path / "abi.c"
    src.write_text(r'''
#include <stdio.h>
#include <string.h>
#include "mj_grpo.h"
#include "mj_norm.h"
#include "mj_sample.h"
#include "mj_grpo_bench.h"
int main(void) {
  MjGrpoDesc d;
  size_t fwd = 0, both = 0;
  memset(&d, 0, sizeof d);
  d.n_tokens = 64; d.hidden = 64; d.vocab = 500; d.ld_hidden = 64; d.ld_w = 500;   /* vocab not a multiple of 8 */
  d.temperature = 1.0f; d.inv_total_valid_tokens = 1.0f; d.grad_loss_scale = 1.0f;
  if (mj_grpo_version() < 100) return 1;
  if (mj_grpo_workspace_bytes(&d, &fwd, &both) != MJ_GRPO_ERR_ALIGN) return 2;
  if (strstr(mj_grpo_last_error(), "multiples of 8") == NULL) return 3;
  d.vocab = 512; d.ld_w = 512;
  if (mj_grpo_workspace_bytes(&d, &fwd, &both) != MJ_GRPO_OK || both <= fwd) return 4;
  if (mj_rmsnorm_workspace_bytes(8, 60, &fwd) != MJ_GRPO_ERR_ALIGN) return 5;
  if (mj_sample_top_k(NULL, 512, 4, 512, 50, 1.0f, NULL, NULL, NULL, NULL, NULL) != MJ_GRPO_ERR_NULL) return 6;
  printf("sizeof(MjGrpoDesc)=%zu\n", sizeof(MjGrpoDesc));
  return 0;
}
''')
    exe = tmp_path / "abi"
    libdir = os.path.dirname(lib.LIB_PATH)
    cmd = [gcc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe),
           "-L", libdir, "-l:libmj_grpo.so", "-Wl,-rpath," + libdir]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True)
    assert run.returncode == 0, (run.returncode, run.stdout, run.stderr)
    assert "sizeof(MjGrpoDesc)=88" in run.stdout


def test_grouped_advantage_estimators_cap_the_batch(lib):
    handle = lib.load()
    rc = handle.mj_grpo_advantages(0, 1, 1, 1, 8193, 1e-4, 0.0, 0, 0.0, None)   # pointers are never touched
    assert rc == 2 and b"8192" in handle.mj_grpo_last_error()
