"""CPU build of the host-side index arithmetic of the tile kernels under the address and
undefined-behaviour sanitizers (no HIP, no GPU): tests/host_plan_check.cpp includes
csrc/tile_map.hpp and csrc/plan.hpp as plain C++ and checks that every (tile row, tile column,
k-split) of a sweep of problems is produced exactly once over the launch's ids, that workspace
regions never overlap and end inside the reported totals, that the vocab splits cover the
vocabulary, and what the workspace-free entry point's chunk search returns.  An indexing mistake in
this code would be an out-of-bounds access on the GPU; it is found here instead."""
import os
import shutil
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_tile_map_and_plan_under_sanitizers(tmp_path):
    gxx = shutil.which("g++")
    if gxx is None:
        pytest.skip("g++ not available")
    exe = tmp_path / "host_plan_check"
    cmd = [gxx, "-std=c++17", "-O1", "-g", "-fsanitize=address,undefined", "-fno-sanitize-recover=all", "-Wall",
           "-Wextra", "-Werror", os.path.join(ROOT, "tests", "host_plan_check.cpp"), "-o", str(exe)]
    res = subprocess.run(cmd, capture_output=True, text=True)
    assert res.returncode == 0, res.stderr
    env = dict(os.environ)
    env.pop("LD_PRELOAD", None)        # the sanitizer runtime must come first in the library list
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=600, env=env)
    assert run.returncode == 0, run.stdout + run.stderr
    assert run.stdout.startswith("ok ") and int(run.stdout.split()[1]) > 1_000_000


def test_plan_headers_do_not_need_hip():
    """The two headers the check includes must stay plain C++: no HIP header, no device code."""
    for name in ("tile_map.hpp", "plan.hpp"):
        text = open(os.path.join(ROOT, "mllm-jax_amd", "csrc", name)).read()
        assert "hip_runtime" not in text and "__global__" not in text and "threadIdx" not in text
