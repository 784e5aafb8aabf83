"""ctypes binding of libmj_grpo.so (declarations: include/mj_grpo.h).

There is no CPU fallback: if the library is missing or a call fails, this raises.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libmj_grpo.so")

OK = 0
FLAG_DW_ACCUMULATE = 1 << 0
FLAG_SFT = 1 << 1
FLAG_SKIP_MASKED = 1 << 2
FLAG_DW_BF16 = 1 << 3

EXPORTS = ("mj_grpo_version", "mj_grpo_last_error", "mj_grpo_workspace_bytes", "mj_grpo_forward",
           "mj_grpo_forward_backward", "mj_grpo_backward", "mj_grpo_forward_noalloc", "mj_grpo_set_trace", "mj_grpo_forward_backward_value",
           "mj_grpo_value_workspace_bytes", "mj_value_head_forward", "mj_grpo_sequence_entropy", "mj_grpo_scale_gradients",
           "mj_grpo_group_advantages", "mj_grpo_advantages", "mj_grpo_gae", "mj_rmsnorm_forward", "mj_sample_logits", "mj_sample_top_k", "mj_rmsnorm_workspace_bytes", "mj_rmsnorm_backward")

KERNEL_NAMES = ("k_logits_stats", "k_finalize", "k_dz", "k_dhidden", "k_dhidden_reduce", "k_dw",
                "k_reduce_loss", "k_scale_hidden", "k_rescue")


class MjGrpoDesc(C.Structure):
    _fields_ = [
        ("n_tokens", C.c_int64), ("hidden", C.c_int64), ("vocab", C.c_int64),
        ("ld_hidden", C.c_int64), ("ld_w", C.c_int64), ("chunk_tokens", C.c_int64),
        ("eps_low", C.c_float), ("eps_high", C.c_float), ("temperature", C.c_float),
        ("softcap", C.c_float), ("inv_total_valid_tokens", C.c_float), ("grad_loss_scale", C.c_float),
        ("flags", C.c_uint32), ("dhidden_splits", C.c_uint32),
        ("entropy_coef", C.c_float), ("inv_entropy_count", C.c_float),
    ]


class MjPpoValue(C.Structure):
    _fields_ = [
        ("value_w", C.c_void_p), ("value_b", C.c_void_p), ("returns", C.c_void_p), ("old_values", C.c_void_p),
        ("value_coef", C.c_float), ("value_clip", C.c_float), ("use_clip", C.c_int32), ("reserved", C.c_int32),
        ("values", C.c_void_p), ("value_loss", C.c_void_p), ("d_value_w", C.c_void_p), ("d_value_b", C.c_void_p),
    ]


class MjGrpoError(RuntimeError):
    def __init__(self, code: int, message: str):
        super().__init__(f"mj_grpo status {code}: {message}")
        self.code = code


_lib = None


def load() -> C.CDLL:
    """Loads the built library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(f"{LIB_PATH} is missing: run `python -m mllm_jax_amd.build` (needs hipcc). "
                           "There is no CPU fallback for the fused GRPO loss.")
    lib = C.CDLL(LIB_PATH)
    vp, fp, ip, sz = C.c_void_p, C.c_void_p, C.c_void_p, C.c_size_t
    dp = C.POINTER(MjGrpoDesc)
    lib.mj_grpo_version.restype = C.c_int
    lib.mj_grpo_last_error.restype = C.c_char_p
    lib.mj_grpo_workspace_bytes.argtypes = [dp, C.POINTER(sz), C.POINTER(sz)]
    lib.mj_grpo_forward.argtypes = [dp, vp, vp, ip, fp, fp, fp, fp, fp, fp, fp, vp, sz, vp]
    lib.mj_grpo_forward_noalloc.argtypes = [dp, vp, vp, ip, fp, fp, fp, fp, fp, fp, fp, vp]
    lib.mj_grpo_set_trace.argtypes = [vp, vp]
    lib.mj_grpo_scale_gradients.argtypes = [vp, C.c_int64, C.c_int64, C.c_int64, vp, C.c_int64, C.c_int64, C.c_int64,
                                            C.c_int, fp, vp]
    lib.mj_grpo_forward_backward.argtypes = [dp, vp, vp, ip, fp, fp, fp, fp, fp, fp, fp, vp, fp, vp, sz, vp]
    lib.mj_grpo_forward_backward_value.argtypes = [dp, C.POINTER(MjPpoValue), vp, vp, ip, fp, fp, fp, fp, fp, fp, fp, vp, fp,
                                                   vp, sz, vp]
    lib.mj_grpo_value_workspace_bytes.argtypes = [dp, C.POINTER(sz)]
    lib.mj_value_head_forward.argtypes = [vp, C.c_int64, fp, fp, fp, C.c_int64, C.c_int64, vp]
    lib.mj_grpo_sequence_entropy.argtypes = [fp, fp, C.c_int64, C.c_int64, fp, fp, vp]
    lib.mj_grpo_backward.argtypes = [dp, vp, vp, ip, fp, fp, fp, fp, fp, vp, fp, vp, sz, vp]
    i64, f32 = C.c_int64, C.c_float
    lib.mj_grpo_group_advantages.argtypes = [fp, ip, fp, i64, f32, vp]
    lib.mj_grpo_advantages.argtypes = [C.c_int, fp, ip, fp, i64, f32, f32, C.c_int, f32, vp]
    lib.mj_grpo_gae.argtypes = [fp, fp, fp, fp, fp, i64, i64, f32, f32, C.c_int, f32, f32, vp]
    lib.mj_sample_logits.argtypes = [vp, i64, vp, i64, fp, i64, i64, i64, i64, f32, vp]
    lib.mj_sample_top_k.argtypes = [fp, i64, i64, i64, C.c_int, f32, fp, ip, ip, fp, vp]
    lib.mj_rmsnorm_forward.argtypes = [vp, i64, fp, vp, i64, fp, i64, i64, f32, vp]
    lib.mj_rmsnorm_workspace_bytes.argtypes = [i64, i64, C.POINTER(sz)]
    lib.mj_rmsnorm_backward.argtypes = [vp, i64, vp, i64, fp, vp, i64, fp, C.c_int, i64, i64, f32, vp, sz, vp]
    for name in EXPORTS:
        getattr(lib, name)
    _lib = lib
    return lib


def check(status: int) -> None:
    if status != OK:
        raise MjGrpoError(status, load().mj_grpo_last_error().decode())


def workspace_bytes(desc: MjGrpoDesc) -> tuple[int, int]:
    f, b = C.c_size_t(0), C.c_size_t(0)
    check(load().mj_grpo_workspace_bytes(C.byref(desc), C.byref(f), C.byref(b)))
    return f.value, b.value


def value_workspace_bytes(desc: MjGrpoDesc) -> int:
    b = C.c_size_t(0)
    check(load().mj_grpo_value_workspace_bytes(C.byref(desc), C.byref(b)))
    return b.value
