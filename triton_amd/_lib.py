"""ctypes binding of libtrinity_hip.so (declared in include/trinity_hip.h).

The library is plain HIP behind a C ABI; torch is used only to own device memory and
to name the current stream.  There is no CPU or eager fallback: if the shared library
is missing, loading raises, and so does every operator.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Optional

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libtrinity_hip.so")

EXPORTS = (
    "trn_version", "trn_status_name", "trn_check_device", "trn_rmsnorm_f16",
    "trn_attn_fwd_f16", "trn_attn_colstats_f16", "trn_prenorm_qkv_f16", "trn_calibration_copy",
    "trn_calibration_mfma", "trn_attn_workspace_bytes", "trn_attn_fwd_ws_f16", "trn_linear_f16", "trn_gate_f16", "trn_attn_fwd_stats_f16",
    "trn_attn_fwd_noalloc_f16", "trn_attn_fwd_kernel_name", "trn_attn_colmeanstd_f16", "trn_attn_fwd_probs_f16",
    "trn_attn_fwd_stats_half_f16", "trn_attn_fwd_stats_ws_f16", "trn_attn_stats_workspace_bytes",
)


class TrnError(RuntimeError):
    """A libtrinity_hip call returned a negative status."""

    def __init__(self, fn: str, status: int, name: str):
        super().__init__(f"{fn} failed: {name} ({status})")
        self.status = status
        self.status_name = name


class AttnDesc(C.Structure):
    """Mirror of `trn_attn_desc`."""
    _fields_ = [
        ("batch", C.c_int32), ("n_q_heads", C.c_int32), ("n_kv_heads", C.c_int32),
        ("seq_q", C.c_int32), ("seq_kv", C.c_int32), ("head_dim", C.c_int32),
        ("q_stride_b", C.c_int64), ("q_stride_h", C.c_int64), ("q_stride_s", C.c_int64),
        ("k_stride_b", C.c_int64), ("k_stride_h", C.c_int64), ("k_stride_s", C.c_int64),
        ("v_stride_b", C.c_int64), ("v_stride_h", C.c_int64), ("v_stride_s", C.c_int64),
        ("o_stride_b", C.c_int64), ("o_stride_h", C.c_int64), ("o_stride_s", C.c_int64),
        ("scale", C.c_float), ("causal", C.c_int32),
        ("q_norm", C.c_int32), ("q_norm_eps", C.c_float),
        ("noise_stride_b", C.c_int64), ("noise_stride_h", C.c_int64), ("noise_stride_s", C.c_int64),
        ("tau", C.c_float),
    ]


_lib: Optional[C.CDLL] = None


def load() -> C.CDLL:
    """Load the shared library (once) and declare prototypes.  Raises if it is not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} is not built; run `python -m triton_amd.build` (needs hipcc). "
            "There is no fallback path.")
    lib = C.CDLL(LIB_PATH)
    vp, i64, f32, i32 = C.c_void_p, C.c_int64, C.c_float, C.c_int32
    lib.trn_version.restype = C.c_int
    lib.trn_version.argtypes = []
    lib.trn_status_name.restype = C.c_char_p
    lib.trn_status_name.argtypes = [C.c_int]
    lib.trn_check_device.restype = C.c_int
    lib.trn_check_device.argtypes = []
    lib.trn_rmsnorm_f16.restype = C.c_int
    lib.trn_rmsnorm_f16.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, i64, f32, vp]
    lib.trn_attn_fwd_f16.restype = C.c_int
    lib.trn_attn_fwd_f16.argtypes = [C.POINTER(AttnDesc), vp, vp, vp, vp, vp, vp, vp, vp, vp]
    lib.trn_attn_fwd_stats_f16.restype = C.c_int
    lib.trn_attn_fwd_stats_f16.argtypes = [C.POINTER(AttnDesc), vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp]
    lib.trn_attn_stats_workspace_bytes.restype = C.c_int64
    lib.trn_attn_stats_workspace_bytes.argtypes = [C.POINTER(AttnDesc)]
    lib.trn_attn_fwd_stats_ws_f16.restype = C.c_int
    lib.trn_attn_fwd_stats_ws_f16.argtypes = [C.POINTER(AttnDesc), vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, vp]
    lib.trn_attn_fwd_stats_half_f16.restype = C.c_int
    lib.trn_attn_fwd_stats_half_f16.argtypes = [C.POINTER(AttnDesc), vp, vp, vp, vp, vp, vp, vp, vp, vp, vp, vp]
    lib.trn_linear_f16.restype = C.c_int
    lib.trn_linear_f16.argtypes = [vp, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.POINTER(vp), C.POINTER(C.c_int64),
                                   C.POINTER(C.c_int64), C.POINTER(vp), C.POINTER(C.c_int64), C.POINTER(vp), vp]
    lib.trn_gate_f16.restype = C.c_int
    lib.trn_gate_f16.argtypes = [vp, vp, vp, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_int32, vp]
    lib.trn_attn_workspace_bytes.restype = C.c_int64
    lib.trn_attn_workspace_bytes.argtypes = [C.POINTER(AttnDesc)]
    lib.trn_attn_fwd_ws_f16.restype = C.c_int
    lib.trn_attn_fwd_ws_f16.argtypes = [C.POINTER(AttnDesc), vp, vp, vp, vp, vp, vp, vp, vp, vp, C.c_int64, vp]
    lib.trn_attn_fwd_noalloc_f16.restype = C.c_int
    lib.trn_attn_fwd_noalloc_f16.argtypes = [C.POINTER(AttnDesc), vp, vp, vp, vp, vp, vp, vp, vp, vp]
    lib.trn_attn_fwd_kernel_name.restype = C.c_char_p
    lib.trn_attn_fwd_kernel_name.argtypes = [C.POINTER(AttnDesc), C.c_int32]
    lib.trn_attn_colstats_f16.restype = C.c_int
    lib.trn_attn_colstats_f16.argtypes = [C.POINTER(AttnDesc), vp, vp, vp, vp, vp, vp, vp]
    lib.trn_attn_fwd_probs_f16.restype = C.c_int
    lib.trn_attn_fwd_probs_f16.argtypes = [C.POINTER(AttnDesc), vp, vp, vp, vp, vp, vp, vp, vp, vp, vp]
    lib.trn_attn_colmeanstd_f16.restype = C.c_int
    lib.trn_attn_colmeanstd_f16.argtypes = [C.POINTER(AttnDesc), vp, vp, vp, vp, vp, vp]
    lib.trn_prenorm_qkv_f16.restype = C.c_int
    lib.trn_prenorm_qkv_f16.argtypes = [vp] * 8 + [i64] * 15 + [f32, i32, vp]
    lib.trn_calibration_copy.restype = C.c_int
    lib.trn_calibration_copy.argtypes = [vp, vp, i64, vp]
    lib.trn_calibration_mfma.restype = C.c_int
    lib.trn_calibration_mfma.argtypes = [vp, vp, i32, i32, vp]
    _lib = lib
    return lib


def check(fn: str, status: int) -> None:
    if status != 0:
        name = load().trn_status_name(status).decode()
        raise TrnError(fn, status, name)


def current_stream_handle(device=None) -> int:
    import torch
    return torch.cuda.current_stream(device).cuda_stream
