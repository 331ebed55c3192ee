"""ctypes binding of libringattn_hip.so (the C ABI declared in include/ring_attention_hip.h)."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# the library built in-tree; RING_ATTENTION_HIP_LIB names another build of the same ABI
LIB_PATH = os.environ.get("RING_ATTENTION_HIP_LIB") or os.path.join(_HERE, "libringattn_hip.so")

RA_BIAS_CAUSAL = 1
RA_BIAS_WINDOW = 2
RA_BIAS_SEGMENT = 4
RA_BIAS_PREFIX = 8
RA_BIAS_ALIBI = 16
RA_BIAS_DENSE = 32
RA_DTYPE_BF16 = 0
RA_ERR_TOO_LARGE = -8  # a whole-ring launch cannot hold the passes: use the split entry points
RA_MAX_SEGMENT_SHARD = 65536  # longest shard that one call takes under a segment bias
RA_MAX_POSITION = (1 << 30) - (1 << 16)  # token positions (offset + index) stay below this
RA_MAX_ROW_STRIDE = 1 << 27  # elements between two rows of a q / k / v / dO view, at most
RA_DTYPE_F32 = 1


class RaTensor(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("stride_b", C.c_int64), ("stride_h", C.c_int64),
                ("stride_l", C.c_int64)]


class RaBias(C.Structure):
    _fields_ = [
        ("flags", C.c_int32), ("window", C.c_int32),
        ("q_offset", C.c_int64), ("kv_offset", C.c_int64),
        ("q_segment_ids", C.c_void_p), ("kv_segment_ids", C.c_void_p),
        ("q_segment_stride_b", C.c_int64), ("kv_segment_stride_b", C.c_int64),
        ("q_prefix", C.c_void_p), ("kv_prefix", C.c_void_p),
        ("q_prefix_stride_b", C.c_int64), ("kv_prefix_stride_b", C.c_int64),
        ("alibi_slopes", C.c_void_p),
        ("dense_bias", C.c_void_p),
        ("dense_stride_b", C.c_int64), ("dense_stride_h", C.c_int64), ("dense_stride_q", C.c_int64),
        ("dense_map", C.c_void_p),
    ]


class RaFwdStepParams(C.Structure):
    _fields_ = [
        ("B", C.c_int32), ("H", C.c_int32), ("Lq", C.c_int32), ("Lk", C.c_int32), ("D", C.c_int32),
        ("sm_scale", C.c_float),
        ("q", RaTensor), ("k", RaTensor), ("v", RaTensor),
        ("o", C.c_void_p), ("m", C.c_void_p), ("l", C.c_void_p),
        ("bias", RaBias),
    ]


class RaBwdStepParams(C.Structure):
    _fields_ = [
        ("B", C.c_int32), ("H", C.c_int32), ("Lq", C.c_int32), ("Lk", C.c_int32), ("D", C.c_int32),
        ("sm_scale", C.c_float),
        ("q", RaTensor), ("k", RaTensor), ("v", RaTensor), ("dout", RaTensor),
        ("lse", C.c_void_p), ("delta", C.c_void_p),
        ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p),
        ("bias", RaBias),
    ]


EXPORTS = {
    "ra_version": (C.c_int, []),
    "ra_last_error": (C.c_char_p, []),
    "ra_fwd_init": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_int32,
                              C.c_int32, C.c_void_p]),
    "ra_fwd_step": (C.c_int, [C.POINTER(RaFwdStepParams), C.c_void_p]),
    "ra_fwd_steps": (C.c_int, [C.POINTER(RaFwdStepParams), C.c_int32, C.c_void_p]),
    "ra_fwd_finalize": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32,
                                  C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_int32, C.c_int32,
                                  C.c_int32, C.c_int32, C.c_void_p]),
    "ra_bwd_delta": (C.c_int, [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64,
                               C.POINTER(RaTensor), C.c_void_p, C.c_int32, C.c_int32, C.c_int32,
                               C.c_int32, C.c_void_p]),
    "ra_bwd_step": (C.c_int, [C.POINTER(RaBwdStepParams), C.c_void_p]),
    "ra_bwd_step_parts": (C.c_int, [C.POINTER(RaBwdStepParams), C.c_int32, C.c_void_p]),
    "ra_bwd_dq_steps": (C.c_int, [C.POINTER(RaBwdStepParams), C.c_int32, C.c_void_p]),
    "ra_bwd_dkdv_steps": (C.c_int, [C.POINTER(RaBwdStepParams), C.c_int32, C.c_void_p]),
    "ra_fwd_passes": (C.c_int, [C.POINTER(RaFwdStepParams), C.POINTER(C.c_int32), C.c_int32, C.c_void_p]),
    "ra_bwd_dq_passes": (C.c_int, [C.POINTER(RaBwdStepParams), C.POINTER(C.c_int32), C.c_int32, C.c_void_p]),
    "ra_bwd_dkdv_passes": (C.c_int, [C.POINTER(RaBwdStepParams), C.POINTER(C.c_int32), C.c_int32, C.c_void_p]),
    "ra_fwd_ring": (C.c_int, [C.POINTER(RaFwdStepParams), C.POINTER(C.c_int32), C.c_int32, C.c_void_p, C.c_int32,
                              C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_void_p]),
    "ra_bwd_dq_ring": (C.c_int, [C.POINTER(RaBwdStepParams), C.POINTER(C.c_int32), C.c_int32, C.c_void_p, C.c_int64,
                                 C.c_int64, C.c_int64, C.c_int64, C.c_void_p]),
    "ra_bwd_dkdv_ring": (C.c_int, [C.POINTER(RaBwdStepParams), C.POINTER(C.c_int32), C.c_int32, C.c_void_p,
                                   C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64, C.c_void_p]),
    "ra_fwd_finalize_passes": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int64,
                                         C.c_int64, C.c_int64, C.c_int64, C.c_void_p, C.c_int32, C.c_int32,
                                         C.c_int32, C.c_int32, C.c_int32, C.c_void_p]),
    "ra_bwd_delta_passes": (C.c_int, [C.c_void_p, C.c_int32, C.c_int64, C.c_int64, C.c_int64, C.c_int64,
                                      C.POINTER(RaTensor), C.c_int64, C.c_void_p, C.c_int32, C.c_int32, C.c_int32,
                                      C.c_int32, C.c_int32, C.c_void_p]),
    "ra_bwd_finalize_passes": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int64,
                                         C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.c_void_p]),
    "ra_bwd_finalize": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int32,
                                  C.c_int32, C.c_int32, C.c_int32, C.c_void_p]),
    "ra_dense_map_bytes": (C.c_int64, [C.c_int64, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_int32]),
    "ra_dense_map": (C.c_int, [C.c_void_p, C.c_int64, C.c_int64, C.c_int64, C.c_int32, C.c_int32, C.c_int32,
                               C.c_int32, C.c_void_p, C.c_void_p]),
    "ra_step_is_skippable": (C.c_int, [C.POINTER(RaBias), C.c_int32, C.c_int32]),
    "ra_fwd_step_check": (C.c_int, [C.POINTER(RaFwdStepParams)]),
    "ra_bwd_step_check": (C.c_int, [C.POINTER(RaBwdStepParams)]),
}

_lib = None


class RingAttentionHipError(RuntimeError):
    """A C-ABI call returned a non-zero code."""

    def __init__(self, fn: str, code: int, text: str):
        super().__init__(f"{fn} failed with code {code}: {text}")
        self.code = code


def load() -> C.CDLL:
    """Load the HIP library built in-tree. There is no fallback: without it nothing runs."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build the gfx950 kernels first (python build.py in the package "
            "directory, or __graft_entry__.build()); there is no CPU or eager fallback")
    lib = C.CDLL(LIB_PATH)
    for name, (res, args) in EXPORTS.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(fn_name: str, code: int) -> None:
    if code != 0:
        raise RingAttentionHipError(fn_name, code, load().ra_last_error().decode())
