"""ctypes binding of liblinearnexus_hip.so (the C-ABI declared in include/linearnexus_hip.h).

There is no fallback: if the library is missing or a call fails, an exception is raised.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "liblinearnexus_hip.so")

LNX_F32, LNX_BF16 = 0, 1
STATIC_SCRATCH_BYTES = 64 << 20  # LNX_STATIC_SCRATCH_BYTES
GATE_NONE, GATE_SCALAR, GATE_VECTOR = 0, 1, 2

EXPORTS = (
    "lnx_abi_version", "lnx_last_error", "lnx_decode_step", "lnx_recurrent_fwd",
    "lnx_chunk_workspace_bytes", "lnx_chunk_fuses_l2norm", "lnx_chunk_fwd", "lnx_chunk_fwd_static", "lnx_chunk_fwd_static_init", "lnx_chunk_bwd", "lnx_l2norm_fwd", "lnx_l2norm_bwd",
    "lnx_conv1d_fwd", "lnx_conv1d_bwd", "lnx_conv1d_cache_bwd", "lnx_conv1d_packed_fwd", "lnx_conv1d_packed_bwd", "lnx_dplr_recurrent_fwd", "lnx_dplr_step", "lnx_dplr_recurrent_bwd", "lnx_dplr_recurrent_bwd_workspace_bytes", "lnx_rmsnorm_gated_fwd", "lnx_rmsnorm_gated_bwd", "lnx_rmsnorm_gated_bwd_workspace_bytes",
    "lnx_gdn_gate_fwd", "lnx_gdn_gate_bwd", "lnx_gdn_gate_bwd_workspace_bytes", "lnx_kda_gate_fwd", "lnx_kda_gate_bwd", "lnx_kda_gate_bwd_workspace_bytes", "lnx_sigmoid_fwd", "lnx_sigmoid_bwd",
    "lnx_profile_enable", "lnx_profile_read",
)


class ScanArgs(C.Structure):
    """Mirror of ``struct lnx_scan_args``."""

    _fields_ = [
        ("B", C.c_int32), ("H", C.c_int32), ("T", C.c_int32), ("dk", C.c_int32), ("dv", C.c_int32),
        ("chunk", C.c_int32), ("dtype", C.c_int32), ("o_dtype", C.c_int32), ("gate", C.c_int32),
        ("use_qk_l2norm", C.c_int32), ("nseq", C.c_int32), ("scale", C.c_float),
        ("forward_only", C.c_int32), ("token_first", C.c_int32),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("beta", C.c_void_p), ("g", C.c_void_p),
        ("initial_state", C.c_void_p), ("cu_seqlens", C.c_void_p), ("o", C.c_void_p),
        ("final_state", C.c_void_p),
        ("d_o", C.c_void_p), ("d_final_state", C.c_void_p), ("d_q", C.c_void_p), ("d_k", C.c_void_p),
        ("d_v", C.c_void_p), ("d_beta", C.c_void_p), ("d_g", C.c_void_p), ("d_initial_state", C.c_void_p),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64),
        ("value_cols", C.c_int32),
        ("gate_raw", C.c_void_p), ("gate_A_log", C.c_void_p), ("gate_bias", C.c_void_p), ("gate_threshold", C.c_float),
        ("d_gate_raw", C.c_void_p), ("d_gate_A_log", C.c_void_p), ("d_gate_bias", C.c_void_p),
        ("test_scan_slab", C.c_int32), ("test_out_slabs", C.c_int32),
    ]


class DplrArgs(C.Structure):
    """Mirror of ``struct lnx_dplr_args``."""

    _fields_ = [
        ("B", C.c_int32), ("H", C.c_int32), ("T", C.c_int32), ("dk", C.c_int32), ("dv", C.c_int32),
        ("dtype", C.c_int32), ("o_dtype", C.c_int32), ("scale", C.c_float),
        ("q", C.c_void_p), ("k", C.c_void_p), ("v", C.c_void_p), ("a", C.c_void_p), ("b", C.c_void_p),
        ("gk", C.c_void_p), ("initial_state", C.c_void_p), ("o", C.c_void_p), ("final_state", C.c_void_p),
    ]


class DplrBwdArgs(C.Structure):
    """Mirror of ``struct lnx_dplr_bwd_args``."""

    _fields_ = [
        ("fwd", DplrArgs), ("d_o", C.c_void_p), ("d_final_state", C.c_void_p),
        ("dq", C.c_void_p), ("dk", C.c_void_p), ("dv", C.c_void_p), ("da", C.c_void_p), ("db", C.c_void_p),
        ("dgk", C.c_void_p), ("d_initial_state", C.c_void_p), ("workspace", C.c_void_p), ("workspace_bytes", C.c_uint64),
    ]


_lib = None


def load() -> C.CDLL:
    """Loads the library once; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -m linearnexus_amd.build` "
            "(there is no CPU or PyTorch fallback for these ops)"
        )
    lib = C.CDLL(LIB_PATH)
    lib.lnx_abi_version.restype = C.c_int
    lib.lnx_last_error.restype = C.c_char_p
    for name in ("lnx_decode_step", "lnx_recurrent_fwd", "lnx_chunk_fwd", "lnx_chunk_fwd_static", "lnx_chunk_bwd"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [C.POINTER(ScanArgs), C.c_void_p]
    lib.lnx_chunk_fwd_static_init.restype = C.c_int
    lib.lnx_chunk_fwd_static_init.argtypes = []
    lib.lnx_chunk_workspace_bytes.restype = C.c_uint64
    lib.lnx_chunk_workspace_bytes.argtypes = [C.POINTER(ScanArgs)]
    lib.lnx_chunk_fuses_l2norm.restype = C.c_int
    lib.lnx_chunk_fuses_l2norm.argtypes = [C.POINTER(ScanArgs)]
    lib.lnx_l2norm_fwd.restype = C.c_int
    lib.lnx_l2norm_fwd.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_void_p]
    lib.lnx_l2norm_bwd.restype = C.c_int
    lib.lnx_l2norm_bwd.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_int32, C.c_int32, C.c_void_p]
    lib.lnx_conv1d_fwd.restype = C.c_int
    lib.lnx_conv1d_fwd.argtypes = [C.c_void_p] * 6 + [C.c_int32] * 6 + [C.c_void_p]
    lib.lnx_conv1d_bwd.restype = C.c_int
    lib.lnx_conv1d_bwd.argtypes = [C.c_void_p] * 8 + [C.c_int32] * 6 + [C.c_void_p]
    lib.lnx_conv1d_cache_bwd.restype = C.c_int
    lib.lnx_conv1d_cache_bwd.argtypes = [C.c_void_p] * 6 + [C.c_int32] * 6 + [C.c_void_p]
    lib.lnx_conv1d_packed_fwd.restype = C.c_int
    lib.lnx_conv1d_packed_fwd.argtypes = [C.c_void_p] * 4 + [C.c_int32] + [C.c_void_p] * 2 + [C.c_int32] * 5 + [C.c_void_p]
    lib.lnx_conv1d_packed_bwd.restype = C.c_int
    lib.lnx_conv1d_packed_bwd.argtypes = [C.c_void_p] * 4 + [C.c_int32] + [C.c_void_p] * 4 + [C.c_int32] * 5 + [C.c_void_p]
    lib.lnx_rmsnorm_gated_fwd.restype = C.c_int
    lib.lnx_rmsnorm_gated_fwd.argtypes = [C.c_void_p] * 4 + [C.c_int64, C.c_int32, C.c_float, C.c_int32, C.c_void_p]
    lib.lnx_rmsnorm_gated_bwd.restype = C.c_int
    lib.lnx_rmsnorm_gated_bwd.argtypes = [C.c_void_p] * 7 + [C.c_int64, C.c_int32, C.c_float, C.c_int32, C.c_void_p, C.c_uint64,
                                          C.c_void_p]
    lib.lnx_rmsnorm_gated_bwd_workspace_bytes.restype = C.c_uint64
    lib.lnx_rmsnorm_gated_bwd_workspace_bytes.argtypes = [C.c_int64, C.c_int32, C.c_int32]
    lib.lnx_kda_gate_fwd.restype = C.c_int
    lib.lnx_kda_gate_fwd.argtypes = [C.c_void_p] * 4 + [C.c_int64, C.c_int32, C.c_int32, C.c_float, C.c_int32, C.c_int32, C.c_void_p]
    lib.lnx_kda_gate_bwd_workspace_bytes.restype = C.c_uint64
    lib.lnx_kda_gate_bwd_workspace_bytes.argtypes = [C.c_int64, C.c_int32, C.c_int32]
    lib.lnx_kda_gate_bwd.restype = C.c_int
    lib.lnx_kda_gate_bwd.argtypes = [C.c_void_p] * 7 + [C.c_int64, C.c_int32, C.c_int32, C.c_float, C.c_int32, C.c_int32,
                                                         C.c_void_p, C.c_uint64, C.c_void_p]
    lib.lnx_gdn_gate_fwd.restype = C.c_int
    lib.lnx_gdn_gate_fwd.argtypes = [C.c_void_p] * 6 + [C.c_int64, C.c_int32, C.c_float, C.c_int32, C.c_void_p]
    lib.lnx_gdn_gate_bwd_workspace_bytes.restype = C.c_uint64
    lib.lnx_gdn_gate_bwd_workspace_bytes.argtypes = [C.c_int64, C.c_int32]
    lib.lnx_gdn_gate_bwd.restype = C.c_int
    lib.lnx_gdn_gate_bwd.argtypes = [C.c_void_p] * 10 + [C.c_int64, C.c_int32, C.c_float, C.c_int32, C.c_void_p, C.c_uint64, C.c_void_p]
    lib.lnx_sigmoid_fwd.restype = C.c_int
    lib.lnx_sigmoid_fwd.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]
    lib.lnx_sigmoid_bwd.restype = C.c_int
    lib.lnx_sigmoid_bwd.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p]
    for name in ("lnx_dplr_recurrent_fwd", "lnx_dplr_step"):
        fn = getattr(lib, name)
        fn.restype = C.c_int
        fn.argtypes = [C.POINTER(DplrArgs), C.c_void_p]
    lib.lnx_dplr_recurrent_bwd.restype = C.c_int
    lib.lnx_dplr_recurrent_bwd.argtypes = [C.POINTER(DplrBwdArgs), C.c_void_p]
    lib.lnx_dplr_recurrent_bwd_workspace_bytes.restype = C.c_uint64
    lib.lnx_dplr_recurrent_bwd_workspace_bytes.argtypes = [C.c_int32] * 5
    lib.lnx_profile_enable.restype = C.c_int
    lib.lnx_profile_enable.argtypes = [C.c_int]
    lib.lnx_profile_read.restype = C.c_int
    lib.lnx_profile_read.argtypes = [C.c_int, C.POINTER(C.c_char_p), C.POINTER(C.c_float)]
    _lib = lib
    return lib


def profile_enable(on: bool) -> None:
    """Turns per-kernel HIP-event timing on or off for the calling thread."""
    load().lnx_profile_enable(int(on))


def profile_read(capacity: int = 8192):
    """Returns [(kernel name, milliseconds), ...] for the kernels launched since the last read."""
    names = (C.c_char_p * capacity)()
    ms = (C.c_float * capacity)()
    n = load().lnx_profile_read(capacity, names, ms)
    return [(names[i].decode(), float(ms[i])) for i in range(min(n, capacity))]


class HipKernelError(RuntimeError):
    """A C-ABI call returned a negative status."""


def check(status: int, what: str) -> None:
    if status != 0:
        msg = load().lnx_last_error().decode("utf-8", "replace")
        raise HipKernelError(f"{what} failed (status {status}): {msg}")
