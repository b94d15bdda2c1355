"""CPU-side checks of the boundary: the shared library loads, exports every symbol the header
declares, validates arguments without touching a GPU, and the Python ops keep the reference's
signatures and error types."""
import ctypes
import inspect
import os
import re

import pytest

import linearnexus_amd as la
from linearnexus_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "linearnexus_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lnx_[a-z0-9_]+)\s*\(", text)))


_dummies = []


def _aligned_dummy():
    """A 16-byte aligned host address for calls that are refused before anything is dereferenced."""
    buf = (ctypes.c_char * 64)()
    _dummies.append(buf)
    return ctypes.c_void_p((ctypes.addressof(buf) + 15) & ~15)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    names = _declared_symbols()
    assert set(names) >= set(_lib.EXPORTS)
    for n in names:
        assert hasattr(lib, n), n
    assert lib.lnx_abi_version() == 8


def test_struct_layout_matches_header():
    # 14 four-byte scalars, then 17 pointers, the workspace pointer and its size, value_cols (+ padding), the fused
    # gate's three pointers, its threshold (+ padding) and three gradient pointers, and the two test hooks
    assert _lib.ScanArgs.q.offset == 56
    assert _lib.ScanArgs.value_cols.offset == 56 + 18 * 8 + 8 == 208
    assert _lib.ScanArgs.gate_raw.offset == 216 and _lib.ScanArgs.gate_threshold.offset == 240
    assert _lib.ScanArgs.d_gate_raw.offset == 248 and _lib.ScanArgs.test_out_slabs.offset == 276
    assert ctypes.sizeof(_lib.ScanArgs) == 280


def test_one_kernel_set_per_shape_and_no_environment_dispatch():
    """The split between the direct-solve and the WY kernels follows from fields the forward and the backward call
    share (dtype, dk, gate) -- not from o_dtype, which the backward does not use, and not from the environment: the
    workspace size (whose layout differs between the splits) does not react to either, and no source under csrc/
    reads the environment."""
    lib = _lib.load()
    a = _lib.ScanArgs()
    a.B, a.H, a.T, a.dk, a.dv, a.chunk = 2, 2, 256, 128, 128, 64
    a.dtype, a.gate = _lib.LNX_BF16, _lib.GATE_SCALAR
    a.o_dtype = _lib.LNX_BF16
    n_bf16 = int(lib.lnx_chunk_workspace_bytes(a))
    a.o_dtype = _lib.LNX_F32
    assert int(lib.lnx_chunk_workspace_bytes(a)) == n_bf16 and lib.lnx_chunk_fuses_l2norm(a) == 1
    os.environ["LNX_CHUNK_DIRECT"] = "0"
    try:
        assert int(lib.lnx_chunk_workspace_bytes(a)) == n_bf16
    finally:
        del os.environ["LNX_CHUNK_DIRECT"]
    a.gate = _lib.GATE_VECTOR
    assert int(lib.lnx_chunk_workspace_bytes(a)) > n_bf16 and lib.lnx_chunk_fuses_l2norm(a) == 0
    a.gate, a.test_scan_slab = _lib.GATE_SCALAR, 48
    a.q = a.k = a.v = a.beta = a.o = a.final_state = a.g = _aligned_dummy()
    assert lib.lnx_chunk_fwd(a, None) == -2 and b"test_scan_slab" in lib.lnx_last_error()
    csrc = os.path.join(ROOT, "linearnexus_amd", "csrc")
    for f in os.listdir(csrc):
        if f.endswith((".hip", ".h")):
            assert "getenv" not in open(os.path.join(csrc, f)).read(), f


def test_argument_validation_without_gpu():
    lib = _lib.load()
    a = _lib.ScanArgs()
    for fn in (lib.lnx_decode_step, lib.lnx_recurrent_fwd, lib.lnx_chunk_fwd, lib.lnx_chunk_bwd):
        assert fn(a, None) == -2 and b"dimensions" in lib.lnx_last_error()  # all-zero struct: H = 0
    a.B, a.H, a.T, a.dk, a.dv, a.chunk = 1, 1, 1, 64, 64, 64
    for fn in (lib.lnx_decode_step, lib.lnx_recurrent_fwd, lib.lnx_chunk_fwd, lib.lnx_chunk_bwd):
        assert fn(a, None) == -1 and b"required" in lib.lnx_last_error()    # null tensors with elements
    a.B = 0  # an empty batch has no elements behind any pointer: accepted, nothing is launched
    for fn in (lib.lnx_decode_step, lib.lnx_recurrent_fwd, lib.lnx_chunk_fwd, lib.lnx_chunk_bwd):
        assert fn(a, None) == 0
    # value_cols (v holds only the leading value columns) is a forward-only feature, in whole 64-column slabs
    a.B, a.dv, a.value_cols = 1, 128, 64
    p = _aligned_dummy()
    base = p.value
    a.q = a.k = a.v = a.beta = a.o = a.final_state = p
    assert lib.lnx_chunk_fwd(a, None) == -2 and b"value_cols" in lib.lnx_last_error()      # forward_only not set
    a.forward_only, a.value_cols = 1, 32
    assert lib.lnx_chunk_fwd(a, None) == -2 and b"value_cols" in lib.lnx_last_error()      # not a whole slab
    a.value_cols = 192
    assert lib.lnx_chunk_fwd(a, None) == -2 and b"value_cols" in lib.lnx_last_error()      # more than dv
    a.value_cols, a.o = 64, None
    assert lib.lnx_chunk_fwd(a, None) == -4 and b"workspace" in lib.lnx_last_error()       # accepted up to the workspace
    a.k = ctypes.c_void_p(base + 2)  # rows are moved as 16-byte vectors
    assert lib.lnx_chunk_fwd(a, None) == -2 and b"16-byte aligned" in lib.lnx_last_error()
    a.k = p
    assert lib.lnx_l2norm_fwd(None, None, 4, 8, 0, None) == -1
    d = _lib.DplrArgs()
    assert lib.lnx_dplr_step(d, None) == -2 and lib.lnx_dplr_recurrent_fwd(d, None) == -2
    d.B, d.H, d.T, d.dk, d.dv = 1, 1, 1, 64, 64
    assert lib.lnx_dplr_step(d, None) == -1 and lib.lnx_dplr_recurrent_fwd(d, None) == -1
    g = _lib.DplrBwdArgs()
    assert lib.lnx_dplr_recurrent_bwd(None, None) == -1 and lib.lnx_dplr_recurrent_bwd(g, None) == -2
    g.fwd = d
    g.fwd.T = 4
    assert lib.lnx_dplr_recurrent_bwd(g, None) == -1 and b"required" in lib.lnx_last_error()
    assert lib.lnx_dplr_recurrent_bwd_workspace_bytes(2, 3, 130, 64, 64) == 2 * 3 * (3 + 64) * 64 * 64 * 4
    assert lib.lnx_dplr_recurrent_bwd_workspace_bytes(0, 3, 130, 64, 64) == 0
    assert lib.lnx_conv1d_fwd(None, None, None, None, None, None, 1, 4, 16, 5, 0, 0, None) == -2  # K > 4
    assert lib.lnx_conv1d_fwd(None, None, None, None, None, None, 1, 4, 18, 4, 0, 0, None) == -2  # D % 4
    assert lib.lnx_conv1d_bwd(None, None, None, None, None, None, None, None, 1, 4, 16, 4, 0, 0, None) == -1


SIGNATURES = {
    # linearnexus/modules/linear_attn/delta_net.py:126-134, :216-225, :357-364
    "delta_rule_recurrent": ["q", "k", "v", "beta", "initial_state", "scale", "backend"],
    "delta_rule_chunkwise": ["q", "k", "v", "beta", "initial_state", "chunk_size", "scale", "backend"],
    "delta_rule_step": ["q", "k", "v", "beta", "state", "scale"],
    # gated_deltanet.py:136-145, :232-242, :539-548
    "gated_delta_rule_recurrent": ["q", "k", "v", "g", "beta", "scale", "initial_state", "use_qk_l2norm"],
    "gated_delta_rule_chunkwise": ["q", "k", "v", "g", "beta", "scale", "initial_state", "chunk_size", "use_qk_l2norm"],
    "gated_delta_rule_step": ["q", "k", "v", "g", "beta", "state", "scale", "use_qk_l2norm"],
    # kda.py:179-188, :350-360, :286-295
    "kda_recurrent": ["q", "k", "v", "g", "beta", "scale", "initial_state", "use_qk_l2norm"],
    "kda_chunkwise": ["q", "k", "v", "g", "beta", "scale", "initial_state", "chunk_size", "use_qk_l2norm"],
    "kda_step": ["q", "k", "v", "g", "beta", "state", "scale", "use_qk_l2norm"],
}


@pytest.mark.parametrize("name", sorted(SIGNATURES))
def test_op_signatures_match_reference(name):
    sig = inspect.signature(getattr(la, name))
    positional = [p.name for p in sig.parameters.values() if p.kind == p.POSITIONAL_OR_KEYWORD]
    assert positional == SIGNATURES[name]
    d = {p.name: p.default for p in sig.parameters.values()}
    if "chunk_size" in d:
        assert d["chunk_size"] == 64
    if "use_qk_l2norm" in d:
        assert d["use_qk_l2norm"] is True
    assert d["scale"] is None


def test_cpu_tensors_are_rejected_loudly():
    import torch
    q = torch.randn(1, 1, 4, 8)
    with pytest.raises(RuntimeError):
        la.delta_rule_recurrent(q, q, q, torch.ones(1, 1, 4))


def test_chunk_size_error_type():
    import torch
    q = torch.randn(1, 1, 4, 8)
    with pytest.raises(ValueError):  # gated_deltanet.py:318-320
        la.gated_delta_rule_chunkwise(q, q, q, torch.zeros(1, 1, 4), torch.ones(1, 1, 4), chunk_size=24)


def test_backend_seam():
    assert la.select_kernel_backend("pallas") is la.KernelBackend.HIP


def test_malformed_cu_seqlens_is_refused_on_the_host():
    """A sequence table held on the host is checked before anything reaches the GPU: it must start at 0, never
    decrease and end at T (every kernel indexes the token tensors with it)."""
    import numpy as np
    import torch
    from linearnexus_amd.linear_attn import _check_cu_seqlens

    assert _check_cu_seqlens([0, 3, 3, 10], 10).tolist() == [0, 3, 3, 10]
    assert _check_cu_seqlens(np.array([0, 10], np.int32), 10).tolist() == [0, 10]
    for bad in ([1, 5, 10], [0, 6, 5, 10], [0, 5, 11], [0, 5, 9], [-1, 10], [0], [[0, 10]], [0.0, 10.0]):
        with pytest.raises(ValueError):
            _check_cu_seqlens(bad, 10)
    with pytest.raises(ValueError):
        _check_cu_seqlens(torch.tensor([0, 4, 2, 10]), 10)


def test_static_scratch_entry_point_refuses_without_gpu():
    """lnx_chunk_fwd_static checks the shape against the library's scratch size before it touches the GPU."""
    lib = _lib.load()
    p = _aligned_dummy()
    a = _lib.ScanArgs()
    a.B, a.H, a.T, a.dk, a.dv, a.chunk = 8, 16, 4096, 128, 128, 64
    a.dtype = a.o_dtype = _lib.LNX_BF16
    a.q = a.k = a.v = a.beta = a.o = a.final_state = p
    assert lib.lnx_chunk_fwd_static(a, None) == -4 and b"forward_only" in lib.lnx_last_error()
    a.forward_only = 1
    assert int(lib.lnx_chunk_workspace_bytes(a)) > _lib.STATIC_SCRATCH_BYTES
    assert lib.lnx_chunk_fwd_static(a, None) == -4 and b"scratch" in lib.lnx_last_error()
