"""lnx_chunk_fwd_static -- the forward entry point that allocates nothing and works on the library's own per-GPU
scratch array -- against lnx_chunk_fwd on a caller-owned workspace, through the C-ABI (ctypes): same kernels on a
different buffer, so the results must be bit-identical.  Two calls in a row, the second on a smaller input (stale
contents of the shared scratch must not leak into it), dense and packed, with an initial state."""
import ctypes

import numpy as np
import pytest
import torch

from linearnexus_amd import _lib
from oracle import recurrent as rc
from oracle.inputs import make_inputs, to_bf16_grid
from conftest import max_rel

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _aligned_dummy():
    """A 16-byte aligned host address for a call that is refused before anything is dereferenced."""
    buf = (ctypes.c_char * 64)()
    _aligned_dummy.keep = buf
    return ctypes.c_void_p((ctypes.addressof(buf) + 15) & ~15)


def _args(x, B, H, T, dk, dv, cu=None):
    a = _lib.ScanArgs()
    a.B, a.H, a.T, a.dk, a.dv, a.chunk = B, H, T, dk, dv, 64
    a.dtype = a.o_dtype = _lib.LNX_BF16
    a.gate = _lib.GATE_SCALAR
    a.scale = dk ** -0.5
    a.forward_only = 1
    a.nseq = 0 if cu is None else cu.numel() - 1
    a.q, a.k, a.v = x["q"].data_ptr(), x["k"].data_ptr(), x["v"].data_ptr()
    a.beta, a.g, a.initial_state = x["beta"].data_ptr(), x["g"].data_ptr(), x["S0"].data_ptr()
    a.cu_seqlens = None if cu is None else cu.data_ptr()
    return a


def _run_both(seed, B, H, T, d, cu_list=None):
    lib = _lib.load()
    nstate = B if cu_list is None else len(cu_list) - 1
    xn = make_inputs(seed, B, H, T, d, d, gate="scalar")
    xn["S0"] = (np.random.default_rng(seed).standard_normal((nstate, H, d, d)) * 0.02).astype(np.float32)
    x = {n: torch.from_numpy(a).to(DEV) for n, a in xn.items()}
    for n in ("q", "k", "v"):
        x[n] = x[n].to(torch.bfloat16).contiguous()
    cu = None if cu_list is None else torch.tensor(cu_list, dtype=torch.int32, device=DEV)
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for static in (False, True):
        o = torch.full((B, H, T, d), float("nan"), dtype=torch.bfloat16, device=DEV)
        sT = torch.full((nstate, H, d, d), float("nan"), dtype=torch.float32, device=DEV)
        a = _args(x, B, H, T, d, d, cu)
        a.o, a.final_state = o.data_ptr(), sT.data_ptr()
        if static:
            a.workspace, a.workspace_bytes = 3, 0  # ignored, whatever they hold
            _lib.check(lib.lnx_chunk_fwd_static(a, stream), "lnx_chunk_fwd_static")
        else:
            n = int(lib.lnx_chunk_workspace_bytes(a))
            ws = torch.empty(n, dtype=torch.uint8, device=DEV)
            a.workspace, a.workspace_bytes = ws.data_ptr(), n
            _lib.check(lib.lnx_chunk_fwd(a, stream), "lnx_chunk_fwd")
        torch.cuda.synchronize()
        outs.append((o, sT))
    (o_ws, s_ws), (o_st, s_st) = outs
    assert torch.equal(o_ws, o_st) and torch.equal(s_ws, s_st)
    return xn, o_st, s_st


def test_static_scratch_forward_matches_workspace_forward_twice():
    # first call: 2 x 4 rows of 5 chunks; second, smaller: 1 x 2 rows of 2 chunks (ragged) on the same scratch
    _run_both(71, 2, 4, 300, 128)
    xn, o, sT = _run_both(72, 1, 2, 100, 128)
    for n in ("q", "k", "v"):
        xn[n] = to_bf16_grid(xn[n])
    o_ref, S_ref = rc.gated_delta_rule_recurrent(xn["q"], xn["k"], xn["v"], xn["g"], xn["beta"], None, xn["S0"], False)
    assert max_rel(o.float().cpu().numpy(), o_ref) < 2e-2 and max_rel(sT.cpu().numpy(), S_ref) < 2e-2


def test_static_scratch_forward_packed_batch():
    _run_both(73, 1, 3, 400, 64, cu_list=[0, 130, 131, 131, 400])
    _run_both(74, 1, 2, 90, 64, cu_list=[0, 64, 90])


def test_static_scratch_forward_refuses_what_does_not_fit():
    lib = _lib.load()
    p = _aligned_dummy()
    a = _lib.ScanArgs()
    a.B, a.H, a.T, a.dk, a.dv, a.chunk = 8, 16, 4096, 128, 128, 64
    a.dtype = a.o_dtype = _lib.LNX_BF16
    a.q = a.k = a.v = a.beta = a.o = a.final_state = p  # never dereferenced: the call is refused before any launch
    assert lib.lnx_chunk_fwd_static(a, None) == -4 and b"forward_only" in lib.lnx_last_error()
    a.forward_only = 1
    assert int(lib.lnx_chunk_workspace_bytes(a)) > _lib.STATIC_SCRATCH_BYTES
    assert lib.lnx_chunk_fwd_static(a, None) == -4 and b"scratch" in lib.lnx_last_error()


def test_static_scratch_forward_under_graph_capture():
    """The entry point exists for callers under HIP graph capture: captured on a stream after
    lnx_chunk_fwd_static_init() (the symbol lookup stays outside the capture), replayed three times with eager work and
    synchronisations in between, every replay bit-identical to lnx_chunk_fwd on a caller-owned workspace."""
    lib = _lib.load()
    assert lib.lnx_chunk_fwd_static_init() == 0
    B, H, T, d = 2, 3, 200, 128
    xn = make_inputs(75, B, H, T, d, d, gate="scalar")
    xn["S0"] = (np.random.default_rng(75).standard_normal((B, H, d, d)) * 0.02).astype(np.float32)
    x = {n: torch.from_numpy(a).to(DEV) for n, a in xn.items()}
    for n in ("q", "k", "v"):
        x[n] = x[n].to(torch.bfloat16).contiguous()
    o = torch.zeros(B, H, T, d, dtype=torch.bfloat16, device=DEV)
    sT = torch.zeros(B, H, d, d, dtype=torch.float32, device=DEV)
    a = _args(x, B, H, T, d, d)
    a.o, a.final_state = o.data_ptr(), sT.data_ptr()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        _lib.check(lib.lnx_chunk_fwd_static(a, torch.cuda.current_stream().cuda_stream), "lnx_chunk_fwd_static (capturing)")
    for rep in range(3):
        # new inputs in the captured buffers; the reference result through the workspace entry point, eagerly
        x["v"].copy_(torch.randn(B, H, T, d, device=DEV).to(torch.bfloat16))
        x["S0"].mul_(0.5)
        o_ref = torch.empty_like(o)
        s_ref = torch.empty_like(sT)
        b = _args(x, B, H, T, d, d)
        b.o, b.final_state = o_ref.data_ptr(), s_ref.data_ptr()
        n = int(lib.lnx_chunk_workspace_bytes(b))
        ws = torch.empty(n, dtype=torch.uint8, device=DEV)
        b.workspace, b.workspace_bytes = ws.data_ptr(), n
        _lib.check(lib.lnx_chunk_fwd(b, torch.cuda.current_stream().cuda_stream), "lnx_chunk_fwd")
        torch.cuda.synchronize()
        o.fill_(float("nan"))
        sT.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, o_ref) and torch.equal(sT, s_ref), f"replay {rep}"
