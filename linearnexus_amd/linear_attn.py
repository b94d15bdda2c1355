"""Delta-rule layer ops on MI355X with the reference's signatures.

The nine ops mirror ``linearnexus.modules.linear_attn`` (names, positional order, defaults,
return conventions; linearnexus/modules/linear_attn/__init__.py:15-58): head-first
``[B, H, T, d]`` tensors in, ``(output, final_state)`` out, fp32 state.  Tensors are
``torch`` CUDA tensors (PyTorch only supplies device memory and the stream); every op
launches hand-written gfx950 kernels through the C-ABI and raises if the library is
missing -- there is no other code path.

Differences from the reference, all additive: ``*_step`` take ``inplace=True`` to update
the state buffer in place; the chunk ops take ``cu_seqlens`` for packed variable-length
batches and are differentiable (``torch.autograd``) through the HIP backward kernels.
"""
from __future__ import annotations

import os

from dataclasses import dataclass
from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import GATE_NONE, GATE_SCALAR, GATE_VECTOR, LNX_BF16, LNX_F32, ScanArgs

Tensor = torch.Tensor
_DT = {torch.float32: LNX_F32, torch.bfloat16: LNX_BF16}
CHUNK = 64  # the kernels' chunk length; results do not depend on it


# --------------------------------------------------------------------------------------
# helpers
# --------------------------------------------------------------------------------------

def _stream(t: Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _ptr(t: Optional[Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _check_inputs(q: Tensor, k: Tensor, v: Tensor) -> int:
    for name, t in (("q", q), ("k", k), ("v", v)):
        if not isinstance(t, torch.Tensor):
            raise TypeError(f"{name} must be a torch.Tensor on an AMD GPU, got {type(t).__name__}")
        if not t.is_cuda:
            raise RuntimeError(f"{name} is on {t.device}; the delta-rule ops run on the GPU only")
    if q.dtype not in _DT:
        raise RuntimeError(f"unsupported dtype {q.dtype}: use float32 or bfloat16")
    if k.dtype != q.dtype or v.dtype != q.dtype:
        raise RuntimeError(f"q, k, v must share one dtype, got {q.dtype}, {k.dtype}, {v.dtype}")
    if q.shape != k.shape or q.shape[:-1] != v.shape[:-1]:
        raise RuntimeError(f"shape mismatch: q {tuple(q.shape)} k {tuple(k.shape)} v {tuple(v.shape)}")
    return _DT[q.dtype]


def _f32(t: Tensor) -> Tensor:
    return t.to(torch.float32).contiguous()


def _wants_grad(*tensors) -> bool:
    """The reference's token-by-token ops are differentiable like everything in JAX, and its blocks call them while
    training (sequences of at most 32 tokens, gated_deltanet.py:836-846).  The token kernels have no backward pass;
    when a gradient is wanted the same function is computed by the chunk kernels, which have one."""
    return torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in tensors)


def _promote(q: Tensor, k: Tensor, v: Tensor):
    """The reference up-casts q, k, v to float32 whatever they are and returns the output in q's dtype
    (delta_net.py:170-179, :213; gated_deltanet.py:167-175, :229).  The kernels take one dtype, float32 or bfloat16:
    anything else -- mixed dtypes (the DeltaNet block normalises q, k in float32 next to a bf16 v,
    delta_net.py:566-575), float16, float64 -- is computed in float32 and the output cast back to q's dtype.
    Returns (q, k, v, dtype to cast the output to or None)."""
    ts = (q, k, v)
    if not all(isinstance(t, torch.Tensor) and t.is_floating_point() for t in ts):
        return q, k, v, None  # _check_inputs reports it
    if q.dtype == k.dtype == v.dtype and q.dtype in _DT:
        return q, k, v, None
    return q.to(torch.float32), k.to(torch.float32), v.to(torch.float32), q.dtype


# Memory layout of the token tensors.  The ops take the reference's head-first [B, H, T, .] shapes; a caller
# whose data lives token-first -- [B, T, H, .], what the reference's blocks hold before they transpose
# (delta_net.py:645-647) -- passes ``x.transpose(1, 2)`` views, and the kernels then read and write that
# memory in place (``token_first`` in the argument block) instead of working on contiguous copies.

def _is_token_first(x: Tensor) -> bool:
    return x.dim() >= 3 and not x.is_contiguous() and x.transpose(1, 2).is_contiguous()


def _as_layout(x: Optional[Tensor], token_first: bool) -> Optional[Tensor]:
    """``x`` (logical [B, H, T, ...]) with dense memory in the chosen layout; no copy when it already has it."""
    if x is None:
        return None
    if x.data_ptr() % 16:  # a dense view that starts inside a 16-byte vector of its storage: the kernels need a copy
        x = x.clone(memory_format=torch.preserve_format)
    if token_first:
        return x if _is_token_first(x) else x.transpose(1, 2).contiguous().transpose(1, 2)
    return x.contiguous()


def _empty_layout(B, H, T, tail, dtype, device, token_first: bool) -> Tensor:
    if token_first:
        return torch.empty((B, T, H) + tuple(tail), dtype=dtype, device=device).transpose(1, 2)
    return torch.empty((B, H, T) + tuple(tail), dtype=dtype, device=device)


def _dense(x: Tensor):
    """A contiguous tensor over x's memory (or a copy) and the function that maps results back to x's layout."""
    if x.is_contiguous():
        return x, (lambda y: y)
    if x.dim() >= 4 and _is_token_first(x):  # with fewer dimensions the transposition would move the last axis itself
        return x.transpose(1, 2), (lambda y: y.transpose(1, 2))
    return x.contiguous(), (lambda y: y)


def _squeeze_beta(beta: Tensor, ndim: int) -> Tensor:
    # delta_net.py:166-167, :257-258, :378-379 -- a trailing singleton is accepted
    return beta.squeeze(-1) if beta.dim() == ndim else beta


def _gate_kind(g: Optional[Tensor], lead_shape, dk: int) -> int:
    if g is None:
        return GATE_NONE
    if tuple(g.shape) == tuple(lead_shape):
        return GATE_SCALAR
    if tuple(g.shape) == tuple(lead_shape) + (dk,):
        return GATE_VECTOR
    raise RuntimeError(f"gate shape {tuple(g.shape)} matches neither {tuple(lead_shape)} nor {tuple(lead_shape) + (dk,)}")


# Test hooks: the tiling overrides of ``lnx_scan_args`` (0 = the library's choice).  The GPU tests set them to reach both
# slab widths of the sequential kernels, and the grouped form of the fp32 output kernel, at small shapes.
_test_hooks = {"scan_slab": 0, "out_slabs": 0}


def _base_args(B, H, T, dk, dv, dtype, o_dtype, gate, l2norm, scale) -> ScanArgs:
    a = ScanArgs()
    a.test_scan_slab, a.test_out_slabs = _test_hooks["scan_slab"], _test_hooks["out_slabs"]
    a.B, a.H, a.T, a.dk, a.dv = B, H, T, dk, dv
    a.chunk = CHUNK
    a.dtype, a.o_dtype, a.gate = dtype, o_dtype, gate
    a.use_qk_l2norm = int(bool(l2norm))
    a.nseq = 0
    a.scale = float(scale)
    return a


# --------------------------------------------------------------------------------------
# state caches (delta_net.py:81-118, gated_deltanet.py:72-128, kda.py:57-113)
# --------------------------------------------------------------------------------------

@dataclass
class DeltaNetState:
    """Cache for DeltaNet generation (delta_net.py:81-118): ``S [batch, heads, key_dim, value_dim]`` float32 and the
    conv cache ``[batch, kernel-1, channels]`` of the block's one convolution over the concatenated q, k, v."""
    S: Tensor
    conv_state: Optional[Tensor] = None

    @classmethod
    def zeros(cls, batch_size, num_heads, key_dim, value_dim, conv_channels=None, conv_size=4, *, device="cuda"):
        S = torch.zeros(batch_size, num_heads, key_dim, value_dim, dtype=torch.float32, device=device)
        conv_state = None
        if conv_channels is not None:
            conv_state = torch.zeros(batch_size, conv_size - 1, conv_channels, dtype=torch.float32, device=device)
        return cls(S=S, conv_state=conv_state)


@dataclass
class _GatedState:
    """``S [batch, num_v_heads, key_dim_per_head, value_dim_per_head]`` float32 and one conv cache each for q, k
    (``[batch, kernel-1, key_dim_total]``) and v (``[batch, kernel-1, value_dim]``)."""
    S: Tensor
    conv_state_q: Optional[Tensor] = None
    conv_state_k: Optional[Tensor] = None
    conv_state_v: Optional[Tensor] = None

    @classmethod
    def zeros(cls, batch_size, num_v_heads, key_dim_per_head, value_dim_per_head, key_dim_total=None, value_dim=None,
              conv_size=4, use_conv=True, *, device="cuda"):
        z = lambda *shape: torch.zeros(*shape, dtype=torch.float32, device=device)
        state = cls(S=z(batch_size, num_v_heads, key_dim_per_head, value_dim_per_head))
        if use_conv and key_dim_total is not None and value_dim is not None:
            state.conv_state_q = z(batch_size, conv_size - 1, key_dim_total)
            state.conv_state_k = z(batch_size, conv_size - 1, key_dim_total)
            state.conv_state_v = z(batch_size, conv_size - 1, value_dim)
        return state


@dataclass
class GatedDeltaNetState(_GatedState):
    """Cache for Gated DeltaNet generation (gated_deltanet.py:72-128)."""


@dataclass
class KDAState(_GatedState):
    """Cache for KDA generation (kda.py:57-113)."""


# --------------------------------------------------------------------------------------
# single-token decode step
# --------------------------------------------------------------------------------------

def _step(q, k, v, g, beta, state, scale, l2norm, o_dtype_from_state, inplace):
    q, k, v, back = _promote(q, k, v)
    if back is not None:
        o, s_out = _step(q, k, v, g, beta, state, scale, l2norm, o_dtype_from_state, inplace)
        return (o if o_dtype_from_state else o.to(back)), s_out
    dt = _check_inputs(q, k, v)
    if q.dim() != 3:
        raise RuntimeError(f"step ops take [B, H, d] vectors, got q {tuple(q.shape)}")
    if _wants_grad(q, k, v, g, beta, state):
        if inplace:
            raise RuntimeError("inplace=True overwrites the state a backward pass would need")
        # the token kernels normalise and compute in fp32 (gated_deltanet.py:193-195): so does this path, so that the
        # values do not depend on whether a gradient is wanted
        up = (lambda t: t.to(torch.float32)) if (l2norm and q.dtype != torch.float32) else (lambda t: t)
        o, s_out = _chunk(up(q)[:, :, None], up(k)[:, :, None], up(v)[:, :, None], None if g is None else g[:, :, None],
                          _squeeze_beta(beta, 3)[:, :, None], scale, state, CHUNK, l2norm,
                          torch.float32 if (o_dtype_from_state or l2norm) else q.dtype, False, None)
        return o[:, :, 0].to(state.dtype if o_dtype_from_state else q.dtype), s_out
    B, H, dk = q.shape
    dv = v.shape[-1]
    beta = _squeeze_beta(beta, 3)
    gate = _gate_kind(g, (B, H), dk)
    if tuple(state.shape) != (B, H, dk, dv):
        raise RuntimeError(f"state shape {tuple(state.shape)} != {(B, H, dk, dv)}")
    if scale is None:
        scale = dk ** -0.5
    if inplace:
        if state.dtype != torch.float32 or not state.is_contiguous():
            raise RuntimeError("inplace=True needs a contiguous float32 state")
        s_in = s_out = state
    else:
        s_in = _f32(state)
        s_out = torch.empty_like(s_in)
    o_t = torch.float32 if o_dtype_from_state else q.dtype
    o = torch.empty(B, H, dv, dtype=o_t, device=q.device)
    q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    beta = _f32(beta)
    g = None if g is None else _f32(g)
    a = _base_args(B, H, 1, dk, dv, dt, _DT[o_t], gate, l2norm, scale)
    a.q, a.k, a.v, a.beta, a.g = _ptr(q), _ptr(k), _ptr(v), _ptr(beta), _ptr(g)
    a.initial_state, a.final_state, a.o = _ptr(s_in), _ptr(s_out), _ptr(o)
    lib = _lib.load()
    _lib.check(lib.lnx_decode_step(a, _stream(q)), "lnx_decode_step")
    return o, s_out


def delta_rule_step(q, k, v, beta, state, scale=None, *, inplace=False) -> Tuple[Tensor, Tensor]:
    """One decode token of plain DeltaNet (delta_net.py:357-397)."""
    return _step(q, k, v, None, beta, state, scale, False, False, inplace)


def gated_delta_rule_step(q, k, v, g, beta, state, scale=None, use_qk_l2norm=True, *, inplace=False):
    """One decode token of Gated DeltaNet, ``g [B,H]`` (gated_deltanet.py:539-597)."""
    return _step(q, k, v, g, beta, state, scale, use_qk_l2norm, False, inplace)


def kda_step(q, k, v, g, beta, state, scale=None, use_qk_l2norm=True, *, inplace=False):
    """One decode token of KDA, ``g [B,H,dk]``; output in the state's dtype (kda.py:286-347)."""
    return _step(q, k, v, g, beta, state, scale, use_qk_l2norm, True, inplace)


# --------------------------------------------------------------------------------------
# token-by-token scan
# --------------------------------------------------------------------------------------

def _seq_setup(q, k, v, g, beta, initial_state, cu_seqlens):
    dt = _check_inputs(q, k, v)
    if q.dim() != 4:
        raise RuntimeError(f"scan ops take [B, H, T, d] tensors, got q {tuple(q.shape)}")
    B, H, T, dk = q.shape
    dv = v.shape[-1]
    beta = _squeeze_beta(beta, 4)
    if tuple(beta.shape) != (B, H, T):
        raise RuntimeError(f"beta shape {tuple(beta.shape)} != {(B, H, T)}")
    gate = _gate_kind(g, (B, H, T), dk)
    nseq = 0
    if cu_seqlens is not None:
        if B != 1:
            raise RuntimeError("cu_seqlens needs a packed batch with B == 1")
        cu_seqlens = _check_cu_seqlens(cu_seqlens, T).to(device=q.device, dtype=torch.int32).contiguous()
        nseq = cu_seqlens.numel() - 1
    nstate = nseq if nseq else B
    if initial_state is not None and tuple(initial_state.shape) != (nstate, H, dk, dv):
        raise RuntimeError(f"initial_state shape {tuple(initial_state.shape)} != {(nstate, H, dk, dv)}")
    return dt, B, H, T, dk, dv, beta, gate, nseq, nstate, cu_seqlens


def _check_cu_seqlens(cu, T: int) -> Tensor:
    """``cu_seqlens`` as an integer tensor.  A table that lives on the host (list, numpy array, CPU tensor) is
    validated here: one-dimensional, at least two entries, ``cu[0] == 0``, non-decreasing, ``cu[-1] == T`` -- every
    token belongs to exactly one sequence; anything else raises ``ValueError``.  A table that is already on the GPU is
    not read back (that would synchronise the stream): the kernels clamp its entries to ``[0, T]`` and treat a
    decreasing pair as an empty sequence, so a malformed table cannot send them outside the tensors, but tokens it
    does not cover then keep unspecified outputs and gradients."""
    if not isinstance(cu, torch.Tensor):
        cu = torch.as_tensor(cu)
    if cu.is_floating_point() or cu.dim() != 1 or cu.numel() < 2:
        raise ValueError(f"cu_seqlens must be a 1-D integer table with at least two entries, got shape {tuple(cu.shape)} {cu.dtype}")
    if not cu.is_cuda:
        c = cu.to(torch.int64)
        if int(c[0]) != 0 or int(c[-1]) != T or bool((c[1:] < c[:-1]).any()):
            raise ValueError(f"cu_seqlens must start at 0, never decrease and end at T = {T}; got {c.tolist()[:8]}"
                             f"{' ...' if c.numel() > 8 else ''} (last {int(c[-1])})")
    return cu


def _recurrent(q, k, v, g, beta, scale, initial_state, l2norm, cu_seqlens=None):
    q, k, v, back = _promote(q, k, v)
    if back is not None:
        o, sT = _recurrent(q, k, v, g, beta, scale, initial_state, l2norm, cu_seqlens)
        return o.to(back), sT
    if _wants_grad(q, k, v, g, beta, initial_state):
        if l2norm and q.dtype != torch.float32:  # fp32 normalisation and arithmetic, like the token kernels
            o, sT = _chunk(q.to(torch.float32), k.to(torch.float32), v.to(torch.float32), g, beta, scale, initial_state, CHUNK,
                           l2norm, torch.float32, False, cu_seqlens)
            return o.to(q.dtype), sT
        return _chunk(q, k, v, g, beta, scale, initial_state, CHUNK, l2norm, q.dtype, False, cu_seqlens)
    dt, B, H, T, dk, dv, beta, gate, nseq, nstate, cu = _seq_setup(q, k, v, g, beta, initial_state, cu_seqlens)
    if scale is None:
        scale = dk ** -0.5
    tf = all(_is_token_first(t) for t in (q, k, v))
    q, k, v = _as_layout(q, tf), _as_layout(k, tf), _as_layout(v, tf)
    beta = _as_layout(beta.to(torch.float32), tf)
    g = None if g is None else _as_layout(g.to(torch.float32), tf)
    s0 = None if initial_state is None else _f32(initial_state)
    o = _empty_layout(B, H, T, (dv,), q.dtype, q.device, tf)
    sT = torch.empty(nstate, H, dk, dv, dtype=torch.float32, device=q.device)
    a = _base_args(B, H, T, dk, dv, dt, dt, gate, l2norm, scale)
    a.nseq = nseq
    a.token_first = int(tf)
    a.q, a.k, a.v, a.beta, a.g = _ptr(q), _ptr(k), _ptr(v), _ptr(beta), _ptr(g)
    a.initial_state, a.final_state, a.o, a.cu_seqlens = _ptr(s0), _ptr(sT), _ptr(o), _ptr(cu)
    lib = _lib.load()
    _lib.check(lib.lnx_recurrent_fwd(a, _stream(q)), "lnx_recurrent_fwd")
    return o, sT


def delta_rule_recurrent(q, k, v, beta, initial_state=None, scale=None, backend=None, *, cu_seqlens=None):
    """Token-by-token DeltaNet scan in fp32 (delta_net.py:126-213)."""
    return _recurrent(q, k, v, None, beta, scale, initial_state, False, cu_seqlens)


def gated_delta_rule_recurrent(q, k, v, g, beta, scale=None, initial_state=None, use_qk_l2norm=True, *,
                               cu_seqlens=None):
    """Token-by-token Gated DeltaNet scan, ``g [B,H,T]`` (gated_deltanet.py:136-229)."""
    return _recurrent(q, k, v, g, beta, scale, initial_state, use_qk_l2norm, cu_seqlens)


def kda_recurrent(q, k, v, g, beta, scale=None, initial_state=None, use_qk_l2norm=True, *, cu_seqlens=None):
    """Token-by-token KDA scan, ``g [B,H,T,dk]`` (kda.py:179-283)."""
    return _recurrent(q, k, v, g, beta, scale, initial_state, use_qk_l2norm, cu_seqlens)


# --------------------------------------------------------------------------------------
# chunked scan (forward + backward)
# --------------------------------------------------------------------------------------

def l2norm_rows(x: Tensor) -> Tensor:
    """``x / (|x|_2 + 1e-6)`` over the last dimension, in x's dtype (gated_deltanet.py:273-275; what the DeltaNet
    block applies to q and k before the op, delta_net.py:566-575).  Differentiable."""
    if _wants_grad(x):
        return _L2Norm.apply(x)
    return _l2norm_rows_fwd(x)


def _l2norm_rows_fwd(x: Tensor) -> Tensor:
    x, back = _dense(x)
    y = torch.empty_like(x)
    d = x.shape[-1]
    _lib.check(_lib.load().lnx_l2norm_fwd(_ptr(x), _ptr(y), x.numel() // d, d, _DT[x.dtype], _stream(x)), "lnx_l2norm_fwd")
    return back(y)


def _l2norm_rows_bwd(x: Tensor, dy: Tensor) -> Tensor:
    x, back = _dense(x)
    dy = back(dy)  # same logical shape; bring it to x's dense memory order (back is its own inverse)
    dy = dy if dy.is_contiguous() else dy.contiguous()
    dx = torch.empty_like(x)
    d = x.shape[-1]
    _lib.check(_lib.load().lnx_l2norm_bwd(_ptr(x), _ptr(dy), _ptr(dx), x.numel() // d, d, _DT[x.dtype], _stream(x)),
               "lnx_l2norm_bwd")
    return back(dx)


class _L2Norm(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        ctx.save_for_backward(x)
        return _l2norm_rows_fwd(x)

    @staticmethod
    def backward(ctx, dy):
        (x,) = ctx.saved_tensors
        return _l2norm_rows_bwd(x, dy.to(x.dtype))


def _chunk_forward(q, k, v, g, beta, initial_state, scale, l2norm, o_dtype, cu_seqlens, forward_only,
                   dv_total=None, want_o=True, raw_gate=None):
    """One lnx_chunk_fwd call.  ``dv_total`` > v's columns: the state has dv_total value columns of which v holds the
    first ones and the others are zero (``value_cols``); ``want_o=False``: final states only.  Both forward-only.
    ``raw_gate = (A_log, g_bias or None, threshold)``: ``g`` is the raw per-channel gate projection in q's dtype and the
    kernels apply kda_gate's activation themselves."""
    dt, B, H, T, dk, dv_in, beta, gate, nseq, nstate, cu = _seq_setup(q, k, v, g, beta, None, cu_seqlens)
    dv = dv_in if dv_total is None else dv_total
    if initial_state is not None and tuple(initial_state.shape) != (nstate, H, dk, dv):
        raise RuntimeError(f"initial_state shape {tuple(initial_state.shape)} != {(nstate, H, dk, dv)}")
    tf = all(_is_token_first(t) for t in (q, k, v))  # [B,T,H,.] memory behind transposed views: used in place
    q_in, k_in = _as_layout(q, tf), _as_layout(k, tf)
    v = _as_layout(v, tf)
    beta_f = _as_layout(beta.to(torch.float32), tf)
    g_f = None if g is None else _as_layout(g if raw_gate is not None else g.to(torch.float32), tf)
    s0 = None if initial_state is None else _f32(initial_state)
    o = _empty_layout(B, H, T, (dv,), o_dtype, q.device, tf) if want_o else None
    sT = torch.empty(nstate, H, dk, dv, dtype=torch.float32, device=q.device)
    a = _base_args(B, H, T, dk, dv, dt, _DT[o_dtype], gate, False, scale)
    lib = _lib.load()
    # The reference's chunk path normalises in the input dtype before anything else (gated_deltanet.py:273-275,
    # kda.py:379-381).  Where the kernels scale the rows themselves (no normalised copies, gradients carried through
    # the normalisation inside lnx_chunk_bwd) they get the raw q and k; otherwise the rows are normalised first.
    fused = bool(l2norm) and bool(lib.lnx_chunk_fuses_l2norm(a))
    a.use_qk_l2norm = int(fused)
    qn = _l2norm_rows_fwd(q_in) if l2norm and not fused else q_in
    kn = _l2norm_rows_fwd(k_in) if l2norm and not fused else k_in
    a.nseq = nseq
    a.token_first = int(tf)
    a.forward_only = int(forward_only)
    a.value_cols = 0 if dv == dv_in else dv_in
    a.q, a.k, a.v, a.beta, a.g = _ptr(qn), _ptr(kn), _ptr(v), _ptr(beta_f), _ptr(g_f)
    a.initial_state, a.final_state, a.o, a.cu_seqlens = _ptr(s0), _ptr(sT), _ptr(o), _ptr(cu)
    gate_keep = ()
    if raw_gate is not None:
        A32 = raw_gate[0].detach().to(torch.float32).contiguous()
        b32 = None if raw_gate[1] is None else raw_gate[1].detach().to(torch.float32).contiguous()
        a.g, a.gate_raw, a.gate_A_log, a.gate_bias, a.gate_threshold = None, _ptr(g_f), _ptr(A32), _ptr(b32), float(raw_gate[2])
        gate_keep = (A32, b32)
    lib = _lib.load()
    nbytes = int(lib.lnx_chunk_workspace_bytes(a))
    if nbytes == 0 and T > 0 and B > 0:
        _lib.check(-2, "lnx_chunk_workspace_bytes")
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=q.device)
    a.workspace, a.workspace_bytes = _ptr(ws), nbytes
    _lib.check(lib.lnx_chunk_fwd(a, _stream(q)), "lnx_chunk_fwd")
    saved = (q_in, k_in, qn, kn, v, beta_f, g_f, s0, cu, ws) + gate_keep
    meta = (dt, B, H, T, dk, dv, gate, nseq, float(scale), bool(l2norm), o_dtype, beta.dtype,
            None if g is None else g.dtype, initial_state is not None, tf, fused)
    return o, sT, saved, meta


class _ChunkScan(torch.autograd.Function):
    """Pairs lnx_chunk_fwd with lnx_chunk_bwd (the role ``jax.custom_vjp`` plays for a JAX caller)."""

    @staticmethod
    def forward(ctx, q, k, v, g, beta, initial_state, scale, l2norm, o_dtype, cu_seqlens, grad_mode=True,
                A_log=None, g_bias=None, threshold=None):
        # nothing to differentiate (inference): the kernels skip what only the backward reads.  `grad_mode` is the
        # caller's torch.is_grad_enabled() -- inside forward() it is always off, and needs_input_grad alone is still set
        # for leaves that require grad under torch.no_grad()
        raw_gate = None if A_log is None else (A_log, g_bias, threshold)
        o, sT, saved, meta = _chunk_forward(q, k, v, g, beta, initial_state, scale, l2norm, o_dtype, cu_seqlens,
                                            forward_only=not (grad_mode and any(ctx.needs_input_grad)), raw_gate=raw_gate)
        ctx.save_for_backward(*saved)
        ctx.meta = meta
        ctx.raw_gate = None if A_log is None else (float(threshold), A_log.dtype, None if g_bias is None else g_bias.dtype)
        # an output that takes no part in the loss arrives in backward() as None, not as a tensor of zeros that a fill
        # kernel wrote and lnx_chunk_bwd would read: a null d_final_state is the kernels' "no gradient"
        ctx.set_materialize_grads(False)
        return o, sT

    @staticmethod
    def backward(ctx, d_o, d_sT):
        q_in, k_in, qn, kn, v, beta_f, g_f, s0, cu, ws = ctx.saved_tensors[:10]
        dt, B, H, T, dk, dv, gate, nseq, scale, l2norm, o_dtype, beta_dt, g_dt, has_s0, tf, fused = ctx.meta
        dev = qn.device
        d_o = torch.zeros(B, H, T, dv, dtype=qn.dtype, device=dev) if d_o is None else d_o.to(qn.dtype)
        d_o = _as_layout(d_o, tf)
        d_sT = None if d_sT is None else _f32(d_sT)
        dq, dk_, dv_ = torch.empty_like(qn), torch.empty_like(kn), torch.empty_like(v)
        dbeta = torch.empty_like(beta_f)
        dg = None if g_f is None else torch.empty_like(g_f)
        nstate = nseq if nseq else B
        ds0 = torch.empty(nstate, H, dk, dv, dtype=torch.float32, device=dev) if has_s0 else None
        a = _base_args(B, H, T, dk, dv, dt, _DT[o_dtype], gate, fused, scale)
        a.nseq = nseq
        a.token_first = int(tf)
        a.q, a.k, a.v, a.beta, a.g = _ptr(qn), _ptr(kn), _ptr(v), _ptr(beta_f), _ptr(g_f)
        a.initial_state, a.cu_seqlens = _ptr(s0), _ptr(cu)
        a.d_o, a.d_final_state = _ptr(d_o), _ptr(d_sT)
        a.d_q, a.d_k, a.d_v, a.d_beta, a.d_g, a.d_initial_state = (_ptr(dq), _ptr(dk_), _ptr(dv_), _ptr(dbeta),
                                                                   _ptr(dg), _ptr(ds0))
        a.workspace, a.workspace_bytes = _ptr(ws), ws.numel()
        dA = dbias = None
        if ctx.raw_gate is not None:  # g is the raw gate projection: its gradient and the activation's parameter gradients
            A32, b32 = ctx.saved_tensors[10:12]
            dA = torch.empty_like(A32)
            dbias = None if b32 is None else torch.empty_like(b32)
            a.g, a.d_g = None, None
            a.gate_raw, a.gate_A_log, a.gate_bias, a.gate_threshold = _ptr(g_f), _ptr(A32), _ptr(b32), ctx.raw_gate[0]
            a.d_gate_raw, a.d_gate_A_log, a.d_gate_bias = _ptr(dg), _ptr(dA), _ptr(dbias)
        _lib.check(_lib.load().lnx_chunk_bwd(a, _stream(qn)), "lnx_chunk_bwd")
        if l2norm and not fused:
            dq = _l2norm_rows_bwd(q_in, dq)
            dk_ = _l2norm_rows_bwd(k_in, dk_)
        dbeta = dbeta.to(beta_dt)
        if dg is not None:
            dg = dg.to(g_dt)
        if ctx.raw_gate is not None:
            dA = dA.to(ctx.raw_gate[1])
            dbias = None if dbias is None else dbias.to(ctx.raw_gate[2])
        return dq, dk_, dv_, dg, dbeta, ds0, None, None, None, None, None, dA, dbias, None


_CHUNK_DK = (64, 128, 256)  # key head dimensions the chunk kernels are built for


def _prefill_segments(B: int, H: int, T: int, dv: int) -> int:
    """How many segments a forward-only call is cut into (1: not at all).  The sequential kernels have one workgroup
    per (batch, head, 64 value columns); a single long prompt leaves most of the 256 CUs without one.  Segments are run
    as independent sequences -- see _segmented_forward -- for three times the scan work spread over nseg times the
    workgroups, so it pays when at most an eighth of the CUs would be busy and every segment keeps >= 64 chunks:
    measured 2.11 -> 0.84 ms for one 65536-token prompt with 4 heads of 128, 4.64 -> 3.36 ms for 131072 tokens with
    16 heads.  LNX_PREFILL_SEGMENTS forces a count (0 or 1: never)."""
    forced = os.environ.get("LNX_PREFILL_SEGMENTS")
    if forced is not None:
        return max(1, min(int(forced), -(-T // CHUNK)))
    wide = B * H * -(-dv // 64)
    if wide > 32 or T < 16384 * max(1, wide // 16):  # measured: no gain at 32 workgroups x 16384 tokens, loss at 64
        return 1
    return max(1, min(256 // wide, T // 4096))


def _segmented_forward(q, k, v, g, beta, scale, initial_state, l2norm, o_dtype, nseg):
    """Forward pass of a long sequence as nseg segments processed in parallel (no gradients).

    The scan is linear in the state: over a segment s, S_out = A_s S_in + B_s with A_s [dk, dk] the product of the
    segment's token transitions and B_s [dk, dv] what the segment writes into a zero state.  One packed call with the
    value columns extended to [v | 0] and every segment started from [0 | I] returns [B_s | A_s] as its final states;
    a short loop chains the segments' entering states; a second packed call with those as initial states gives the
    outputs.  (The same (A_s, B_s) pair is what ranks would exchange if a sequence were split across GPUs.)"""
    B, H, T, dk = q.shape
    dv = v.shape[-1]
    rows = B * H
    seg = -(-(-(-T // CHUNK)) // nseg) * CHUNK                      # whole chunks per segment
    bounds = list(range(0, T, seg)) + [T]
    nseg = len(bounds) - 1
    cu = torch.tensor(bounds, dtype=torch.int32, device=q.device)
    fold = lambda t: None if t is None else t.reshape(1, rows, *t.shape[2:])   # batch rows become heads of a packed batch
    q1, k1, v1, g1, beta1 = fold(q), fold(k), fold(v), fold(g), fold(_squeeze_beta(beta, 4))
    s_ext = torch.zeros(nseg, rows, dk, dv + dk, dtype=torch.float32, device=q.device)
    s_ext[..., dv:] = torch.eye(dk, dtype=torch.float32, device=q.device)
    _, ab, _, _ = _chunk_forward(q1, k1, v1, g1, beta1, s_ext, scale, l2norm, o_dtype, cu, forward_only=True,
                                 dv_total=dv + dk, want_o=False)  # v's columns followed by dk zero columns
    del s_ext
    Bs, As = ab[..., :dv], ab[..., dv:]
    s_in = torch.empty(nseg, rows, dk, dv, dtype=torch.float32, device=q.device)
    cur = torch.zeros(rows, dk, dv, dtype=torch.float32, device=q.device) if initial_state is None \
        else _f32(initial_state).reshape(rows, dk, dv)
    for i in range(nseg):
        s_in[i] = cur
        if i + 1 < nseg:
            cur = torch.baddbmm(Bs[i], As[i], cur)
    o, sT = _ChunkScan.apply(q1, k1, v1, g1, beta1, s_in, scale, l2norm, o_dtype, cu, torch.is_grad_enabled())
    return o.reshape(B, H, T, dv), sT[nseg - 1].reshape(B, H, dk, dv)


def _chunk(q, k, v, g, beta, scale, initial_state, chunk_size, l2norm, o_dtype, need_mult16, cu_seqlens):
    if need_mult16 and chunk_size % 16 != 0:
        # gated_deltanet.py:318-320, kda.py:438-440
        raise ValueError(f"chunk_size (BT={chunk_size}) must be divisible by BC=16.")
    if chunk_size <= 0:
        raise ValueError(f"chunk_size must be positive, got {chunk_size}")
    if scale is None:
        scale = q.shape[-1] ** -0.5
    q, k, v, back = _promote(q, k, v)
    if back is not None:  # computed in float32; o_dtype is what the caller gets
        o, sT = _chunk(q, k, v, g, beta, scale, initial_state, chunk_size, l2norm, torch.float32, need_mult16, cu_seqlens)
        return o.to(o_dtype), sT
    dk, dv = q.shape[-1], v.shape[-1]
    dkp = next((c for c in _CHUNK_DK if dk <= c), None)
    dvp = -(-dv // 64) * 64
    if dkp is None or q.dim() != 4 or (dkp, dvp) == (dk, dv):
        if dkp is not None and q.dim() == 4 and cu_seqlens is None and not _wants_grad(q, k, v, g, beta, initial_state):
            nseg = _prefill_segments(q.shape[0], q.shape[1], q.shape[2], dv)
            if nseg > 1:
                return _segmented_forward(q, k, v, g, beta, scale, initial_state, l2norm, o_dtype, nseg)
        return _ChunkScan.apply(q, k, v, g, beta, initial_state, scale, l2norm, o_dtype, cu_seqlens, torch.is_grad_enabled())
    # Head dimensions between the kernels' sizes (the reference's own tests use dk = 8, 16, dv = 8, 32):
    # zero channels are exact.  A zero key/query channel adds nothing to any <q,k>, <k,k> or |x|_2, the state rows
    # and columns it would feed stay zero, and the padded value columns are independent of the others; autograd
    # slices the gradients back.  `scale` was fixed above from the true dk.
    pad = torch.nn.functional.pad
    q, k, v = pad(q, (0, dkp - dk)), pad(k, (0, dkp - dk)), pad(v, (0, dvp - dv))
    if g is not None and g.dim() == 4 and g.shape[-1] == dk:
        g = pad(g, (0, dkp - dk))
    if initial_state is not None:
        initial_state = pad(initial_state, (0, dvp - dv, 0, dkp - dk))
    o, sT = _ChunkScan.apply(q, k, v, g, beta, initial_state, scale, l2norm, o_dtype, cu_seqlens, torch.is_grad_enabled())
    return o[..., :dv], sT[..., :dk, :dv]


def delta_rule_chunkwise(q, k, v, beta, initial_state=None, chunk_size=64, scale=None, backend=None, *,
                         cu_seqlens=None):
    """Chunked (WY) DeltaNet scan (delta_net.py:216-354).  ``chunk_size`` is validated and then
    ignored: the kernels always use 64-token chunks, which the result does not depend on."""
    return _chunk(q, k, v, None, beta, scale, initial_state, chunk_size, False, q.dtype, False, cu_seqlens)


def gated_delta_rule_chunkwise(q, k, v, g, beta, scale=None, initial_state=None, chunk_size=64,
                               use_qk_l2norm=True, *, cu_seqlens=None):
    """Chunked Gated DeltaNet scan, ``g [B,H,T]`` (gated_deltanet.py:232-534)."""
    return _chunk(q, k, v, g, beta, scale, initial_state, chunk_size, use_qk_l2norm, q.dtype, True, cu_seqlens)


def kda_chunkwise(q, k, v, g, beta, scale=None, initial_state=None, chunk_size=64, use_qk_l2norm=True, *,
                  cu_seqlens=None, output_dtype=torch.float32):
    """Chunked KDA scan, ``g [B,H,T,dk]`` (kda.py:350-655).  Like the reference, the output is
    float32 whatever the input dtype (kda.py:416, :655); pass ``output_dtype`` to change that."""
    return _chunk(q, k, v, g, beta, scale, initial_state, chunk_size, use_qk_l2norm, output_dtype, True, cu_seqlens)


def kda_chunkwise_raw_gate(q, k, v, g_raw, beta, A_log, g_bias=None, scale=None, initial_state=None, chunk_size=64,
                           use_qk_l2norm=True, *, threshold=20.0, cu_seqlens=None, output_dtype=torch.float32):
    """``kda_gate`` (kda.py:120-172) and ``kda_chunkwise`` (kda.py:350-655) as one op: the KDA block's two steps between
    its projections and its output norm without the fp32 log-decay tensor in between.

    ``g_raw [B,H,T,dk]`` is the raw gate projection in q's dtype -- the block's ``[B,T,H*dk]`` viewed as
    ``[B,T,H,dk].transpose(1, 2)`` is used in place, like q, k, v; ``A_log [H]``, ``g_bias [H*dk]`` as in ``kda_gate``.
    Equal to ``kda_chunkwise(q, k, v, kda_gate(g_raw, A_log, dk, g_bias, out_dtype=float32)[0], beta, ...)`` with the
    activation computed in fp32 inside the chunk kernels; differentiable with respect to q, k, v, g_raw, beta,
    initial_state, A_log and g_bias.  dk must be 64, 128 or 256 and dv a multiple of 64."""
    if chunk_size % 16 != 0:
        raise ValueError(f"chunk_size (BT={chunk_size}) must be divisible by BC=16.")  # kda.py:438-440
    if q.dim() != 4 or q.shape[-1] not in _CHUNK_DK or v.shape[-1] % 64 != 0:
        raise RuntimeError(f"kda_chunkwise_raw_gate needs [B,H,T,d] inputs with dk in {_CHUNK_DK} and dv % 64 == 0, "
                           f"got q {tuple(q.shape)}, v {tuple(v.shape)}")
    if not (q.dtype == k.dtype == v.dtype == g_raw.dtype) or q.dtype not in _DT:
        raise RuntimeError("q, k, v and g_raw must share one of the dtypes float32 / bfloat16")
    if tuple(g_raw.shape) != tuple(q.shape):
        raise RuntimeError(f"g_raw {tuple(g_raw.shape)} must have q's shape {tuple(q.shape)}")
    H, dk = q.shape[1], q.shape[-1]
    if tuple(A_log.shape) != (H,) or (g_bias is not None and tuple(g_bias.shape) != (H * dk,)):
        raise RuntimeError(f"A_log must be [{H}] and g_bias [{H * dk}]")
    if scale is None:
        scale = dk ** -0.5
    return _ChunkScan.apply(q, k, v, g_raw, beta, initial_state, scale, use_qk_l2norm, output_dtype, cu_seqlens,
                            torch.is_grad_enabled(), A_log, g_bias, float(threshold))
