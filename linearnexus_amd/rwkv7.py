"""RWKV-7's diagonal-plus-low-rank delta rule on MI355X behind the reference's op names.

``dplr_delta_rule_recurrent(q, k, v, a, b, gk, scale=1.0, initial_state=None)`` and
``dplr_delta_rule_step(q, k, v, a, b, gk, state, scale=1.0)`` mirror
linearnexus/modules/linear_attn/rwkv7.py:114-265 (names, positional order, defaults, ``(output, state)`` returns,
output in ``q.dtype``, fp32 state).  The reference has no chunked form of this recurrence, and neither has this
module.  Both ops are differentiable with respect to q, k, v, a, b, gk and the state, as the reference's are under
jax.grad (its RWKV-7 block trains through the scan): the HIP backward kernel recomputes the states from checkpoints.
Additive: ``dplr_delta_rule_step(..., inplace=True)`` updates the state buffer in place (not differentiable).  There
is no other code path: the ops raise if the library is missing.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import DplrArgs, DplrBwdArgs
from .linear_attn import _DT, _check_inputs, _f32, _ptr, _stream

Tensor = torch.Tensor


def _args(q, k, v, a, b, gk, lead_dims):
    dt = _check_inputs(q, k, v)
    if q.dim() != lead_dims + 1:
        raise RuntimeError(f"expected {lead_dims + 1}-dimensional q, got {tuple(q.shape)}")
    for name, t in (("a", a), ("b", b), ("gk", gk)):
        if tuple(t.shape) != tuple(q.shape):
            raise RuntimeError(f"{name} shape {tuple(t.shape)} != q shape {tuple(q.shape)}")
    if a.dtype != q.dtype or b.dtype != q.dtype:
        raise RuntimeError(f"a and b must have q's dtype {q.dtype}, got {a.dtype}, {b.dtype}")
    return dt


def _fill(args, step, q, k, v, a, b, gk, s_in, scale):
    args.B, args.H = q.shape[0], q.shape[1]
    args.T = 1 if step else q.shape[2]
    args.dk, args.dv = q.shape[-1], v.shape[-1]
    args.dtype = args.o_dtype = _DT[q.dtype]
    args.scale = float(scale)
    args.q, args.k, args.v, args.a, args.b, args.gk = (_ptr(x) for x in (q, k, v, a, b, gk))
    args.initial_state = _ptr(s_in)


def _call(fn_name, step, q, k, v, a, b, gk, s_in, s_out, scale):
    o = torch.empty(v.shape, dtype=q.dtype, device=q.device)
    q, k, v, a, b = (x.contiguous() for x in (q, k, v, a, b))
    gk = _f32(gk)
    args = DplrArgs()
    _fill(args, step, q, k, v, a, b, gk, s_in, scale)
    args.final_state, args.o = _ptr(s_out), _ptr(o)
    lib = _lib.load()
    _lib.check(getattr(lib, fn_name)(args, _stream(q)), fn_name)
    return o


class _DplrScan(torch.autograd.Function):
    """The scan under autograd: forward = lnx_dplr_recurrent_fwd, backward = lnx_dplr_recurrent_bwd."""

    @staticmethod
    def forward(ctx, q, k, v, a, b, gk, s0, scale):
        B, H, _, dk = q.shape
        q, k, v, a, b = (x.detach().contiguous() for x in (q, k, v, a, b))
        gk32 = _f32(gk.detach())
        s_in = None if s0 is None else _f32(s0.detach())
        s_out = torch.empty(B, H, dk, v.shape[-1], dtype=torch.float32, device=q.device)
        o = _call("lnx_dplr_recurrent_fwd", False, q, k, v, a, b, gk32, s_in, s_out, scale)
        ctx.save_for_backward(q, k, v, a, b, gk32, s_in)
        ctx.meta = (float(scale), gk.dtype, None if s0 is None else s0.dtype)
        return o, s_out

    @staticmethod
    def backward(ctx, d_o, d_s):
        q, k, v, a, b, gk32, s_in = ctx.saved_tensors
        scale, gk_dt, s0_dt = ctx.meta
        B, H, T, dk = q.shape
        dv = v.shape[-1]
        dev = q.device
        lib = _lib.load()
        g = DplrBwdArgs()
        _fill(g.fwd, False, q, k, v, a, b, gk32, s_in, scale)
        d_o = torch.zeros_like(v) if d_o is None else d_o.to(q.dtype).contiguous()
        d_s = None if d_s is None else _f32(d_s)
        new = lambda *shape: torch.empty(*shape, dtype=torch.float32, device=dev)
        dq, dk_, da, db, dgk = (new(B, H, T, dk) for _ in range(5))
        dv_ = new(B, H, T, dv)
        ds0 = new(B, H, dk, dv) if (s_in is not None and ctx.needs_input_grad[6]) else None
        nbytes = int(lib.lnx_dplr_recurrent_bwd_workspace_bytes(B, H, T, dk, dv))
        ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=dev)
        g.d_o, g.d_final_state = _ptr(d_o), _ptr(d_s)
        g.dq, g.dk, g.dv, g.da, g.db, g.dgk = (_ptr(x) for x in (dq, dk_, dv_, da, db, dgk))
        g.d_initial_state, g.workspace, g.workspace_bytes = _ptr(ds0), _ptr(ws), nbytes
        _lib.check(lib.lnx_dplr_recurrent_bwd(g, _stream(q)), "lnx_dplr_recurrent_bwd")
        dt = q.dtype
        return (dq.to(dt), dk_.to(dt), dv_.to(dt), da.to(dt), db.to(dt), dgk.to(gk_dt),
                None if ds0 is None else ds0.to(s0_dt), None)


def _wants_grad(*tensors):
    return torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in tensors)


def dplr_delta_rule_recurrent(q: Tensor, k: Tensor, v: Tensor, a: Tensor, b: Tensor, gk: Tensor, scale: float = 1.0,
                              initial_state: Optional[Tensor] = None) -> Tuple[Tensor, Tensor]:
    """Token-by-token DPLR scan over ``[B,H,T,.]`` tensors (rwkv7.py:114-213)."""
    _args(q, k, v, a, b, gk, 3)
    B, H, _, dk = q.shape
    dv = v.shape[-1]
    s_in = None
    if initial_state is not None:
        if tuple(initial_state.shape) != (B, H, dk, dv):
            raise RuntimeError(f"initial_state shape {tuple(initial_state.shape)} != {(B, H, dk, dv)}")
        s_in = _f32(initial_state)
    if _wants_grad(q, k, v, a, b, gk, initial_state):
        if dv > 256:
            raise RuntimeError(f"the DPLR backward kernel takes dv <= 256, got {dv}")
        return _DplrScan.apply(q, k, v, a, b, gk, initial_state, scale)
    s_out = torch.empty(B, H, dk, dv, dtype=torch.float32, device=q.device)
    return _call("lnx_dplr_recurrent_fwd", False, q, k, v, a, b, gk, s_in, s_out, scale), s_out


def dplr_delta_rule_step(q: Tensor, k: Tensor, v: Tensor, a: Tensor, b: Tensor, gk: Tensor, state: Tensor,
                         scale: float = 1.0, *, inplace: bool = False) -> Tuple[Tensor, Tensor]:
    """One decode token of the DPLR rule on ``[B,H,.]`` vectors (rwkv7.py:216-265)."""
    _args(q, k, v, a, b, gk, 2)
    B, H, dk = q.shape
    dv = v.shape[-1]
    if tuple(state.shape) != (B, H, dk, dv):
        raise RuntimeError(f"state shape {tuple(state.shape)} != {(B, H, dk, dv)}")
    if _wants_grad(q, k, v, a, b, gk, state):
        if inplace:
            raise RuntimeError("cannot differentiate through a step that updates its state in place")
        o, s_out = dplr_delta_rule_recurrent(*(x.unsqueeze(2) for x in (q, k, v, a, b, gk)), scale, state)
        return o.squeeze(2), s_out
    if inplace:
        if state.dtype != torch.float32 or not state.is_contiguous():
            raise RuntimeError("inplace=True needs a contiguous float32 state")
        s_in = s_out = state
    else:
        s_in = _f32(state)
        s_out = torch.empty_like(s_in)
    return _call("lnx_dplr_step", True, q, k, v, a, b, gk, s_in, s_out, scale), s_out
