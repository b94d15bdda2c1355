"""RWKV-7's diagonal-plus-low-rank delta rule on MI355X behind the reference's op names.

``dplr_delta_rule_recurrent(q, k, v, a, b, gk, scale=1.0, initial_state=None)`` and
``dplr_delta_rule_step(q, k, v, a, b, gk, state, scale=1.0)`` mirror
linearnexus/modules/linear_attn/rwkv7.py:114-265 (names, positional order, defaults, ``(output, state)`` returns,
output in ``q.dtype``, fp32 state).  The reference has no chunked form of this recurrence, and neither has this
module.  Additive: ``dplr_delta_rule_step(..., inplace=True)`` updates the state buffer in place.  There is no
other code path: the ops raise if the library is missing.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib
from ._lib import DplrArgs
from .linear_attn import _DT, _check_inputs, _f32, _ptr, _stream

Tensor = torch.Tensor


def _args(q, k, v, a, b, gk, lead_dims):
    dt = _check_inputs(q, k, v)
    if torch.is_grad_enabled() and any(t.requires_grad for t in (q, k, v, a, b, gk)):
        # no silent loss of gradients: the rule has a forward (decode / prefill) kernel only
        raise RuntimeError("the DPLR delta rule has no backward pass here: call it under torch.no_grad() or on "
                           "detached tensors")
    if q.dim() != lead_dims + 1:
        raise RuntimeError(f"expected {lead_dims + 1}-dimensional q, got {tuple(q.shape)}")
    for name, t in (("a", a), ("b", b), ("gk", gk)):
        if tuple(t.shape) != tuple(q.shape):
            raise RuntimeError(f"{name} shape {tuple(t.shape)} != q shape {tuple(q.shape)}")
    if a.dtype != q.dtype or b.dtype != q.dtype:
        raise RuntimeError(f"a and b must have q's dtype {q.dtype}, got {a.dtype}, {b.dtype}")
    return dt


def _call(fn_name, step, q, k, v, a, b, gk, s_in, s_out, scale):
    dt = _DT[q.dtype]
    B, H = q.shape[0], q.shape[1]
    T = 1 if step else q.shape[2]
    dk, dv = q.shape[-1], v.shape[-1]
    o = torch.empty(v.shape, dtype=q.dtype, device=q.device)
    q, k, v, a, b = (x.contiguous() for x in (q, k, v, a, b))
    gk = _f32(gk)
    args = DplrArgs()
    args.B, args.H, args.T, args.dk, args.dv = B, H, T, dk, dv
    args.dtype = args.o_dtype = dt
    args.scale = float(scale)
    args.q, args.k, args.v, args.a, args.b, args.gk = (_ptr(x) for x in (q, k, v, a, b, gk))
    args.initial_state, args.final_state, args.o = _ptr(s_in), _ptr(s_out), _ptr(o)
    lib = _lib.load()
    _lib.check(getattr(lib, fn_name)(args, _stream(q)), fn_name)
    return o


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
    if inplace:
        if state.dtype != torch.float32 or not state.is_contiguous():
            raise RuntimeError("inplace=True needs a contiguous float32 state")
        s_in = s_out = state
    else:
        s_in = _f32(state)
        s_out = torch.empty_like(s_in)
    return _call("lnx_dplr_step", True, q, k, v, a, b, gk, s_in, s_out, scale), s_out
