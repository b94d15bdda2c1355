"""Gated RMSNorm output epilogue on MI355X: ``rmsnorm_gated(x, gate, weight, eps)`` computes what the reference's
``FusedRMSNormGated`` module does in its ``__call__`` (linearnexus/modules/linear_attn/kda.py:664-700):
``RMSNorm(x) * weight * sigmoid(gate)`` over the last dimension; ``gate=None`` gives the plain RMSNorm the blocks
use without an output gate (gated_deltanet.py:861-862).  Differentiable with respect to x, gate and weight through
the HIP backward kernel.  There is no other code path: the op raises if the library is missing.
"""
from __future__ import annotations

from typing import Optional

import torch

from . import _lib
from .linear_attn import _DT, _ptr, _stream

Tensor = torch.Tensor


class _RmsNormGated(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, gate, weight, eps):
        d = x.shape[-1]
        x2 = x.contiguous().view(-1, d)
        g2 = None if gate is None else gate.to(x.dtype).contiguous().view(-1, d)
        w32 = weight.detach().to(torch.float32).contiguous()
        y = torch.empty_like(x2)
        _lib.check(_lib.load().lnx_rmsnorm_gated_fwd(_ptr(x2), _ptr(g2), _ptr(w32), _ptr(y), x2.shape[0], d, float(eps),
                                                     _DT[x.dtype], _stream(x)), "lnx_rmsnorm_gated_fwd")
        ctx.save_for_backward(x2, g2, w32)
        ctx.meta = (float(eps), x.shape, weight.dtype, None if gate is None else gate.dtype)
        return y.view(x.shape)

    @staticmethod
    def backward(ctx, dy):
        x2, g2, w32 = ctx.saved_tensors
        eps, shape, wdt, gdt = ctx.meta
        d = x2.shape[-1]
        dy2 = dy.to(x2.dtype).contiguous().view(-1, d)
        dx = torch.empty_like(x2)
        dg = None if g2 is None else torch.empty_like(g2)
        dw = torch.empty_like(w32)
        lib = _lib.load()
        nws = lib.lnx_rmsnorm_gated_bwd_workspace_bytes(x2.shape[0], d, _DT[x2.dtype])
        ws = torch.empty(max(int(nws), 1), dtype=torch.uint8, device=x2.device)
        _lib.check(lib.lnx_rmsnorm_gated_bwd(_ptr(x2), _ptr(g2), _ptr(w32), _ptr(dy2), _ptr(dx), _ptr(dg), _ptr(dw),
                                             x2.shape[0], d, eps, _DT[x2.dtype], _ptr(ws), int(nws), _stream(x2)),
                   "lnx_rmsnorm_gated_bwd")
        return dx.view(shape), None if dg is None else dg.view(shape).to(gdt), dw.to(wdt), None


def rmsnorm_gated(x: Tensor, gate: Optional[Tensor], weight: Tensor, eps: float = 1e-5) -> Tensor:
    """``x * rsqrt(mean(x^2, -1) + eps) * weight * sigmoid(gate)`` (kda.py:683-700); ``x, gate [..., d]``, ``weight [d]``."""
    if not isinstance(x, torch.Tensor) or not x.is_cuda:
        raise RuntimeError("x must be a torch.Tensor on the GPU; the op runs on the GPU only")
    if x.dtype not in _DT:
        raise RuntimeError(f"unsupported dtype {x.dtype}: use float32 or bfloat16")
    if gate is not None and gate.shape != x.shape:
        raise RuntimeError(f"gate shape {tuple(gate.shape)} != x shape {tuple(x.shape)}")
    if tuple(weight.shape) != (x.shape[-1],):
        raise RuntimeError(f"weight must be [{x.shape[-1]}], got {tuple(weight.shape)}")
    return _RmsNormGated.apply(x, gate, weight, eps)
