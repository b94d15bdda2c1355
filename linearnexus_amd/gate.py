"""KDA's gate activation on MI355X behind the reference's function name.

``kda_gate(g, A_log, head_k_dim, g_bias=None, beta=None, threshold=20.0)`` mirrors
linearnexus/modules/linear_attn/kda.py:120-172: ``g [B,T,H*dk]`` -> ``-exp(A_log)[h] * softplus(g + g_bias)`` reshaped
to ``[B,T,H,dk]``, plus ``sigmoid(beta)`` in fp32 when ``beta`` is given.  Additive: ``out_dtype`` (default: the
input's dtype, like the reference; ``torch.float32`` feeds ``kda_chunkwise`` without a cast and without rounding the
log-decay to bf16).  Differentiable with respect to g, A_log, g_bias and beta through the HIP kernels; there is no
other code path.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib
from .linear_attn import _DT, _ptr, _stream

Tensor = torch.Tensor


class _KdaGate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, g, A_log, g_bias, dk, threshold, out_dtype):
        B, T, D = g.shape
        H = A_log.shape[0]
        g2 = g.contiguous()
        a32 = A_log.detach().to(torch.float32).contiguous()
        b32 = None if g_bias is None else g_bias.detach().to(torch.float32).contiguous()
        out = torch.empty(B, T, H, dk, dtype=out_dtype, device=g.device)
        _lib.check(_lib.load().lnx_kda_gate_fwd(_ptr(g2), _ptr(a32), _ptr(b32), _ptr(out), B * T, H, dk, float(threshold),
                                                _DT[g.dtype], _DT[out_dtype], _stream(g)), "lnx_kda_gate_fwd")
        ctx.save_for_backward(g2, a32, b32)
        ctx.meta = (dk, float(threshold), out_dtype, A_log.dtype, None if g_bias is None else g_bias.dtype)
        return out

    @staticmethod
    def backward(ctx, d_out):
        g2, a32, b32 = ctx.saved_tensors
        dk, threshold, out_dtype, adt, bdt = ctx.meta
        B, T, D = g2.shape
        H = a32.shape[0]
        d_out = d_out.to(out_dtype).contiguous()
        d_g = torch.empty_like(g2)
        d_a = torch.empty_like(a32)
        d_b = None if b32 is None else torch.empty_like(b32)
        lib = _lib.load()
        nws = int(lib.lnx_kda_gate_bwd_workspace_bytes(B * T, H, dk))
        ws = torch.empty(max(nws, 1), dtype=torch.uint8, device=g2.device)
        _lib.check(lib.lnx_kda_gate_bwd(_ptr(g2), _ptr(a32), _ptr(b32), _ptr(d_out), _ptr(d_g), _ptr(d_a), _ptr(d_b), B * T, H, dk,
                                        threshold, _DT[g2.dtype], _DT[out_dtype], _ptr(ws), nws, _stream(g2)), "lnx_kda_gate_bwd")
        return d_g, d_a.to(adt), None if d_b is None else d_b.to(bdt), None, None, None


class _Sigmoid(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x):
        x32 = x.to(torch.float32).contiguous()
        y = torch.empty_like(x32)
        _lib.check(_lib.load().lnx_sigmoid_fwd(_ptr(x32), _ptr(y), x32.numel(), _stream(x)), "lnx_sigmoid_fwd")
        ctx.save_for_backward(y)
        ctx.xdt = x.dtype
        return y

    @staticmethod
    def backward(ctx, dy):
        (y,) = ctx.saved_tensors
        dy = dy.to(torch.float32).contiguous()
        dx = torch.empty_like(y)
        _lib.check(_lib.load().lnx_sigmoid_bwd(_ptr(y), _ptr(dy), _ptr(dx), y.numel(), _stream(y)), "lnx_sigmoid_bwd")
        return dx.to(ctx.xdt)


def kda_gate(g: Tensor, A_log: Tensor, head_k_dim: int, g_bias: Optional[Tensor] = None, beta: Optional[Tensor] = None,
             threshold: float = 20.0, *, out_dtype: Optional[torch.dtype] = None) -> Tuple[Tensor, Optional[Tensor]]:
    """KDA gate computation (kda.py:120-172): returns ``(g_out [B,T,H,dk], sigmoid(beta) or None)``."""
    if not isinstance(g, torch.Tensor) or not g.is_cuda:
        raise RuntimeError("g must be a torch.Tensor on the GPU; the op runs on the GPU only")
    if g.dtype not in _DT:
        raise RuntimeError(f"unsupported dtype {g.dtype}: use float32 or bfloat16")
    if g.dim() != 3 or A_log.dim() != 1 or g.shape[-1] != A_log.shape[0] * head_k_dim:
        raise RuntimeError(f"g {tuple(g.shape)} must be [batch, seq, {A_log.shape[0]} * {head_k_dim}]")
    if g_bias is not None and tuple(g_bias.shape) != (g.shape[-1],):
        raise RuntimeError(f"g_bias must be [{g.shape[-1]}], got {tuple(g_bias.shape)}")
    out_dtype = g.dtype if out_dtype is None else out_dtype
    if out_dtype not in _DT:
        raise RuntimeError(f"unsupported out_dtype {out_dtype}")
    g_out = _KdaGate.apply(g, A_log, g_bias, int(head_k_dim), threshold, out_dtype)
    beta_out = None if beta is None else _Sigmoid.apply(beta)
    return g_out, beta_out
