"""Gate activations of the KDA and Gated DeltaNet blocks on MI355X.

``kda_gate(g, A_log, head_k_dim, g_bias=None, beta=None, threshold=20.0)`` mirrors
linearnexus/modules/linear_attn/kda.py:120-172: ``g [B,T,H*dk]`` -> ``-exp(A_log)[h] * softplus(g + g_bias)`` reshaped
to ``[B,T,H,dk]``, plus ``sigmoid(beta)`` in fp32 when ``beta`` is given.  Additive: ``out_dtype`` (default: the
input's dtype, like the reference; ``torch.float32`` feeds ``kda_chunkwise`` without a cast and without rounding the
log-decay to bf16).  Differentiable with respect to g, A_log, g_bias and beta through the HIP kernels; there is no
other code path.

``gated_deltanet_gate(a, A_log, dt_bias, b=None, allow_neg_eigval=False)`` is what the Gated DeltaNet block computes
inline between its projections and the scan (gated_deltanet.py:804-815): ``g = -exp(A_log) * softplus(a + dt_bias)`` and
``beta = sigmoid(b)`` (times 2 with ``allow_neg_eigval``), both ``[..., H]`` in fp32 like the reference's.
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


class _GdnGate(torch.autograd.Function):
    @staticmethod
    def forward(ctx, a, b, A_log, dt_bias, beta_scale):
        H = A_log.shape[0]
        a2 = a.contiguous()
        b2 = None if b is None else b.to(a.dtype).contiguous()
        A32 = A_log.detach().to(torch.float32).contiguous()
        bias32 = None if dt_bias is None else dt_bias.detach().to(torch.float32).contiguous()
        g = torch.empty(a.shape, dtype=torch.float32, device=a.device)
        beta = None if b is None else torch.empty(a.shape, dtype=torch.float32, device=a.device)
        rows = a2.numel() // H
        _lib.check(_lib.load().lnx_gdn_gate_fwd(_ptr(a2), _ptr(b2), _ptr(A32), _ptr(bias32), _ptr(g), _ptr(beta), rows, H,
                                                float(beta_scale), _DT[a.dtype], _stream(a)), "lnx_gdn_gate_fwd")
        ctx.save_for_backward(a2, b2, A32, bias32)
        ctx.meta = (float(beta_scale), A_log.dtype, None if dt_bias is None else dt_bias.dtype, None if b is None else b.dtype)
        return g, beta

    @staticmethod
    def backward(ctx, d_g, d_beta):
        a2, b2, A32, bias32 = ctx.saved_tensors
        beta_scale, adt, biasdt, bdt = ctx.meta
        H = A32.shape[0]
        rows = a2.numel() // H
        d_g = None if d_g is None else d_g.to(torch.float32).contiguous()
        d_beta = None if (d_beta is None or b2 is None) else d_beta.to(torch.float32).contiguous()
        d_a = torch.empty_like(a2)
        d_b = None if b2 is None else torch.empty_like(b2)
        d_A = torch.empty_like(A32)
        d_bias = None if bias32 is None else torch.empty_like(bias32)
        lib = _lib.load()
        nws = int(lib.lnx_gdn_gate_bwd_workspace_bytes(rows, H))
        ws = torch.empty(max(nws, 1), dtype=torch.uint8, device=a2.device)
        _lib.check(lib.lnx_gdn_gate_bwd(_ptr(a2), _ptr(b2), _ptr(A32), _ptr(bias32), _ptr(d_g), _ptr(d_beta), _ptr(d_a), _ptr(d_b),
                                        _ptr(d_A), _ptr(d_bias), rows, H, beta_scale, _DT[a2.dtype], _ptr(ws), nws, _stream(a2)),
                   "lnx_gdn_gate_bwd")
        return (d_a, None if d_b is None else d_b.to(bdt), d_A.to(adt), None if d_bias is None else d_bias.to(biasdt), None)


def gated_deltanet_gate(a: Tensor, A_log: Tensor, dt_bias: Optional[Tensor] = None, b: Optional[Tensor] = None,
                        allow_neg_eigval: bool = False) -> Tuple[Tensor, Optional[Tensor]]:
    """Gated DeltaNet's decay gate and learning rate (gated_deltanet.py:804-815): returns ``(g, beta or None)`` in fp32,
    shaped like ``a`` (``[..., H]``: the block's ``[batch, seq, num_v_heads]``, which it then transposes)."""
    if not isinstance(a, torch.Tensor) or not a.is_cuda:
        raise RuntimeError("a must be a torch.Tensor on the GPU; the op runs on the GPU only")
    if a.dtype not in _DT:
        raise RuntimeError(f"unsupported dtype {a.dtype}: use float32 or bfloat16")
    if A_log.dim() != 1 or a.dim() < 1 or a.shape[-1] != A_log.shape[0]:
        raise RuntimeError(f"a {tuple(a.shape)} must end in the {A_log.shape[0]} heads of A_log")
    if dt_bias is not None and tuple(dt_bias.shape) != tuple(A_log.shape):
        raise RuntimeError(f"dt_bias must be [{A_log.shape[0]}], got {tuple(dt_bias.shape)}")
    if b is not None and tuple(b.shape) != tuple(a.shape):
        raise RuntimeError(f"b {tuple(b.shape)} must have a's shape {tuple(a.shape)}")
    return _GdnGate.apply(a, b, A_log, dt_bias, 2.0 if allow_neg_eigval else 1.0)
