"""Short causal depthwise convolution (+ fused SiLU) on MI355X behind the reference's helper name.

``depthwise_conv1d_causal(inputs, weight, bias, *, cache=None)`` mirrors linearnexus/core/conv.py:13-68:
``inputs [B,T,D]``, ``weight [K,D]`` (K <= 4), ``bias [D]`` or None, ``cache [B,K-1,D]`` or None; returns
``(output, new_cache)``.  Additive: ``activation="silu"`` fuses the SiLU the blocks apply right after
(gated_deltanet.py:765-779), ``inplace_cache=True`` writes the new cache over the old one (decode) and
``cu_seqlens`` makes the batch packed (``inputs [1,T,D]``: the taps stop at the start of each sequence, as if
every sequence went through the function on its own with a zero cache -- the layout the chunk ops take).
Differentiable with respect to inputs, weight, bias and the carry-in cache through the HIP backward kernels.
There is no other code path: the ops raise if the library is missing.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch

from . import _lib
from .linear_attn import _DT, _check_cu_seqlens, _ptr, _stream

Tensor = torch.Tensor
_ACT = {None: 0, "none": 0, "silu": 1}


def _check(inputs: Tensor, weight: Tensor, bias: Optional[Tensor], cache: Optional[Tensor]):
    if not isinstance(inputs, torch.Tensor) or not inputs.is_cuda:
        raise RuntimeError("inputs must be a torch.Tensor on the GPU; the convolution runs on the GPU only")
    if inputs.dim() != 3:
        raise RuntimeError(f"inputs must be [batch, seq, channels], got {tuple(inputs.shape)}")
    if inputs.dtype not in _DT:
        raise RuntimeError(f"unsupported dtype {inputs.dtype}: use float32 or bfloat16")
    B, T, D = inputs.shape
    if weight.dim() != 2 or weight.shape[1] != D:
        raise RuntimeError(f"weight must be [kernel, {D}], got {tuple(weight.shape)}")
    K = weight.shape[0]
    if K < 1:
        raise ValueError("kernel_size must be >= 1")  # conv.py:36-37
    if K > 4:
        raise RuntimeError(f"kernel_size {K} is not supported (1..4)")
    if bias is not None and tuple(bias.shape) != (D,):
        raise RuntimeError(f"bias must be [{D}], got {tuple(bias.shape)}")
    if cache is not None and K > 1 and tuple(cache.shape) != (B, K - 1, D):
        raise ValueError(  # conv.py:49-53
            f"cache shape must be (batch, kernel-1, channels); got {tuple(cache.shape)} for kernel_size={K}")
    return B, T, D, K


class _Conv(torch.autograd.Function):
    @staticmethod
    def forward(ctx, x, weight, bias, cache, act, inplace_cache, cu):
        B, T, D = x.shape
        K = weight.shape[0]
        lib = _lib.load()
        x = x.contiguous()
        w32 = weight.detach().to(torch.float32).contiguous()
        b32 = None if bias is None else bias.detach().to(torch.float32).contiguous()
        if cache is not None and K > 1:
            if inplace_cache:
                if cache.dtype != x.dtype or not cache.is_contiguous():
                    raise RuntimeError("inplace_cache=True needs a contiguous cache of the inputs' dtype")
                cin = new_cache = cache
            else:
                cin = cache.detach().to(x.dtype).contiguous()
                new_cache = torch.empty_like(cin)
        else:
            cin = None
            new_cache = torch.empty(B, K - 1, D, dtype=x.dtype, device=x.device)
        y = torch.empty_like(x)
        if cu is None:
            _lib.check(lib.lnx_conv1d_fwd(_ptr(x), _ptr(w32), _ptr(b32), _ptr(cin), _ptr(y), _ptr(new_cache),
                                          B, T, D, K, _DT[x.dtype], act, _stream(x)), "lnx_conv1d_fwd")
        else:
            _lib.check(lib.lnx_conv1d_packed_fwd(_ptr(x), _ptr(w32), _ptr(b32), _ptr(cu), cu.numel() - 1, _ptr(y), _ptr(new_cache),
                                                 T, D, K, _DT[x.dtype], act, _stream(x)), "lnx_conv1d_packed_fwd")
        ctx.save_for_backward(x, w32, b32, None if inplace_cache else cin, cu)
        ctx.meta = (act, weight.dtype, None if bias is None else bias.dtype, inplace_cache and cin is not None,
                    None if cache is None else cache.dtype)
        ctx.mark_non_differentiable(new_cache)
        return y, new_cache

    @staticmethod
    def backward(ctx, dy, _dcache):
        x, w32, b32, cin, cu = ctx.saved_tensors
        act, wdt, bdt, lost_cache, cdt = ctx.meta
        if lost_cache:
            raise RuntimeError("cannot differentiate through a convolution whose cache was updated in place")
        B, T, D = x.shape
        K = w32.shape[0]
        dy = dy.to(x.dtype).contiguous()
        dx = torch.empty_like(x)
        dw = torch.empty_like(w32)
        db = None if b32 is None else torch.empty_like(b32)
        lib = _lib.load()
        if cu is None:
            _lib.check(lib.lnx_conv1d_bwd(_ptr(x), _ptr(w32), _ptr(b32), _ptr(cin), _ptr(dy), _ptr(dx), _ptr(dw),
                                          _ptr(db), B, T, D, K, _DT[x.dtype], act, _stream(x)), "lnx_conv1d_bwd")
        else:
            _lib.check(lib.lnx_conv1d_packed_bwd(_ptr(x), _ptr(w32), _ptr(b32), _ptr(cu), cu.numel() - 1, _ptr(dy), _ptr(dx),
                                                 _ptr(dw), _ptr(db), T, D, K, _DT[x.dtype], act, _stream(x)), "lnx_conv1d_packed_bwd")
        dc = None
        if cin is not None and ctx.needs_input_grad[3] and K > 1:
            dc = torch.empty_like(cin)
            _lib.check(lib.lnx_conv1d_cache_bwd(_ptr(x), _ptr(w32), _ptr(b32), _ptr(cin), _ptr(dy), _ptr(dc), B, T, D, K,
                                                _DT[x.dtype], act, _stream(x)), "lnx_conv1d_cache_bwd")
            dc = dc.to(cdt)
        return dx, dw.to(wdt), None if db is None else db.to(bdt), dc, None, None, None


def depthwise_conv1d_causal(inputs: Tensor, weight: Tensor, bias: Optional[Tensor] = None, *,
                            cache: Optional[Tensor] = None, activation: Optional[str] = None,
                            inplace_cache: bool = False, cu_seqlens=None) -> Tuple[Tensor, Tensor]:
    """Depthwise causal conv1d with optional cache warm-start (linearnexus/core/conv.py:13-68)."""
    B, T, D, K = _check(inputs, weight, bias, cache)
    if activation not in _ACT:
        raise ValueError(f"activation must be None or 'silu', got {activation!r}")
    cu = None
    if cu_seqlens is not None:
        if B != 1:
            raise RuntimeError("cu_seqlens needs a packed batch with B == 1")
        if cache is not None:
            raise RuntimeError("a packed batch starts every sequence from a zero cache: pass cache=None")
        cu = _check_cu_seqlens(cu_seqlens, T).to(device=inputs.device, dtype=torch.int32).contiguous()
    return _Conv.apply(inputs, weight, bias, cache, _ACT[activation], bool(inplace_cache), cu)
