"""fp64 restatement of the reference's short causal depthwise convolution -- TEST INFRASTRUCTURE ONLY.

Follows linearnexus/core/conv.py:13-68 (``depthwise_conv1d_causal``) and the SiLU the blocks apply to its
output (gated_deltanet.py:765-779).  Pinned in tests/test_oracle_conv.py by scipy's FIR filter
(``lfilter`` with the taps reversed), by the step-by-step == whole-sequence property the reference tests
(tests/test_comprehensive.py:57-83), by a brute-force triple loop, and -- the gradient -- by central finite
differences and an independent ``torch.nn.functional.conv1d`` + autograd.
"""
import numpy as np


def silu(z):
    return z / (1.0 + np.exp(-z))


def depthwise_conv1d_causal(inputs, weight, bias=None, cache=None, activation=None):
    """inputs [B,T,D], weight [K,D], bias [D]|None, cache [B,K-1,D]|None -> (y [B,T,D], new_cache [B,K-1,D]).

    conv.py:56-67: the cache (zeros when absent) is put in front of the inputs, a VALID cross-correlation
    runs over that, the last T outputs are kept, and the new cache is the last K-1 rows of the
    concatenation.  conv.py:39-44: a width-1 kernel is the identity (+ bias) with an empty cache."""
    x = np.asarray(inputs, np.float64)
    w = np.asarray(weight, np.float64)
    B, T, D = x.shape
    K = w.shape[0]
    if K < 1:
        raise ValueError("kernel_size must be >= 1")
    if cache is None:
        cache = np.zeros((B, K - 1, D))
    cache = np.asarray(cache, np.float64)
    if cache.shape != (B, K - 1, D):
        raise ValueError(f"cache shape must be (batch, kernel-1, channels); got {cache.shape}")
    xin = np.concatenate([cache, x], axis=1)
    z = np.zeros((B, T, D))
    for j in range(K):
        z += (1.0 if K == 1 else w[j]) * xin[:, j:j + T]  # conv.py:39-44: a width-1 kernel ignores its weight
    if bias is not None:
        z = z + np.asarray(bias, np.float64)
    y = silu(z) if activation == "silu" else z
    return y, xin[:, xin.shape[1] - (K - 1):]


def depthwise_conv1d_causal_grad(inputs, weight, bias, dy, cache=None, activation=None, with_cache=False):
    """Gradients of <y, dy> with respect to inputs, weight and bias -- and the carry-in cache with ``with_cache``."""
    x = np.asarray(inputs, np.float64)
    w = np.asarray(weight, np.float64)
    dy = np.asarray(dy, np.float64)
    B, T, D = x.shape
    K = w.shape[0]
    if cache is None:
        cache = np.zeros((B, K - 1, D))
    xin = np.concatenate([np.asarray(cache, np.float64), x], axis=1)
    wk = np.ones_like(w) if K == 1 else w
    z = sum(wk[j] * xin[:, j:j + T] for j in range(K))
    if bias is not None:
        z = z + np.asarray(bias, np.float64)
    if activation == "silu":
        s = 1.0 / (1.0 + np.exp(-z))
        dz = dy * s * (1.0 + z * (1.0 - s))
    else:
        dz = dy
    dxin = np.zeros_like(xin)
    dw = np.zeros_like(w)
    for j in range(K):
        dxin[:, j:j + T] += wk[j] * dz
        if K > 1:
            dw[j] = (dz * xin[:, j:j + T]).sum((0, 1))
    if with_cache:
        return dxin[:, K - 1:], dw, dz.sum((0, 1)), dxin[:, :K - 1]
    return dxin[:, K - 1:], dw, dz.sum((0, 1))


def packed(fn, cu_seqlens, inputs, *args, **kw):
    """``fn`` applied to each sequence [cu[s], cu[s+1]) of a packed batch ``inputs [1,T,D]`` on its own (zero cache); the
    first result of every call concatenated along T, the others summed (parameter gradients)."""
    outs = [fn(inputs[:, a:b], *[x[:, a:b] if (hasattr(x, "ndim") and x.ndim == 3) else x for x in args], **kw)
            for a, b in zip(cu_seqlens[:-1], cu_seqlens[1:])]
    first = np.concatenate([o[0] for o in outs], axis=1)
    return (first,) + tuple(sum(o[i] for o in outs) for i in range(1, len(outs[0])))
