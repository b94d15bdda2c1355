"""fp64 restatement of the reference's gated RMSNorm epilogue -- TEST INFRASTRUCTURE ONLY.

Follows FusedRMSNormGated.__call__ (linearnexus/modules/linear_attn/kda.py:683-700).  Pinned in
tests/test_oracle_norm.py by torch's own ``rms_norm`` + ``sigmoid`` (a library routine) with autograd, and by
central finite differences.
"""
import numpy as np


def rmsnorm_gated(x, gate, weight, eps=1e-5):
    """x, gate [..., d] (gate None = no gate), weight [d]."""
    x = np.asarray(x, np.float64)
    variance = np.mean(x ** 2, axis=-1, keepdims=True)                  # kda.py:694
    y = x / np.sqrt(variance + eps) * np.asarray(weight, np.float64)    # :695-696
    if gate is not None:
        y = y / (1.0 + np.exp(-np.asarray(gate, np.float64)))           # :699
    return y


def rmsnorm_gated_grad(x, gate, weight, dy, eps=1e-5):
    """Gradients of <y, dy>: (dx, dgate or None, dweight)."""
    x, w, dy = (np.asarray(a, np.float64) for a in (x, weight, dy))
    d = x.shape[-1]
    rstd = 1.0 / np.sqrt(np.mean(x ** 2, axis=-1, keepdims=True) + eps)
    xn = x * rstd
    s = np.ones_like(x) if gate is None else 1.0 / (1.0 + np.exp(-np.asarray(gate, np.float64)))
    u = dy * s * w
    dx = rstd * (u - xn * np.sum(u * xn, -1, keepdims=True) / d)
    dgate = None if gate is None else dy * xn * w * s * (1.0 - s)
    dw = (dy * xn * s).reshape(-1, d).sum(0)
    return dx, dgate, dw
