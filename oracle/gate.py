"""fp64 restatement of the reference's KDA gate activation -- TEST INFRASTRUCTURE ONLY.

Follows kda_gate (linearnexus/modules/linear_attn/kda.py:120-172).  Pinned in tests/test_oracle_gate.py by torch's
``softplus(threshold=...)`` + autograd (a library routine), finite differences, and the closed forms at 0 and above
the threshold.
"""
import numpy as np


def kda_gate(g, A_log, head_k_dim, g_bias=None, beta=None, threshold=20.0):
    """g [B,T,H*dk], A_log [H], g_bias [H*dk]|None, beta [B,T,H]|None -> (g_out [B,T,H,dk], sigmoid(beta)|None)."""
    g = np.asarray(g, np.float64)
    if g_bias is not None:
        g = g + np.asarray(g_bias, np.float64)                                  # kda.py:146-147
    B, T, _ = g.shape
    H = np.shape(A_log)[0]
    g = g.reshape(B, T, H, head_k_dim)                                          # :150-152
    a_exp = -np.exp(np.asarray(A_log, np.float64))                              # :155
    sp = np.where(g > threshold, g, np.log1p(np.exp(np.minimum(g, threshold))))  # :158-163
    out = a_exp[None, None, :, None] * sp                                       # :166
    beta_out = None if beta is None else 1.0 / (1.0 + np.exp(-np.asarray(beta, np.float64)))  # :169-170
    return out, beta_out


def kda_gate_grad(g, A_log, head_k_dim, d_out, g_bias=None, threshold=20.0):
    """Gradients of <g_out, d_out>: (d_g [B,T,H*dk], d_A_log [H], d_bias [H*dk])."""
    g = np.asarray(g, np.float64)
    x = g if g_bias is None else g + np.asarray(g_bias, np.float64)
    B, T, D = x.shape
    H = np.shape(A_log)[0]
    x4 = x.reshape(B, T, H, head_k_dim)
    a_exp = -np.exp(np.asarray(A_log, np.float64))[None, None, :, None]
    sp = np.where(x4 > threshold, x4, np.log1p(np.exp(np.minimum(x4, threshold))))
    dsp = np.where(x4 > threshold, 1.0, 1.0 / (1.0 + np.exp(-x4)))
    d_out = np.asarray(d_out, np.float64)
    d_g = (d_out * a_exp * dsp).reshape(B, T, D)
    return d_g, (d_out * a_exp * sp).sum((0, 1, 3)), d_g.sum((0, 1))
