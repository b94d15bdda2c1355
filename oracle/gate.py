"""fp64 restatement of the reference's gate activations -- TEST INFRASTRUCTURE ONLY.

``kda_gate`` follows kda_gate (linearnexus/modules/linear_attn/kda.py:120-172); ``gdn_gate`` follows the lines of the
Gated DeltaNet block between its projections and the scan (gated_deltanet.py:804-815).  Pinned in
tests/test_oracle_gate.py by torch's ``softplus`` + autograd (a library routine), finite differences, and closed forms.
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


def gdn_gate(a, A_log, dt_bias=None, b=None, allow_neg_eigval=False):
    """a, b [..., H], A_log, dt_bias [H] -> (g = -exp(A_log) softplus(a + dt_bias), beta = sigmoid(b) (* 2) | None)."""
    x = np.asarray(a, np.float64) + (0.0 if dt_bias is None else np.asarray(dt_bias, np.float64))
    g = -np.exp(np.asarray(A_log, np.float64)) * (np.maximum(x, 0.0) + np.log1p(np.exp(-np.abs(x))))  # :811-814
    beta = None
    if b is not None:
        beta = 1.0 / (1.0 + np.exp(-np.asarray(b, np.float64)))                                     # :804
        if allow_neg_eigval:
            beta = beta * 2.0                                                                        # :806-807
    return g, beta


def gdn_gate_grad(a, A_log, d_g, dt_bias=None, b=None, d_beta=None, allow_neg_eigval=False):
    """Gradients of <g, d_g> + <beta, d_beta>: (d_a, d_A_log [H], d_dt_bias [H], d_b | None)."""
    x = np.asarray(a, np.float64) + (0.0 if dt_bias is None else np.asarray(dt_bias, np.float64))
    na = -np.exp(np.asarray(A_log, np.float64))
    d_g = np.asarray(d_g, np.float64)
    sp = np.maximum(x, 0.0) + np.log1p(np.exp(-np.abs(x)))
    d_a = d_g * na / (1.0 + np.exp(-x))
    red = tuple(range(x.ndim - 1))
    d_b = None
    if b is not None:
        s = 1.0 / (1.0 + np.exp(-np.asarray(b, np.float64)))
        d_b = np.asarray(d_beta, np.float64) * (2.0 if allow_neg_eigval else 1.0) * s * (1.0 - s)
    return d_a, (d_g * na * sp).sum(red), d_a.sum(red), d_b
