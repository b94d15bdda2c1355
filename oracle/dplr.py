"""fp64 restatement of the reference's RWKV-7 diagonal-plus-low-rank recurrence -- TEST INFRASTRUCTURE ONLY.

Follows linearnexus/modules/linear_attn/rwkv7.py:114-213 (scan) and :216-265 (step).  Pinned in
tests/test_oracle_dplr.py by the explicit transition-matrix form on tiny inputs, by its reduction to the KDA
recurrence (a = -exp(g) k, b = beta k, key beta k: the two oracles are independent code), by the pure-decay
closed form (a = b = 0), by step == scan(T=1) and by split invariance.
"""
import numpy as np


def dplr_delta_rule_step(q, k, v, a, b, gk, state, scale=1.0):
    """q,k,a,b,gk [B,H,dk], v [B,H,dv], state [B,H,dk,dv] -> (o [B,H,dv], new state).  rwkv7.py:250-263."""
    q, k, v, a, b, gk, h = (np.asarray(x, np.float64) for x in (q, k, v, a, b, gk, state))
    a_h = np.einsum("bhk,bhkv->bhv", a, h)                                      # :252
    h = np.exp(gk)[..., None] * h + b[..., None] * a_h[..., None, :]            # :253
    h = h + np.einsum("bhk,bhv->bhkv", k, v)                                    # :256-257
    return np.einsum("bhkv,bhk->bhv", h, q * scale), h                          # :260


def dplr_delta_rule_recurrent(q, k, v, a, b, gk, scale=1.0, initial_state=None):
    """[B,H,T,.] tensors; returns (o [B,H,T,dv], final state [B,H,dk,dv]).  rwkv7.py:148-213."""
    B, H, T, dk = np.shape(q)
    dv = np.shape(v)[-1]
    h = np.zeros((B, H, dk, dv)) if initial_state is None else np.asarray(initial_state, np.float64)
    o = np.zeros((B, H, T, dv))
    for t in range(T):
        sl = lambda x: np.asarray(x)[:, :, t]
        o[:, :, t], h = dplr_delta_rule_step(sl(q), sl(k), sl(v), sl(a), sl(b), sl(gk), h, scale)
    return o, h
