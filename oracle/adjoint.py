"""Token-level reverse recurrence: the gradient of the recurrent delta rule (numpy).

TEST INFRASTRUCTURE.  The reference has no backward code: gradients there come from
JAX autodiff through ``lax.scan`` over the recurrent step
(linearnexus/train/sft.py:108-137 -> gated_deltanet.py:185-215, kda.py:227-269,
delta_net.py:181-200).  This file is the hand-derived adjoint of that step; it is
pinned by central finite differences and by ``torch.autograd`` in the tests.

Forward step (alpha = exp(g_t): 1 for DeltaNet, scalar for Gated, a dk-vector for KDA):
    S' = alpha * S_prev ; r = v - S'^T k ; d = beta r ; S = S' + k d^T ; o = S^T (scale * qh)
with qh, kh the (optionally) L2-normalised q, k.
"""

from __future__ import annotations

import numpy as np

from .recurrent import L2_EPS, _prep_beta


def _l2_fwd(x):
    n = np.sqrt(np.sum(x * x, -1, keepdims=True))
    return x / (n + L2_EPS), n


def _l2_bwd(x, n, dy):
    # y = x / (n + eps):  dx = dy/(n+eps) - x <x,dy> / (n (n+eps)^2)
    s = n + L2_EPS
    inner = np.sum(x * dy, -1, keepdims=True)
    return dy / s - x * inner / (np.maximum(n, 1e-300) * s * s)


def delta_rule_adjoint(
    q, k, v, beta, dO, g=None, dS_T=None, scale=None, initial_state=None,
    use_qk_l2norm=False, dtype=np.float64,
):
    """Gradients of (o, S_T) wrt (q, k, v, beta, g, S0) contracted with (dO, dS_T).

    ``g`` is None (DeltaNet), ``[B,H,T]`` (Gated) or ``[B,H,T,dk]`` (KDA).
    Returns a dict with keys dq, dk, dv, dbeta, dg (None without a gate), dS0.
    """
    B, H, T, dk = q.shape
    dv_ = v.shape[-1]
    if scale is None:
        scale = dk ** -0.5
    beta = np.asarray(_prep_beta(np.asarray(beta), 4), dtype)
    q = np.asarray(q, dtype)
    k = np.asarray(k, dtype)
    v = np.asarray(v, dtype)
    dO = np.asarray(dO, dtype)
    if g is not None:
        g = np.asarray(g, dtype)
    vector_gate = g is not None and g.ndim == 4
    if use_qk_l2norm:
        qh, qn = _l2_fwd(q)
        kh, kn = _l2_fwd(k)
    else:
        qh, kh = q, k
    S = np.zeros((B, H, dk, dv_), dtype) if initial_state is None else np.array(initial_state, dtype)

    def alpha_of(t):
        if g is None:
            return None
        a = np.exp(g[:, :, t])
        return a[..., None] if vector_gate else a[..., None, None]

    prev, resid = [], []
    for t in range(T):  # forward sweep, keeping S_{t-1} and r_t
        prev.append(S)
        a = alpha_of(t)
        Sp = S if a is None else S * a
        r = v[:, :, t] - np.einsum("bhkv,bhk->bhv", Sp, kh[:, :, t])
        resid.append(r)
        S = Sp + np.einsum("bhk,bhv->bhkv", kh[:, :, t], beta[:, :, t][..., None] * r)

    dS = np.zeros_like(S) if dS_T is None else np.array(dS_T, dtype)
    dqh = np.zeros_like(q)
    dkh = np.zeros_like(k)
    dv = np.zeros_like(v)
    dbeta = np.zeros_like(beta)
    dg = None if g is None else np.zeros_like(g)
    S_t = S
    for t in range(T - 1, -1, -1):
        k_t, b_t, r = kh[:, :, t], beta[:, :, t][..., None], resid[t]
        a = alpha_of(t)
        Sp = prev[t] if a is None else prev[t] * a
        dS = dS + np.einsum("bhk,bhv->bhkv", qh[:, :, t] * scale, dO[:, :, t])
        dqh[:, :, t] = scale * np.einsum("bhkv,bhv->bhk", S_t, dO[:, :, t])
        dd = np.einsum("bhkv,bhk->bhv", dS, k_t)
        dkh[:, :, t] = np.einsum("bhkv,bhv->bhk", dS, b_t * r) - np.einsum("bhkv,bhv->bhk", Sp, b_t * dd)
        dbeta[:, :, t] = np.sum(dd * r, -1)
        dv[:, :, t] = b_t * dd
        dSp = dS - np.einsum("bhk,bhv->bhkv", k_t, b_t * dd)
        if a is None:
            dS = dSp
        else:
            if vector_gate:
                dg[:, :, t] = np.sum(dSp * prev[t], -1) * a[..., 0]
            else:
                dg[:, :, t] = np.sum(dSp * prev[t], (-1, -2)) * a[..., 0, 0]
            dS = dSp * a
        S_t = prev[t]
    if use_qk_l2norm:
        dq = _l2_bwd(q, qn, dqh)
        dk_ = _l2_bwd(k, kn, dkh)
    else:
        dq, dk_ = dqh, dkh
    return {"dq": dq, "dk": dk_, "dv": dv, "dbeta": dbeta, "dg": dg, "dS0": dS}
