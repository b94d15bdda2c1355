"""Token-by-token delta-rule recurrences and single decode steps (numpy).

TEST INFRASTRUCTURE: the ground truth the HIP kernels are checked against.

Each public function restates one reference op; tensors are head-first
``[B, H, T, d]`` like the reference's.  ``dtype`` selects the arithmetic type
(``np.float64`` for truth, ``np.float32`` to mimic the reference's precision).

Reference lines followed:
  delta_rule_recurrent        linearnexus/modules/linear_attn/delta_net.py:158-213
  delta_rule_step             linearnexus/modules/linear_attn/delta_net.py:378-397
  gated_delta_rule_recurrent  linearnexus/modules/linear_attn/gated_deltanet.py:165-229
  gated_delta_rule_step       linearnexus/modules/linear_attn/gated_deltanet.py:565-597
  kda_recurrent               linearnexus/modules/linear_attn/kda.py:215-283
  kda_step                    linearnexus/modules/linear_attn/kda.py:312-347
"""

from __future__ import annotations

import numpy as np

L2_EPS = 1e-6


def l2norm(x: np.ndarray) -> np.ndarray:
    """``x / (||x||_2 + 1e-6)`` over the last axis (gated_deltanet.py:193-195)."""
    n = np.sqrt(np.sum(x * x, axis=-1, keepdims=True))
    return x / (n + x.dtype.type(L2_EPS))


def _prep_beta(beta: np.ndarray, ndim: int) -> np.ndarray:
    # delta_net.py:166-167 -- a trailing singleton on beta is squeezed.
    if beta.ndim == ndim:
        beta = beta[..., 0]
    return beta


def delta_rule_recurrent(q, k, v, beta, initial_state=None, scale=None, dtype=np.float64):
    """Plain DeltaNet: v_old=S^T k; d=beta(v-v_old); S+=k d^T; o=S^T (scale q)."""
    B, H, T, dk = q.shape
    dv = v.shape[-1]
    if scale is None:
        scale = dk ** -0.5
    beta = _prep_beta(np.asarray(beta), 4)
    q = np.asarray(q, dtype) * dtype(scale)  # delta_net.py:170
    k = np.asarray(k, dtype)
    v = np.asarray(v, dtype)
    beta = np.asarray(beta, dtype)
    S = np.zeros((B, H, dk, dv), dtype) if initial_state is None else np.array(initial_state, dtype)
    o = np.empty((B, H, T, dv), dtype)
    for t in range(T):
        k_t, v_t, q_t, b_t = k[:, :, t], v[:, :, t], q[:, :, t], beta[:, :, t]
        v_old = np.einsum("bhkv,bhk->bhv", S, k_t)  # :189
        v_delta = b_t[..., None] * (v_t - v_old)  # :192
        S = S + np.einsum("bhk,bhv->bhkv", k_t, v_delta)  # :195
        o[:, :, t] = np.einsum("bhk,bhkv->bhv", q_t, S)  # :198
    return o, S


def delta_rule_step(q, k, v, beta, state, scale=None, dtype=np.float64):
    """One token of :func:`delta_rule_recurrent` on ``[B, H, d]`` vectors."""
    beta = _prep_beta(np.asarray(beta), 3)
    o, S = delta_rule_recurrent(
        q[:, :, None], k[:, :, None], v[:, :, None], beta[:, :, None], state, scale, dtype
    )
    return o[:, :, 0], S


def gated_delta_rule_recurrent(
    q, k, v, g, beta, scale=None, initial_state=None, use_qk_l2norm=True, dtype=np.float64
):
    """Gated DeltaNet: S'=exp(g_t) S, then the delta rule on S' (scalar gate per head)."""
    B, H, T, dk = q.shape
    dv = v.shape[-1]
    if scale is None:
        scale = dk ** -0.5
    beta = _prep_beta(np.asarray(beta), 4)
    q = np.asarray(q, dtype)
    k = np.asarray(k, dtype)
    v = np.asarray(v, dtype)
    g = np.asarray(g, dtype)
    beta = np.asarray(beta, dtype)
    S = np.zeros((B, H, dk, dv), dtype) if initial_state is None else np.array(initial_state, dtype)
    o = np.empty((B, H, T, dv), dtype)
    for t in range(T):
        k_t, v_t, q_t = k[:, :, t], v[:, :, t], q[:, :, t]
        if use_qk_l2norm:  # :193-195
            q_t = l2norm(q_t)
            k_t = l2norm(k_t)
        q_t = q_t * dtype(scale)  # :197
        S = S * np.exp(g[:, :, t])[..., None, None]  # :200-201
        v_old = np.einsum("bhkv,bhk->bhv", S, k_t)  # :204
        v_delta = beta[:, :, t][..., None] * (v_t - v_old)  # :207
        S = S + np.einsum("bhk,bhv->bhkv", k_t, v_delta)  # :210
        o[:, :, t] = np.einsum("bhk,bhkv->bhv", q_t, S)  # :213
    return o, S


def gated_delta_rule_step(q, k, v, g, beta, state, scale=None, use_qk_l2norm=True, dtype=np.float64):
    beta = _prep_beta(np.asarray(beta), 3)
    o, S = gated_delta_rule_recurrent(
        q[:, :, None], k[:, :, None], v[:, :, None], np.asarray(g)[:, :, None], beta[:, :, None],
        scale, state, use_qk_l2norm, dtype,
    )
    return o[:, :, 0], S


def kda_recurrent(
    q, k, v, g, beta, scale=None, initial_state=None, use_qk_l2norm=True, dtype=np.float64
):
    """KDA: S'=diag(exp(g_t)) S; r=v-S'^T k; S=S'+(beta k) r^T (vector gate over dk)."""
    B, H, T, dk = q.shape
    dv = v.shape[-1]
    if scale is None:
        scale = dk ** -0.5
    beta = _prep_beta(np.asarray(beta), 4)
    q = np.asarray(q, dtype)
    k = np.asarray(k, dtype)
    v = np.asarray(v, dtype)
    g = np.asarray(g, dtype)
    beta = np.asarray(beta, dtype)
    S = np.zeros((B, H, dk, dv), dtype) if initial_state is None else np.array(initial_state, dtype)
    o = np.empty((B, H, T, dv), dtype)
    for t in range(T):
        k_t, v_t, q_t = k[:, :, t], v[:, :, t], q[:, :, t]
        if use_qk_l2norm:  # :243-245
            q_t = l2norm(q_t)
            k_t = l2norm(k_t)
        q_t = q_t * dtype(scale)  # :247
        S = S * np.exp(g[:, :, t])[..., None]  # :251-252
        v_old = np.einsum("bhk,bhkv->bhv", k_t, S)  # :257
        v_delta = v_t - v_old  # :260 (no beta here)
        S = S + np.einsum("bhk,bhv->bhkv", beta[:, :, t][..., None] * k_t, v_delta)  # :264
        o[:, :, t] = np.einsum("bhk,bhkv->bhv", q_t, S)  # :267
    return o, S


def kda_step(q, k, v, g, beta, state, scale=None, use_qk_l2norm=True, dtype=np.float64):
    beta = _prep_beta(np.asarray(beta), 3)
    o, S = kda_recurrent(
        q[:, :, None], k[:, :, None], v[:, :, None], np.asarray(g)[:, :, None], beta[:, :, None],
        scale, state, use_qk_l2norm, dtype,
    )
    return o[:, :, 0], S


def varlen(fn, cu_seqlens, *seq_args, initial_state=None, **kw):
    """Packed variable-length batch: run ``fn`` once per sequence slice.

    ``seq_args`` are ``[1, H, T, ...]`` tensors packed along T; ``cu_seqlens`` is
    ``[0, l1, l1+l2, ..., T]``; ``initial_state`` is ``[Nseq, H, dk, dv]`` or None.
    Returns ``o [1,H,T,dv]`` and ``S_T [Nseq,H,dk,dv]``.  This is the definition
    of the state reset at sequence boundaries (the reference has no such op).
    """
    outs, states = [], []
    for s in range(len(cu_seqlens) - 1):
        a, b = int(cu_seqlens[s]), int(cu_seqlens[s + 1])
        sl = [x[:, :, a:b] for x in seq_args]
        s0 = None if initial_state is None else initial_state[s : s + 1]
        o, S = fn(*sl, initial_state=s0, **kw)
        outs.append(o)
        states.append(S)
    return np.concatenate(outs, axis=2), np.concatenate(states, axis=0)
