"""Chunk-parallel (WY) forms of the delta rule, restated in numpy.

TEST INFRASTRUCTURE.  A second restatement, independent of ``recurrent.py``:
it follows the reference's chunk algorithms step by step, so that
chunk == recurrent (which the reference's own tests assert only loosely) can be
asserted here at fp64 round-off.

Reference lines followed:
  delta_rule_chunkwise        linearnexus/modules/linear_attn/delta_net.py:250-354
  gated_delta_rule_chunkwise  linearnexus/modules/linear_attn/gated_deltanet.py:265-534
  kda_chunkwise               linearnexus/modules/linear_attn/kda.py:372-655
"""

from __future__ import annotations

import numpy as np

from .recurrent import l2norm, _prep_beta

BC = 16  # sub-block edge used for M / Aqk (gated_deltanet.py:318, kda.py:438)


def _pad_T(x, pad):
    if pad == 0:
        return x
    width = [(0, 0)] * x.ndim
    width[2] = (0, pad)
    return np.pad(x, width)


def delta_rule_chunkwise(q, k, v, beta, initial_state=None, chunk_size=64, scale=None, dtype=np.float64):
    B, H, T, dk = q.shape
    dv = v.shape[-1]
    if scale is None:
        scale = dk ** -0.5
    beta = _prep_beta(np.asarray(beta), 4)
    q = np.asarray(q, dtype) * dtype(scale)  # :261
    k = np.asarray(k, dtype)
    v = np.asarray(v, dtype)
    beta = np.asarray(beta, dtype)
    C = chunk_size
    pad = (C - T % C) % C  # :267
    q, k, v, beta = (_pad_T(x, pad) for x in (q, k, v, beta))
    N = (T + pad) // C
    S = np.zeros((B, H, dk, dv), dtype) if initial_state is None else np.array(initial_state, dtype)
    eye = np.eye(C, dtype=dtype)
    tril_incl = np.tril(np.ones((C, C), dtype))
    o = np.empty((B, H, N * C, dv), dtype)
    for n in range(N):
        sl = slice(n * C, (n + 1) * C)
        q_c, k_c, v_c, b_c = q[:, :, sl], k[:, :, sl], v[:, :, sl], beta[:, :, sl]
        kk = np.einsum("bhik,bhjk->bhij", k_c, k_c)  # :297
        A = np.tril(b_c[..., :, None] * kk, -1)  # :298
        A_inv = np.linalg.solve(eye + A, np.broadcast_to(eye, A.shape))  # :301-311
        w = np.einsum("bhij,bhjk->bhik", A_inv, k_c * b_c[..., None])  # :314-316
        u = np.einsum("bhij,bhjv->bhiv", A_inv, v_c * b_c[..., None])  # :317
        v_new = u - np.einsum("bhik,bhkv->bhiv", w, S)  # :320-321
        qk = np.einsum("bhik,bhjk->bhij", q_c, k_c) * tril_incl  # :325-326
        o[:, :, sl] = np.einsum("bhik,bhkv->bhiv", q_c, S) + np.einsum("bhij,bhjv->bhiv", qk, v_new)
        S = S + np.einsum("bhik,bhiv->bhkv", k_c, v_new)  # :330
    return o[:, :, :T], S


def _gated_chunk_core(q, k, v, G, beta, S, C, dtype):
    """Shared body of the Gated / KDA chunk forms with ``G [B,H,N*C,dk]`` per-chunk cumsums.

    Builds M and Aqk from 16x16 blocks -- diagonal blocks by masked exponentials of gate
    differences, off-diagonal blocks through a per-row-block reference gate so that both
    exponentials are <= 1 -- then forward-substitutes ``M [w|u] = [beta k e^G | beta v]``
    and scans the chunks (kda.py:483-523, :569-648; gated_deltanet.py:353-398, :444-523).
    """
    B, H, TT, dk = q.shape
    dv = v.shape[-1]
    N = TT // C
    if C % BC != 0:
        raise ValueError(f"chunk_size (BT={C}) must be divisible by BC={BC}.")
    NC = C // BC
    o = np.empty((B, H, TT, dv), dtype)
    incl = np.tril(np.ones((BC, BC), bool))
    strict = np.tril(np.ones((BC, BC), bool), -1)
    for n in range(N):
        sl = slice(n * C, (n + 1) * C)
        q_c, k_c, v_c, g_c, b_c = q[:, :, sl], k[:, :, sl], v[:, :, sl], G[:, :, sl], beta[:, :, sl]
        M = np.zeros((B, H, C, C), dtype)
        Aqk = np.zeros((B, H, C, C), dtype)
        for i in range(NC):
            r = slice(i * BC, (i + 1) * BC)
            g_ref = g_c[:, :, i * BC]  # first row of the row block
            # diagonal block: exponent differences masked *before* exp
            d = g_c[:, :, r, None, :] - g_c[:, :, None, r, :]  # [B,H,BC,BC,dk]
            e_strict = np.exp(np.where(strict[None, None, :, :, None], d, -np.inf))
            e_incl = np.exp(np.where(incl[None, None, :, :, None], d, -np.inf))
            kk = k_c[:, :, r, None, :] * k_c[:, :, None, r, :]
            qk = q_c[:, :, r, None, :] * k_c[:, :, None, r, :]
            M[:, :, r, r] = np.eye(BC, dtype=dtype) + (kk * e_strict).sum(-1) * b_c[:, :, r, None]
            Aqk[:, :, r, r] = (qk * e_incl).sum(-1)
            row_scale = np.exp(np.minimum(g_c[:, :, r] - g_ref[:, :, None], 0))
            for j in range(i):
                c = slice(j * BC, (j + 1) * BC)
                col_scale = np.exp(np.minimum(g_ref[:, :, None] - g_c[:, :, c], 0))
                kc = k_c[:, :, c] * col_scale
                M[:, :, r, c] = np.einsum("bhik,bhjk->bhij", k_c[:, :, r] * row_scale, kc) * b_c[:, :, r, None]
                Aqk[:, :, r, c] = np.einsum("bhik,bhjk->bhij", q_c[:, :, r] * row_scale, kc)
        eg = np.exp(g_c)
        rhs = np.concatenate([b_c[..., None] * k_c * eg, b_c[..., None] * v_c], -1)
        X = np.zeros_like(rhs)
        for t in range(C):  # unit-lower forward substitution (kda.py:575-596)
            X[:, :, t] = rhs[:, :, t] - np.einsum("bhj,bhjd->bhd", M[:, :, t, :t], X[:, :, :t])
        w, u = X[..., :dk], X[..., dk:]
        v_i = u - np.einsum("bhck,bhkv->bhcv", w, S)
        o[:, :, sl] = np.einsum("bhck,bhkv->bhcv", q_c * eg, S) + np.einsum("bhij,bhjv->bhiv", Aqk, v_i)
        g_last = g_c[:, :, -1]  # [B,H,dk]
        ratio = np.exp(np.minimum(g_last[:, :, None] - g_c, 0))
        S = S * eg[:, :, -1][..., None] + np.einsum("bhck,bhcv->bhkv", ratio * k_c, v_i)
    return o, S


def _gated_common(q, k, v, g, beta, scale, initial_state, chunk_size, use_qk_l2norm, dtype, vector_gate):
    B, H, T, dk = q.shape
    dv = v.shape[-1]
    if scale is None:
        scale = dk ** -0.5
    beta = _prep_beta(np.asarray(beta), 4)
    q = np.asarray(q, dtype)
    k = np.asarray(k, dtype)
    if use_qk_l2norm:
        q, k = l2norm(q), l2norm(k)
    q = q * dtype(scale)
    v = np.asarray(v, dtype)
    g = np.asarray(g, dtype)
    beta = np.asarray(beta, dtype)
    C = chunk_size
    pad = (C - T % C) % C
    q, k, v, g, beta = (_pad_T(x, pad) for x in (q, k, v, g, beta))
    N = (T + pad) // C
    gshape = g.shape
    G = np.cumsum(g.reshape(B, H, N, C, *gshape[3:]), axis=3).reshape(gshape)
    if not vector_gate:
        G = np.broadcast_to(G[..., None], (B, H, N * C, dk))
    S = np.zeros((B, H, dk, dv), dtype) if initial_state is None else np.array(initial_state, dtype)
    o, S = _gated_chunk_core(q, k, v, G, beta, S, C, dtype)
    return o[:, :, :T], S


def gated_delta_rule_chunkwise(
    q, k, v, g, beta, scale=None, initial_state=None, chunk_size=64, use_qk_l2norm=True, dtype=np.float64
):
    return _gated_common(q, k, v, g, beta, scale, initial_state, chunk_size, use_qk_l2norm, dtype, False)


def kda_chunkwise(
    q, k, v, g, beta, scale=None, initial_state=None, chunk_size=64, use_qk_l2norm=True, dtype=np.float64
):
    return _gated_common(q, k, v, g, beta, scale, initial_state, chunk_size, use_qk_l2norm, dtype, True)
