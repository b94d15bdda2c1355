"""Chunk-level forward and backward, split the way the HIP kernels are split (numpy).

TEST INFRASTRUCTURE.  Every intermediate tensor a kernel writes to its workspace is exposed
here under the same name, so a kernel can be checked stage by stage.  The forward follows
the WY chunk algorithm of linearnexus/modules/linear_attn/gated_deltanet.py:444-523 and
kda.py:569-648 (delta_net.py:296-330 is the gate-free case); the backward is its hand-derived
adjoint (the reference has none) and is pinned against ``adjoint.py`` / autograd in the tests.

Notation per (batch, head) and chunk of C tokens, S = state entering the chunk:
  G = cumsum(g) inside the chunk, Gam = exp(G), E_ij = exp(G_i - G_j) (inside the dk sum for
  a vector gate), GC = G at the chunk's last row.
  X_ij = <k_i, k_j>_E (i>j)        A = diag(beta) X         Tm = (I + A)^-1
  P_ij = scale <q_i, k_j>_E (i>=j)
  W = Tm diag(beta) (K*Gam)        U = Tm diag(beta) V
  D = U - W S                      O = scale (Q*Gam) S + P D
  S' = exp(GC) * S + (K * exp(GC - G))^T D
"""
from __future__ import annotations

import numpy as np

C = 64


def _chunks(x, T):
    """[B,H,T,...] -> [B,H,N,C,...] zero padded."""
    pad = (C - T % C) % C
    if pad:
        w = [(0, 0)] * x.ndim
        w[2] = (0, pad)
        x = np.pad(x, w)
    return x.reshape(x.shape[0], x.shape[1], -1, C, *x.shape[3:])


def _gate_tensors(g, B, H, N, dk, dtype):
    """Returns G [B,H,N,C,dkg] with dkg = 1 (none / scalar) or dk (vector)."""
    if g is None:
        return np.zeros((B, H, N, C, 1), dtype)
    if g.ndim == 4:  # chunked scalar gate [B,H,N,C]
        return np.cumsum(g, 3)[..., None]
    return np.cumsum(g, 3)


def _pair_products(a, b, G, strict):
    """sum_c a_i[c] b_j[c] exp(G_i[c]-G_j[c]) on the (strict) lower triangle, else 0."""
    idx = np.arange(C)
    mask = (idx[:, None] > idx[None, :]) if strict else (idx[:, None] >= idx[None, :])
    if G.shape[-1] == 1:
        E = np.exp(np.where(mask, G[..., :, None, 0] - G[..., None, :, 0], -np.inf))
        return np.einsum("...ik,...jk->...ij", a, b) * E
    E = np.exp(np.where(mask[..., None], G[..., :, None, :] - G[..., None, :, :], -np.inf))
    return np.einsum("...ik,...jk,...ijk->...ij", a, b, E)


def forward(q, k, v, beta, g=None, scale=None, initial_state=None, dtype=np.float64):
    """Returns (o, S_T, ws) with ws the dict of per-chunk intermediates."""
    B, H, T, dk = q.shape
    dv = v.shape[-1]
    if scale is None:
        scale = dk ** -0.5
    qc, kc, vc = (_chunks(np.asarray(x, dtype), T) for x in (q, k, v))
    bc = _chunks(np.asarray(beta, dtype), T)
    gc = None if g is None else _chunks(np.asarray(g, dtype), T)
    N = qc.shape[2]
    G = _gate_tensors(gc, B, H, N, dk, dtype)
    Gam = np.exp(G)
    GC = G[:, :, :, -1:, :]
    X = _pair_products(kc, kc, G, strict=True)
    A = bc[..., None] * X
    Tm = np.linalg.inv(np.eye(C, dtype=dtype) + A)
    P = scale * _pair_products(qc, kc, G, strict=False)
    W = Tm @ (bc[..., None] * kc * Gam)
    U = Tm @ (bc[..., None] * vc)
    Kr = kc * np.exp(GC - G)
    S = np.zeros((B, H, dk, dv), dtype) if initial_state is None else np.array(initial_state, dtype)
    Sn = np.empty((B, H, N, dk, dv), dtype)
    D = np.empty_like(vc)
    O = np.empty_like(vc)
    for n in range(N):
        Sn[:, :, n] = S
        D[:, :, n] = U[:, :, n] - W[:, :, n] @ S
        O[:, :, n] = scale * (qc[:, :, n] * Gam[:, :, n]) @ S + P[:, :, n] @ D[:, :, n]
        S = S * np.swapaxes(np.broadcast_to(np.exp(GC[:, :, n]), (B, H, 1, dk)), -1, -2) + np.swapaxes(Kr[:, :, n], -1, -2) @ D[:, :, n]
    o = O.reshape(B, H, N * C, dv)[:, :, :T]
    ws = dict(q=qc, k=kc, v=vc, beta=bc, G=G, X=X, Tm=Tm, P=P, W=W, U=U, D=D, Sn=Sn, Kr=Kr, N=N, scale=scale)
    return o, S, ws


def backward(ws, dO, dS_T=None, dtype=np.float64):
    """Gradients for the inputs of :func:`forward`, given its ``ws``.  Also returns the
    intermediates of the reverse scan (dD, dSn) for stage-wise kernel checks."""
    q, k, v, beta, G, X, Tm, P, W, U, D, Sn, Kr = (ws[n] for n in ("q", "k", "v", "beta", "G", "X", "Tm", "P", "W", "U", "D", "Sn", "Kr"))
    scale, N = ws["scale"], ws["N"]
    B, H, _, _, dk = q.shape
    dv = v.shape[-1]
    T = dO.shape[2]
    dOc = _chunks(np.asarray(dO, dtype), T)
    vector = G.shape[-1] != 1
    Gam = np.exp(G)
    GC = G[:, :, :, -1:, :]
    eGC = np.exp(GC)  # [B,H,N,1,dkg]
    decay_to_end = np.exp(GC - G)
    Qg = scale * q * Gam

    # ---- reverse scan over chunks: dD and the state gradient entering each chunk's output
    dS = np.zeros((B, H, dk, dv), dtype) if dS_T is None else np.array(dS_T, dtype)
    dD = np.empty_like(v)
    dSn = np.empty_like(Sn)  # gradient wrt the state LEAVING chunk n
    for n in range(N - 1, -1, -1):
        dSn[:, :, n] = dS
        dD[:, :, n] = np.swapaxes(P[:, :, n], -1, -2) @ dOc[:, :, n] + Kr[:, :, n] @ dS
        row_decay = np.swapaxes(np.broadcast_to(eGC[:, :, n], (B, H, 1, dk)), -1, -2)
        dS = dS * row_decay + np.swapaxes(Qg[:, :, n], -1, -2) @ dOc[:, :, n] - np.swapaxes(W[:, :, n], -1, -2) @ dD[:, :, n]
    dS0 = dS

    # ---- chunk-parallel part
    idx = np.arange(C)
    incl = idx[:, None] >= idx[None, :]
    strict = idx[:, None] > idx[None, :]
    dP = np.where(incl, dOc @ np.swapaxes(D, -1, -2), 0.0)
    dQg = dOc @ np.swapaxes(Sn, -1, -2)
    dKr = D @ np.swapaxes(dSn, -1, -2)
    dW = -dD @ np.swapaxes(Sn, -1, -2)
    TmT = np.swapaxes(Tm, -1, -2)
    dBw = TmT @ dW
    dBu = TmT @ dD
    dA = np.where(strict, -(dBw @ np.swapaxes(W, -1, -2) + dBu @ np.swapaxes(U, -1, -2)), 0.0)
    dX = beta[..., None] * dA
    Kg = k * Gam

    dv_ = beta[..., None] * dBu
    dbeta = np.sum(dBu * v, -1) + np.sum(dBw * Kg, -1) + np.sum(dA * X, -1)
    dq = dQg * Gam * scale
    dk_ = dKr * decay_to_end + beta[..., None] * dBw * Gam
    # gate gradient wrt the cumulative gate G (row-wise), accumulated per channel group
    dG = dQg * Qg - dKr * Kr + beta[..., None] * dBw * Kg
    dGC = np.sum(dKr * Kr, 3, keepdims=True)
    state_term = np.sum(dSn * Sn, -1)  # [B,H,N,dk]
    if vector:
        dGC = dGC + (state_term * eGC[:, :, :, 0, :])[:, :, :, None, :]
    else:
        dG = np.sum(dG, -1, keepdims=True)
        dGC = np.sum(dGC, -1, keepdims=True) + (np.sum(state_term, -1)[..., None, None] * eGC)

    # pairwise terms  X_ij = <k_i,k_j>_E ,  P_ij = scale <q_i,k_j>_E
    if not vector:
        E = np.exp(np.where(incl, G[..., :, None, 0] - G[..., None, :, 0], -np.inf))
        dXe = dX * E
        dPe = dP * E * scale
        dq = dq + dPe @ k
        dk_ = dk_ + np.swapaxes(dPe, -1, -2) @ q + dXe @ k + np.swapaxes(dXe, -1, -2) @ k
        R = dX * X + dP * P
        dG = dG + (R.sum(-1) - R.sum(-2))[..., None]
    else:
        Ev = np.exp(np.where(incl[..., None], G[..., :, None, :] - G[..., None, :, :], -np.inf))  # [..,i,j,c]
        dq_intra = scale * np.einsum("...ij,...ijc,...jc->...ic", dP, Ev, k)
        dk_row = np.einsum("...ij,...ijc,...jc->...ic", dX, Ev, k)
        dk_col = np.einsum("...ij,...ijc,...ic->...jc", dX, Ev, k) + scale * np.einsum("...ij,...ijc,...ic->...jc", dP, Ev, q)
        dq = dq + dq_intra
        dk_ = dk_ + dk_row + dk_col
        dG = dG + q * dq_intra + k * dk_row - k * dk_col
    dG[:, :, :, -1:, :] += dGC
    dg = np.flip(np.cumsum(np.flip(dG, 3), 3), 3)  # reverse cumsum inside the chunk

    def unchunk(x):
        return x.reshape(B, H, N * C, *x.shape[4:])[:, :, :T]

    out = {"dq": unchunk(dq), "dk": unchunk(dk_), "dv": unchunk(dv_), "dbeta": unchunk(dbeta), "dS0": dS0,
           "dg": unchunk(dg if vector else dg[..., 0]),
           "ws": dict(dD=dD, dSn=dSn, dW=dW, dBw=dBw, dBu=dBu, dA=dA, dP=dP, dQg=dQg, dKr=dKr, dG=dG)}
    return out
