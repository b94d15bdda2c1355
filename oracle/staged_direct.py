"""Chunk-level forward and backward in the "direct solve" split of the HIP kernels for 2-byte inputs
with dk <= 128 and no / a scalar gate (numpy).

TEST INFRASTRUCTURE.  Same algorithm as ``staged.py`` -- the chunk form of
linearnexus/modules/linear_attn/gated_deltanet.py:444-523 (delta_net.py:296-330 without a gate) -- but the
triangular system is applied to the right-hand side of each chunk instead of being folded into W and U first:

  G = cumsum(g) inside the chunk, gam = exp(G), r = exp(G_C - G), E_ij = exp(G_i - G_j)
  X = K K^T                       A = tril(diag(beta) (E * X), -1)      Tm = (I + A)^-1
  Pm = scale * tril(E * (Q K^T))  (diagonal included)
  Y = K S                         R = diag(beta) (V - diag(gam) Y)      D = Tm R
  O = scale diag(gam) (Q S) + Pm D
  S' = exp(G_C) S + (diag(r) K)^T D

(gated_deltanet.py:450-477 solves M [w | u] = rhs by forward substitution; D = u - w S is the same solve applied to
rhs_u - rhs_w S.)  Tm, Pm and G leave the chunk-parallel prepare kernel; the forward scan keeps the states entering
the chunks (Sn) and D; the reverse scan keeps the state gradients leaving the chunks (dSn) and dR, and writes dv.

Reverse scan, given dO and the gradient dS' of the state leaving the chunk:
  dD = Pm^T dO + diag(r) K dS'        dR = Tm^T dD        dV = diag(beta) dR        dY = -diag(beta gam) dR
  dS = exp(G_C) dS' + scale (diag(gam) Q)^T dO + K^T dY
The chunk-local kernel then needs only products that contract over the value columns plus an epilogue over the
chunk's tokens; they are listed in :func:`backward`.
"""
from __future__ import annotations

import numpy as np

from .staged import C, _chunks


def forward(q, k, v, beta, g=None, scale=None, initial_state=None, dtype=np.float64):
    """Returns (o, S_T, ws): ws holds what the kernels keep per chunk (G, Tm, Pm, Sn) and the chunked inputs."""
    B, H, T, dk = q.shape
    dv = v.shape[-1]
    if scale is None:
        scale = dk ** -0.5
    qc, kc, vc = (_chunks(np.asarray(x, dtype), T) for x in (q, k, v))
    bc = _chunks(np.asarray(beta, dtype), T)
    N = qc.shape[2]
    G = np.zeros((B, H, N, C), dtype) if g is None else np.cumsum(_chunks(np.asarray(g, dtype), T), 3)
    idx = np.arange(C)
    incl = idx[:, None] >= idx[None, :]
    strict = idx[:, None] > idx[None, :]
    E = np.exp(np.where(incl, G[..., :, None] - G[..., None, :], -np.inf))
    X = kc @ np.swapaxes(kc, -1, -2)
    A = np.where(strict, bc[..., None] * E * X, 0.0)
    Tm = np.linalg.inv(np.eye(C, dtype=dtype) + A)
    Pm = scale * E * (qc @ np.swapaxes(kc, -1, -2))
    gam = np.exp(G)[..., None]
    r = np.exp(G[..., -1:] - G)[..., None]
    S = np.zeros((B, H, dk, dv), dtype) if initial_state is None else np.array(initial_state, dtype)
    Sn = np.empty((B, H, N, dk, dv), dtype)
    D = np.empty_like(vc)
    O = np.empty_like(vc)
    for n in range(N):
        Sn[:, :, n] = S
        Y = kc[:, :, n] @ S
        R = bc[:, :, n, :, None] * (vc[:, :, n] - gam[:, :, n] * Y)
        D[:, :, n] = Tm[:, :, n] @ R
        O[:, :, n] = scale * gam[:, :, n] * (qc[:, :, n] @ S) + Pm[:, :, n] @ D[:, :, n]
        S = np.exp(G[:, :, n, -1])[..., None, None] * S + np.swapaxes(r[:, :, n] * kc[:, :, n], -1, -2) @ D[:, :, n]
    o = O.reshape(B, H, N * C, dv)[:, :, :T]
    ws = dict(q=qc, k=kc, v=vc, beta=bc, G=G, Tm=Tm, Pm=Pm, Sn=Sn, D=D, N=N, scale=scale, gated=g is not None)
    return o, S, ws


def backward(ws, dO, dS_T=None, dtype=np.float64):
    """Gradients for the inputs of :func:`forward`; also the reverse scan's per-chunk tensor dSn."""
    q, k, v, beta, G, Tm, Pm, Sn = (ws[n] for n in ("q", "k", "v", "beta", "G", "Tm", "Pm", "Sn"))
    scale, N = ws["scale"], ws["N"]
    B, H, _, _, dk = q.shape
    dv = v.shape[-1]
    T = dO.shape[2]
    dOc = _chunks(np.asarray(dO, dtype), T)
    gam = np.exp(G)[..., None]
    GC = G[..., -1]
    r = np.exp(GC[..., None] - G)[..., None]
    TmT = np.swapaxes(Tm, -1, -2)
    bg = beta[..., None] * gam

    # ---- reverse scan: needs K, Q, dO, Tm, Pm, G, beta only (no forward state) ----
    dS = np.zeros((B, H, dk, dv), dtype) if dS_T is None else np.array(dS_T, dtype)
    dSn = np.empty_like(Sn)  # gradient with respect to the state LEAVING chunk n
    for n in range(N - 1, -1, -1):
        dSn[:, :, n] = dS
        dD = np.swapaxes(Pm[:, :, n], -1, -2) @ dOc[:, :, n] + r[:, :, n] * (k[:, :, n] @ dS)
        dY = -bg[:, :, n] * (TmT[:, :, n] @ dD)
        dS = (np.exp(GC[:, :, n])[..., None, None] * dS + np.swapaxes(scale * gam[:, :, n] * q[:, :, n], -1, -2) @ dOc[:, :, n]
              + np.swapaxes(k[:, :, n], -1, -2) @ dY)
    dS0 = dS

    # ---- reverse scan, continued: per chunk it also leaves dR and dv = beta dR ----
    # (recomputed here for all chunks at once from the saved dSn)
    D = ws["D"]
    Z = k @ dSn
    dD = np.swapaxes(Pm, -1, -2) @ dOc + r * Z
    dR = TmT @ dD
    dv_ = beta[..., None] * dR

    # ---- chunk-local kernel: reads q, k, v, dO, Pm's gate factors (G), beta, Sn, dSn, D, dR ----
    idx = np.arange(C)
    incl = idx[:, None] >= idx[None, :]
    strict = idx[:, None] > idx[None, :]
    E = np.exp(np.where(incl, G[..., :, None] - G[..., None, :], -np.inf))
    # loop over the value columns (every product contracts over v)
    dQa = dOc @ np.swapaxes(Sn, -1, -2)        # [C, dk]
    dK1 = dR @ np.swapaxes(Sn, -1, -2)
    dK2 = D @ np.swapaxes(dSn, -1, -2)
    dPm = dOc @ np.swapaxes(D, -1, -2)         # [C, C], masked below
    dAm = dR @ np.swapaxes(D, -1, -2)
    rd_v = np.sum(dR * v, -1)                  # row dots <dR_t, v_t>
    ss = np.sum(dSn * Sn, (-1, -2))            # <dS', S> per chunk
    # epilogue over the chunk's tokens
    dPe = np.where(incl, scale * E * dPm, 0.0)
    dXa = np.where(strict, -E * dAm, 0.0)      # dA * E
    dXe = beta[..., None] * dXa
    dq = scale * gam * dQa + dPe @ k
    row = dXa @ k - gam * dK1                  # row-type part of dk before its factor beta
    m = np.sum(k * row, -1)
    dk_ = beta[..., None] * row + r * dK2 + np.swapaxes(dPe, -1, -2) @ q + np.swapaxes(dXe, -1, -2) @ k
    dbeta = rd_v + m
    dG = np.sum(q * dq, -1) - np.sum(k * dk_, -1) + 2.0 * beta * m
    dG[..., -1] += np.sum(r * dK2 * k, (-1, -2)) + np.exp(GC) * ss
    dg = np.flip(np.cumsum(np.flip(dG, 3), 3), 3)

    def unchunk(x):
        return x.reshape(B, H, N * C, *x.shape[4:])[:, :, :T]

    return {"dq": unchunk(dq), "dk": unchunk(dk_), "dv": unchunk(dv_), "dbeta": unchunk(dbeta), "dS0": dS0,
            "dg": unchunk(dg) if ws["gated"] else None, "ws": dict(dSn=dSn, D=D, dD=dD, dR=dR, dPe=dPe, dXa=dXa)}
