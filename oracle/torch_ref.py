"""Torch (CPU) restatement of the recurrent and chunk forms, differentiable by autograd.

TEST INFRASTRUCTURE.  Two uses: (1) ``torch.autograd`` through ``recurrent`` is an
independent check of ``adjoint.py`` and the gradient oracle for the HIP backward kernels;
(2) ``chunkwise`` + autograd on all host cores is the CPU baseline the benchmark times,
the closest stand-in for the reference's JAX-CPU path (forward
gated_deltanet.py:265-534 / kda.py:372-655, backward by autodiff as in
linearnexus/train/sft.py:126-127).
"""

from __future__ import annotations

import torch

L2_EPS = 1e-6


def l2norm(x):
    return x / (x.norm(dim=-1, keepdim=True) + L2_EPS)


def recurrent(q, k, v, beta, g=None, scale=None, initial_state=None, use_qk_l2norm=False):
    """Generic recurrent form; ``g`` None / [B,H,T] / [B,H,T,dk].  Returns (o, S_T)."""
    B, H, T, dk = q.shape
    dv = v.shape[-1]
    if scale is None:
        scale = dk ** -0.5
    if use_qk_l2norm:
        q, k = l2norm(q), l2norm(k)
    q = q * scale
    S = q.new_zeros(B, H, dk, dv) if initial_state is None else initial_state
    outs = []
    for t in range(T):
        if g is not None:
            a = torch.exp(g[:, :, t])
            S = S * (a[..., None] if g.dim() == 4 else a[..., None, None])
        k_t = k[:, :, t]
        r = v[:, :, t] - torch.einsum("bhkv,bhk->bhv", S, k_t)
        S = S + torch.einsum("bhk,bhv->bhkv", k_t, beta[:, :, t, None] * r)
        outs.append(torch.einsum("bhk,bhkv->bhv", q[:, :, t], S))
    return torch.stack(outs, 2), S


def chunkwise(q, k, v, beta, g=None, scale=None, initial_state=None, chunk_size=64, use_qk_l2norm=False):
    """Chunk form batched over all chunks (what a CPU backend would run)."""
    B, H, T, dk = q.shape
    dv = v.shape[-1]
    C = chunk_size
    if scale is None:
        scale = dk ** -0.5
    if use_qk_l2norm:
        q, k = l2norm(q), l2norm(k)
    q = q * scale
    pad = (C - T % C) % C
    if pad:
        P = torch.nn.functional.pad
        q, k, v = (P(x, (0, 0, 0, pad)) for x in (q, k, v))
        beta = P(beta, (0, pad))
        if g is not None:
            g = P(g, (0, 0, 0, pad)) if g.dim() == 4 else P(g, (0, pad))
    N = (T + pad) // C
    q, k, v = (x.reshape(B, H, N, C, -1) for x in (q, k, v))
    beta = beta.reshape(B, H, N, C)
    if g is None:
        G = q.new_zeros(B, H, N, C, 1)
    elif g.dim() == 3:
        G = g.reshape(B, H, N, C).cumsum(3)[..., None]
    else:
        G = g.reshape(B, H, N, C, dk).cumsum(3)
    # pairwise decays exp(G_i - G_j), masked before exponentiating
    idx = torch.arange(C)
    lower = (idx[:, None] >= idx[None, :])[..., None]
    D = torch.exp(torch.where(lower, G[..., :, None, :] - G[..., None, :, :], torch.full_like(G[..., :1, None, :], -float("inf"))))
    if D.shape[-1] == 1:
        KK = torch.einsum("bhnik,bhnjk->bhnij", k, k) * D[..., 0]
        QK = torch.einsum("bhnik,bhnjk->bhnij", q, k) * D[..., 0]
    else:
        KK = torch.einsum("bhnik,bhnjk,bhnijk->bhnij", k, k, D)
        QK = torch.einsum("bhnik,bhnjk,bhnijk->bhnij", q, k, D)
    eye = torch.eye(C, dtype=q.dtype)
    M = eye + torch.tril(KK * beta[..., None], -1)
    eg = torch.exp(G)
    rhs = torch.cat([beta[..., None] * k * eg, beta[..., None] * v], -1)
    X = torch.linalg.solve_triangular(M, rhs, upper=False, unitriangular=True)
    w, u = X[..., :dk], X[..., dk:]
    kr = k * torch.exp(G[..., -1:, :] - G)
    qg = q * eg
    S = q.new_zeros(B, H, dk, dv) if initial_state is None else initial_state
    outs = []
    for n in range(N):
        d = u[:, :, n] - w[:, :, n] @ S
        outs.append(qg[:, :, n] @ S + QK[:, :, n] @ d)
        S = S * eg[:, :, n, -1].expand(B, H, dk)[..., None] + kr[:, :, n].transpose(-1, -2) @ d
    o = torch.stack(outs, 2).reshape(B, H, N * C, dv)[:, :, :T]
    return o, S


def grads(fn, inputs, dO, dS, **kw):
    """Runs ``fn`` on leaf copies of ``inputs`` (dict of tensors or None) and back-propagates
    ``<o,dO> + <S_T,dS>``.  Returns (o, S_T, {name: grad})."""
    leaves = {n: (x.detach().clone().requires_grad_(True) if x is not None else None) for n, x in inputs.items()}
    o, S = fn(**leaves, **kw)
    loss = (o * dO).sum() + ((S * dS).sum() if dS is not None else 0.0)
    loss.backward()
    return o.detach(), S.detach(), {n: (x.grad if x is not None else None) for n, x in leaves.items()}
