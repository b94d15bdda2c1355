"""fp64 restatement of the reference's RWKV-7 diagonal-plus-low-rank recurrence -- TEST INFRASTRUCTURE ONLY.

Follows linearnexus/modules/linear_attn/rwkv7.py:114-213 (scan) and :216-265 (step).  Pinned in
tests/test_oracle_dplr.py by the explicit transition-matrix form on tiny inputs, by its reduction to the KDA
recurrence (a = -exp(g) k, b = beta k, key beta k: the two oracles are independent code), by the pure-decay
closed form (a = b = 0), by step == scan(T=1) and by split invariance; the adjoint by central finite differences and by
torch.autograd through the transition-matrix form (an independent statement of the recurrence).
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


def dplr_delta_rule_adjoint(q, k, v, a, b, gk, d_o, d_final_state=None, scale=1.0, initial_state=None):
    """Gradients of  <o, d_o> + <final state, d_final_state>  with respect to q, k, v, a, b, gk and the initial state:
    reverse-mode differentiation of the scan above by hand (the reference differentiates its lax.scan, rwkv7.py:148-213,
    with jax.grad).  Per token, with h' the state before it, w = exp(gk), u = h'^T a and D the gradient of the state
    after it (the later tokens' share plus scale q d_o^T):
      dq = scale h d_o;  dv = D^T k;  dk = D v;  db = D u;  du = D^T b;  da = h' du;  dgk = w (.) rowsum(D (.) h');
      gradient of h' = w (.) D + a du^T.
    Returns a dict with dq, dk, dv, da, db, dgk, dS0."""
    q, k, v, a, b, gk, d_o = (np.asarray(x, np.float64) for x in (q, k, v, a, b, gk, d_o))
    B, H, T, dk = q.shape
    dv_ = v.shape[-1]
    h = np.zeros((B, H, dk, dv_)) if initial_state is None else np.asarray(initial_state, np.float64).copy()
    before = np.zeros((T, B, H, dk, dv_))  # the state each token starts from
    for t in range(T):
        before[t] = h
        _, h = dplr_delta_rule_step(q[:, :, t], k[:, :, t], v[:, :, t], a[:, :, t], b[:, :, t], gk[:, :, t], h, scale)
    D = np.zeros_like(h) if d_final_state is None else np.asarray(d_final_state, np.float64).copy()
    g = {n: np.zeros_like(x) for n, x in (("dq", q), ("dk", k), ("dv", v), ("da", a), ("db", b), ("dgk", gk))}
    for t in range(T - 1, -1, -1):
        hp = before[t]
        w = np.exp(gk[:, :, t])
        u = np.einsum("bhk,bhkv->bhv", a[:, :, t], hp)
        h_t = w[..., None] * hp + b[:, :, t][..., None] * u[..., None, :] + k[:, :, t][..., None] * v[:, :, t][..., None, :]
        g["dq"][:, :, t] = scale * np.einsum("bhkv,bhv->bhk", h_t, d_o[:, :, t])
        D = D + scale * q[:, :, t][..., None] * d_o[:, :, t][..., None, :]
        g["dv"][:, :, t] = np.einsum("bhkv,bhk->bhv", D, k[:, :, t])
        g["dk"][:, :, t] = np.einsum("bhkv,bhv->bhk", D, v[:, :, t])
        g["db"][:, :, t] = np.einsum("bhkv,bhv->bhk", D, u)
        du = np.einsum("bhkv,bhk->bhv", D, b[:, :, t])
        g["da"][:, :, t] = np.einsum("bhkv,bhv->bhk", hp, du)
        g["dgk"][:, :, t] = w * (D * hp).sum(-1)
        D = w[..., None] * D + a[:, :, t][..., None] * du[..., None, :]
    g["dS0"] = D
    return g
