"""Pins oracle/dplr.py without the reference."""
import numpy as np

from oracle import dplr, recurrent as rc


def _data(seed, B, H, T, dk, dv):
    r = np.random.default_rng(seed)
    f = lambda *s: r.standard_normal(s)
    return dict(q=f(B, H, T, dk), k=f(B, H, T, dk), v=f(B, H, T, dv), a=f(B, H, T, dk) * 0.3, b=f(B, H, T, dk) * 0.3,
                gk=-np.abs(f(B, H, T, dk)) * 0.2, h0=f(B, H, dk, dv) * 0.5)


def test_explicit_transition_matrix_form():
    # rwkv7.py:129-130: S_t = S_{t-1} (D_t + a_t b_t^T) + v_t k_t^T with S = h^T [dv x dk]
    x = _data(1, 1, 1, 6, 3, 2)
    S = x["h0"][0, 0].T.copy()
    outs = []
    for t in range(6):
        a, b, k, v, q = (x[n][0, 0, t] for n in ("a", "b", "k", "v", "q"))
        S = S @ (np.diag(np.exp(x["gk"][0, 0, t])) + np.outer(a, b)) + np.outer(v, k)
        outs.append(S @ (0.7 * q))
    o, h = dplr.dplr_delta_rule_recurrent(x["q"], x["k"], x["v"], x["a"], x["b"], x["gk"], 0.7, x["h0"])
    assert np.allclose(o[0, 0], np.stack(outs), atol=1e-13) and np.allclose(h[0, 0], S.T, atol=1e-13)


def test_reduces_to_kda():
    # S <- diag(alpha) S;  S += beta k (v - S^T k)^T   ==   (diag(alpha) - beta k (alpha k)^T) S + beta k v^T
    x = _data(2, 2, 2, 9, 4, 5)
    r = np.random.default_rng(3)
    beta = 1 / (1 + np.exp(-r.standard_normal((2, 2, 9))))
    g = x["gk"]
    o_ref, S_ref = rc.kda_recurrent(x["q"], x["k"], x["v"], g, beta, 0.5, x["h0"], False)
    bk = beta[..., None] * x["k"]
    o, h = dplr.dplr_delta_rule_recurrent(x["q"], bk, x["v"], -np.exp(g) * x["k"], bk, g, 0.5, x["h0"])
    assert np.allclose(o, o_ref, atol=1e-12) and np.allclose(h, S_ref, atol=1e-12)


def test_pure_decay_closed_form():
    # a = b = 0: h_T = prod(w) h0 + sum_t (prod_{s>t} w_s) k_t v_t^T; the reference's decay test (tests/test_rwkv7.py:655-682)
    x = _data(4, 1, 2, 7, 3, 4)
    z = np.zeros_like(x["a"])
    _, h = dplr.dplr_delta_rule_recurrent(x["q"], x["k"], x["v"], z, z, x["gk"], 1.0, x["h0"])
    G = np.cumsum(x["gk"], 2)
    ref = np.exp(G[:, :, -1])[..., None] * x["h0"]
    for t in range(7):
        ref += (np.exp(G[:, :, -1] - G[:, :, t]) * x["k"][:, :, t])[..., None] * x["v"][:, :, t][:, :, None, :]
    assert np.allclose(h, ref, atol=1e-13)


def test_step_equals_scan_of_one_token_and_split_invariance():
    x = _data(5, 2, 3, 8, 4, 4)
    names = ("q", "k", "v", "a", "b", "gk")
    o, h = dplr.dplr_delta_rule_recurrent(*(x[n] for n in names), 1.0, x["h0"])
    o1, h1 = dplr.dplr_delta_rule_recurrent(*(x[n][:, :, :3] for n in names), 1.0, x["h0"])
    o2, h2 = dplr.dplr_delta_rule_recurrent(*(x[n][:, :, 3:] for n in names), 1.0, h1)
    assert np.allclose(np.concatenate([o1, o2], 2), o, atol=1e-13) and np.allclose(h2, h, atol=1e-13)
    os_, hs = dplr.dplr_delta_rule_step(*(x[n][:, :, 0] for n in names), x["h0"], 1.0)  # tests/test_rwkv7.py:160-203
    ot, ht = dplr.dplr_delta_rule_recurrent(*(x[n][:, :, :1] for n in names), 1.0, x["h0"])
    assert np.allclose(os_, ot[:, :, 0], atol=1e-14) and np.allclose(hs, ht, atol=1e-14)


def test_adjoint_against_finite_differences_and_torch_autograd():
    """The hand-derived adjoint against central differences of the forward oracle (every input, a few entries each) and
    against torch.autograd through an independent torch statement of the recurrence (the transition-matrix form)."""
    import torch
    x = _data(7, 2, 2, 7, 4, 3)
    r = np.random.default_rng(8)
    dO, dS = r.standard_normal((2, 2, 7, 3)), r.standard_normal((2, 2, 4, 3))
    names = ("q", "k", "v", "a", "b", "gk")
    g = dplr.dplr_delta_rule_adjoint(*(x[n] for n in names), dO, dS, 0.6, x["h0"])

    def loss(**over):
        y = dict(x, **over)
        o, h = dplr.dplr_delta_rule_recurrent(*(y[n] for n in names), 0.6, y["h0"])
        return (o * dO).sum() + (h * dS).sum()
    for n, gn in (("q", "dq"), ("k", "dk"), ("v", "dv"), ("a", "da"), ("b", "db"), ("gk", "dgk"), ("h0", "dS0")):
        for _ in range(6):
            i = tuple(r.integers(0, s) for s in x[n].shape)
            p, m = x[n].copy(), x[n].copy()
            p[i] += 1e-6
            m[i] -= 1e-6
            fd = (loss(**{n: p}) - loss(**{n: m})) / 2e-6
            assert abs(fd - g[gn][i]) < 1e-6 * max(1.0, abs(fd)), (n, i, fd, g[gn][i])
    # torch: S_t = S_{t-1} (diag(w_t) + a_t b_t^T) + v_t k_t^T with S = h^T (rwkv7.py:129-130), o_t = S_t (scale q_t)
    t = {n: torch.tensor(x[n], requires_grad=True) for n in names + ("h0",)}
    S = t["h0"].transpose(-1, -2)
    outs = []
    for i in range(7):
        M = torch.diag_embed(torch.exp(t["gk"][:, :, i])) + t["a"][:, :, i, :, None] * t["b"][:, :, i, None, :]
        S = S @ M + t["v"][:, :, i, :, None] * t["k"][:, :, i, None, :]
        outs.append((S @ (0.6 * t["q"][:, :, i, :, None]))[..., 0])
    ((torch.stack(outs, 2) * torch.tensor(dO)).sum() + (S.transpose(-1, -2) * torch.tensor(dS)).sum()).backward()
    for n, gn in (("q", "dq"), ("k", "dk"), ("v", "dv"), ("a", "da"), ("b", "db"), ("gk", "dgk"), ("h0", "dS0")):
        assert np.allclose(g[gn], t[n].grad.numpy(), atol=1e-11), gn


def test_adjoint_without_state_gradients():
    x = _data(9, 1, 2, 5, 3, 4)
    dO = np.random.default_rng(10).standard_normal((1, 2, 5, 4))
    names = ("q", "k", "v", "a", "b", "gk")
    g0 = dplr.dplr_delta_rule_adjoint(*(x[n] for n in names), dO)
    g1 = dplr.dplr_delta_rule_adjoint(*(x[n] for n in names), dO, np.zeros((1, 2, 3, 4)), 1.0, np.zeros((1, 2, 3, 4)))
    assert all(np.allclose(g0[n], g1[n], atol=1e-14) for n in g0)
