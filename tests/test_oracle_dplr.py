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
