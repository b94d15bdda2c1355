"""Pins oracle/gate.py: torch's thresholded softplus + autograd, finite differences, closed forms."""
import numpy as np
import torch

from oracle import gate as og


def test_against_torch_softplus_and_autograd():
    r = np.random.default_rng(1)
    g = r.standard_normal((2, 5, 12)) * 8  # some entries above the threshold used below
    A, bias, dy = r.standard_normal(3) * 0.5, r.standard_normal(12), r.standard_normal((2, 5, 3, 4))
    beta = r.standard_normal((2, 5, 3))
    tg, tA, tb = (torch.tensor(a, requires_grad=True) for a in (g, A, bias))
    sp = torch.nn.functional.softplus(tg + tb, beta=1.0, threshold=6.0).view(2, 5, 3, 4)
    out = -torch.exp(tA)[None, None, :, None] * sp
    (out * torch.tensor(dy)).sum().backward()
    o, b = og.kda_gate(g, A, 4, bias, beta, 6.0)
    assert np.allclose(o, out.detach().numpy(), atol=1e-12) and np.allclose(b, torch.sigmoid(torch.tensor(beta)).numpy(), atol=1e-14)
    dg, dA, db = og.kda_gate_grad(g, A, 4, dy, bias, 6.0)
    assert np.allclose(dg, tg.grad.numpy(), atol=1e-12) and np.allclose(dA, tA.grad.numpy(), atol=1e-12)
    assert np.allclose(db, tb.grad.numpy(), atol=1e-12)


def test_closed_forms_and_finite_differences():
    # softplus(0) = ln 2; above the threshold the gate is linear: g_out = -e^A g
    o, b = og.kda_gate(np.zeros((1, 1, 4)), np.array([0.0, np.log(2.0)]), 2)
    assert np.allclose(o[0, 0], [[-np.log(2)] * 2, [-2 * np.log(2)] * 2]) and b is None
    o, _ = og.kda_gate(np.full((1, 1, 2), 30.0), np.array([0.5]), 2)
    assert np.allclose(o, -np.exp(0.5) * 30.0)
    r = np.random.default_rng(2)
    g, A, dy = r.standard_normal((1, 3, 4)), r.standard_normal(2), r.standard_normal((1, 3, 2, 2))
    dg, dA, _ = og.kda_gate_grad(g, A, 2, dy)
    f = lambda g_, A_: (og.kda_gate(g_, A_, 2)[0] * dy).sum()
    for arr, grad, which in ((g, dg, 0), (A, dA, 1)):
        for i in np.ndindex(arr.shape):
            p, m = arr.copy(), arr.copy()
            p[i] += 1e-6
            m[i] -= 1e-6
            ap, am = [g, A], [g, A]
            ap[which], am[which] = p, m
            assert abs((f(*ap) - f(*am)) / 2e-6 - grad[i]) < 1e-6


def test_gdn_gate_against_torch_autograd_and_closed_forms():
    """gated_deltanet.py:804-815 with torch's softplus / sigmoid + autograd; softplus(0) = ln 2, sigmoid(0) = 1/2."""
    r = np.random.default_rng(3)
    a, b = r.standard_normal((2, 7, 5)) * 10, r.standard_normal((2, 7, 5)) * 3  # softplus far into both tails
    A, bias = r.standard_normal(5) * 0.5, r.standard_normal(5)
    dg, dbeta = r.standard_normal((2, 7, 5)), r.standard_normal((2, 7, 5))
    for neg in (False, True):
        ta, tb, tA, tbias = (torch.tensor(x, requires_grad=True) for x in (a, b, A, bias))
        g_t = -torch.exp(tA) * torch.nn.functional.softplus(ta + tbias, threshold=1e9)
        beta_t = torch.sigmoid(tb) * (2.0 if neg else 1.0)
        ((g_t * torch.tensor(dg)).sum() + (beta_t * torch.tensor(dbeta)).sum()).backward()
        g, beta = og.gdn_gate(a, A, bias, b, neg)
        assert np.allclose(g, g_t.detach().numpy(), atol=1e-12) and np.allclose(beta, beta_t.detach().numpy(), atol=1e-14)
        d_a, d_A, d_bias, d_b = og.gdn_gate_grad(a, A, dg, bias, b, dbeta, neg)
        assert np.allclose(d_a, ta.grad.numpy(), atol=1e-12) and np.allclose(d_b, tb.grad.numpy(), atol=1e-12)
        assert np.allclose(d_A, tA.grad.numpy(), atol=1e-11) and np.allclose(d_bias, tbias.grad.numpy(), atol=1e-11)
    g, beta = og.gdn_gate(np.zeros((1, 2)), np.array([0.0, np.log(3.0)]), None, np.zeros((1, 2)), True)
    assert np.allclose(g, [[-np.log(2), -3 * np.log(2)]]) and np.allclose(beta, 1.0)
    assert og.gdn_gate(np.zeros((1, 2)), np.zeros(2))[1] is None
