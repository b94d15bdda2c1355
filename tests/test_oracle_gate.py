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
