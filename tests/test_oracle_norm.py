"""Pins oracle/norm.py: torch's rms_norm + sigmoid with autograd, and finite differences."""
import numpy as np
import pytest
import torch

from oracle import norm as on


@pytest.mark.parametrize("gated", [False, True])
def test_against_torch_rms_norm_and_autograd(gated):
    r = np.random.default_rng(1)
    x, g, dy = (r.standard_normal((3, 5, 16)) for _ in range(3))
    w = r.standard_normal(16)
    tx, tg, tw = (torch.tensor(a, requires_grad=True) for a in (x, g, w))
    y = torch.nn.functional.rms_norm(tx, (16,), tw, 1e-5)
    if gated:
        y = y * torch.sigmoid(tg)
    (y * torch.tensor(dy)).sum().backward()
    gate = g if gated else None
    assert np.allclose(on.rmsnorm_gated(x, gate, w), y.detach().numpy(), atol=1e-12)
    dx, dg, dw = on.rmsnorm_gated_grad(x, gate, w, dy)
    assert np.allclose(dx, tx.grad.numpy(), atol=1e-12) and np.allclose(dw, tw.grad.numpy(), atol=1e-12)
    if gated:
        assert np.allclose(dg, tg.grad.numpy(), atol=1e-12)
    else:
        assert dg is None


def test_finite_differences_and_unit_rows():
    r = np.random.default_rng(2)
    x, g, dy = (r.standard_normal((4, 8)) for _ in range(3))
    w = r.standard_normal(8)
    dx, dg, dw = on.rmsnorm_gated_grad(x, g, w, dy)
    f = lambda x_, g_, w_: (on.rmsnorm_gated(x_, g_, w_) * dy).sum()
    eps = 1e-6
    for arr, grad, which in ((x, dx, 0), (g, dg, 1), (w, dw, 2)):
        for i in np.ndindex(arr.shape):
            p, m = arr.copy(), arr.copy()
            p[i] += eps
            m[i] -= eps
            ap, am = [x, g, w], [x, g, w]
            ap[which], am[which] = p, m
            assert abs((f(*ap) - f(*am)) / (2 * eps) - grad[i]) < 1e-6
    # a row of equal entries c normalises to sign(c) (up to eps); gate 0 halves it
    y = on.rmsnorm_gated(np.full((1, 8), 3.0), np.zeros((1, 8)), np.ones(8), 0.0)
    assert np.allclose(y, 0.5)
