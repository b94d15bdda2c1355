"""GPU parity of the gated RMSNorm kernels against the fp64 oracle, through the C-ABI.
Tolerances as max|x - ref| / max|ref|: 1e-5 (fp32) / 2e-2 (bf16 storage, fp32 arithmetic)."""
import numpy as np
import pytest
import torch

from oracle import norm as on
from oracle.inputs import to_bf16_grid
from conftest import max_rel

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _t(a, dt=None, grad=False):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    if dt is not None:
        t = t.to(dt)
    return t.requires_grad_(grad)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("shape", [(2, 7, 4, 128), (1, 33, 2, 64), (5, 256), (1, 1, 1, 32), (3, 100, 256), (1000, 16),
                                   (2, 9, 3, 512), (3, 11, 80), (70, 1024), (5, 40), (2, 3, 200)])
def test_forward_backward_match_oracle(shape, gated, bf16):
    import linearnexus_amd as la
    r = np.random.default_rng(91)
    rnd = (lambda a: to_bf16_grid(a.astype(np.float32))) if bf16 else (lambda a: a.astype(np.float32))
    x, g, dy = (rnd(r.standard_normal(shape)) for _ in range(3))
    w = (1 + 0.3 * r.standard_normal(shape[-1])).astype(np.float32)
    dt = torch.bfloat16 if bf16 else torch.float32
    gate = g if gated else None
    y_ref = on.rmsnorm_gated(x, gate, w, 1e-5)
    dx_ref, dg_ref, dw_ref = on.rmsnorm_gated_grad(x, gate, w, dy, 1e-5)
    tx, tw = _t(x, dt, True), _t(w, None, True)
    tg = _t(g, dt, True) if gated else None
    y = la.rmsnorm_gated(tx, tg, tw, 1e-5)
    assert y.dtype == dt and y.shape == shape
    (y.float() * _t(dy)).sum().backward()
    tol = 2e-2 if bf16 else 1e-5
    assert max_rel(y.detach().float().cpu().numpy(), y_ref) < tol
    assert max_rel(tx.grad.float().cpu().numpy(), dx_ref) < tol
    assert max_rel(tw.grad.cpu().numpy(), dw_ref) < (2e-2 if bf16 else 1e-4)
    if gated:
        assert max_rel(tg.grad.float().cpu().numpy(), dg_ref) < tol


def test_errors_and_empty():
    import linearnexus_amd as la
    w = torch.ones(22, device=DEV)
    with pytest.raises(RuntimeError):
        la.rmsnorm_gated(torch.randn(4, 22, device=DEV), None, w)  # 22 floats: no whole number of 16-byte vectors
    with pytest.raises(RuntimeError):
        la.rmsnorm_gated(torch.randn(2, 2048, device=DEV), None, torch.ones(2048, device=DEV))  # 512 vectors: too wide
    with pytest.raises(RuntimeError):
        la.rmsnorm_gated(torch.randn(4, 32), None, torch.ones(32))
    with pytest.raises(RuntimeError):
        la.rmsnorm_gated(torch.randn(4, 32, device=DEV), torch.randn(4, 16, device=DEV), torch.ones(32, device=DEV))
    y = la.rmsnorm_gated(torch.randn(0, 32, device=DEV), None, torch.ones(32, device=DEV))
    assert y.shape == (0, 32)


def test_full_size_scale_invariance():
    """At a full layer's size ([8, 4096, 16, 128] bf16) RMSNorm ignores a power-of-two rescaling of its input
    exactly (eps = 0): y(4x) == y(x) bit for bit, gate and weight unchanged."""
    import linearnexus_amd as la
    torch.manual_seed(1)
    x = torch.randn(8, 4096, 16, 128, device=DEV).bfloat16()
    g = torch.randn(8, 4096, 16, 128, device=DEV).bfloat16()
    w = torch.rand(128, device=DEV) + 0.5
    assert torch.equal(la.rmsnorm_gated(x, g, w, 0.0), la.rmsnorm_gated(x * 4, g, w, 0.0))
