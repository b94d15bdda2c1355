"""GPU parity of the RWKV-7 DPLR token kernels against the fp64 oracle, through the C-ABI.
Tolerances as max|x - ref| / max|ref|: 1e-4 (fp32 inputs) / 2e-2 (bf16 inputs)."""
import numpy as np
import pytest
import torch

from oracle import dplr as od
from oracle.inputs import to_bf16_grid
from conftest import max_rel

pytestmark = pytest.mark.gpu
DEV = "cuda"
NAMES = ("q", "k", "v", "a", "b", "gk")


def _data(seed, B, H, T, dk, dv, bf16):
    # the distributions of the reference's tests (tests/test_rwkv7.py:116-127): small a, b; gk <= 0
    r = np.random.default_rng(seed)
    f = lambda *s: r.standard_normal(s).astype(np.float32)
    x = dict(q=f(B, H, T, dk), k=f(B, H, T, dk), v=f(B, H, T, dv), a=f(B, H, T, dk) * 0.1, b=f(B, H, T, dk) * 0.1,
             gk=-np.abs(f(B, H, T, dk)) * 0.1, h0=f(B, H, dk, dv) * 0.5)
    if bf16:
        for n in ("q", "k", "v", "a", "b"):
            x[n] = to_bf16_grid(x[n])
    return x


def _t(a, dt=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    return t.to(dt) if dt is not None else t


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("shape", [(2, 4, 16, 32, 32), (1, 2, 130, 64, 64), (2, 2, 40, 128, 128), (1, 3, 17, 8, 8),
                                   (1, 2, 20, 16, 100)])
def test_scan_matches_oracle(shape, bf16):
    import linearnexus_amd as la
    B, H, T, dk, dv = shape
    x = _data(81, B, H, T, dk, dv, bf16)
    dt = torch.bfloat16 if bf16 else torch.float32
    o_ref, h_ref = od.dplr_delta_rule_recurrent(*(x[n] for n in NAMES), 0.5, x["h0"])
    ins = [_t(x[n], dt) for n in NAMES[:5]] + [_t(x["gk"])]
    o, h = la.dplr_delta_rule_recurrent(*ins, 0.5, _t(x["h0"]))
    assert o.dtype == dt and o.shape == (B, H, T, dv) and h.dtype == torch.float32 and h.shape == (B, H, dk, dv)
    tol = 2e-2 if bf16 else 1e-4
    assert max_rel(o.float().cpu().numpy(), o_ref) < tol and max_rel(h.cpu().numpy(), h_ref) < tol
    o0, h0 = la.dplr_delta_rule_recurrent(*ins)  # defaults: scale 1, zero state (rwkv7.py:121-122)
    o0_ref, h0_ref = od.dplr_delta_rule_recurrent(*(x[n] for n in NAMES))
    assert max_rel(o0.float().cpu().numpy(), o0_ref) < tol and max_rel(h0.cpu().numpy(), h0_ref) < tol


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("shape", [(3, 4, 128, 128), (2, 2, 64, 64), (2, 4, 8, 8), (1, 2, 32, 200)])
def test_step_matches_oracle_and_first_scan_step(shape, bf16):
    # tests/test_rwkv7.py:160-203
    import linearnexus_amd as la
    B, H, dk, dv = shape
    x = _data(82, B, H, 1, dk, dv, bf16)
    dt = torch.bfloat16 if bf16 else torch.float32
    sq = lambda n: x[n][:, :, 0]
    o_ref, h_ref = od.dplr_delta_rule_step(*(sq(n) for n in NAMES), x["h0"], 1.0)
    ins = [_t(sq(n), dt) for n in NAMES[:5]] + [_t(sq("gk"))]
    state = _t(x["h0"])
    keep = state.clone()
    o, h = la.dplr_delta_rule_step(*ins, state)
    assert torch.equal(state, keep)
    tol = 2e-2 if bf16 else 1e-4
    assert max_rel(o.float().cpu().numpy(), o_ref) < tol and max_rel(h.cpu().numpy(), h_ref) < 1e-5 + tol * bf16
    o2, h2 = la.dplr_delta_rule_recurrent(*(t[:, :, None] for t in ins), 1.0, state)
    assert torch.allclose(o2[:, :, 0].float(), o.float(), rtol=1e-4, atol=1e-6) and torch.allclose(h2, h, rtol=1e-4, atol=1e-6)
    o3, h3 = la.dplr_delta_rule_step(*ins, state, inplace=True)
    assert h3.data_ptr() == state.data_ptr() and torch.equal(h3, h) and torch.equal(o3, o)


def test_decay_only_shrinks_the_state():
    # tests/test_rwkv7.py:655-682 with its closed form: zero k, v, a, b and gk = -0.5 over 10 tokens -> h0 * exp(-5)
    import linearnexus_amd as la
    B, H, T, d = 2, 2, 10, 16
    z = torch.zeros(B, H, T, d, device=DEV)
    h0 = torch.full((B, H, d, d), 10.0, device=DEV)
    _, h = la.dplr_delta_rule_recurrent(torch.randn(B, H, T, d, device=DEV) * 0.01, z, z, z, z, z - 0.5, initial_state=h0)
    assert torch.allclose(h, h0 * float(np.exp(-5.0)), rtol=1e-5)


def test_reduces_to_kda_kernel_on_gpu():
    """a = -exp(g) k, b = beta k, key beta k: the DPLR kernel must agree with the KDA token kernel."""
    import linearnexus_amd as la
    B, H, T, d = 1, 2, 50, 64
    x = _data(83, B, H, T, d, d, False)
    beta = torch.sigmoid(torch.randn(B, H, T, device=DEV))
    q, k, v, g = _t(x["q"]), _t(x["k"]) * 0.3, _t(x["v"]), _t(x["gk"])
    o_ref, S_ref = la.kda_recurrent(q, k, v, g, beta, 0.5, _t(x["h0"]), False)
    bk = beta[..., None] * k
    o, S = la.dplr_delta_rule_recurrent(q, bk, v, -torch.exp(g) * k, bk, g, 0.5, _t(x["h0"]))
    assert max_rel(o.cpu().numpy(), o_ref.cpu().numpy()) < 1e-4 and max_rel(S.cpu().numpy(), S_ref.cpu().numpy()) < 1e-4


def test_errors_and_empty():
    import linearnexus_amd as la
    q = torch.randn(1, 2, 4, 16, device=DEV)
    with pytest.raises(RuntimeError):
        la.dplr_delta_rule_recurrent(q, q, q, q[..., :8], q, q)
    with pytest.raises(RuntimeError):
        la.dplr_delta_rule_recurrent(q[..., :12], q[..., :12], q, q[..., :12], q[..., :12], q[..., :12])  # dk = 12
    with pytest.raises(RuntimeError):
        la.dplr_delta_rule_recurrent(q.cpu(), q, q, q, q, q)
    e = q[:, :, :0]
    h0 = torch.randn(1, 2, 16, 16, device=DEV)
    o, h = la.dplr_delta_rule_recurrent(e, e, e, e, e, e, initial_state=h0)
    assert o.shape == (1, 2, 0, 16) and torch.equal(h, h0)


def test_wanted_gradient_is_refused_loudly():
    import linearnexus_amd as la
    t = lambda *s: torch.randn(*s, device="cuda")
    q = t(1, 2, 8, 64).requires_grad_(True)
    with pytest.raises(RuntimeError, match="no backward pass"):
        la.dplr_delta_rule_recurrent(q, t(1, 2, 8, 64), t(1, 2, 8, 64), t(1, 2, 8, 64), t(1, 2, 8, 64), -t(1, 2, 8, 64).abs())
