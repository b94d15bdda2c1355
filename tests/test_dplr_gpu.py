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


GRADS = (("q", "dq"), ("k", "dk"), ("v", "dv"), ("a", "da"), ("b", "db"), ("gk", "dgk"), ("h0", "dS0"))


def _grad_check(x, bf16, with_state, with_ds, scale, tol):
    import linearnexus_amd as la
    dt = torch.bfloat16 if bf16 else torch.float32
    r = np.random.default_rng(99)
    B, H, T, dk = x["q"].shape
    dv = x["v"].shape[-1]
    dO = r.standard_normal((B, H, T, dv)).astype(np.float32)
    if bf16:
        dO = to_bf16_grid(dO)
    dS = r.standard_normal((B, H, dk, dv)).astype(np.float32) if with_ds else None
    t = {n: _t(x[n], dt if n in ("q", "k", "v", "a", "b") else None).requires_grad_(True) for n in NAMES + ("h0",)}
    o, h = la.dplr_delta_rule_recurrent(*(t[n] for n in NAMES), scale, t["h0"] if with_state else None)
    assert o.requires_grad and h.requires_grad and o.dtype == dt and h.dtype == torch.float32
    loss = (o.float() * _t(dO)).sum()
    if with_ds:
        loss = loss + (h * _t(dS)).sum()
    loss.backward()
    ref = od.dplr_delta_rule_adjoint(*(x[n] for n in NAMES), dO, dS, scale, x["h0"] if with_state else None)
    errs = {}
    for n, gn in GRADS:
        if n == "h0" and not with_state:
            assert t[n].grad is None
            continue
        assert t[n].grad.dtype == t[n].dtype and t[n].grad.shape == t[n].shape
        errs[gn] = max_rel(t[n].grad.float().cpu().numpy(), ref[gn])
    assert all(e < tol for e in errs.values()), errs


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("shape", [(2, 3, 16, 32, 32), (1, 2, 130, 64, 64), (1, 2, 70, 128, 128), (1, 3, 17, 8, 8),
                                   (1, 2, 65, 16, 100), (1, 1, 64, 64, 256)])
def test_scan_gradients_match_the_adjoint_oracle(shape, bf16):
    """Backward kernel (checkpoints every 64 tokens, segment tapes) against the hand-derived fp64 adjoint: sequence
    lengths below, at and across segment boundaries, value widths that leave lanes and whole waves partly idle."""
    x = _data(21, *shape, bf16)
    _grad_check(x, bf16, with_state=True, with_ds=True, scale=0.7, tol=2e-2 if bf16 else 1e-4)


@pytest.mark.parametrize("with_state,with_ds", [(False, False), (True, False), (False, True)])
def test_scan_gradients_without_state_or_state_gradient(with_state, with_ds):
    x = _data(22, 2, 2, 75, 64, 64, False)
    _grad_check(x, False, with_state, with_ds, 1.0, 1e-4)


def test_step_is_differentiable_and_backward_repeats_exactly():
    import linearnexus_amd as la
    x = _data(23, 2, 3, 1, 64, 64, False)
    t = {n: _t(x[n][:, :, 0] if n != "h0" else x[n]).requires_grad_(True) for n in NAMES + ("h0",)}
    o, h = la.dplr_delta_rule_step(*(t[n] for n in NAMES), t["h0"], 0.5)
    r = np.random.default_rng(5)
    dO, dS = r.standard_normal((2, 3, 64)).astype(np.float32), r.standard_normal((2, 3, 64, 64)).astype(np.float32)
    ((o * _t(dO)).sum() + (h * _t(dS)).sum()).backward()
    ref = od.dplr_delta_rule_adjoint(*(x[n] for n in NAMES), dO[:, :, None], dS, 0.5, x["h0"])
    for n, gn in GRADS:
        want = ref[gn][:, :, 0] if n != "h0" else ref[gn]
        assert max_rel(t[n].grad.cpu().numpy(), want) < 1e-4, gn
    with pytest.raises(RuntimeError, match="in place"):
        la.dplr_delta_rule_step(*(t[n] for n in NAMES), t["h0"].detach().clone().requires_grad_(True), 0.5, inplace=True)
    # no atomics anywhere: two backward passes of the same scan give the same bits
    y = _data(24, 1, 2, 200, 64, 64, False)
    grads = []
    for _ in range(2):
        u = {n: _t(y[n]).requires_grad_(True) for n in NAMES}
        o, _ = la.dplr_delta_rule_recurrent(*(u[n] for n in NAMES), 1.0)
        o.sum().backward()
        grads.append([u[n].grad.clone() for n in NAMES])
    assert all(torch.equal(g0, g1) for g0, g1 in zip(*grads))


def test_backward_through_the_c_abi_rejects_bad_arguments():
    import ctypes as C
    from linearnexus_amd import _lib
    lib = _lib.load()
    g = _lib.DplrBwdArgs()
    g.fwd.B, g.fwd.H, g.fwd.T, g.fwd.dk, g.fwd.dv = 1, 1, 4, 64, 64
    g.fwd.dtype = g.fwd.o_dtype = 0
    assert lib.lnx_dplr_recurrent_bwd(g, None) == -1          # NULL tensors
    assert lib.lnx_dplr_recurrent_bwd(None, None) == -1
    g.fwd.dv = 512
    assert lib.lnx_dplr_recurrent_bwd(g, None) == -2          # dv beyond one workgroup
    g.fwd.dv, g.fwd.dk = 64, 12
    z = torch.zeros(1 * 1 * 4 * 64, device=DEV)
    for f in ("q", "k", "v", "a", "b", "gk"):
        setattr(g.fwd, f, z.data_ptr())
    for f in ("d_o", "dq", "dk", "dv", "da", "db", "dgk"):
        setattr(g, f, z.data_ptr())
    assert lib.lnx_dplr_recurrent_bwd(g, None) == -4          # no workspace
    ws = torch.empty(int(lib.lnx_dplr_recurrent_bwd_workspace_bytes(1, 1, 4, 12, 64)), dtype=torch.uint8, device=DEV)
    g.workspace, g.workspace_bytes = ws.data_ptr(), ws.numel()
    assert lib.lnx_dplr_recurrent_bwd(g, None) == -2          # dk = 12
    assert lib.lnx_dplr_recurrent_bwd_workspace_bytes(2, 3, 130, 64, 64) == 2 * 3 * (3 + 64) * 64 * 64 * 4


def test_gradients_of_empty_scans():
    """No tokens: the state passes through and so does its gradient; no batch rows: empty gradients."""
    import linearnexus_amd as la
    e = torch.zeros(1, 2, 0, 16, device=DEV, requires_grad=True)
    h0 = torch.randn(1, 2, 16, 16, device=DEV, requires_grad=True)
    o, h = la.dplr_delta_rule_recurrent(e, e, e, e, e, e, initial_state=h0)
    dS = torch.randn_like(h)
    (h * dS).sum().backward()
    assert o.shape == (1, 2, 0, 16) and torch.equal(h0.grad, dS) and e.grad.shape == e.shape
    z = torch.zeros(0, 2, 5, 16, device=DEV, requires_grad=True)
    o, h = la.dplr_delta_rule_recurrent(z, z, z, z, z, z)
    (o.sum() + h.sum()).backward()
    assert z.grad.shape == z.shape
