"""GPU parity of the KDA gate kernels against the fp64 oracle, through the C-ABI.
Tolerances as max|x - ref| / max|ref|: 1e-5 (fp32) / 2e-2 (bf16 storage, fp32 arithmetic)."""
import numpy as np
import pytest
import torch

from oracle import gate as og
from oracle.inputs import to_bf16_grid
from conftest import max_rel

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _t(a, dt=None, grad=False):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    if dt is not None:
        t = t.to(dt)
    return t.requires_grad_(grad)


@pytest.mark.parametrize("bf16,out32", [(False, True), (True, False), (True, True)])
@pytest.mark.parametrize("bias", [False, True])
@pytest.mark.parametrize("shape", [(2, 16, 4, 32), (1, 100, 3, 128), (3, 33, 2, 8), (1, 1, 1, 4), (2, 1000, 16, 128)])
def test_forward_backward_match_oracle(shape, bias, bf16, out32):
    import linearnexus_amd as la
    B, T, H, dk = shape
    r = np.random.default_rng(95)
    rnd = (lambda a: to_bf16_grid(a.astype(np.float32))) if bf16 else (lambda a: a.astype(np.float32))
    g = rnd(r.standard_normal((B, T, H * dk)) * 6)  # a few entries above the threshold of 12 used here
    A = (r.standard_normal(H) * 0.5).astype(np.float32)
    gb = (r.standard_normal(H * dk)).astype(np.float32) if bias else None
    beta = r.standard_normal((B, T, H)).astype(np.float32)
    dy = r.standard_normal((B, T, H, dk)).astype(np.float32)
    if not out32:
        dy = to_bf16_grid(dy)
    dbeta = r.standard_normal((B, T, H)).astype(np.float32)
    o_ref, b_ref = og.kda_gate(g, A, dk, gb, beta, 12.0)
    dg_ref, dA_ref, db_ref = og.kda_gate_grad(g, A, dk, dy, gb, 12.0)
    dt = torch.bfloat16 if bf16 else torch.float32
    tg, tA, tbeta = _t(g, dt, True), _t(A, None, True), _t(beta, None, True)
    tgb = _t(gb, None, True) if bias else None
    o, b = la.kda_gate(tg, tA, dk, tgb, tbeta, 12.0, out_dtype=torch.float32 if out32 else None)
    assert o.shape == (B, T, H, dk) and o.dtype == (torch.float32 if out32 else dt) and b.dtype == torch.float32
    ((o.float() * _t(dy)).sum() + (b * _t(dbeta)).sum()).backward()
    tol_o = 1e-5 if out32 else 2e-2
    tol_g = 2e-2 if bf16 else 1e-5
    assert max_rel(o.detach().float().cpu().numpy(), o_ref) < tol_o
    assert max_rel(b.detach().cpu().numpy(), b_ref) < 1e-6
    assert max_rel(tg.grad.float().cpu().numpy(), dg_ref) < tol_g
    assert max_rel(tA.grad.cpu().numpy(), dA_ref) < 1e-4
    if bias:
        assert max_rel(tgb.grad.cpu().numpy(), db_ref) < 1e-4
    s = 1 / (1 + np.exp(-beta.astype(np.float64)))
    assert max_rel(tbeta.grad.cpu().numpy(), dbeta * s * (1 - s)) < 1e-5


def test_feeds_the_kda_scan_and_gradients_are_deterministic():
    """fp32 gate output goes straight into kda_chunkwise; two backward passes give bit-identical parameter gradients."""
    import linearnexus_amd as la
    B, T, H, d = 1, 130, 2, 128
    torch.manual_seed(4)
    raw = torch.randn(B, T, H * d, device=DEV).bfloat16().requires_grad_(True)
    A = torch.zeros(H, device=DEV, requires_grad=True)
    nrm = lambda x: x / (x.norm(dim=-1, keepdim=True) + 1e-6)
    q, k = (nrm(torch.randn(B, T, H, d, device=DEV)).bfloat16() for _ in range(2))
    v = torch.randn(B, T, H, d, device=DEV).bfloat16()
    beta_raw = torch.randn(B, T, H, device=DEV)
    grads = []
    for _ in range(2):
        raw.grad = A.grad = None
        g, beta = la.kda_gate(raw * 0.1 - 3, A, d, beta=beta_raw, out_dtype=torch.float32)
        o, _ = la.kda_chunkwise(q.transpose(1, 2), k.transpose(1, 2), v.transpose(1, 2), g.transpose(1, 2), beta.transpose(1, 2),
                                use_qk_l2norm=False)
        o.square().sum().backward()
        grads.append((raw.grad.clone(), A.grad.clone()))
    assert torch.isfinite(grads[0][0]).all() and grads[0][1].abs().sum() > 0
    assert torch.equal(grads[0][1], grads[1][1]) or (grads[0][1] - grads[1][1]).abs().max() <= 1e-5 * grads[0][1].abs().max()


def test_errors_and_empty():
    import linearnexus_amd as la
    A = torch.zeros(2, device=DEV)
    with pytest.raises(RuntimeError):
        la.kda_gate(torch.randn(1, 4, 10, device=DEV), A, 4)
    with pytest.raises(RuntimeError):
        la.kda_gate(torch.randn(1, 4, 8), A, 4)
    with pytest.raises(RuntimeError):
        la.kda_gate(torch.randn(1, 4, 4, device=DEV), A, 2)  # dk = 2 is not a multiple of 4
    o, b = la.kda_gate(torch.randn(1, 0, 8, device=DEV), A, 4)
    assert o.shape == (1, 0, 2, 4) and b is None


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("shape", [(2, 16, 4), (1, 1000, 16), (3, 33, 6), (1, 1, 1), (8, 4096, 16)])
@pytest.mark.parametrize("neg,with_b,with_bias", [(False, True, True), (True, True, False), (False, False, True)])
def test_gated_deltanet_gate_matches_oracle(shape, bf16, neg, with_b, with_bias):
    """g = -exp(A_log) softplus(a + dt_bias), beta = sigmoid(b) (* 2) and every gradient (gated_deltanet.py:804-815)."""
    import linearnexus_amd as la
    B, T, H = shape
    r = np.random.default_rng(96)
    rnd = (lambda x: to_bf16_grid(x.astype(np.float32))) if bf16 else (lambda x: x.astype(np.float32))
    a, b = rnd(r.standard_normal((B, T, H)) * 6), rnd(r.standard_normal((B, T, H)) * 3)
    A, bias = (r.standard_normal(H) * 0.5).astype(np.float32), r.standard_normal(H).astype(np.float32)
    dg, dbeta = r.standard_normal((B, T, H)).astype(np.float32), r.standard_normal((B, T, H)).astype(np.float32)
    g_ref, beta_ref = og.gdn_gate(a, A, bias if with_bias else None, b if with_b else None, neg)
    da_ref, dA_ref, dbias_ref, db_ref = og.gdn_gate_grad(a, A, dg, bias if with_bias else None, b if with_b else None, dbeta, neg)
    dt = torch.bfloat16 if bf16 else torch.float32
    ta, tA = _t(a, dt, True), _t(A, None, True)
    tb = _t(b, dt, True) if with_b else None
    tbias = _t(bias, None, True) if with_bias else None
    g, beta = la.gated_deltanet_gate(ta, tA, tbias, tb, neg)
    assert g.dtype == torch.float32 and g.shape == (B, T, H) and (beta is None) == (not with_b)
    loss = (g * _t(dg)).sum()
    if with_b:
        loss = loss + (beta * _t(dbeta)).sum()
    loss.backward()
    assert max_rel(g.detach().cpu().numpy(), g_ref) < 1e-5
    tol = 2e-2 if bf16 else 1e-5
    assert max_rel(ta.grad.float().cpu().numpy(), da_ref) < tol
    assert max_rel(tA.grad.cpu().numpy(), dA_ref) < 1e-4
    if with_bias:
        assert max_rel(tbias.grad.cpu().numpy(), dbias_ref) < 1e-4
    if with_b:
        assert max_rel(beta.detach().cpu().numpy(), beta_ref) < 1e-6
        assert max_rel(tb.grad.float().cpu().numpy(), db_ref) < tol


def test_gated_deltanet_gate_errors_and_empty():
    import linearnexus_amd as la
    A = torch.zeros(4, device=DEV)
    with pytest.raises(RuntimeError):
        la.gated_deltanet_gate(torch.randn(2, 3, 5, device=DEV), A)
    with pytest.raises(RuntimeError):
        la.gated_deltanet_gate(torch.randn(2, 3, 4), A)
    with pytest.raises(RuntimeError):
        la.gated_deltanet_gate(torch.randn(2, 3, 4, device=DEV), A, torch.zeros(3, device=DEV))
    g, beta = la.gated_deltanet_gate(torch.randn(2, 0, 4, device=DEV), A)
    assert g.shape == (2, 0, 4) and beta is None
