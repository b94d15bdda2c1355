"""Benchmark-shaped parity checks on the GPU.

The fp64 oracle finishes in seconds only on slices, so at the full benchmark shapes the checks
are (a) the oracle on a slice of the (batch, head) rows of the very same launch and
(b) size-independent properties: MFMA chunk path == fp32 token-by-token kernel, the adjoint
identity <dO, o(v)> = <dv, v>, and var-len == per-sequence launches."""
import numpy as np
import pytest
import torch

from oracle import recurrent as rc
from oracle.adjoint import delta_rule_adjoint
from oracle.inputs import make_cu_seqlens
from conftest import max_rel

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _nrm(x):
    return x / (x.norm(dim=-1, keepdim=True) + 1e-6)


def _rel(a, b):
    a, b = a.detach(), b.detach()
    return float((a.double() - b.double()).abs().max() / b.double().abs().max())


def _row_grads_against_oracle(grads, inputs, dO, b, h, t0, t1, s0_row, tol=2e-2):
    """One (batch, head) row of a full-shape launch, tokens [t0, t1), against the token-level adjoint in fp64: every
    gradient the backward pass returns, after the whole chain of carried state gradients."""
    f = lambda t: t.detach()[b:b + 1, h:h + 1, t0:t1].float().cpu().numpy()
    g = inputs.get("g")
    ref = delta_rule_adjoint(f(inputs["q"]), f(inputs["k"]), f(inputs["v"]), f(inputs["beta"]), f(dO),
                             None if g is None else f(g), None, None, s0_row, False)
    for name in ("dq", "dk", "dv", "dbeta") + (("dg",) if g is not None else ()):
        err = max_rel(f(grads[name]), ref[name])
        assert err < tol, (name, err)
    return ref


def test_config2_gradients_of_one_full_row():
    """Gated DeltaNet chunk fwd+bwd at B8 H16 T4096 d128 bf16: dq, dk, dv, dbeta, dg and dS0 of one (batch, head) row of
    the full launch against the fp64 token-level adjoint over all 4096 tokens (64 chunks of carried dS)."""
    import linearnexus_amd as la
    torch.manual_seed(2)
    B, H, T, d = 8, 16, 4096, 128
    q = _nrm(torch.randn(B, H, T, d, device=DEV)).bfloat16().requires_grad_(True)
    k = _nrm(torch.randn(B, H, T, d, device=DEV)).bfloat16().requires_grad_(True)
    v = torch.randn(B, H, T, d, device=DEV).bfloat16().requires_grad_(True)
    beta = torch.sigmoid(torch.randn(B, H, T, device=DEV)).requires_grad_(True)
    g = (-torch.nn.functional.softplus(torch.randn(B, H, T, device=DEV)) * 0.1).requires_grad_(True)
    S0 = torch.zeros(B, H, d, d, device=DEV, requires_grad=True)
    dO = torch.randn(B, H, T, d, device=DEV).bfloat16()
    o, _ = la.gated_delta_rule_chunkwise(q, k, v, g, beta, None, S0, 64, False)
    o.backward(dO)
    grads = dict(dq=q.grad, dk=k.grad, dv=v.grad, dbeta=beta.grad, dg=g.grad)
    for b, h in ((5, 11), (0, 0)):
        ref = _row_grads_against_oracle(grads, dict(q=q, k=k, v=v, beta=beta, g=g), dO, b, h, 0, T,
                                        np.zeros((1, 1, d, d)))
        assert max_rel(S0.grad[b:b + 1, h:h + 1].cpu().numpy(), ref["dS0"]) < 2e-2


def test_config3_kda_gradients_of_one_full_row():
    """KDA chunk fwd+bwd at B4 H16 T8192 d128 bf16 with a random S0: all gradients of one row over all 8192 tokens."""
    import linearnexus_amd as la
    torch.manual_seed(33)
    B, H, T, d = 4, 16, 8192, 128
    q = _nrm(torch.randn(B, H, T, d, device=DEV)).bfloat16().requires_grad_(True)
    k = _nrm(torch.randn(B, H, T, d, device=DEV)).bfloat16().requires_grad_(True)
    v = torch.randn(B, H, T, d, device=DEV).bfloat16().requires_grad_(True)
    beta = torch.sigmoid(torch.randn(B, H, T, device=DEV)).requires_grad_(True)
    g = (-torch.nn.functional.softplus(torch.randn(B, H, T, d, device=DEV)) * 0.05).requires_grad_(True)
    S0 = (torch.randn(B, H, d, d, device=DEV) * 0.02).requires_grad_(True)
    dO = torch.randn(B, H, T, d, device=DEV)
    o, _ = la.kda_chunkwise(q, k, v, g, beta, None, S0, 64, False)
    o.backward(dO)
    grads = dict(dq=q.grad, dk=k.grad, dv=v.grad, dbeta=beta.grad, dg=g.grad)
    b, h = 2, 9
    ref = _row_grads_against_oracle(grads, dict(q=q, k=k, v=v, beta=beta, g=g), dO, b, h, 0, T,
                                    S0.detach()[b:b + 1, h:h + 1].cpu().numpy())
    assert max_rel(S0.grad[b:b + 1, h:h + 1].cpu().numpy(), ref["dS0"]) < 2e-2


def test_config3_kda_full_shape():
    """KDA chunk fwd+bwd at B4 H16 T8192 d128 bf16, vector gate, random S0."""
    import linearnexus_amd as la
    torch.manual_seed(3)
    B, H, T, d = 4, 16, 8192, 128
    q = _nrm(torch.randn(B, H, T, d, device=DEV)).bfloat16()
    k = _nrm(torch.randn(B, H, T, d, device=DEV)).bfloat16()
    v = torch.randn(B, H, T, d, device=DEV).bfloat16().requires_grad_(True)
    beta = torch.sigmoid(torch.randn(B, H, T, device=DEV))
    g = -torch.nn.functional.softplus(torch.randn(B, H, T, d, device=DEV)) * 0.05
    S0 = torch.randn(B, H, d, d, device=DEV) * 0.02
    o1, S1 = la.kda_recurrent(q, k, v.detach(), g, beta, None, S0, False)
    o2, S2 = la.kda_chunkwise(q, k, v, g, beta, None, S0, 64, False)
    assert o2.dtype == torch.float32  # kda.py:655
    assert _rel(o2, o1.float()) < 2e-2 and _rel(S2, S1) < 2e-2
    # oracle on one (batch, head) row of the same launch, first 512 tokens
    sl = lambda t: t.detach()[1:2, 3:4, :512].float().cpu().numpy()
    o_ref, _ = rc.kda_recurrent(sl(q), sl(k), sl(v.detach()), sl(g), sl(beta), None, S0[1:2, 3:4].cpu().numpy(), False)
    assert max_rel(o2.detach()[1:2, 3:4, :512].cpu().numpy(), o_ref) < 2e-2
    # adjoint identity with S0 = 0 (o linear in v)
    dO = torch.randn(B, H, T, d, device=DEV)
    o3, _ = la.kda_chunkwise(q, k, v, g, beta, None, None, 64, False)
    o3.backward(dO)
    tl, tr = o3.detach().double() * dO.bfloat16().double(), v.grad.double() * v.detach().double()
    lhs, rhs = tl.sum(), tr.sum()
    # o leaves the kernels as bf16 and dv is bf16: independent relative errors, uniform within +-2^-9, on each of the
    # 6.7e7 terms of either sum; sigma is the standard deviation of their accumulated effect.  The tiles between the
    # kernels (D, dD, the states, W, U, the scaled pair operands) are rounded the same way, hence 8 sigma, not 4.
    sigma = 2.0 ** -9 / 3 ** 0.5 * torch.sqrt((tl * tl).sum() + (tr * tr).sum())
    ratio = float(abs(lhs - rhs) / sigma)
    print(f"adjoint identity at config 3: |<o,dO> - <dv,v>| = {ratio:.2f} sigma, {float(abs(lhs - rhs) / abs(lhs)):.2e} of <o,dO>")
    assert ratio <= 8, (float(lhs), float(rhs), float(sigma), ratio)


def test_config5_deltanet_long_packed():
    """DeltaNet chunk fwd+bwd at B1 H32 T32768 d128 bf16, 8 packed sequences in [1024, 8192]."""
    import linearnexus_amd as la
    torch.manual_seed(5)
    H, T, d = 32, 32768, 128
    cu = make_cu_seqlens(5, 8, T, 1024, 8192)
    q = _nrm(torch.randn(1, H, T, d, device=DEV)).bfloat16().requires_grad_(True)
    k = _nrm(torch.randn(1, H, T, d, device=DEV)).bfloat16().requires_grad_(True)
    v = torch.randn(1, H, T, d, device=DEV).bfloat16().requires_grad_(True)
    beta = torch.sigmoid(torch.randn(1, H, T, device=DEV)).requires_grad_(True)
    S0 = (torch.randn(8, H, d, d, device=DEV) * 0.02).requires_grad_(True)
    dO = torch.randn(1, H, T, d, device=DEV).bfloat16()
    cu_t = torch.from_numpy(cu).to(DEV)
    o, S = la.delta_rule_chunkwise(q, k, v, beta, S0, cu_seqlens=cu_t)
    o.backward(dO)
    assert tuple(S.shape) == (8, H, d, d) and all(t.grad is not None for t in (q, k, v, beta, S0))
    # (a) packed == the token-by-token kernel on the packed batch
    o_r, S_r = la.delta_rule_recurrent(q.detach(), k.detach(), v.detach(), beta.detach(), S0.detach(), cu_seqlens=cu_t)
    assert _rel(o, o_r) < 2e-2 and _rel(S, S_r) < 2e-2
    # (b) packed == one launch per sequence, outputs and every gradient (sequence 2 and the last)
    for s in (2, 7):
        a, b = int(cu[s]), int(cu[s + 1])
        leaf = lambda t: t.detach()[:, :, a:b].clone().requires_grad_(True)
        qs, ks, vs, bs = leaf(q), leaf(k), leaf(v), leaf(beta)
        s0 = S0.detach()[s:s + 1].clone().requires_grad_(True)
        o_s, S_s = la.delta_rule_chunkwise(qs, ks, vs, bs, s0)
        o_s.backward(dO[:, :, a:b])
        assert _rel(o[:, :, a:b], o_s) < 1e-3 and _rel(S[s:s + 1], S_s) < 1e-3
        for full, part in ((q.grad, qs.grad), (k.grad, ks.grad), (v.grad, vs.grad), (beta.grad, bs.grad)):
            assert _rel(full[:, :, a:b], part) < 1e-3
        assert _rel(S0.grad[s:s + 1], s0.grad) < 1e-3
    # (c) every gradient of one whole sequence of one head (its packed neighbours in place) against the fp64 adjoint
    for s_, h in ((3, 17), (7, 0)):
        a, b = int(cu[s_]), int(cu[s_ + 1])
        grads = dict(dq=q.grad, dk=k.grad, dv=v.grad, dbeta=beta.grad)
        ref = _row_grads_against_oracle(grads, dict(q=q, k=k, v=v, beta=beta), dO, 0, h, a, b,
                                        S0.detach()[s_:s_ + 1, h:h + 1].cpu().numpy())
        assert max_rel(S0.grad[s_:s_ + 1, h:h + 1].cpu().numpy(), ref["dS0"]) < 2e-2
    # (d) oracle on the first 300 tokens of sequence 0, head 5
    a = int(cu[0])
    sl = lambda t: t.detach()[:, 5:6, a:a + 300].float().cpu().numpy()
    o_ref, _ = rc.delta_rule_recurrent(sl(q), sl(k), sl(v), sl(beta), S0.detach()[0:1, 5:6].cpu().numpy())
    assert max_rel(o.detach()[:, 5:6, a:a + 300].float().cpu().numpy(), o_ref) < 2e-2


def test_config4_decode_full_shape_one_step_and_1000_steps():
    """Gated decode step at B256 H32 d128: one in-place step against the oracle on a slice of
    the rows, then 1000 back-to-back steps on a smaller batch against the oracle scan."""
    import linearnexus_amd as la
    torch.manual_seed(4)
    B, H, d = 256, 32, 128
    S = torch.randn(B, H, d, d, device=DEV) * 0.02
    S_before = S[:2, :4].clone()
    q = _nrm(torch.randn(B, H, d, device=DEV)).bfloat16()
    k = _nrm(torch.randn(B, H, d, device=DEV)).bfloat16()
    v = torch.randn(B, H, d, device=DEV).bfloat16()
    beta = torch.sigmoid(torch.randn(B, H, device=DEV))
    g = -torch.nn.functional.softplus(torch.randn(B, H, device=DEV)) * 0.1
    o, S2 = la.gated_delta_rule_step(q, k, v, g, beta, S, use_qk_l2norm=False, inplace=True)
    assert S2.data_ptr() == S.data_ptr()
    n = lambda t: t[:2, :4].float().cpu().numpy()
    o_ref, S_ref = rc.gated_delta_rule_step(n(q), n(k), n(v), n(g), n(beta), S_before.cpu().numpy(), None, False)
    assert max_rel(o[:2, :4].float().cpu().numpy(), o_ref) < 2e-2 and max_rel(S[:2, :4].cpu().numpy(), S_ref) < 2e-2
    # 1000 steps, B=4 H=4
    B, H, T = 4, 4, 1000
    S = torch.randn(B, H, d, d, device=DEV) * 0.02
    S0 = S.clone()
    q = _nrm(torch.randn(B, H, T, d, device=DEV)).bfloat16()
    k = _nrm(torch.randn(B, H, T, d, device=DEV)).bfloat16()
    v = torch.randn(B, H, T, d, device=DEV).bfloat16()
    beta = torch.sigmoid(torch.randn(B, H, T, device=DEV))
    g = -torch.nn.functional.softplus(torch.randn(B, H, T, device=DEV)) * 0.1
    outs = []
    for t in range(T):
        o, _ = la.gated_delta_rule_step(q[:, :, t], k[:, :, t], v[:, :, t], g[:, :, t], beta[:, :, t], S,
                                        use_qk_l2norm=False, inplace=True)
        outs.append(o)
    o = torch.stack(outs, 2)
    f = lambda t: t.float().cpu().numpy()
    o_ref, S_ref = rc.gated_delta_rule_recurrent(f(q), f(k), f(v), f(g), f(beta), None, f(S0), False)
    assert max_rel(f(o), o_ref) < 2e-2 and max_rel(f(S), S_ref) < 2e-2


def test_config4_decode_1000_steps_at_the_full_shape():
    """Config 4 as BASELINE states it: 1000 back-to-back in-place gated_delta_rule_step calls on the fp32 state
    [256, 32, 128, 128] (gated_deltanet.py:539-597), checked after all of them -- the last step's outputs and the final
    state of eight (batch, head) rows against the fp64 token-by-token oracle run over the same 1000 tokens.  The token
    inputs cycle through eight distinct tokens (the state evolves, the inputs may repeat)."""
    import linearnexus_amd as la
    torch.manual_seed(44)
    B, H, d, T, NTOK = 256, 32, 128, 1000, 8
    S = torch.randn(B, H, d, d, device=DEV) * 0.02
    rows_b, rows_h = [0, 255], [0, 7, 19, 31]
    S0 = S[rows_b][:, rows_h].clone()
    q = _nrm(torch.randn(NTOK, B, H, d, device=DEV)).bfloat16()
    k = _nrm(torch.randn(NTOK, B, H, d, device=DEV)).bfloat16()
    v = torch.randn(NTOK, B, H, d, device=DEV).bfloat16()
    beta = torch.sigmoid(torch.randn(NTOK, B, H, device=DEV))
    g = -torch.nn.functional.softplus(torch.randn(NTOK, B, H, device=DEV)) * 0.1
    o = None
    for t in range(T):
        i = t % NTOK
        o, S2 = la.gated_delta_rule_step(q[i], k[i], v[i], g[i], beta[i], S, use_qk_l2norm=False, inplace=True)
    assert S2.data_ptr() == S.data_ptr()
    torch.cuda.synchronize()
    # the same 1000 tokens as a [2, 4, 1000, .] sequence for the oracle
    idx = torch.arange(T, device=DEV) % NTOK
    seq = lambda t: t[idx][:, rows_b][:, :, rows_h].permute(1, 2, 0, *range(3, t.dim())).float().cpu().numpy()
    o_ref, S_ref = rc.gated_delta_rule_recurrent(seq(q), seq(k), seq(v), seq(g), seq(beta), None, S0.cpu().numpy(), False)
    assert max_rel(o[rows_b][:, rows_h].float().cpu().numpy(), o_ref[:, :, -1]) < 2e-2
    assert max_rel(S[rows_b][:, rows_h].cpu().numpy(), S_ref) < 2e-2
    assert torch.isfinite(S).all()
