"""GPU parity of the chunked backward kernels: gradients from torch.autograd through the HIP
ops against the fp64 token-level adjoint oracle (= autodiff of the recurrent form).
Metric max|x - ref| / max|ref| per tensor: 1e-4 for fp32 inputs, 2e-2 for bf16 inputs."""
import numpy as np
import pytest
import torch

from oracle.adjoint import delta_rule_adjoint
from oracle.inputs import make_inputs, to_bf16_grid
from conftest import max_rel

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _t(a, dtype=None, grad=False):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    if dtype is not None:
        t = t.to(dtype)
    return t.requires_grad_(grad)


def gpu_grads(x, gate, dt, l2=False, cu=None, with_state=True, with_dS=True):
    import linearnexus_amd as la
    q, k, v = _t(x["q"], dt, True), _t(x["k"], dt, True), _t(x["v"], dt, True)
    beta = _t(x["beta"], None, True)
    g = _t(x["g"], None, True) if gate != "none" else None
    s0 = _t(x["S0"], None, True) if with_state else None
    cu_t = None if cu is None else torch.from_numpy(cu).to(DEV)
    if gate == "none":
        o, S = la.delta_rule_chunkwise(q, k, v, beta, s0, cu_seqlens=cu_t)
    elif gate == "scalar":
        o, S = la.gated_delta_rule_chunkwise(q, k, v, g, beta, None, s0, 64, l2, cu_seqlens=cu_t)
    else:
        o, S = la.kda_chunkwise(q, k, v, g, beta, None, s0, 64, l2, cu_seqlens=cu_t)
    loss = (o.float() * _t(x["dO"])).sum()
    if with_dS:
        loss = loss + (S * _t(x["dS"])).sum()
    loss.backward()
    out = {"dq": q.grad, "dk": k.grad, "dv": v.grad, "dbeta": beta.grad}
    if g is not None:
        out["dg"] = g.grad
    if s0 is not None:
        out["dS0"] = s0.grad
    return {n: t.float().cpu().numpy() for n, t in out.items()}


def check(got, ref, tol):
    errs = {n: max_rel(got[n], ref[n]) for n in got}
    bad = {n: e for n, e in errs.items() if not e < tol}
    assert not bad, (bad, errs)


def _prep(x, bf16):
    if not bf16:
        return x, torch.float32
    y = dict(x)
    for n in ("q", "k", "v", "dO"):
        y[n] = to_bf16_grid(x[n])
    return y, torch.bfloat16


GATES = ["none", "scalar", "vector"]


@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("shape", [(2, 2, 128, 64, 64), (1, 2, 200, 128, 128), (1, 2, 70, 128, 64), (1, 1, 256, 64, 128)])
def test_chunk_backward_matches_adjoint_oracle(gate, bf16, shape):
    B, H, T, dk, dv = shape
    x = make_inputs(51, B, H, T, dk, dv, gate=gate, with_state=True, with_grad=True)
    x, dt = _prep(x, bf16)
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x.get("g"), x["dS"], None, x["S0"], False)
    got = gpu_grads(x, gate, dt)
    check(got, ref, 2e-2 if bf16 else 1e-4)


@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("dk,dv", [(128, 192), (64, 320), (128, 64)])
def test_chunk_backward_slab_buffer_rotation(gate, dk, dv):
    """bf16 inputs: the chunk-local backward kernels take the value dimension in 32-column slabs that arrive through
    loads straight to LDS into two or three buffers in rotation; 2, 6 and 10 slabs leave the rotation at every buffer."""
    x = make_inputs(57, 1, 2, 150, dk, dv, gate=gate, with_state=True, with_grad=True)
    x, dt = _prep(x, True)
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x.get("g"), x["dS"], None, x["S0"], False)
    check(gpu_grads(x, gate, dt), ref, 2e-2)


@pytest.mark.parametrize("gate", GATES)
def test_backward_without_state_gradients(gate):
    """Zero initial state, no gradient flowing into the final state."""
    x = make_inputs(52, 1, 2, 192, 128, 128, gate=gate, with_grad=True)
    x, dt = _prep(x, True)
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x.get("g"))
    got = gpu_grads(x, gate, dt, with_state=False, with_dS=False)
    check(got, ref, 2e-2)


@pytest.mark.parametrize("gate", ["scalar", "vector"])
def test_backward_through_l2norm(gate):
    x = make_inputs(53, 1, 2, 130, 128, 128, gate=gate, with_state=True, with_grad=True, normalize=False)
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x["g"], x["dS"], None, x["S0"], True)
    got = gpu_grads(x, gate, torch.float32, l2=True)
    check(got, ref, 1e-4)


@pytest.mark.parametrize("shape", [(2, 2, 200, 128, 128), (1, 2, 130, 64, 128), (1, 3, 64, 128, 64)])
@pytest.mark.parametrize("packed", [False, True])
def test_backward_through_l2norm_inside_the_chunk_kernels(shape, packed):
    """bf16 inputs with no per-channel gate: the kernels scale the q and k rows themselves (no normalised copies) and
    lnx_chunk_bwd returns the gradients of the raw rows (gated_deltanet.py:273-275 normalises inside the op).  Rows of
    very different lengths."""
    import linearnexus_amd as la
    from linearnexus_amd import _lib
    B, H, T, dk, dv = shape
    if packed:
        B = 1
    x = make_inputs(57, B, H, T, dk, dv, gate="scalar", with_state=not packed, with_grad=True, normalize=False)
    rng = np.random.default_rng(58)
    x["q"] = x["q"] * np.exp(rng.standard_normal((B, H, T, 1))).astype(np.float32)
    x["k"] = x["k"] * np.exp(rng.standard_normal((B, H, T, 1))).astype(np.float32)
    x, dt = _prep(x, True)
    a = _lib.ScanArgs(B=B, H=H, T=T, dk=dk, dv=dv, chunk=64, dtype=_lib.LNX_BF16, o_dtype=_lib.LNX_BF16, gate=_lib.GATE_SCALAR)
    assert _lib.load().lnx_chunk_fuses_l2norm(a) == 1
    if packed:
        cu = np.array([0, 3, T // 2, T], np.int32)
        x["S0"] = (rng.standard_normal((3, H, dk, dv)) * 0.02).astype(np.float32)
        x["dS"] = (rng.standard_normal((3, H, dk, dv)) * 0.1).astype(np.float32)
        parts = []
        for s_ in range(3):
            lo, hi = cu[s_], cu[s_ + 1]
            sl = lambda n: x[n][:, :, lo:hi]
            parts.append(delta_rule_adjoint(sl("q"), sl("k"), sl("v"), sl("beta"), sl("dO"), sl("g"), x["dS"][s_:s_ + 1], None,
                                            x["S0"][s_:s_ + 1], True))
        ref = {n: np.concatenate([p_[n] for p_ in parts], 2) for n in ("dq", "dk", "dv", "dbeta", "dg")}
        ref["dS0"] = np.concatenate([p_["dS0"] for p_ in parts], 0)
        got = gpu_grads(x, "scalar", dt, l2=True, cu=cu)
    else:
        ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x["g"], x["dS"], None, x["S0"], True)
        got = gpu_grads(x, "scalar", dt, l2=True)
    assert all(np.isfinite(t).all() for t in got.values())
    check(got, ref, 2e-2)


@pytest.mark.parametrize("gate", GATES)
def test_backward_packed_sequences(gate):
    H, T, d = 2, 300, 128
    x = make_inputs(54, 1, H, T, d, d, gate=gate, with_grad=True)
    cu = np.array([0, 64, 70, 200, 300], np.int32)
    rng = np.random.default_rng(6)
    x["S0"] = (rng.standard_normal((4, H, d, d)) * 0.02).astype(np.float32)
    x["dS"] = (rng.standard_normal((4, H, d, d)) * 0.1).astype(np.float32)
    x, dt = _prep(x, True)
    parts = []
    for s in range(4):
        a, b = cu[s], cu[s + 1]
        sl = lambda n: x[n][:, :, a:b]
        parts.append(delta_rule_adjoint(sl("q"), sl("k"), sl("v"), sl("beta"), sl("dO"), sl("g") if gate != "none" else None,
                                        x["dS"][s:s + 1], None, x["S0"][s:s + 1], False))
    ref = {n: np.concatenate([p[n] for p in parts], 2) for n in ("dq", "dk", "dv", "dbeta") + (("dg",) if gate != "none" else ())}
    ref["dS0"] = np.concatenate([p["dS0"] for p in parts], 0)
    got = gpu_grads(x, gate, dt, cu=cu)
    check(got, ref, 2e-2)


def test_backward_packed_sequences_of_four_to_eight_chunks():
    """Per-channel gate, packed sequences of 4, 5, 7 and 8 chunks behind one another: the scans take two chunks per loop
    round once a sequence has four, with an odd or even remainder, and start every sequence on the first of their two
    tile buffers whatever the parity of its first chunk in the batch."""
    H, d = 1, 128
    lens = [256, 300, 448, 512]
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T = int(cu[-1])
    x = make_inputs(58, 1, H, T, d, d, gate="vector", with_grad=True)
    rng = np.random.default_rng(8)
    x["S0"] = (rng.standard_normal((4, H, d, d)) * 0.02).astype(np.float32)
    x["dS"] = (rng.standard_normal((4, H, d, d)) * 0.1).astype(np.float32)
    x, dt = _prep(x, True)
    parts = []
    for s in range(4):
        a, b = cu[s], cu[s + 1]
        sl = lambda n: x[n][:, :, a:b]
        parts.append(delta_rule_adjoint(sl("q"), sl("k"), sl("v"), sl("beta"), sl("dO"), sl("g"), x["dS"][s:s + 1], None,
                                        x["S0"][s:s + 1], False))
    ref = {n: np.concatenate([p[n] for p in parts], 2) for n in ("dq", "dk", "dv", "dbeta", "dg")}
    ref["dS0"] = np.concatenate([p["dS0"] for p in parts], 0)
    check(gpu_grads(x, "vector", dt, cu=cu), ref, 2e-2)


def test_backward_adjoint_identity_at_full_config2_size():
    """Size-independent check at B8 H16 T4096 d128 bf16 with S0 = 0: o is linear in v, so
    <dO, o(v)> == <dv, v> must hold for the dv the backward kernels return."""
    import linearnexus_amd as la
    torch.manual_seed(3)
    B, H, T, d = 8, 16, 4096, 128
    q = torch.nn.functional.normalize(torch.randn(B, H, T, d, device=DEV), dim=-1).bfloat16()
    k = torch.nn.functional.normalize(torch.randn(B, H, T, d, device=DEV), dim=-1).bfloat16()
    v = torch.randn(B, H, T, d, device=DEV).bfloat16().requires_grad_(True)
    beta = torch.sigmoid(torch.randn(B, H, T, device=DEV))
    g = -torch.nn.functional.softplus(torch.randn(B, H, T, device=DEV)) * 0.1
    dO = torch.randn(B, H, T, d, device=DEV).bfloat16()
    o, _ = la.gated_delta_rule_chunkwise(q, k, v, g, beta, use_qk_l2norm=False)
    o.backward(dO)
    tl, tr = o.detach().double() * dO.double(), v.grad.double() * v.detach().double()
    lhs, rhs = tl.sum(), tr.sum()
    # o and dv are rounded to bf16: independent relative errors, uniform within +-2^-9, on each of the
    # 6.7e7 terms of either sum.  sigma is the standard deviation of their accumulated effect (the sums
    # themselves are small against it: ~30 against 0.14); the two sides must agree within 4 sigma.
    sigma = 2.0 ** -9 / 3 ** 0.5 * torch.sqrt((tl * tl).sum() + (tr * tr).sum())
    assert abs(lhs - rhs) <= 4 * sigma, (float(lhs), float(rhs), float(sigma))
