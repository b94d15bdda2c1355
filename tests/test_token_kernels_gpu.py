"""GPU parity of the token-level kernels (decode step, token-by-token scan) against the
fp64 oracle, through the C-ABI.  Tolerances: 1e-4 (fp32) / 2e-2 (bf16 inputs), as
max|x - ref| / max|ref|."""
import numpy as np
import pytest
import torch

from oracle import recurrent as rc
from oracle.inputs import make_inputs, to_bf16_grid
from conftest import max_rel

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _t(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    return t.to(dtype) if dtype is not None else t


def _prep(x, bf16):
    """Casts q,k,v to the kernel dtype; the oracle sees exactly the values the kernel sees."""
    if not bf16:
        return x, torch.float32
    y = dict(x)
    for n in ("q", "k", "v"):
        y[n] = to_bf16_grid(x[n])
    return y, torch.bfloat16


def _oracle_rec(x, gate, l2):
    if gate == "none":
        return rc.delta_rule_recurrent(x["q"], x["k"], x["v"], x["beta"], x.get("S0"))
    fn = rc.gated_delta_rule_recurrent if gate == "scalar" else rc.kda_recurrent
    return fn(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x.get("S0"), l2)


def _gpu_rec(x, gate, l2, dt, cu=None):
    import linearnexus_amd as la
    q, k, v = _t(x["q"], dt), _t(x["k"], dt), _t(x["v"], dt)
    s0 = _t(x["S0"]) if "S0" in x else None
    cu_t = None if cu is None else _t(cu)
    if gate == "none":
        return la.delta_rule_recurrent(q, k, v, _t(x["beta"]), s0, cu_seqlens=cu_t)
    fn = la.gated_delta_rule_recurrent if gate == "scalar" else la.kda_recurrent
    return fn(q, k, v, _t(x["g"]), _t(x["beta"]), None, s0, l2, cu_seqlens=cu_t)


@pytest.mark.parametrize("gate", ["none", "scalar", "vector"])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("shape", [(2, 4, 96, 64, 64), (1, 2, 130, 128, 128), (2, 2, 33, 16, 32), (1, 3, 17, 8, 8),
                                   (1, 1, 40, 256, 64), (1, 2, 20, 32, 100)])
def test_recurrent_scan_matches_oracle(gate, bf16, shape):
    B, H, T, dk, dv = shape
    l2 = gate != "none"
    x = make_inputs(21, B, H, T, dk, dv, gate=gate, with_state=True, normalize=not l2)
    x, dt = _prep(x, bf16)
    o_ref, S_ref = _oracle_rec(x, gate, l2)
    o, S = _gpu_rec(x, gate, l2, dt)
    assert o.dtype == dt and S.dtype == torch.float32
    tol = 2e-2 if bf16 else 1e-4
    assert max_rel(o.float().cpu().numpy(), o_ref) < tol
    assert max_rel(S.cpu().numpy(), S_ref) < (1e-4 if not bf16 else 2e-2)


def test_recurrent_scan_config1_shape_fp32():
    """B2 H4 T512 d64 fp32, zero initial state: the fp32 parity configuration."""
    x = make_inputs(1, 2, 4, 512, 64, 64)
    o_ref, S_ref = _oracle_rec(x, "none", False)
    o, S = _gpu_rec(x, "none", False, torch.float32)
    assert max_rel(o.cpu().numpy(), o_ref) < 1e-4 and max_rel(S.cpu().numpy(), S_ref) < 1e-4


def test_recurrent_scan_packed_sequences():
    x = make_inputs(22, 1, 3, 200, 64, 64, gate="scalar")
    cu = np.array([0, 70, 71, 160, 200], np.int32)
    S0 = (np.random.default_rng(3).standard_normal((4, 3, 64, 64)) * 0.02).astype(np.float32)
    o_ref, S_ref = rc.varlen(
        lambda q, k, v, g, b, initial_state=None: rc.gated_delta_rule_recurrent(q, k, v, g, b, None, initial_state, False),
        cu, x["q"], x["k"], x["v"], x["g"], x["beta"], initial_state=S0)
    x["S0"] = S0
    o, S = _gpu_rec(x, "scalar", False, torch.float32, cu)
    assert tuple(S.shape) == (4, 3, 64, 64)
    assert max_rel(o.cpu().numpy(), o_ref) < 1e-4 and max_rel(S.cpu().numpy(), S_ref) < 1e-4


def test_orthonormal_keys_closed_form_on_gpu():
    # tests/test_deltanet.py:330-346 with its closed form: S_T = V, o_t = dk^-1/2 v_t
    import linearnexus_amd as la
    dk = 8
    k = torch.eye(dk, device=DEV)[None, None]
    v = torch.randn(1, 1, dk, dk, device=DEV)
    o, S = la.delta_rule_recurrent(k.clone(), k, v, torch.ones(1, 1, dk, device=DEV))
    assert torch.allclose(S[0, 0], v[0, 0], atol=1e-6) and torch.allclose(o, dk ** -0.5 * v, atol=1e-6)


@pytest.mark.parametrize("gate", ["none", "scalar", "vector"])
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("shape", [(3, 4, 128, 128), (2, 2, 64, 64), (2, 4, 16, 32), (2, 4, 8, 8), (1, 2, 32, 200),
                                   (2, 3, 256, 512)])
def test_decode_step_matches_oracle(gate, bf16, shape):
    import linearnexus_amd as la
    B, H, dk, dv = shape
    l2 = gate != "none"
    x = make_inputs(23, B, H, 1, dk, dv, gate=gate, with_state=True, normalize=not l2)
    x, dt = _prep(x, bf16)
    sq = lambda a: a[:, :, 0]
    q, k, v, beta = (_t(sq(x[n]), dt if n != "beta" else None) for n in ("q", "k", "v", "beta"))
    S0 = _t(x["S0"])
    keep = S0.clone()
    if gate == "none":
        o_ref, S_ref = rc.delta_rule_step(sq(x["q"]), sq(x["k"]), sq(x["v"]), sq(x["beta"]), x["S0"])
        o, S = la.delta_rule_step(q, k, v, beta, S0)
    elif gate == "scalar":
        o_ref, S_ref = rc.gated_delta_rule_step(sq(x["q"]), sq(x["k"]), sq(x["v"]), sq(x["g"]), sq(x["beta"]), x["S0"])
        o, S = la.gated_delta_rule_step(q, k, v, _t(sq(x["g"])), beta[..., None], S0)
    else:
        o_ref, S_ref = rc.kda_step(sq(x["q"]), sq(x["k"]), sq(x["v"]), sq(x["g"]), sq(x["beta"]), x["S0"])
        o, S = la.kda_step(q, k, v, _t(sq(x["g"])), beta, S0)
    assert torch.equal(S0, keep), "the functional form must not touch the input state"
    assert o.dtype == (torch.float32 if gate == "vector" else dt)  # kda.py:347 returns state.dtype
    tol = 2e-2 if bf16 else 1e-4
    assert max_rel(o.float().cpu().numpy(), o_ref) < tol
    assert max_rel(S.cpu().numpy(), S_ref) < (1e-5 if not bf16 else 2e-2)


def test_decode_step_inplace_many_steps_follow_the_scan():
    """In-place steps chained 64 times equal the oracle scan over the same 64 tokens."""
    import linearnexus_amd as la
    B, H, T, d = 2, 3, 64, 128
    x = make_inputs(24, B, H, T, d, d, gate="scalar", with_state=True)
    x, dt = _prep(x, True)
    o_ref, S_ref = rc.gated_delta_rule_recurrent(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["S0"], False)
    S = _t(x["S0"]).clone()
    ptr = S.data_ptr()
    q, k, v, g, beta = _t(x["q"], dt), _t(x["k"], dt), _t(x["v"], dt), _t(x["g"]), _t(x["beta"])
    outs = []
    for t in range(T):
        o, S2 = la.gated_delta_rule_step(q[:, :, t], k[:, :, t], v[:, :, t], g[:, :, t], beta[:, :, t], S,
                                         use_qk_l2norm=False, inplace=True)
        assert S2.data_ptr() == ptr
        outs.append(o)
    o = torch.stack(outs, 2)
    assert max_rel(o.float().cpu().numpy(), o_ref) < 2e-2 and max_rel(S.cpu().numpy(), S_ref) < 2e-2


def test_beta_zero_leaves_zero_state_on_gpu():
    # tests/test_deltanet.py:281-297
    import linearnexus_amd as la
    q = torch.randn(1, 2, 4, 16, device=DEV)
    o, S = la.delta_rule_recurrent(q, q.clone(), torch.randn(1, 2, 4, 32, device=DEV), torch.zeros(1, 2, 4, device=DEV))
    assert torch.count_nonzero(S) == 0 and torch.count_nonzero(o) == 0


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("rows,d", [(37, 128), (1, 64), (1000, 256), (130, 16), (5, 100), (9, 512), (0, 128)])
def test_l2norm_rows_fwd_bwd(rows, d, bf16):
    """x / (|x| + 1e-6) and its gradient; covers the vector kernels (16-byte row pieces, 4..64 lanes per
    row), the scalar fallback for other row lengths, ragged last passes and an empty tensor."""
    import linearnexus_amd as la
    from linearnexus_amd.linear_attn import _l2norm_rows_bwd
    dt = torch.bfloat16 if bf16 else torch.float32
    x = torch.randn(rows, d, device=DEV).to(dt).float().requires_grad_(True)
    y_ref = x / (x.norm(dim=-1, keepdim=True) + 1e-6)
    dy = torch.randn(rows, d, device=DEV).to(dt).float()
    y_ref.backward(dy)
    tol = 1e-2 if bf16 else 1e-5
    y = la.l2norm_rows(x.detach().to(dt))
    dx = _l2norm_rows_bwd(x.detach().to(dt), dy.to(dt))
    assert y.shape == (rows, d) and y.dtype == dt
    assert torch.allclose(y.float(), y_ref, atol=tol) and torch.allclose(dx.float(), x.grad, atol=tol * 4)
    if rows:  # and through autograd on the public op
        xa = x.detach().to(dt).requires_grad_(True)
        la.l2norm_rows(xa).backward(dy.to(dt))
        assert torch.equal(xa.grad, dx)


def test_l2norm_rows_on_transposed_views():
    """A non-contiguous [B, T, d] view whose transpose(1, 2) is contiguous is normalised over its LAST axis (forward
    and backward), and a [B, H, T, d] view over token-first memory keeps its memory order."""
    import linearnexus_amd as la
    base = torch.randn(3, 16, 5, device=DEV)          # memory [B, d, T]
    x = base.transpose(1, 2).requires_grad_(True)     # view [B, T, d], non-contiguous
    assert not x.is_contiguous() and x.transpose(1, 2).is_contiguous()
    xr = x.detach().clone().requires_grad_(True)
    dy = torch.randn(3, 5, 16, device=DEV)
    la.l2norm_rows(x).backward(dy)
    (xr / (xr.norm(dim=-1, keepdim=True) + 1e-6)).backward(dy)
    assert torch.allclose(la.l2norm_rows(x.detach()), xr.detach() / (xr.detach().norm(dim=-1, keepdim=True) + 1e-6), atol=1e-6)
    assert torch.allclose(x.grad, xr.grad, atol=1e-5)
    tf = torch.randn(2, 7, 3, 16, device=DEV).transpose(1, 2)  # [B, H, T, d] over [B, T, H, d] memory
    y = la.l2norm_rows(tf)
    assert y.stride() == tf.stride() and torch.allclose(y, tf / (tf.norm(dim=-1, keepdim=True) + 1e-6), atol=1e-6)
