"""The token-by-token ops under autograd.  The reference's *_recurrent and *_step ops are differentiable (JAX), and
its blocks call *_recurrent while training on sequences of at most 32 tokens (gated_deltanet.py:836-846); here a
wanted gradient sends the same function through the chunk kernels.  Gradients against the fp64 adjoint oracle:
1e-4 (fp32), 2e-2 (bf16)."""
import numpy as np
import pytest
import torch

from oracle import recurrent as rc
from oracle.adjoint import delta_rule_adjoint
from oracle.inputs import make_inputs
from conftest import max_rel
from test_chunk_bwd_gpu import _prep, check

pytestmark = pytest.mark.gpu
DEV = "cuda"
GATES = ["none", "scalar", "vector"]


def _leaves(x, names, dt):
    out = {}
    for n in names:
        t = torch.from_numpy(np.ascontiguousarray(x[n])).to(DEV)
        out[n] = (t.to(dt) if n in ("q", "k", "v") else t).requires_grad_(True)
    return out


@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("shape", [(2, 2, 24, 64, 64), (1, 3, 32, 16, 32), (1, 2, 100, 128, 128)])
def test_recurrent_ops_are_differentiable(gate, bf16, shape):
    import linearnexus_amd as la
    B, H, T, dk, dv = shape
    x = make_inputs(71, B, H, T, dk, dv, gate=gate, with_state=True, with_grad=True, normalize=(gate == "none"))
    x, dt = _prep(x, bf16)
    l2 = gate != "none"
    names = ["q", "k", "v", "beta", "S0"] + (["g"] if gate != "none" else [])
    t = _leaves(x, names, dt)
    if gate == "none":
        o, S = la.delta_rule_recurrent(t["q"], t["k"], t["v"], t["beta"], t["S0"])
    else:
        fn = la.gated_delta_rule_recurrent if gate == "scalar" else la.kda_recurrent
        o, S = fn(t["q"], t["k"], t["v"], t["g"], t["beta"], None, t["S0"], True)
    assert o.dtype == dt and o.requires_grad and S.requires_grad
    ((o.float() * torch.from_numpy(x["dO"]).to(DEV)).sum() + (S * torch.from_numpy(x["dS"]).to(DEV)).sum()).backward()
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x.get("g"), x["dS"], None, x["S0"], l2)
    got = {"dq": t["q"].grad, "dk": t["k"].grad, "dv": t["v"].grad, "dbeta": t["beta"].grad, "dS0": t["S0"].grad}
    if gate != "none":
        got["dg"] = t["g"].grad
    check({n: g.float().cpu().numpy() for n, g in got.items()}, ref, 2e-2 if bf16 else 1e-4)
    # without a wanted gradient the token kernel runs, and the two paths agree
    with torch.no_grad():
        if gate == "none":
            o2, S2 = la.delta_rule_recurrent(t["q"], t["k"], t["v"], t["beta"], t["S0"])
        else:
            o2, S2 = fn(t["q"], t["k"], t["v"], t["g"], t["beta"], None, t["S0"], True)
    tol = 2e-2 if bf16 else 1e-4
    assert not o2.requires_grad
    assert max_rel(o2.float().cpu().numpy(), o.detach().float().cpu().numpy()) < tol


@pytest.mark.parametrize("gate", GATES)
def test_step_ops_are_differentiable(gate):
    import linearnexus_amd as la
    B, H, dk, dv = 2, 3, 128, 64
    x = make_inputs(72, B, H, 1, dk, dv, gate=gate, with_state=True, with_grad=True, normalize=(gate == "none"))
    l2 = gate != "none"
    names = ["q", "k", "v", "beta", "S0"] + (["g"] if gate != "none" else [])
    t = _leaves(x, names, torch.float32)
    tok = lambda n: t[n][:, :, 0]
    if gate == "none":
        o, S = la.delta_rule_step(tok("q"), tok("k"), tok("v"), tok("beta"), t["S0"])
    else:
        fn = la.gated_delta_rule_step if gate == "scalar" else la.kda_step
        o, S = fn(tok("q"), tok("k"), tok("v"), tok("g"), tok("beta"), t["S0"])
    ((o * torch.from_numpy(x["dO"][:, :, 0]).to(DEV)).sum() + (S * torch.from_numpy(x["dS"]).to(DEV)).sum()).backward()
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x.get("g"), x["dS"], None, x["S0"], l2)
    got = {"dq": t["q"].grad, "dk": t["k"].grad, "dv": t["v"].grad, "dbeta": t["beta"].grad, "dS0": t["S0"].grad}
    if gate != "none":
        got["dg"] = t["g"].grad
    check({n: g.float().cpu().numpy() for n, g in got.items()}, ref, 1e-4)
    with pytest.raises(RuntimeError):
        la.delta_rule_step(tok("q"), tok("k"), tok("v"), tok("beta"), t["S0"].detach().clone(), inplace=True)
