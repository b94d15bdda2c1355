"""Pins the gradient oracle: the hand-derived token-level adjoint must equal central
finite differences of the fp64 recurrent form, ``torch.autograd`` through an independent
torch restatement, and satisfy the adjoint identity <dO, J dx> = <J^T dO, dx>.
The reference has no backward code and checks no gradient numerically."""
import numpy as np
import pytest
import torch

from oracle import recurrent as rc
from oracle import torch_ref as tr
from oracle.adjoint import delta_rule_adjoint
from oracle.inputs import make_inputs
from conftest import max_rel


def _forward(x, gate, l2):
    if gate == "none":
        assert not l2
        return rc.delta_rule_recurrent(x["q"], x["k"], x["v"], x["beta"], x["S0"])
    fn = rc.gated_delta_rule_recurrent if gate == "scalar" else rc.kda_recurrent
    return fn(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["S0"], l2)


def _loss(x, gate, l2):
    o, S = _forward(x, gate, l2)
    return float((o * x["dO"]).sum() + (S * x["dS"]).sum())


@pytest.mark.parametrize("gate,l2", [("none", False), ("scalar", False), ("scalar", True), ("vector", False), ("vector", True)])
def test_adjoint_vs_finite_differences(gate, l2):
    x = make_inputs(11, 1, 2, 5, 4, 3, gate=gate, with_state=True, with_grad=True, normalize=not l2, gate_scale=1.0)
    x = {n: a.astype(np.float64) for n, a in x.items()}
    x["S0"] *= 20
    gr = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x.get("g"), x["dS"], None, x["S0"], l2)
    rng = np.random.default_rng(0)
    eps = 1e-6
    for name, key in [("q", "dq"), ("k", "dk"), ("v", "dv"), ("beta", "dbeta"), ("g", "dg"), ("S0", "dS0")]:
        if name not in x:
            continue
        for _ in range(6):  # random directional derivatives
            d = rng.standard_normal(x[name].shape)
            xp, xm = dict(x), dict(x)
            xp[name] = x[name] + eps * d
            xm[name] = x[name] - eps * d
            fd = (_loss(xp, gate, l2) - _loss(xm, gate, l2)) / (2 * eps)
            an = float((gr[key] * d).sum())
            assert abs(fd - an) <= 1e-6 * max(1.0, abs(an)), (name, fd, an)


@pytest.mark.parametrize("gate,l2", [("none", False), ("scalar", True), ("vector", True), ("vector", False)])
def test_adjoint_vs_torch_autograd(gate, l2):
    x = make_inputs(12, 2, 2, 40, 8, 6, gate=gate, with_state=True, with_grad=True, normalize=not l2)
    t = {n: torch.from_numpy(a.astype(np.float64)) for n, a in x.items()}
    inp = {"q": t["q"], "k": t["k"], "v": t["v"], "beta": t["beta"], "g": t.get("g"), "initial_state": t["S0"]}
    o, S, g = tr.grads(tr.recurrent, inp, t["dO"], t["dS"], use_qk_l2norm=l2)
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x.get("g"), x["dS"], None, x["S0"], l2)
    o_np, S_np = _forward({n: a.astype(np.float64) for n, a in x.items()}, gate, l2)
    assert max_rel(o.numpy(), o_np) < 1e-12 and max_rel(S.numpy(), S_np) < 1e-12
    for a, b in [("q", "dq"), ("k", "dk"), ("v", "dv"), ("beta", "dbeta"), ("g", "dg"), ("initial_state", "dS0")]:
        if g[a] is None:
            continue
        assert max_rel(g[a].numpy(), ref[b]) < 1e-10, a


def test_torch_chunk_equals_torch_recurrent_with_grads():
    for gate in ("none", "scalar", "vector"):
        x = make_inputs(13, 1, 2, 100, 8, 8, gate=gate, with_state=True, with_grad=True)
        t = {n: torch.from_numpy(a.astype(np.float64)) for n, a in x.items()}
        inp = {"q": t["q"], "k": t["k"], "v": t["v"], "beta": t["beta"], "g": t.get("g"), "initial_state": t["S0"]}
        o1, S1, g1 = tr.grads(tr.recurrent, inp, t["dO"], t["dS"])
        o2, S2, g2 = tr.grads(tr.chunkwise, inp, t["dO"], t["dS"], chunk_size=32)
        assert max_rel(o2, o1) < 1e-10 and max_rel(S2, S1) < 1e-10
        for n in g1:
            if g1[n] is not None:
                assert max_rel(g2[n], g1[n]) < 1e-9, (gate, n)


def test_adjoint_identity():
    # o is linear in v for fixed q,k,beta,g and S0=0:  <dO, o(v)> == <dv, v>
    x = make_inputs(14, 1, 2, 30, 8, 8, gate="vector", with_grad=True)
    gr = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x["g"])
    o, _ = rc.kda_recurrent(x["q"], x["k"], x["v"], x["g"], x["beta"], use_qk_l2norm=False)
    assert abs((o * x["dO"]).sum() - (gr["dv"] * x["v"]).sum()) < 1e-9 * abs((o * x["dO"]).sum())
