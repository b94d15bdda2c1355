"""The kernel-shaped chunk forward/backward (oracle/staged.py) must equal the recurrent form
and its token-level adjoint at fp64 round-off -- this is what licenses the HIP kernels'
decomposition."""
import numpy as np
import pytest

from oracle import recurrent as rc
from oracle import staged
from oracle.adjoint import delta_rule_adjoint
from oracle.inputs import make_inputs
from conftest import max_rel


@pytest.mark.parametrize("gate", ["none", "scalar", "vector"])
@pytest.mark.parametrize("T", [64, 150])
def test_staged_forward_backward(gate, T):
    x = make_inputs(31, 2, 2, T, 8, 6, gate=gate, with_state=True, with_grad=True, gate_scale=0.3)
    x = {n: a.astype(np.float64) for n, a in x.items()}
    g = x.get("g")
    if gate == "none":
        o_ref, S_ref = rc.delta_rule_recurrent(x["q"], x["k"], x["v"], x["beta"], x["S0"])
    elif gate == "scalar":
        o_ref, S_ref = rc.gated_delta_rule_recurrent(x["q"], x["k"], x["v"], g, x["beta"], None, x["S0"], False)
    else:
        o_ref, S_ref = rc.kda_recurrent(x["q"], x["k"], x["v"], g, x["beta"], None, x["S0"], False)
    o, S, ws = staged.forward(x["q"], x["k"], x["v"], x["beta"], g, None, x["S0"])
    assert max_rel(o, o_ref) < 1e-11 and max_rel(S, S_ref) < 1e-11
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], g, x["dS"], None, x["S0"], False)
    got = staged.backward(ws, x["dO"], x["dS"])
    for n in ("dq", "dk", "dv", "dbeta", "dS0") + (("dg",) if gate != "none" else ()):
        assert max_rel(got[n], ref[n]) < 1e-10, n


@pytest.mark.parametrize("gate", ["none", "scalar"])
@pytest.mark.parametrize("T", [64, 150])
def test_direct_solve_split_forward_backward(gate, T):
    """The split the kernels for 2-byte inputs use (the inverse applied to each chunk's right-hand side, nothing but
    Tm, Pm, G and the per-chunk states kept) against the recurrent form and the token-level adjoint."""
    from oracle import staged_direct as sd
    x = make_inputs(32, 2, 2, T, 8, 6, gate=gate, with_state=True, with_grad=True, gate_scale=0.3)
    x = {n: a.astype(np.float64) for n, a in x.items()}
    g = x.get("g")
    if gate == "none":
        o_ref, S_ref = rc.delta_rule_recurrent(x["q"], x["k"], x["v"], x["beta"], x["S0"])
    else:
        o_ref, S_ref = rc.gated_delta_rule_recurrent(x["q"], x["k"], x["v"], g, x["beta"], None, x["S0"], False)
    o, S, ws = sd.forward(x["q"], x["k"], x["v"], x["beta"], g, None, x["S0"])
    assert max_rel(o, o_ref) < 1e-11 and max_rel(S, S_ref) < 1e-11
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], g, x["dS"], None, x["S0"], False)
    got = sd.backward(ws, x["dO"], x["dS"])
    for n in ("dq", "dk", "dv", "dbeta", "dS0") + (("dg",) if gate != "none" else ()):
        assert max_rel(got[n], ref[n]) < 1e-10, n
