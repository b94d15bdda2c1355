"""CPU checks of the committed golden fixtures (tests/golden/*.npz, written by
tests/golden/make_fixtures.py from the fp64 token-by-token oracle).

The fixtures freeze numbers; these tests make sure that three independent routes still land on
them: the recurrent oracle itself (drift guard), the chunk-algorithm restatement
(oracle.chunkwise, a different algorithm), and torch.autograd through the torch restatement
(an independent gradient).  Tolerance 2e-6 relative to the tensor's maximum: the fixtures
are stored in fp32."""
import os

import numpy as np
import pytest
import torch

from oracle import adjoint, chunkwise, recurrent, torch_ref
from conftest import max_rel

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
DENSE = {"deltanet": "none", "gated": "scalar", "kda": "vector"}
TOL = 2e-6


def load(name):
    with np.load(os.path.join(GOLD, name), allow_pickle=False) as z:
        return {k: z[k] for k in z.files}


def test_fixture_files_present():
    names = sorted(f for f in os.listdir(GOLD) if f.endswith(".npz"))
    assert names == ["deltanet_B1H1T80d64.npz", "deltanet_varlen_3seq_T100d64.npz", "gated_B1H1T80d64.npz",
                     "kda_B1H1T80d64.npz", "steps_B1H2d64.npz"]


@pytest.mark.parametrize("name", sorted(DENSE))
def test_recurrent_and_chunk_oracles_reproduce_fixture(name):
    f = load(f"{name}_B1H1T80d64.npz")
    gate = DENSE[name]
    q, k, v, beta, S0 = (f[f"in_{n}"] for n in ("q", "k", "v", "beta", "S0"))
    if gate == "none":
        o1, S1 = recurrent.delta_rule_recurrent(q, k, v, beta, S0)
        o2, S2 = chunkwise.delta_rule_chunkwise(q, k, v, beta, S0, 64)
    else:
        g = f["in_g"]
        rec = recurrent.gated_delta_rule_recurrent if gate == "scalar" else recurrent.kda_recurrent
        chk = chunkwise.gated_delta_rule_chunkwise if gate == "scalar" else chunkwise.kda_chunkwise
        o1, S1 = rec(q, k, v, g, beta, None, S0, False)
        o2, S2 = chk(q, k, v, g, beta, None, S0, 64, False)
    for o, S in ((o1, S1), (o2, S2)):
        assert max_rel(o, f["o"]) < TOL and max_rel(S, f["S_T"]) < TOL


@pytest.mark.parametrize("name", sorted(DENSE))
def test_adjoint_and_autograd_reproduce_fixture_gradients(name):
    f = load(f"{name}_B1H1T80d64.npz")
    gate = DENSE[name]
    g = f["in_g"] if gate != "none" else None
    a = adjoint.delta_rule_adjoint(f["in_q"], f["in_k"], f["in_v"], f["in_beta"], f["in_dO"], g=g, dS_T=f["in_dS"],
                                   initial_state=f["in_S0"])
    td = lambda x: None if x is None else torch.from_numpy(np.asarray(x, np.float64))
    _, _, t = torch_ref.grads(torch_ref.recurrent, dict(q=td(f["in_q"]), k=td(f["in_k"]), v=td(f["in_v"]),
                                                        beta=td(f["in_beta"]), g=td(g), initial_state=td(f["in_S0"])),
                              td(f["in_dO"]), td(f["in_dS"]))
    names = {"dq": "q", "dk": "k", "dv": "v", "dbeta": "beta", "dS0": "initial_state"}
    if gate != "none":
        names["dg"] = "g"
    for gn, tn in names.items():
        assert max_rel(a[gn], f[gn]) < TOL, gn
        assert max_rel(t[tn].numpy(), f[gn]) < TOL, gn


def test_varlen_fixture_is_the_per_sequence_loop():
    f = load("deltanet_varlen_3seq_T100d64.npz")
    cu = f["in_cu_seqlens"]
    assert cu.dtype == np.int32 and list(cu) == [0, 20, 84, 100]
    for s in range(3):
        a, b = int(cu[s]), int(cu[s + 1])
        o, S = chunkwise.delta_rule_chunkwise(f["in_q"][:, :, a:b], f["in_k"][:, :, a:b], f["in_v"][:, :, a:b],
                                              f["in_beta"][:, :, a:b], f["in_S0"][s:s + 1], 64)
        assert max_rel(o, f["o"][:, :, a:b]) < TOL and max_rel(S[0], f["S_T"][s]) < TOL


def test_step_fixture_equals_one_token_scan():
    f = load("steps_B1H2d64.npz")
    for name, gate in DENSE.items():
        q, k, v, beta, S0 = (f[f"{name}_in_{n}"] for n in ("q", "k", "v", "beta", "S0"))
        x = lambda a: a[:, :, None]
        if gate == "none":
            o, S = recurrent.delta_rule_recurrent(x(q), x(k), x(v), x(beta), S0)
        else:
            fn = recurrent.gated_delta_rule_recurrent if gate == "scalar" else recurrent.kda_recurrent
            o, S = fn(x(q), x(k), x(v), x(f[f"{name}_in_g"]), x(beta), None, S0, False)
        assert max_rel(o[:, :, 0], f[f"{name}_o"]) < TOL and max_rel(S, f[f"{name}_S"]) < TOL
