"""The decode driver: steps replayed from a captured HIP graph equal the eager steps and the oracle scan.
Every replay is checked, with eager work and synchronisations between replays."""
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


@pytest.mark.parametrize("variant,gate", [("delta", "none"), ("gated", "scalar"), ("kda", "vector")])
def test_graph_replays_follow_eager_steps_and_oracle(variant, gate):
    import linearnexus_amd as la
    from linearnexus_amd.decode import DecodeGraph
    B, H, T, dk, dv, L = 2, 4, 10, 128, 64, 3
    xs = []
    for layer in range(L):
        x = make_inputs(70 + layer, B, H, T, dk, dv, gate=gate, with_state=True)
        for n in ("q", "k", "v"):
            x[n] = to_bf16_grid(x[n])
        xs.append(x)
    states = [_t(x["S0"]).clone() for x in xs]
    ptrs = [s.data_ptr() for s in states]
    dg = DecodeGraph(variant, B, H, dk, dv, layers=L, dtype=torch.bfloat16, use_qk_l2norm=False, states=states)
    for s, x in zip(states, xs):  # building the graph must not have moved the states
        assert torch.equal(s, _t(x["S0"]))
    eager_S = [_t(x["S0"]).clone() for x in xs]
    outs = [[] for _ in range(L)]
    for t in range(T):
        for layer, x in enumerate(xs):
            tok = lambda n, dt=None: _t(x[n][:, :, t], dt)
            dg.step(tok("q", torch.bfloat16), tok("k", torch.bfloat16), tok("v", torch.bfloat16), tok("beta"),
                    None if gate == "none" else tok("g"), layer=layer)
        o_graph = [o.clone() for o in dg.replay()]
        torch.cuda.synchronize()
        for layer, x in enumerate(xs):  # eager work between replays: the same step through the plain op
            tok = lambda n, dt=None: _t(x[n][:, :, t], dt)
            q, k, v = tok("q", torch.bfloat16), tok("k", torch.bfloat16), tok("v", torch.bfloat16)
            if variant == "delta":
                o, S = la.delta_rule_step(q, k, v, tok("beta"), eager_S[layer])
            elif variant == "gated":
                o, S = la.gated_delta_rule_step(q, k, v, tok("g"), tok("beta"), eager_S[layer], use_qk_l2norm=False)
            else:
                o, S = la.kda_step(q, k, v, tok("g"), tok("beta"), eager_S[layer], use_qk_l2norm=False)
            eager_S[layer] = S
            assert torch.equal(o, o_graph[layer]), (t, layer)
            assert torch.equal(S, dg.state[layer]), (t, layer)
            outs[layer].append(o_graph[layer])
    for layer, x in enumerate(xs):
        assert dg.state[layer].data_ptr() == ptrs[layer]
        if gate == "none":
            o_ref, S_ref = rc.delta_rule_recurrent(x["q"], x["k"], x["v"], x["beta"], x["S0"])
        else:
            fn = rc.gated_delta_rule_recurrent if gate == "scalar" else rc.kda_recurrent
            o_ref, S_ref = fn(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["S0"], False)
        o = torch.stack(outs[layer], 2).float().cpu().numpy()
        assert max_rel(o, o_ref) < 2e-2 and max_rel(dg.state[layer].cpu().numpy(), S_ref) < 2e-2


def test_graph_rejects_bad_states():
    from linearnexus_amd.decode import DecodeGraph
    with pytest.raises(RuntimeError):
        DecodeGraph("gated", 1, 2, 64, 64, states=[torch.zeros(1, 2, 64, 64, dtype=torch.bfloat16, device=DEV)])
    with pytest.raises(ValueError):
        DecodeGraph("rwkv", 1, 2, 64, 64)
