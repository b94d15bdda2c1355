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


@pytest.mark.parametrize("variant", ["gated", "kda"])
def test_chunk_forward_backward_under_graph_capture(variant):
    """A whole differentiable chunk step (forward kernels, autograd, backward kernels) captured in one HIP graph:
    every replay must reproduce the eager results bit for bit -- o, S and all five gradients (the row and chunk sums
    behind dg and dbeta are added in a fixed order) -- with new inputs copied into the captured buffers and eager work
    between the replays."""
    import linearnexus_amd as la
    B, H, T, d = 2, 4, 200, 128
    gate = "scalar" if variant == "gated" else "vector"
    op = la.gated_delta_rule_chunkwise if variant == "gated" else la.kda_chunkwise

    def inputs(seed):
        x = make_inputs(seed, B, H, T, d, d, gate=gate, with_grad=True)
        return [_t(x[n], torch.bfloat16) for n in ("q", "k", "v")] + [_t(x["g"]), _t(x["beta"]), _t(x["dO"], torch.bfloat16)]

    def run(q, k, v, g, beta, dO):
        leaves = [t.detach().requires_grad_(True) for t in (q, k, v, g, beta)]
        o, S = op(*leaves, use_qk_l2norm=False)
        grads = torch.autograd.grad(o, leaves, dO.to(o.dtype))
        return [o, S, *grads]

    static = inputs(60)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        run(*static)  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = run(*static)
    for seed in (61, 62, 61):
        fresh = inputs(seed)
        for dst, src in zip(static, fresh):
            dst.copy_(src)
        graph.replay()
        got = [t.clone() for t in outs]
        torch.cuda.synchronize()
        ref = run(*fresh)  # eager work between the replays
        torch.cuda.synchronize()
        for i, (a, b) in enumerate(zip(got, ref)):
            assert torch.equal(a, b), (seed, i)
