"""The pieces composed the way the reference's Gated DeltaNet block composes them between its projections
(gated_deltanet.py:763-859): short causal conv + SiLU on the projected q, k, v -> [B, T, H, d] views transposed to
head-first -> beta = sigmoid(b), g = -exp(A_log) softplus(a + dt_bias) -> gated_delta_rule_chunkwise with the L2
norm inside the op -> transpose back -> gated RMSNorm.  Outputs and the gradients of every input of the pipeline
are checked against an fp64 torch restatement (autograd through oracle/torch_ref.py's recurrent form,
torch.nn.functional.conv1d, and the RMSNorm formula of kda.py:683-700).
Metric max|x - ref| / max|ref| <= 1e-4 (fp32) or 2e-2 (bf16 activations).  In bf16 the two per-head parameter
gradients, sums of B*T signed terms, are measured against the sum of the terms' magnitudes, at 5e-2: the error of
dg_t, a reverse cumulative sum inside each chunk, is shared by the tokens before t and does not average out over the
sum (the fp32 run of the same pipeline pins the algebra at 1e-4)."""
import dataclasses

import numpy as np
import pytest
import torch

from oracle import torch_ref as tr

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _inputs(seed, B, T, H, dk, dv, K):
    r = np.random.default_rng(seed)
    n = lambda *s, sc=1.0: (r.standard_normal(s) * sc).astype(np.float32)
    return {
        "q": n(B, T, H * dk), "k": n(B, T, H * dk), "v": n(B, T, H * dv), "gate": n(B, T, H, dv),
        "wq": n(K, H * dk, sc=0.5), "wk": n(K, H * dk, sc=0.5), "wv": n(K, H * dv, sc=0.5),
        "a": n(B, T, H), "b": n(B, T, H), "A_log": n(H, sc=0.3), "dt_bias": n(H, sc=0.3),
        "norm_w": (1.0 + 0.1 * r.standard_normal(dv)).astype(np.float32), "dy": n(B, T, H, dv),
    }


def _reference(x, B, T, H, dk, dv, bf16):
    # bf16 activations: the stages hand bf16 tensors to each other, so the restatement rounds at the same stage
    # boundaries (straight-through in the backward pass) and both sides feed every stage the same values
    rnd = (lambda u: u + (u.detach().float().bfloat16().double() - u.detach())) if bf16 else (lambda u: u)
    t = {n: torch.from_numpy(a).double().requires_grad_(n != "dy") for n, a in x.items()}

    def conv(u, w):  # causal depthwise cross-correlation, zero history (conv.py:56-67), then SiLU
        K = w.shape[0]
        y = torch.nn.functional.conv1d(torch.nn.functional.pad(u.transpose(1, 2), (K - 1, 0)), w.t().unsqueeze(1),
                                       groups=u.shape[-1])
        return rnd(torch.nn.functional.silu(y.transpose(1, 2)))

    q = conv(t["q"], t["wq"]).view(B, T, H, dk).transpose(1, 2)
    k = conv(t["k"], t["wk"]).view(B, T, H, dk).transpose(1, 2)
    v = conv(t["v"], t["wv"]).view(B, T, H, dv).transpose(1, 2)
    beta = torch.sigmoid(t["b"]).transpose(1, 2)
    g = (-torch.exp(t["A_log"]) * torch.nn.functional.softplus(t["a"] + t["dt_bias"])).transpose(1, 2)
    g.retain_grad()
    o, S = tr.recurrent(q, k, v, beta, g, None, None, True)
    o = rnd(o.transpose(1, 2))
    y = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + 1e-5) * t["norm_w"] * torch.sigmoid(t["gate"])
    (y * t["dy"]).sum().backward()
    grads = {n: t[n].grad.numpy() for n in t if n != "dy"}
    # the two per-head parameters collect B*T signed terms each: sum_t dg_t g_t and sum_t da_t.  Their un-cancelled
    # sizes are the yardstick for the bf16 comparison (rounding noise of the terms does not cancel with them).
    mass = {"A_log": (g.grad * g).abs().sum((0, 2)).detach().numpy(), "dt_bias": t["a"].grad.abs().sum((0, 1)).numpy()}
    return y.detach().numpy(), S.detach().numpy(), grads, mass


def _pipeline(x, B, T, H, dk, dv, dt):
    import linearnexus_amd as la
    act = ("q", "k", "v", "gate", "dy")
    t = {n: torch.from_numpy(a).to(DEV).to(dt if n in act else torch.float32).requires_grad_(n != "dy")
         for n, a in x.items()}
    q, _ = la.depthwise_conv1d_causal(t["q"], t["wq"], None, activation="silu")
    k, _ = la.depthwise_conv1d_causal(t["k"], t["wk"], None, activation="silu")
    v, _ = la.depthwise_conv1d_causal(t["v"], t["wv"], None, activation="silu")
    q = q.view(B, T, H, dk).transpose(1, 2)  # token-first memory behind head-first views: used in place
    k = k.view(B, T, H, dk).transpose(1, 2)
    v = v.view(B, T, H, dv).transpose(1, 2)
    g, beta = la.gated_deltanet_gate(t["a"], t["A_log"], t["dt_bias"], t["b"])  # [B, T, H] each, fp32
    g, beta = g.transpose(1, 2), beta.transpose(1, 2)
    o, S = la.gated_delta_rule_chunkwise(q, k, v, g, beta, None, None, 64, True)
    y = la.rmsnorm_gated(o.transpose(1, 2), t["gate"], t["norm_w"])
    (y.float() * t["dy"].float()).sum().backward()
    grads = {n: t[n].grad.float().cpu().numpy() for n in t if n != "dy"}
    return y.detach().float().cpu().numpy(), S.detach().cpu().numpy(), grads


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("shape", [(2, 150, 2, 64, 128), (1, 96, 3, 256, 512), (2, 70, 2, 128, 128)])
def test_gated_deltanet_mixer_forward_and_backward(shape, bf16):
    B, T, H, dk, dv = shape
    x = _inputs(95, B, T, H, dk, dv, 4)
    dt = torch.bfloat16 if bf16 else torch.float32
    if bf16:  # both sides see the activations on the bf16 grid
        for n in ("q", "k", "v", "gate", "dy"):
            x[n] = torch.from_numpy(x[n]).bfloat16().float().numpy()
    y_ref, S_ref, g_ref, mass = _reference(x, B, T, H, dk, dv, bf16)
    y, S, g = _pipeline(x, B, T, H, dk, dv, dt)
    tol = 2e-2 if bf16 else 1e-4
    rel = lambda a, b: float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))
    errs = {"y": rel(y, y_ref), "S": rel(S, S_ref), **{"d" + n: rel(g[n], g_ref[n]) for n in g_ref}}
    if bf16:
        for n in mass:
            errs["d" + n] = float((np.abs(g[n] - g_ref[n]) / mass[n]).max())
    bad = {n: e for n, e in errs.items() if not e < (5e-2 if bf16 and n[1:] in mass else tol)}
    assert not bad, (bad, errs)


def _kda_reference(x, B, T, H, dk, dv):
    t = {n: torch.from_numpy(a).double().requires_grad_(n != "dy") for n, a in x.items()}

    def conv(u, w):
        K = w.shape[0]
        y = torch.nn.functional.conv1d(torch.nn.functional.pad(u.transpose(1, 2), (K - 1, 0)), w.t().unsqueeze(1),
                                       groups=u.shape[-1])
        return torch.nn.functional.silu(y.transpose(1, 2))

    q = conv(t["q"], t["wq"]).view(B, T, H, dk).transpose(1, 2)
    k = conv(t["k"], t["wk"]).view(B, T, H, dk).transpose(1, 2)
    v = conv(t["v"], t["wv"]).view(B, T, H, dv).transpose(1, 2)
    # kda.py:120-172: g = -exp(A_log) softplus(g_in + bias) per key channel, beta = sigmoid(b)
    g = -torch.exp(t["A_log"])[None, None, :, None] * torch.nn.functional.softplus((t["g_in"] + t["g_bias"]).view(B, T, H, dk))
    beta = torch.sigmoid(t["b"]).transpose(1, 2)
    o, S = tr.recurrent(q, k, v, beta, g.transpose(1, 2), None, None, True)
    o = o.transpose(1, 2)
    y = o * torch.rsqrt((o * o).mean(-1, keepdim=True) + 1e-5) * t["norm_w"] * torch.sigmoid(t["gate"])
    (y * t["dy"]).sum().backward()
    return y.detach().numpy(), S.detach().numpy(), {n: t[n].grad.numpy() for n in t if n != "dy"}


def _kda_pipeline(x, B, T, H, dk, dv):
    import linearnexus_amd as la
    t = {n: torch.from_numpy(a).to(DEV).requires_grad_(n != "dy") for n, a in x.items()}
    q, _ = la.depthwise_conv1d_causal(t["q"], t["wq"], None, activation="silu")
    k, _ = la.depthwise_conv1d_causal(t["k"], t["wk"], None, activation="silu")
    v, _ = la.depthwise_conv1d_causal(t["v"], t["wv"], None, activation="silu")
    q = q.view(B, T, H, dk).transpose(1, 2)
    k = k.view(B, T, H, dk).transpose(1, 2)
    v = v.view(B, T, H, dv).transpose(1, 2)
    g, beta = la.kda_gate(t["g_in"], t["A_log"], dk, t["g_bias"], t["b"])  # [B, T, H, dk], [B, T, H]
    o, S = la.kda_chunkwise(q, k, v, g.transpose(1, 2), beta.transpose(1, 2), None, None, 64, True)
    y = la.rmsnorm_gated(o.transpose(1, 2), t["gate"], t["norm_w"])
    (y * t["dy"]).sum().backward()
    return y.detach().cpu().numpy(), S.detach().cpu().numpy(), {n: t[n].grad.cpu().numpy() for n in t if n != "dy"}


@pytest.mark.parametrize("shape", [(2, 100, 2, 128, 128), (1, 130, 3, 64, 64)])
def test_kda_mixer_forward_and_backward_fp32(shape):
    """The KDA block's composition (kda.py:864-975): conv + SiLU, the per-channel gate activation, the chunk scan with
    the L2 norm inside, the gated RMSNorm -- fp32 end to end at 1e-4."""
    B, T, H, dk, dv = shape
    x = _inputs(96, B, T, H, dk, dv, 4)
    r = np.random.default_rng(97)
    x["g_in"] = r.standard_normal((B, T, H * dk)).astype(np.float32)
    x["g_bias"] = (0.3 * r.standard_normal(H * dk)).astype(np.float32)
    del x["a"], x["dt_bias"]
    y_ref, S_ref, g_ref = _kda_reference(x, B, T, H, dk, dv)
    y, S, g = _kda_pipeline(x, B, T, H, dk, dv)
    rel = lambda a, b: float(np.abs(a - b).max() / max(np.abs(b).max(), 1e-30))
    errs = {"y": rel(y, y_ref), "S": rel(S, S_ref), **{"d" + n: rel(g[n], g_ref[n]) for n in g_ref}}
    bad = {n: e for n, e in errs.items() if not e < 1e-4}
    assert not bad, (bad, errs)


def test_prefill_then_token_by_token_decode_equals_whole_sequence():
    """Generation the way the reference's block runs it (gated_deltanet.py:756-779, :829-841, :868-876): the prompt goes
    through the chunk path once and leaves a GatedDeltaNetState (scan state + the three conv caches); every further
    token is one conv step on the caches and one gated_delta_rule_step.  The outputs must equal the whole sequence
    through the chunk path (the step-by-step == whole-sequence property of tests/test_comprehensive.py:57-83)."""
    import linearnexus_amd as la
    B, T, H, dk, dv, K, T0 = 2, 90, 2, 64, 128, 4, 70
    x = {n: torch.from_numpy(a).to(DEV) for n, a in _inputs(98, B, T, H, dk, dv, K).items()}

    def mixer(sl, state):
        q, cq = la.depthwise_conv1d_causal(x["q"][:, sl], x["wq"], None, cache=state.conv_state_q, activation="silu")
        k, ck = la.depthwise_conv1d_causal(x["k"][:, sl], x["wk"], None, cache=state.conv_state_k, activation="silu")
        v, cv = la.depthwise_conv1d_causal(x["v"][:, sl], x["wv"], None, cache=state.conv_state_v, activation="silu")
        n = q.shape[1]
        q, k, v = (t.view(B, n, H, -1).transpose(1, 2) for t in (q, k, v))
        g, beta = la.gated_deltanet_gate(x["a"][:, sl], x["A_log"], x["dt_bias"], x["b"][:, sl])
        g, beta = g.transpose(1, 2), beta.transpose(1, 2)
        if n == 1:
            o, S = la.gated_delta_rule_step(q[:, :, 0], k[:, :, 0], v[:, :, 0], g[:, :, 0], beta[:, :, 0], state.S)
            o = o[:, :, None]
        else:
            o, S = la.gated_delta_rule_chunkwise(q, k, v, g, beta, None, state.S, 64, True)
        y = la.rmsnorm_gated(o.transpose(1, 2), x["gate"][:, sl], x["norm_w"])
        return y, la.GatedDeltaNetState(S=S, conv_state_q=cq, conv_state_k=ck, conv_state_v=cv)

    zero = lambda: la.GatedDeltaNetState.zeros(B, H, dk, dv, key_dim_total=H * dk, value_dim=H * dv, conv_size=K)
    y_full, s_full = mixer(slice(0, T), zero())
    y, state = mixer(slice(0, T0), zero())
    assert (y - y_full[:, :T0]).abs().max() <= 1e-4 * y_full.abs().max()
    for t in range(T0, T):
        y, state = mixer(slice(t, t + 1), state)
        assert (y[:, 0] - y_full[:, t]).abs().max() <= 1e-4 * y_full.abs().max(), t
    assert (state.S - s_full.S).abs().max() <= 1e-4 * s_full.S.abs().max()
    for n in ("conv_state_q", "conv_state_k", "conv_state_v"):
        assert torch.equal(getattr(state, n), getattr(s_full, n))


def test_whole_mixer_decode_step_replayed_from_one_graph():
    """Serving: one token of the whole mixer (three conv steps on their caches, gates, the decode step on the state
    in place, gated RMSNorm) captured once in a HIP graph; every replay on new token inputs must equal the eager
    step bit for bit, with eager work and synchronisations between the replays."""
    import linearnexus_amd as la
    B, T, H, dk, dv, K = 4, 12, 3, 256, 512, 4
    x = {n: torch.from_numpy(a).to(DEV) for n, a in _inputs(99, B, T, H, dk, dv, K).items()}

    def new_state():
        return la.GatedDeltaNetState.zeros(B, H, dk, dv, key_dim_total=H * dk, value_dim=H * dv, conv_size=K)

    def step(tok, st):  # tok: dict of [B, 1, ...] inputs of one token; the state is updated in place
        q, _ = la.depthwise_conv1d_causal(tok["q"], x["wq"], None, cache=st.conv_state_q, activation="silu", inplace_cache=True)
        k, _ = la.depthwise_conv1d_causal(tok["k"], x["wk"], None, cache=st.conv_state_k, activation="silu", inplace_cache=True)
        v, _ = la.depthwise_conv1d_causal(tok["v"], x["wv"], None, cache=st.conv_state_v, activation="silu", inplace_cache=True)
        beta = torch.sigmoid(tok["b"][:, 0])
        g = -torch.exp(x["A_log"]) * torch.nn.functional.softplus(tok["a"][:, 0] + x["dt_bias"])
        o, _ = la.gated_delta_rule_step(q.view(B, H, dk), k.view(B, H, dk), v.view(B, H, dv), g, beta, st.S, inplace=True)
        return la.rmsnorm_gated(o, tok["gate"][:, 0], x["norm_w"])

    names = ("q", "k", "v", "a", "b", "gate")
    token = lambda t: {n: x[n][:, t:t + 1].contiguous() for n in names}
    eager_state, graph_state = new_state(), new_state()
    static = {n: torch.zeros_like(v_) for n, v_ in token(0).items()}
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(static, new_state())  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.no_grad(), torch.cuda.graph(graph):
        y_static = step(static, graph_state)
    for f in dataclasses.fields(graph_state):  # the capture itself ran nothing: start from zeros
        getattr(graph_state, f.name).zero_()
    for t in range(T):
        for n in names:
            static[n].copy_(token(t)[n])
        graph.replay()
        y_graph = y_static.clone()
        torch.cuda.synchronize()
        with torch.no_grad():
            y_eager = step(token(t), eager_state)  # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(y_graph, y_eager), t
        for f in dataclasses.fields(graph_state):
            assert torch.equal(getattr(graph_state, f.name), getattr(eager_state, f.name)), (t, f.name)
