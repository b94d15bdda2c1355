"""GPU parity on the edges of the input space: empty and one-token inputs, packed batches with
empty and one-token sequences, wide value heads, hand-over of the state between two calls, and
the closed forms the reference's tests use (beta = 0, test_deltanet.py:281-297).  Tolerances as
everywhere: max|x - ref| / max|ref| below 1e-4 for fp32 inputs and 2e-2 for bf16 inputs."""
import numpy as np
import pytest
import torch

from linearnexus_amd import linear_attn
from oracle import recurrent as rc
from oracle.adjoint import delta_rule_adjoint
from oracle.inputs import make_inputs, to_bf16_grid
from conftest import max_rel
from test_chunk_bwd_gpu import gpu_grads, check, _prep as _prep_bwd
from test_chunk_fwd_gpu import gpu_chunk_fwd, oracle_fwd, _prep

pytestmark = pytest.mark.gpu
DEV = "cuda"
GATES = ["none", "scalar", "vector"]


@pytest.mark.parametrize("gate", GATES)
def test_empty_sequence_returns_initial_state(gate):
    import linearnexus_amd as la
    B, H, d = 2, 3, 64
    z = lambda *s: torch.zeros(*s, device=DEV)
    S0 = torch.randn(B, H, d, d, device=DEV)
    q = k = v = z(B, H, 0, d)
    beta = z(B, H, 0)
    if gate == "none":
        o, S = la.delta_rule_chunkwise(q, k, v, beta, S0)
        o2, S2 = la.delta_rule_recurrent(q, k, v, beta, S0)
    else:
        g = z(B, H, 0) if gate == "scalar" else z(B, H, 0, d)
        fn = (la.gated_delta_rule_chunkwise, la.gated_delta_rule_recurrent) if gate == "scalar" else (la.kda_chunkwise, la.kda_recurrent)
        o, S = fn[0](q, k, v, g, beta, None, S0)
        o2, S2 = fn[1](q, k, v, g, beta, None, S0)
    assert o.shape == (B, H, 0, d) and o2.shape == (B, H, 0, d)
    assert torch.equal(S, S0) and torch.equal(S2, S0)


@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("T", [1, 63, 64, 65])
def test_lengths_around_one_chunk(gate, T):
    x = make_inputs(61, 1, 2, T, 64, 64, gate=gate, with_state=True, with_grad=True)
    o_ref, S_ref = oracle_fwd(x, gate)
    o, S = gpu_chunk_fwd(x, gate, torch.float32)
    assert max_rel(o.float().cpu().numpy(), o_ref) < 1e-4 and max_rel(S.cpu().numpy(), S_ref) < 1e-4
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x.get("g"), x["dS"], None, x["S0"], False)
    check(gpu_grads(x, gate, torch.float32), ref, 1e-4)


@pytest.mark.parametrize("gate", GATES)
def test_packed_batch_with_empty_and_one_token_sequences(gate):
    H, d = 2, 64
    cu = np.array([0, 0, 1, 66, 66, 130, 131], np.int32)  # lengths 0, 1, 65, 0, 64, 1
    T, nseq = int(cu[-1]), len(cu) - 1
    x = make_inputs(62, 1, H, T, d, d, gate=gate, with_grad=True)
    rng = np.random.default_rng(62)
    x["S0"] = (rng.standard_normal((nseq, H, d, d)) * 0.02).astype(np.float32)
    x["dS"] = (rng.standard_normal((nseq, H, d, d)) * 0.1).astype(np.float32)

    def one(q, k, v, *rest, initial_state=None):
        y = {"q": q, "k": k, "v": v, "beta": rest[-1], "S0": initial_state}
        if gate != "none":
            y["g"] = rest[0]
        return oracle_fwd(y, gate)

    args = [x["q"], x["k"], x["v"]] + ([x["g"]] if gate != "none" else []) + [x["beta"]]
    o_ref, S_ref = rc.varlen(one, cu, *args, initial_state=x["S0"])
    o, S = gpu_chunk_fwd(x, gate, torch.float32, cu=cu)
    assert max_rel(o.cpu().numpy(), o_ref) < 1e-4 and max_rel(S.cpu().numpy(), S_ref) < 1e-4
    assert np.array_equal(S[0].cpu().numpy(), x["S0"][0]) and np.array_equal(S[3].cpu().numpy(), x["S0"][3])
    parts = []
    for s in range(nseq):
        a, b = cu[s], cu[s + 1]
        sl = lambda n: x[n][:, :, a:b]
        parts.append(delta_rule_adjoint(sl("q"), sl("k"), sl("v"), sl("beta"), sl("dO"), sl("g") if gate != "none" else None,
                                        x["dS"][s:s + 1], None, x["S0"][s:s + 1], False))
    names = ("dq", "dk", "dv", "dbeta") + (("dg",) if gate != "none" else ())
    ref = {n: np.concatenate([p[n] for p in parts], 2) for n in names}
    ref["dS0"] = np.concatenate([p["dS0"] for p in parts], 0)
    check(gpu_grads(x, gate, torch.float32, cu=cu), ref, 1e-4)


@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("bf16", [False, True])
def test_wide_value_head(gate, bf16):
    """dv = 256 with dk = 64: four value slabs per state."""
    x = make_inputs(63, 1, 2, 150, 64, 256, gate=gate, with_state=True, with_grad=True)
    xf, dt = _prep(x, bf16)
    o_ref, S_ref = oracle_fwd(xf, gate)
    o, S = gpu_chunk_fwd(xf, gate, dt)
    tol = 2e-2 if bf16 else 1e-4
    assert max_rel(o.float().cpu().numpy(), o_ref) < tol and max_rel(S.cpu().numpy(), S_ref) < tol
    xb, dt = _prep_bwd(x, bf16)
    ref = delta_rule_adjoint(xb["q"], xb["k"], xb["v"], xb["beta"], xb["dO"], xb.get("g"), xb["dS"], None, xb["S0"], False)
    check(gpu_grads(xb, gate, dt), ref, tol)


@pytest.mark.parametrize("gate", GATES)
def test_state_hand_over_between_calls(gate):
    """[0, T1) followed by [T1, T) with the first call's final state == one call over [0, T)."""
    T, T1 = 200, 77
    x = make_inputs(64, 2, 2, T, 128, 128, gate=gate, with_state=True)
    o_full, S_full = gpu_chunk_fwd(x, gate, torch.float32)
    cut = lambda a, b: {n: (t[:, :, a:b] if n not in ("S0",) else t) for n, t in x.items()}
    x1 = cut(0, T1)
    o1, S1 = gpu_chunk_fwd(x1, gate, torch.float32)
    x2 = cut(T1, T)
    x2["S0"] = S1.cpu().numpy()
    o2, S2 = gpu_chunk_fwd(x2, gate, torch.float32)
    o12 = torch.cat([o1, o2], 2)
    assert max_rel(o12.cpu().numpy(), o_full.cpu().numpy()) < 1e-4
    assert max_rel(S2.cpu().numpy(), S_full.cpu().numpy()) < 1e-4


@pytest.mark.parametrize("gate", GATES)
def test_beta_zero_closed_form(gate):
    """beta = 0: S_T = (prod alpha) S0 and o_t = scale * (e^{G_t} S0)^T q_t."""
    B, H, T, d = 1, 2, 100, 64
    x = make_inputs(65, B, H, T, d, d, gate=gate, with_state=True)
    x["beta"] = np.zeros_like(x["beta"])
    o, S = gpu_chunk_fwd(x, gate, torch.float32)
    if gate == "none":
        G = np.zeros((B, H, T, d))
    elif gate == "scalar":
        G = np.cumsum(x["g"].astype(np.float64), 2)[..., None] * np.ones(d)
    else:
        G = np.cumsum(x["g"].astype(np.float64), 2)
    S0 = x["S0"].astype(np.float64)
    S_ref = np.exp(G[:, :, -1])[..., None] * S0
    o_ref = d ** -0.5 * np.einsum("bhtk,bhkv->bhtv", x["q"].astype(np.float64) * np.exp(G), S0)
    assert max_rel(S.cpu().numpy(), S_ref) < 1e-4 and max_rel(o.cpu().numpy(), o_ref) < 1e-4


@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("bf16", [False, True])
def test_forward_without_gradients_skips_nothing_visible(gate, bf16):
    """Under torch.no_grad() the op sets forward_only (the kernels do not write what only the backward
    reads); outputs and final state must be bit-identical to the differentiable call."""
    x = make_inputs(66, 2, 2, 300, 128, 128, gate=gate, with_state=True)
    x, dt = _prep(x, bf16)
    with torch.no_grad():
        o1, S1 = gpu_chunk_fwd(x, gate, dt)
    import linearnexus_amd as la
    q, k, v = (torch.from_numpy(x[n]).to(DEV).to(dt).requires_grad_(True) for n in ("q", "k", "v"))
    beta, s0 = torch.from_numpy(x["beta"]).to(DEV), torch.from_numpy(x["S0"]).to(DEV)
    if gate == "none":
        o2, S2 = la.delta_rule_chunkwise(q, k, v, beta, s0)
    else:
        fn = la.gated_delta_rule_chunkwise if gate == "scalar" else la.kda_chunkwise
        o2, S2 = fn(q, k, v, torch.from_numpy(x["g"]).to(DEV), beta, None, s0, 64, False)
    assert o2.requires_grad and not o1.requires_grad
    assert torch.equal(o1, o2.detach()) and torch.equal(S1, S2.detach())


@pytest.mark.parametrize("slab", ["32", "64"])
@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("bf16", [True, False])
def test_both_slab_widths_of_the_sequential_kernels(gate, slab, bf16, monkeypatch):
    """dk = 128 has 32- and 64-column variants of the two scans (chosen by the number of workgroups; the 64-column
    backward scan of 4-byte inputs lets K and Q share an LDS tile); the test_scan_slab field of the argument block forces either so that both meet
    the oracle at a small shape."""
    monkeypatch.setitem(linear_attn._test_hooks, "scan_slab", int(slab))
    x = make_inputs(67, 1, 2, 200, 128, 128, gate=gate, with_state=True, with_grad=True)
    tol = 2e-2 if bf16 else 1e-4
    xf, dt = _prep(x, bf16)
    o_ref, S_ref = oracle_fwd(xf, gate)
    o, S = gpu_chunk_fwd(xf, gate, dt)
    assert max_rel(o.float().cpu().numpy(), o_ref) < tol and max_rel(S.cpu().numpy(), S_ref) < tol
    xb, dt = _prep_bwd(x, bf16)
    ref = delta_rule_adjoint(xb["q"], xb["k"], xb["v"], xb["beta"], xb["dO"], xb.get("g"), xb["dS"], None, xb["S0"], False)
    check(gpu_grads(xb, gate, dt), ref, tol)


@pytest.mark.parametrize("spw", ["1", "3", "8"])
@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("dk,dv", [(128, 320), (256, 160), (64, 192)])
def test_output_kernel_slabs_per_workgroup(gate, spw, dk, dv, monkeypatch):
    """4-byte inputs form the outputs in a kernel of their own, which takes several value slabs per workgroup at
    large shapes (Q and P staged once); the test_out_slabs field of the argument block forces the count, here with a ragged last group."""
    monkeypatch.setitem(linear_attn._test_hooks, "out_slabs", int(spw))
    x = make_inputs(68, 1, 2, 150, dk, dv, gate=gate, with_state=True)
    o_ref, S_ref = oracle_fwd(x, gate)
    o, S = gpu_chunk_fwd(x, gate, torch.float32)
    assert max_rel(o.cpu().numpy(), o_ref) < 1e-4 and max_rel(S.cpu().numpy(), S_ref) < 1e-4


def _tf(x):
    """The same logical [B, H, T, ...] tensor on [B, T, H, ...] memory."""
    return x.transpose(1, 2).contiguous().transpose(1, 2)


@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("packed", [False, True])
def test_token_first_memory_is_used_in_place(gate, bf16, packed):
    """Transposed views of [B, T, H, .] tensors (the layout the reference's blocks hold, delta_net.py:645-647)
    go to the kernels without copies (token_first = 1); outputs and gradients come back on the same kind of
    memory and are bit-identical to the head-first call."""
    import linearnexus_amd as la
    B, H, T, d = (1, 3, 200, 128) if packed else (2, 3, 150, 128)
    x = make_inputs(68, B, H, T, d, d, gate=gate, with_grad=True)
    dt = torch.bfloat16 if bf16 else torch.float32
    cu = torch.tensor([0, 70, 71, 200], dtype=torch.int32, device=DEV) if packed else None
    nstate = 3 if packed else B
    S0 = torch.randn(nstate, H, d, d, device=DEV) * 0.02
    dS = torch.randn(nstate, H, d, d, device=DEV) * 0.1

    def run(layout, l2, chunk):
        leaves = {n: layout(torch.from_numpy(x[n]).to(DEV).to(dt if n in ("q", "k", "v") else torch.float32)).requires_grad_(True)
                  for n in ("q", "k", "v", "beta") + (("g",) if gate != "none" else ())}
        s0 = S0.clone().requires_grad_(True)
        q, k, v, beta = leaves["q"], leaves["k"], leaves["v"], leaves["beta"]
        if gate == "none":
            fn = la.delta_rule_chunkwise if chunk else la.delta_rule_recurrent
            o, S = fn(q, k, v, beta, s0, cu_seqlens=cu)
        else:
            fn = {("scalar", True): la.gated_delta_rule_chunkwise, ("scalar", False): la.gated_delta_rule_recurrent,
                  ("vector", True): la.kda_chunkwise, ("vector", False): la.kda_recurrent}[(gate, chunk)]
            o, S = fn(q, k, v, leaves["g"], beta, None, s0, use_qk_l2norm=l2, cu_seqlens=cu)
        grads = None
        if chunk:
            dO = layout(torch.from_numpy(x["dO"]).to(DEV).to(o.dtype))
            ((o * dO).sum() + (S * dS).sum()).backward()
            grads = {n: t.grad for n, t in leaves.items()}
            grads["S0"] = s0.grad
        return o, S, grads

    for l2 in ((False, True) if gate != "none" else (False,)):
        o1, S1, g1 = run(lambda t: t, l2, True)
        o2, S2, g2 = run(_tf, l2, True)
        assert o2.transpose(1, 2).is_contiguous() and (not o2.is_contiguous() or H == 1)
        assert torch.equal(o1, o2) and torch.equal(S1, S2)
        for n in g1:
            if n in ("beta", "g"):  # row sums go through LDS atomics, whose order is not fixed: equal up to fp32 rounding
                scale_ = float(g1[n].float().abs().max())
                assert float((g1[n].float() - g2[n].float()).abs().max()) <= 2e-5 * scale_, n
            else:
                assert torch.equal(g1[n], g2[n]), n
        for n in ("q", "k", "v"):
            assert g2[n].transpose(1, 2).is_contiguous(), n
    o1, S1, _ = run(lambda t: t, False, False)
    o2, S2, _ = run(_tf, False, False)
    assert torch.equal(o1, o2) and torch.equal(S1, S2) and o2.transpose(1, 2).is_contiguous()


@pytest.mark.parametrize("kind", ["mixed", "float16", "float64"])
def test_other_input_dtypes_are_computed_in_float32(kind):
    """The reference up-casts q, k, v to float32 whatever they are and returns o in q's dtype (delta_net.py:170-179,
    :213).  Its DeltaNet block hands float32 q, k (normalised in float32, delta_net.py:566-575) next to a v in the model
    dtype; float16 and float64 inputs go the same way.  Chunk (with gradients), token scan and decode step."""
    import linearnexus_amd as la
    x = make_inputs(69, 1, 2, 100, 64, 64, gate="scalar", with_state=True, with_grad=True)
    if kind == "mixed":
        x["v"] = to_bf16_grid(x["v"])
        dts = (torch.float32, torch.float32, torch.bfloat16)
    elif kind == "float16":
        for n in ("q", "k", "v"):
            x[n] = x[n].astype(np.float16).astype(np.float32)
        dts = (torch.float16,) * 3
    else:
        dts = (torch.float64,) * 3
    q, k, v = (torch.from_numpy(x[n]).to(DEV).to(dt).requires_grad_(True) for n, dt in zip(("q", "k", "v"), dts))
    g, beta, s0 = (torch.from_numpy(x[n]).to(DEV) for n in ("g", "beta", "S0"))
    o_ref, S_ref = oracle_fwd(x, "scalar")
    tol = 2e-3 if kind == "float16" else 1e-4  # o is rounded to q's dtype on the way out
    o, S = la.gated_delta_rule_chunkwise(q, k, v, g, beta, None, s0, 64, False)
    assert o.dtype == dts[0] and S.dtype == torch.float32
    assert max_rel(o.detach().float().cpu().numpy(), o_ref) < tol and max_rel(S.detach().cpu().numpy(), S_ref) < 1e-4
    (o.float() * torch.from_numpy(x["dO"]).to(DEV)).sum().backward()
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x["g"], None, None, x["S0"], False)
    assert q.grad.dtype == dts[0] and v.grad.dtype == dts[2]
    gtol = 2e-2 if kind != "float64" else 1e-4  # gradients come back rounded to the leaves' dtypes
    for n, t in (("dq", q), ("dk", k), ("dv", v)):
        assert max_rel(t.grad.float().cpu().numpy(), ref[n]) < gtol, n
    o2, S2 = la.gated_delta_rule_recurrent(q.detach(), k.detach(), v.detach(), g, beta, None, s0, False)
    assert o2.dtype == dts[0] and max_rel(o2.float().cpu().numpy(), o_ref) < tol and max_rel(S2.cpu().numpy(), S_ref) < 1e-4
    o3, S3 = la.gated_delta_rule_step(q.detach()[:, :, 0], k.detach()[:, :, 0], v.detach()[:, :, 0], g[:, :, 0], beta[:, :, 0], s0,
                                      use_qk_l2norm=False)
    assert o3.dtype == dts[0] and max_rel(o3.float().cpu().numpy(), o_ref[:, :, 0]) < tol


@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("bf16", [False, True])
def test_beta_up_to_two_and_extreme_gates(gate, bf16):
    """allow_neg_eigval doubles beta (gated_deltanet.py:803-805): learning rates in (0, 2), so I - beta k k^T has
    eigenvalues down to -1.  Together with gates from 0 (no decay) to -30 per token (state wiped), exact zeros in
    beta and a run of all-zero keys (padding tokens inside a sequence)."""
    x = make_inputs(73, 1, 2, 200, 128, 128, gate=gate, with_state=True, with_grad=True)
    r = np.random.default_rng(73)
    x["beta"] = r.uniform(0.0, 2.0, x["beta"].shape).astype(np.float32)
    x["beta"][:, :, 50:60] = 0.0
    x["beta"][:, :, 60:64] = 2.0
    x["k"][:, :, 100:110] = 0.0
    if gate != "none":
        g = x["g"]
        g[:, :, 20:30] = 0.0
        g[:, :, 120:124] = -30.0
    xf, dt = _prep(x, bf16)
    o_ref, S_ref = oracle_fwd(xf, gate)
    o, S = gpu_chunk_fwd(xf, gate, dt)
    tol = 2e-2 if bf16 else 1e-4
    assert torch.isfinite(o).all() and torch.isfinite(S).all()
    assert max_rel(o.float().cpu().numpy(), o_ref) < tol and max_rel(S.cpu().numpy(), S_ref) < tol
    xb, dt = _prep_bwd(x, bf16)
    ref = delta_rule_adjoint(xb["q"], xb["k"], xb["v"], xb["beta"], xb["dO"], xb.get("g"), xb["dS"], None, xb["S0"], False)
    check(gpu_grads(xb, gate, dt), ref, tol)


@pytest.mark.parametrize("gate", ["none", "vector"])
def test_packed_batch_with_hundreds_of_short_sequences(gate):
    """More sequences than the table builder has threads, most of them a few tokens long, some empty."""
    H, d = 2, 64
    r = np.random.default_rng(74)
    lens = r.integers(0, 6, 300)
    lens[::37] = r.integers(60, 140, len(lens[::37]))
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T, nseq = int(cu[-1]), len(lens)
    x = make_inputs(74, 1, H, T, d, d, gate=gate, with_grad=True)
    x["S0"] = (r.standard_normal((nseq, H, d, d)) * 0.02).astype(np.float32)
    x["dS"] = (r.standard_normal((nseq, H, d, d)) * 0.1).astype(np.float32)
    parts, o_ref, S_ref = [], np.zeros((1, H, T, d)), []
    for s in range(nseq):
        a, b = cu[s], cu[s + 1]
        sl = lambda n: x[n][:, :, a:b]
        y = {"q": sl("q"), "k": sl("k"), "v": sl("v"), "beta": sl("beta"), "S0": x["S0"][s:s + 1]}
        if gate != "none":
            y["g"] = sl("g")
        o_s, S_s = oracle_fwd(y, gate)
        o_ref[:, :, a:b] = o_s
        S_ref.append(S_s)
        parts.append(delta_rule_adjoint(sl("q"), sl("k"), sl("v"), sl("beta"), sl("dO"), sl("g") if gate != "none" else None,
                                        x["dS"][s:s + 1], None, x["S0"][s:s + 1], False))
    o, S = gpu_chunk_fwd(x, gate, torch.float32, cu=cu)
    assert max_rel(o.cpu().numpy(), o_ref) < 1e-4 and max_rel(S.cpu().numpy(), np.concatenate(S_ref, 0)) < 1e-4
    names = ("dq", "dk", "dv", "dbeta") + (("dg",) if gate != "none" else ())
    ref = {n: np.concatenate([p[n] for p in parts], 2) for n in names}
    ref["dS0"] = np.concatenate([p["dS0"] for p in parts], 0)
    check(gpu_grads(x, gate, torch.float32, cu=cu), ref, 1e-4)


@pytest.mark.parametrize("gate", ["none", "scalar"])
@pytest.mark.parametrize("slab", [32, 64])
def test_bf16_inputs_with_fp32_outputs_take_the_same_kernels(gate, slab, monkeypatch):
    """o_dtype does not select kernels: bf16 q, k, v with an fp32 output tensor run the direct-solve kernels like the
    bf16-output call (the outputs are formed in fp32, rounded to bf16 -- the precision the reference returns for such
    inputs, gated_deltanet.py:534 -- and widened on their way out), the backward pass reads the same workspace layout,
    and values and gradients equal the bf16-output call's exactly."""
    monkeypatch.setitem(linear_attn._test_hooks, "scan_slab", slab)
    x = make_inputs(91, 2, 3, 150, 128, 128, gate=gate, with_state=True, with_grad=True)
    xb, dt = _prep_bwd(x, True)
    g = None if gate == "none" else torch.from_numpy(xb["g"]).to(DEV)
    res = []
    for o_dtype in (torch.bfloat16, torch.float32):
        leaves = [torch.from_numpy(xb[n]).to(DEV).to(torch.bfloat16).requires_grad_(True) for n in ("q", "k", "v")]
        beta = torch.from_numpy(xb["beta"]).to(DEV).requires_grad_(True)
        s0 = torch.from_numpy(xb["S0"]).to(DEV).requires_grad_(True)
        o, S = linear_attn._chunk(*leaves, g, beta, None, s0, 64, False, o_dtype, True, None)
        assert o.dtype == o_dtype
        dO = torch.from_numpy(xb["dO"]).to(DEV).to(torch.bfloat16)
        grads = torch.autograd.grad([o, S], leaves + [beta, s0], [dO.to(o_dtype), torch.from_numpy(xb["dS"]).to(DEV)])
        res.append([o.detach().float(), S.detach(), *[t.float() for t in grads]])
    for a, b in zip(*res):
        assert torch.equal(a, b)
    o_ref, S_ref = oracle_fwd(xb, gate)
    assert max_rel(res[1][0].cpu().numpy(), o_ref) < 2e-2 and max_rel(res[1][1].cpu().numpy(), S_ref) < 2e-2


def test_views_that_start_inside_a_16_byte_vector_are_copied_and_the_abi_refuses_them():
    """The kernels move rows as 16-byte vectors.  The Python ops copy a dense view whose first element does not sit on
    a 16-byte boundary of its storage (same values and gradients as from aligned tensors); the C-ABI refuses such a
    pointer instead of launching."""
    import linearnexus_amd as la
    from linearnexus_amd import _lib
    B, H, T, d = 1, 2, 130, 64
    x = make_inputs(93, B, H, T, d, d, gate="scalar")
    n = B * H * T * d

    def leaves(offset):
        out = []
        for name in ("q", "k", "v"):
            flat = torch.zeros(n + 8, dtype=torch.bfloat16, device=DEV)
            flat[offset:offset + n] = torch.from_numpy(x[name]).to(DEV).to(torch.bfloat16).flatten()
            out.append(flat[offset:offset + n].view(B, H, T, d).detach().requires_grad_(True))
        return out

    g, beta = torch.from_numpy(x["g"]).to(DEV), torch.from_numpy(x["beta"]).to(DEV)
    res = []
    for offset in (0, 1):  # 0 and 2 bytes into the storage
        q, k, v = leaves(offset)
        assert q.data_ptr() % 16 == 2 * offset
        o, S = la.gated_delta_rule_chunkwise(q, k, v, g, beta, use_qk_l2norm=False)
        grads = torch.autograd.grad([o, S], [q, k, v], [torch.ones_like(o), torch.ones_like(S)])
        res.append([o, S, *grads])
    for a, b in zip(*res):
        assert torch.equal(a, b)
    lib = _lib.load()
    q, k, v = leaves(1)
    a = _lib.ScanArgs()
    a.B, a.H, a.T, a.dk, a.dv, a.chunk = B, H, T, d, d, 64
    a.dtype = a.o_dtype = _lib.LNX_BF16
    a.gate, a.scale, a.forward_only = _lib.GATE_SCALAR, d ** -0.5, 1
    o = torch.empty(B, H, T, d, dtype=torch.bfloat16, device=DEV)
    sT = torch.empty(B, H, d, d, dtype=torch.float32, device=DEV)
    a.q, a.k, a.v, a.beta, a.g = q.data_ptr(), k.data_ptr(), v.data_ptr(), beta.data_ptr(), g.data_ptr()
    a.o, a.final_state = o.data_ptr(), sT.data_ptr()
    ws = torch.empty(int(lib.lnx_chunk_workspace_bytes(a)), dtype=torch.uint8, device=DEV)
    a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel()
    assert lib.lnx_chunk_fwd(a, None) == -2 and b"16-byte aligned" in lib.lnx_last_error()
