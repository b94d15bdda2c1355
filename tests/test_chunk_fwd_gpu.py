"""GPU parity of the chunked forward kernels against the fp64 recurrent oracle, through the
Python ops -> C-ABI -> HIP path.  Metric: max|x - ref| / max|ref| <= 1e-4 (fp32 inputs) or
<= 2e-2 (bf16 inputs, fp32 accumulation)."""
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
    if not bf16:
        return x, torch.float32
    y = dict(x)
    for n in ("q", "k", "v"):
        y[n] = to_bf16_grid(x[n])
    return y, torch.bfloat16


def oracle_fwd(x, gate, l2=False):
    if gate == "none":
        return rc.delta_rule_recurrent(x["q"], x["k"], x["v"], x["beta"], x.get("S0"))
    fn = rc.gated_delta_rule_recurrent if gate == "scalar" else rc.kda_recurrent
    return fn(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x.get("S0"), l2)


def gpu_chunk_fwd(x, gate, dt, l2=False, cu=None):
    import linearnexus_amd as la
    q, k, v = _t(x["q"], dt), _t(x["k"], dt), _t(x["v"], dt)
    s0 = _t(x["S0"]) if "S0" in x else None
    cu_t = None if cu is None else _t(cu)
    if gate == "none":
        return la.delta_rule_chunkwise(q, k, v, _t(x["beta"]), s0, cu_seqlens=cu_t)
    fn = la.gated_delta_rule_chunkwise if gate == "scalar" else la.kda_chunkwise
    return fn(q, k, v, _t(x["g"]), _t(x["beta"]), None, s0, 64, l2, cu_seqlens=cu_t)


GATES = ["none", "scalar", "vector"]
SHAPES = [(2, 2, 128, 64, 64), (1, 2, 200, 128, 128), (1, 3, 64, 128, 64), (2, 1, 37, 64, 128), (1, 2, 513, 128, 128)]


@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("with_state", [False, True])
def test_chunk_forward_matches_oracle(gate, bf16, shape, with_state):
    B, H, T, dk, dv = shape
    x = make_inputs(41, B, H, T, dk, dv, gate=gate, with_state=with_state)
    x, dt = _prep(x, bf16)
    o_ref, S_ref = oracle_fwd(x, gate)
    o, S = gpu_chunk_fwd(x, gate, dt)
    assert S.dtype == torch.float32
    assert o.dtype == (torch.float32 if gate == "vector" else dt)  # kda.py:655 returns fp32
    tol = 2e-2 if bf16 else 1e-4
    eo, eS = max_rel(o.float().cpu().numpy(), o_ref), max_rel(S.cpu().numpy(), S_ref)
    assert eo < tol and eS < tol, (eo, eS)


def test_config1_deltanet_fp32():
    """Benchmark configuration 1: B2 H4 T512 dk=dv=64 fp32, zero initial state."""
    x = make_inputs(1, 2, 4, 512, 64, 64)
    o_ref, S_ref = oracle_fwd(x, "none")
    o, S = gpu_chunk_fwd(x, "none", torch.float32)
    assert max_rel(o.cpu().numpy(), o_ref) < 1e-4 and max_rel(S.cpu().numpy(), S_ref) < 1e-4


@pytest.mark.parametrize("gate", GATES)
def test_l2norm_inside_op(gate):
    if gate == "none":
        pytest.skip("delta_rule_chunkwise has no l2norm flag (delta_net.py:216-225)")
    x = make_inputs(42, 1, 2, 130, 128, 128, gate=gate, normalize=False)
    x, dt = _prep(x, True)
    o_ref, S_ref = oracle_fwd(x, gate, l2=True)
    o, S = gpu_chunk_fwd(x, gate, dt, l2=True)
    assert max_rel(o.float().cpu().numpy(), o_ref) < 2e-2 and max_rel(S.cpu().numpy(), S_ref) < 2e-2


@pytest.mark.parametrize("dk", [64, 128])
def test_l2norm_inside_the_chunk_kernels_zero_rows(dk):
    """bf16, scalar gate: the kernels normalise the rows themselves; an all-zero q row and an all-zero k row normalise
    to zero (x / (|x| + 1e-6)) and everything stays finite."""
    x = make_inputs(45, 2, 2, 150, dk, 128, gate="scalar", normalize=False)
    x["q"] = x["q"] * np.exp(np.random.default_rng(46).standard_normal((2, 2, 150, 1))).astype(np.float32)
    x["q"][0, 0, 5] = 0.0
    x["k"][1, 1, 70] = 0.0
    x, dt = _prep(x, True)
    o_ref, S_ref = oracle_fwd(x, "scalar", l2=True)
    o, S = gpu_chunk_fwd(x, "scalar", dt, l2=True)
    assert torch.isfinite(o).all() and torch.isfinite(S).all()
    assert max_rel(o.float().cpu().numpy(), o_ref) < 2e-2 and max_rel(S.cpu().numpy(), S_ref) < 2e-2


@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("bf16", [False, True])
def test_packed_sequences(gate, bf16):
    H, T, d = 2, 400, 128
    x = make_inputs(43, 1, H, T, d, d, gate=gate)
    x, dt = _prep(x, bf16)
    cu = np.array([0, 64, 65, 200, 330, 400], np.int32)
    S0 = (np.random.default_rng(5).standard_normal((5, H, d, d)) * 0.02).astype(np.float32)

    def one(q, k, v, *rest, initial_state=None):
        y = {"q": q, "k": k, "v": v, "beta": rest[-1], "S0": initial_state}
        if gate != "none":
            y["g"] = rest[0]
        return oracle_fwd(y, gate)

    args = [x["q"], x["k"], x["v"]] + ([x["g"]] if gate != "none" else []) + [x["beta"]]
    o_ref, S_ref = rc.varlen(one, cu, *args, initial_state=S0)
    x["S0"] = S0
    o, S = gpu_chunk_fwd(x, gate, dt, cu=cu)
    tol = 2e-2 if bf16 else 1e-4
    assert tuple(S.shape) == (5, H, d, d)
    assert max_rel(o.float().cpu().numpy(), o_ref) < tol and max_rel(S.cpu().numpy(), S_ref) < tol


@pytest.mark.parametrize("gate", ["scalar", "vector"])
def test_strong_decay_stays_finite(gate):
    # gates down to -10 per token as in bench_kda_kernels.py:123-129
    x = make_inputs(44, 1, 2, 192, 128, 128, gate=gate)
    x["g"] = (-np.random.default_rng(44).uniform(0, 10, x["g"].shape)).astype(np.float32)
    x, dt = _prep(x, True)
    o_ref, S_ref = oracle_fwd(x, gate)
    o, S = gpu_chunk_fwd(x, gate, dt)
    assert torch.isfinite(o).all() and torch.isfinite(S).all()
    assert max_rel(o.float().cpu().numpy(), o_ref) < 2e-2 and max_rel(S.cpu().numpy(), S_ref) < 2e-2


@pytest.mark.parametrize("shape", [(1, 2, 200, 128, 128), (1, 3, 330, 128, 64)])
def test_vector_gate_two_byte_output_is_the_rounded_fp32_output(shape):
    """The per-channel-gate scan stages its outputs through LDS in either precision; kda_chunkwise only ever asks for
    fp32 (kda.py:655), so the 2-byte branch is reached through the internal entry: same arithmetic, one rounding at the
    store, hence bit-equal to the rounded fp32 result.  Ragged lengths: the last chunk's rows past T are not written."""
    from linearnexus_amd import linear_attn as la_int
    B, H, T, dk, dv = shape
    x, dt = _prep(make_inputs(46, B, H, T, dk, dv, gate="vector", with_state=True), True)
    q, k, v = _t(x["q"], dt), _t(x["k"], dt), _t(x["v"], dt)
    args = (q, k, v, _t(x["g"]), _t(x["beta"]), None, _t(x["S0"]), 64, False)
    o32, S32 = la_int._chunk(*args, torch.float32, True, None)
    o16, S16 = la_int._chunk(*args, torch.bfloat16, True, None)
    assert o16.dtype == torch.bfloat16 and o32.dtype == torch.float32
    assert torch.equal(o16, o32.to(torch.bfloat16)) and torch.equal(S16, S32)


def test_chunk_equals_recurrent_kernel_at_full_config2_size():
    """Size-independent check at B8 H16 T4096 d128 bf16: the MFMA chunk path and the fp32
    token-by-token kernel (itself checked against the oracle) must agree."""
    import linearnexus_amd as la
    torch.manual_seed(2)
    B, H, T, d = 8, 16, 4096, 128
    q = torch.nn.functional.normalize(torch.randn(B, H, T, d, device=DEV), dim=-1).bfloat16()
    k = torch.nn.functional.normalize(torch.randn(B, H, T, d, device=DEV), dim=-1).bfloat16()
    v = torch.randn(B, H, T, d, device=DEV).bfloat16()
    beta = torch.sigmoid(torch.randn(B, H, T, device=DEV))
    g = -torch.nn.functional.softplus(torch.randn(B, H, T, device=DEV)) * 0.1
    o1, S1 = la.gated_delta_rule_recurrent(q, k, v, g, beta, use_qk_l2norm=False)
    o2, S2 = la.gated_delta_rule_chunkwise(q, k, v, g, beta, use_qk_l2norm=False)
    eo = (o1.float() - o2.float()).abs().max() / o1.float().abs().max()
    eS = (S1 - S2).abs().max() / S1.abs().max()
    assert eo < 2e-2 and eS < 2e-2, (float(eo), float(eS))


def test_unsupported_dims_raise_runtime_error():
    # same error type as the reference's accelerated path (kernels/pallas/delta_rule.py:108-115)
    import linearnexus_amd as la
    q = torch.randn(1, 1, 64, 272, device=DEV)  # key heads wider than 256 (narrower ones are embedded with zero channels)
    with pytest.raises(RuntimeError):
        la.delta_rule_chunkwise(q, q, torch.randn(1, 1, 64, 64, device=DEV), torch.ones(1, 1, 64, device=DEV))


@pytest.mark.parametrize("gate", ["none", "scalar", "vector"])
def test_no_grad_with_leaves_that_require_grad_is_the_forward_only_path(gate, monkeypatch):
    """Evaluation of a model whose parameters require grad, under torch.no_grad(): the op must not save for a backward
    pass (it used to, going by the leaves alone) and must return what the differentiable call returns, bit for bit."""
    import linearnexus_amd as la
    from linearnexus_amd import linear_attn
    x, dt = _prep(make_inputs(31, 2, 2, 200, 128, 128, gate=gate, with_state=True), True)
    q, k, v = _t(x["q"], dt), _t(x["k"], dt), _t(x["v"], dt)
    beta, s0 = _t(x["beta"]), _t(x["S0"])
    g = _t(x["g"]) if gate != "none" else None
    for t in (q, k, v, beta, s0) + ((g,) if g is not None else ()):
        t.requires_grad_(True)

    def call():
        if gate == "none":
            return la.delta_rule_chunkwise(q, k, v, beta, s0)
        fn = la.gated_delta_rule_chunkwise if gate == "scalar" else la.kda_chunkwise
        return fn(q, k, v, g, beta, None, s0, 64, False)

    seen = []
    inner = linear_attn._chunk_forward

    def spy(*a, forward_only, **kw):
        seen.append(forward_only)
        return inner(*a, forward_only=forward_only, **kw)

    monkeypatch.setattr(linear_attn, "_chunk_forward", spy)
    o1, s1 = call()
    with torch.no_grad():
        o2, s2 = call()
    assert seen == [False, True]
    assert o1.requires_grad and not o2.requires_grad
    assert torch.equal(o1.detach(), o2) and torch.equal(s1.detach(), s2)
