"""Key head dimension 256 (the Gated DeltaNet presets of the reference: models.py:142-143, :369-370 use
head_dim 256 with expand_v 2, i.e. dk = 256, dv = 512): chunk forward and backward for 2-byte inputs against
the fp64 oracles, for every gate kind, ragged lengths, packed batches and token-first memory.
Metric max|x - ref| / max|ref| <= 2e-2 (bf16 inputs, fp32 accumulation) or <= 1e-4 (fp32 inputs)."""
import numpy as np
import pytest
import torch

from linearnexus_amd import linear_attn
from oracle import recurrent as rc
from oracle.adjoint import delta_rule_adjoint
from oracle.inputs import make_inputs
from conftest import max_rel
from test_chunk_bwd_gpu import _prep, check, gpu_grads
from test_chunk_fwd_gpu import gpu_chunk_fwd, oracle_fwd

pytestmark = pytest.mark.gpu
DEV = "cuda"
GATES = ["none", "scalar", "vector"]


# 2-byte inputs have a 32-column variant of the two sequential kernels and a 64-column one in which two operand tiles
# share LDS space (chosen by the number of workgroups); the test_scan_slab field of the argument block forces either.
SLABS = ["32", "64"]


@pytest.mark.parametrize("slab", SLABS)
@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("shape", [(1, 2, 200, 256, 128), (2, 1, 64, 256, 64), (1, 1, 130, 256, 512)])
@pytest.mark.parametrize("with_state", [False, True])
def test_forward_dk256(gate, shape, with_state, slab, monkeypatch):
    monkeypatch.setitem(linear_attn._test_hooks, "scan_slab", int(slab))
    B, H, T, dk, dv = shape
    x = make_inputs(81, B, H, T, dk, dv, gate=gate, with_state=with_state, with_grad=True)
    x, dt = _prep(x, True)
    o_ref, S_ref = oracle_fwd(x, gate)
    o, S = gpu_chunk_fwd(x, gate, dt)
    eo, eS = max_rel(o.float().cpu().numpy(), o_ref), max_rel(S.cpu().numpy(), S_ref)
    assert eo < 2e-2 and eS < 2e-2, (eo, eS)


@pytest.mark.parametrize("slab", SLABS)
@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("shape", [(1, 2, 200, 256, 128), (2, 1, 70, 256, 64), (1, 1, 128, 256, 512)])
def test_backward_dk256(gate, shape, slab, monkeypatch):
    monkeypatch.setitem(linear_attn._test_hooks, "scan_slab", int(slab))
    B, H, T, dk, dv = shape
    x = make_inputs(82, B, H, T, dk, dv, gate=gate, with_state=True, with_grad=True)
    x, dt = _prep(x, True)
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x.get("g"), x["dS"], None, x["S0"], False)
    check(gpu_grads(x, gate, dt), ref, 2e-2)


@pytest.mark.parametrize("slab", SLABS)
@pytest.mark.parametrize("gate", ["scalar", "vector"])
def test_packed_dk256(gate, slab, monkeypatch):
    monkeypatch.setitem(linear_attn._test_hooks, "scan_slab", int(slab))
    H, T, dk, dv = 2, 300, 256, 128
    x = make_inputs(83, 1, H, T, dk, dv, gate=gate, with_grad=True)
    cu = np.array([0, 64, 70, 200, 300], np.int32)
    rng = np.random.default_rng(7)
    x["S0"] = (rng.standard_normal((4, H, dk, dv)) * 0.02).astype(np.float32)
    x["dS"] = (rng.standard_normal((4, H, dk, dv)) * 0.1).astype(np.float32)
    x, dt = _prep(x, True)
    parts = []
    for s in range(4):
        a, b = cu[s], cu[s + 1]
        sl = lambda n: x[n][:, :, a:b]
        parts.append(delta_rule_adjoint(sl("q"), sl("k"), sl("v"), sl("beta"), sl("dO"), sl("g"), x["dS"][s:s + 1], None,
                                        x["S0"][s:s + 1], False))
    ref = {n: np.concatenate([p[n] for p in parts], axis=2) for n in ("dq", "dk", "dv", "dbeta", "dg")}
    ref["dS0"] = np.concatenate([p["dS0"] for p in parts], axis=0)
    check(gpu_grads(x, gate, dt, cu=cu), ref, 2e-2)


@pytest.mark.parametrize("slab", SLABS)
def test_token_first_dk256(slab, monkeypatch):
    """[B, T, H, d] memory (the layout the reference's blocks hold before their transpose) through the same kernels."""
    monkeypatch.setitem(linear_attn._test_hooks, "scan_slab", int(slab))
    import linearnexus_amd as la
    B, H, T, dk, dv = 2, 3, 150, 256, 128
    x = make_inputs(84, B, H, T, dk, dv, gate="scalar", with_state=True)
    x, dt = _prep({**x, "dO": x["v"]}, True)
    o_ref, S_ref = rc.gated_delta_rule_recurrent(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["S0"], False)
    tf = lambda a, d=None: torch.from_numpy(np.ascontiguousarray(np.swapaxes(a, 1, 2))).to(DEV).to(d or torch.float32).transpose(1, 2)
    o, S = la.gated_delta_rule_chunkwise(tf(x["q"], dt), tf(x["k"], dt), tf(x["v"], dt), tf(x["g"]), tf(x["beta"]), None,
                                         torch.from_numpy(x["S0"]).to(DEV), 64, False)
    assert max_rel(o.float().cpu().numpy(), o_ref) < 2e-2 and max_rel(S.cpu().numpy(), S_ref) < 2e-2


@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("shape", [(1, 2, 200, 256, 128), (2, 1, 70, 256, 64), (1, 1, 128, 256, 512)])
def test_fp32_dk256(gate, shape):
    """4-byte inputs: K, Q and W of a chunk take turns in one LDS tile in the sequential kernels.  Tolerance 1e-4."""
    B, H, T, dk, dv = shape
    x = make_inputs(85, B, H, T, dk, dv, gate=gate, with_state=True, with_grad=True)
    o_ref, S_ref = oracle_fwd(x, gate)
    o, S = gpu_chunk_fwd(x, gate, torch.float32)
    eo, eS = max_rel(o.cpu().numpy(), o_ref), max_rel(S.cpu().numpy(), S_ref)
    assert eo < 1e-4 and eS < 1e-4, (eo, eS)
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x.get("g"), x["dS"], None, x["S0"], False)
    check(gpu_grads(x, gate, torch.float32), ref, 1e-4)


def test_fp32_dk256_packed():
    H, T, dk, dv = 2, 300, 256, 128
    x = make_inputs(86, 1, H, T, dk, dv, gate="scalar", with_grad=True)
    cu = np.array([0, 64, 70, 200, 300], np.int32)
    rng = np.random.default_rng(8)
    x["S0"] = (rng.standard_normal((4, H, dk, dv)) * 0.02).astype(np.float32)
    x["dS"] = (rng.standard_normal((4, H, dk, dv)) * 0.1).astype(np.float32)
    parts = []
    for s in range(4):
        a, b = cu[s], cu[s + 1]
        sl = lambda n: x[n][:, :, a:b]
        parts.append(delta_rule_adjoint(sl("q"), sl("k"), sl("v"), sl("beta"), sl("dO"), sl("g"), x["dS"][s:s + 1], None,
                                        x["S0"][s:s + 1], False))
    ref = {n: np.concatenate([p[n] for p in parts], axis=2) for n in ("dq", "dk", "dv", "dbeta", "dg")}
    ref["dS0"] = np.concatenate([p["dS0"] for p in parts], axis=0)
    check(gpu_grads(x, "scalar", torch.float32, cu=cu), ref, 1e-4)


@pytest.mark.parametrize("slab", SLABS)
def test_reference_preset_shape_against_token_kernel(slab, monkeypatch):
    """The presets' head shape (dk 256, dv 512) at a few thousand tokens: the chunk path and the fp32
    token-by-token kernel (itself checked against the oracle) must agree."""
    import linearnexus_amd as la
    monkeypatch.setitem(linear_attn._test_hooks, "scan_slab", int(slab))
    torch.manual_seed(3)
    B, H, T, dk, dv = 2, 4, 2048, 256, 512
    q = torch.nn.functional.normalize(torch.randn(B, H, T, dk, device=DEV), dim=-1).bfloat16()
    k = torch.nn.functional.normalize(torch.randn(B, H, T, dk, device=DEV), dim=-1).bfloat16()
    v = torch.randn(B, H, T, dv, device=DEV).bfloat16()
    beta = torch.sigmoid(torch.randn(B, H, T, device=DEV))
    g = -torch.nn.functional.softplus(torch.randn(B, H, T, device=DEV)) * 0.1
    o1, S1 = la.gated_delta_rule_recurrent(q, k, v, g, beta, use_qk_l2norm=False)
    o2, S2 = la.gated_delta_rule_chunkwise(q, k, v, g, beta, use_qk_l2norm=False)
    eo = (o1.float() - o2.float()).abs().max() / o1.float().abs().max()
    eS = (S1 - S2).abs().max() / S1.abs().max()
    assert eo < 2e-2 and eS < 2e-2, (float(eo), float(eS))
