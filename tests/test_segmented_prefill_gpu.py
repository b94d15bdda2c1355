"""Forward-only calls on few long sequences are cut into segments that run in parallel (the scan is linear in the
state: S_out = A_s S_in + B_s per segment).  The result must be the sequential one: against the fp64 oracle for
every gate kind, with and without an initial state, ragged lengths, forced segment counts; and at a long prompt's
size against the unsegmented kernels.  1e-4 (fp32), 2e-2 (bf16)."""
import numpy as np
import pytest
import torch

from oracle.inputs import make_inputs
from conftest import max_rel
from test_chunk_fwd_gpu import _prep, gpu_chunk_fwd, oracle_fwd

pytestmark = pytest.mark.gpu
DEV = "cuda"
GATES = ["none", "scalar", "vector"]


@pytest.mark.parametrize("nseg", ["2", "5"])
@pytest.mark.parametrize("gate", GATES)
@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("shape,with_state", [((2, 2, 1000, 64, 128), True), ((1, 3, 700, 128, 64), False),
                                              ((1, 2, 330, 256, 128), True)])
def test_forced_segments_match_oracle(gate, bf16, shape, with_state, nseg, monkeypatch):
    monkeypatch.setenv("LNX_PREFILL_SEGMENTS", nseg)
    B, H, T, dk, dv = shape
    x = make_inputs(101, B, H, T, dk, dv, gate=gate, with_state=with_state)
    x, dt = _prep(x, bf16)
    o_ref, S_ref = oracle_fwd(x, gate)
    with torch.no_grad():
        o, S = gpu_chunk_fwd(x, gate, dt)
    tol = 2e-2 if bf16 else 1e-4
    assert tuple(o.shape) == (B, H, T, dv) and tuple(S.shape) == (B, H, dk, dv)
    eo, eS = max_rel(o.float().cpu().numpy(), o_ref), max_rel(S.cpu().numpy(), S_ref)
    assert eo < tol and eS < tol, (eo, eS)


def test_l2norm_inside_and_gradients_bypass(monkeypatch):
    """The in-op L2 norm goes through both passes; a call that wants gradients is never segmented."""
    import linearnexus_amd as la
    monkeypatch.setenv("LNX_PREFILL_SEGMENTS", "4")
    x = make_inputs(102, 1, 2, 600, 128, 128, gate="scalar", with_state=True, normalize=False)
    o_ref, S_ref = oracle_fwd(x, "scalar", l2=True)
    with torch.no_grad():
        o, S = gpu_chunk_fwd(x, "scalar", torch.float32, l2=True)
    assert max_rel(o.cpu().numpy(), o_ref) < 1e-4 and max_rel(S.cpu().numpy(), S_ref) < 1e-4
    t = {n: torch.from_numpy(x[n]).to(DEV) for n in ("q", "k", "v", "g", "beta")}
    t["q"].requires_grad_(True)
    o2, _ = la.gated_delta_rule_chunkwise(t["q"], t["k"], t["v"], t["g"], t["beta"], None, None, 64, True)
    o2.sum().backward()
    assert t["q"].grad is not None


def test_long_prompt_agrees_with_the_sequential_kernels(monkeypatch):
    """One prompt of 65536 tokens, 8 heads, d = 128, bf16: segmented automatically; same result as one long chain."""
    import time
    import linearnexus_amd as la
    torch.manual_seed(4)
    B, H, T, d = 1, 8, 65536, 128
    q = torch.nn.functional.normalize(torch.randn(B, H, T, d, device=DEV), dim=-1).bfloat16()
    k = torch.nn.functional.normalize(torch.randn(B, H, T, d, device=DEV), dim=-1).bfloat16()
    v = torch.randn(B, H, T, d, device=DEV).bfloat16()
    beta = torch.sigmoid(torch.randn(B, H, T, device=DEV))
    g = -torch.nn.functional.softplus(torch.randn(B, H, T, device=DEV)) * 0.1

    def run():
        with torch.no_grad():
            for _ in range(2):
                out = la.gated_delta_rule_chunkwise(q, k, v, g, beta, use_qk_l2norm=False)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            out = la.gated_delta_rule_chunkwise(q, k, v, g, beta, use_qk_l2norm=False)
            torch.cuda.synchronize()
        return out, (time.perf_counter() - t0) * 1e3

    monkeypatch.setenv("LNX_PREFILL_SEGMENTS", "1")
    (o1, S1), ms1 = run()
    monkeypatch.delenv("LNX_PREFILL_SEGMENTS")
    (o2, S2), ms2 = run()
    print(f"65536-token prompt: one chain {ms1:.2f} ms, segmented {ms2:.2f} ms")
    eo = (o1.float() - o2.float()).abs().max() / o1.float().abs().max()
    eS = (S1 - S2).abs().max() / S1.abs().max()
    assert eo < 2e-2 and eS < 2e-2, (float(eo), float(eS))
