"""Seeded random sweep over the configuration space of the chunk ops (gate kind, dtype, head dims, ragged
lengths, packed batches, initial state, token-first memory) against the fp64 oracles.  Tolerances as everywhere:
max|x - ref| / max|ref| below 1e-4 for fp32 inputs and 2e-2 for bf16 inputs."""
import numpy as np
import pytest
import torch

from oracle import recurrent as rc
from oracle.adjoint import delta_rule_adjoint
from oracle.inputs import make_inputs, to_bf16_grid
from conftest import max_rel

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _cases():
    r = np.random.default_rng(2024)
    out = []
    for i in range(36):
        gate = ("none", "scalar", "vector")[i % 3]
        bf16 = bool(r.integers(2))
        dk = int(r.choice([64, 128]))
        dv = int(r.choice([64, 128, 256] if bf16 or dk == 64 else [64, 128]))
        H = int(r.integers(1, 4))
        packed = bool(r.integers(3) == 0)
        B = 1 if packed else int(r.integers(1, 3))
        T = int(r.integers(1, 330))
        nseq = int(r.integers(1, 5)) if packed else 0
        out.append((i, gate, bf16, B, H, T, dk, dv, nseq, bool(r.integers(2)), bool(r.integers(2))))
    # a second list (its own generator, so the first keeps its cases): the wide key heads of the reference's presets,
    # head sizes between the kernels' sizes, either dtype
    r = np.random.default_rng(2025)
    for i in range(36, 60):
        gate = ("none", "scalar", "vector")[i % 3]
        bf16 = bool(r.integers(2))
        dk = int(r.choice([256, 256, 96, 200, 16]))
        dv = int(r.choice([64, 128, 512, 80, 32] if bf16 or dk < 256 else [64, 128, 80]))
        H = int(r.integers(1, 3))
        packed = bool(r.integers(3) == 0)
        B = 1 if packed else int(r.integers(1, 3))
        T = int(r.integers(1, 200))
        nseq = int(r.integers(1, 5)) if packed else 0
        out.append((i, gate, bf16, B, H, T, dk, dv, nseq, bool(r.integers(2)), bool(r.integers(2))))
    # a third list: the in-op L2 normalisation (the reference's default) on rows of very different lengths -- inside the
    # kernels for bf16 with a scalar gate, stand-alone kernels around them otherwise
    r = np.random.default_rng(2026)
    for i in range(60, 84):
        gate = ("scalar", "scalar", "vector")[i % 3]
        bf16 = bool(r.integers(4) > 0)
        dk = int(r.choice([64, 128, 128, 96, 256]))
        dv = int(r.choice([64, 128, 256, 80] if bf16 or dk < 256 else [64, 128]))
        H = int(r.integers(1, 4))
        packed = bool(r.integers(3) == 0)
        B = 1 if packed else int(r.integers(1, 3))
        T = int(r.integers(1, 300))
        nseq = int(r.integers(1, 5)) if packed else 0
        out.append((i, gate, bf16, B, H, T, dk, dv, nseq, bool(r.integers(2)), bool(r.integers(2)), True))
    return out


@pytest.mark.parametrize("case", _cases(), ids=lambda c: f"{c[0]}-{c[1]}-{'bf16' if c[2] else 'f32'}-B{c[3]}H{c[4]}T{c[5]}k{c[6]}v{c[7]}s{c[8]}{'-l2' if len(c) > 11 else ''}")
def test_random_configuration(case):
    import linearnexus_amd as la
    i, gate, bf16, B, H, T, dk, dv, nseq, with_state, token_first = case[:11]
    l2 = len(case) > 11 and case[11]
    x = make_inputs(500 + i, B, H, T, dk, dv, gate=gate, with_grad=True, normalize=not l2)
    r = np.random.default_rng(900 + i)
    if l2:
        x["q"] = x["q"] * np.exp(r.standard_normal((B, H, T, 1))).astype(np.float32)
        x["k"] = x["k"] * np.exp(r.standard_normal((B, H, T, 1))).astype(np.float32)
    cu = None
    nstate = B
    if nseq:
        cuts = np.sort(r.integers(0, T + 1, nseq - 1))
        cu = np.concatenate([[0], cuts, [T]]).astype(np.int32)
        nstate = nseq
    x["dS"] = (r.standard_normal((nstate, H, dk, dv)) * 0.1).astype(np.float32)
    if with_state:
        x["S0"] = (r.standard_normal((nstate, H, dk, dv)) * 0.02).astype(np.float32)
    dt = torch.bfloat16 if bf16 else torch.float32
    if bf16:
        for n in ("q", "k", "v", "dO"):
            x[n] = to_bf16_grid(x[n])

    # oracle: every sequence on its own
    spans = [(0, T)] if cu is None else list(zip(cu[:-1], cu[1:]))
    names = ("dq", "dk", "dv", "dbeta") + (("dg",) if gate != "none" else ())
    o_ref = np.zeros((B, H, T, dv))
    g_ref = {n: [] for n in names}
    S_ref, dS0_ref = [], []
    for s, (a, b) in enumerate(spans):
        sl = lambda n: x[n][:, :, a:b]
        st = slice(s, s + 1) if cu is not None else slice(None)
        S0 = x["S0"][st] if with_state else None
        gg = sl("g") if gate != "none" else None
        if gate == "none":
            o_s, S_s = rc.delta_rule_recurrent(sl("q"), sl("k"), sl("v"), sl("beta"), S0)
        else:
            fn = rc.gated_delta_rule_recurrent if gate == "scalar" else rc.kda_recurrent
            o_s, S_s = fn(sl("q"), sl("k"), sl("v"), gg, sl("beta"), None, S0, l2)
        o_ref[:, :, a:b] = o_s
        S_ref.append(S_s)
        ad = delta_rule_adjoint(sl("q"), sl("k"), sl("v"), sl("beta"), sl("dO"), gg, x["dS"][st], None, S0, l2)
        for n in names:
            g_ref[n].append(ad[n])
        dS0_ref.append(ad["dS0"])
    S_ref = np.concatenate(S_ref, 0) if cu is not None else S_ref[0]
    dS0_ref = np.concatenate(dS0_ref, 0) if cu is not None else dS0_ref[0]
    g_ref = {n: np.concatenate(v, 2) for n, v in g_ref.items()}

    def dev(a, d=None):
        t = torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
        t = t.to(d) if d is not None else t
        if token_first and t.dim() >= 3:  # same values, [B,T,H,.] memory behind a [B,H,T,.] view
            t = t.transpose(1, 2).contiguous().transpose(1, 2)
        return t.requires_grad_(True)

    q, k, v = dev(x["q"], dt), dev(x["k"], dt), dev(x["v"], dt)
    beta = dev(x["beta"])
    g = dev(x["g"]) if gate != "none" else None
    S0 = torch.from_numpy(x["S0"]).to(DEV).requires_grad_(True) if with_state else None
    cu_t = None if cu is None else torch.from_numpy(cu).to(DEV)
    if gate == "none":
        o, S = la.delta_rule_chunkwise(q, k, v, beta, S0, cu_seqlens=cu_t)
    elif gate == "scalar":
        o, S = la.gated_delta_rule_chunkwise(q, k, v, g, beta, None, S0, 64, l2, cu_seqlens=cu_t)
    else:
        o, S = la.kda_chunkwise(q, k, v, g, beta, None, S0, 64, l2, cu_seqlens=cu_t)
    dO = torch.from_numpy(x["dO"]).to(DEV)
    ((o.float() * dO).sum() + (S * torch.from_numpy(x["dS"]).to(DEV)).sum()).backward()
    tol = 2e-2 if bf16 else 1e-4
    errs = {"o": max_rel(o.detach().float().cpu().numpy(), o_ref) if T else 0.0, "S": max_rel(S.detach().cpu().numpy(), S_ref)}
    got = {"dq": q.grad, "dk": k.grad, "dv": v.grad, "dbeta": beta.grad}
    if g is not None:
        got["dg"] = g.grad
    for n, t in got.items():
        errs[n] = max_rel(t.float().cpu().numpy(), g_ref[n]) if T else 0.0
    if with_state:
        errs["dS0"] = max_rel(S0.grad.cpu().numpy(), dS0_ref)
    bad = {n: e for n, e in errs.items() if not e < tol}
    assert not bad, (bad, errs)
