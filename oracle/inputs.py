"""Shared synthetic inputs for oracle, tests and benchmark (numpy ``default_rng``).

TEST INFRASTRUCTURE.  One generator feeds the oracle and the HIP kernels the same
values.  Distributions follow the benchmark configurations: q, k ~ N(0,1) then
``x / (||x|| + 1e-6)`` in fp32 (the caller-side normalisation of
linearnexus/modules/linear_attn/delta_net.py:571-575), v ~ N(0,1),
beta = sigmoid(N(0,1)) (delta_net.py:654-655), scalar gate
``g = -softplus(N(0,1)) * 0.1`` and vector gate ``-softplus(N(0,1)) * 0.05``
(shapes of gated_deltanet.py:811-815 and kda.py:153-165), S0 ~ N(0, 0.02).
"""

from __future__ import annotations

import numpy as np

from .recurrent import l2norm


def _sigmoid(x):
    return 1.0 / (1.0 + np.exp(-x))


def _softplus(x):
    return np.log1p(np.exp(-np.abs(x))) + np.maximum(x, 0)


def make_inputs(seed, B, H, T, dk, dv, gate="none", with_state=False, with_grad=False,
                gate_scale=None, normalize=True):
    """Returns a dict of fp32 arrays: q,k,v,beta[,g][,S0][,dO,dS]."""
    rng = np.random.default_rng(seed)
    f = np.float32
    q = rng.standard_normal((B, H, T, dk), dtype=f)
    k = rng.standard_normal((B, H, T, dk), dtype=f)
    if normalize:
        q, k = l2norm(q), l2norm(k)
    v = rng.standard_normal((B, H, T, dv), dtype=f)
    beta = _sigmoid(rng.standard_normal((B, H, T), dtype=f)).astype(f)
    out = {"q": q, "k": k, "v": v, "beta": beta}
    if gate == "scalar":
        s = 0.1 if gate_scale is None else gate_scale
        out["g"] = (-_softplus(rng.standard_normal((B, H, T), dtype=f)) * s).astype(f)
    elif gate == "vector":
        s = 0.05 if gate_scale is None else gate_scale
        out["g"] = (-_softplus(rng.standard_normal((B, H, T, dk), dtype=f)) * s).astype(f)
    elif gate != "none":
        raise ValueError(gate)
    if with_state:
        out["S0"] = (rng.standard_normal((B, H, dk, dv), dtype=f) * 0.02).astype(f)
    if with_grad:
        out["dO"] = rng.standard_normal((B, H, T, dv), dtype=f)
        out["dS"] = (rng.standard_normal((B, H, dk, dv), dtype=f) * 0.1).astype(f)
    return out


def make_cu_seqlens(seed, nseq, total, lo, hi, max_tries=1000):
    """``nseq`` lengths uniform in [lo, hi], deterministically adjusted to sum to ``total``."""
    rng = np.random.default_rng(seed)
    for _ in range(max_tries):
        lens = rng.integers(lo, hi + 1, size=nseq).astype(np.int64)
        lens = np.floor(lens * (total / lens.sum())).astype(np.int64)
        lens[-1] += total - lens.sum()
        if lens.min() >= lo and lens.max() <= hi:
            return np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    raise RuntimeError("could not draw sequence lengths in range")


def to_bf16_grid(x):
    """Round fp32 to the nearest bf16 value (ties to even), returned as fp32."""
    u = np.ascontiguousarray(x, np.float32).view(np.uint32)
    r = ((u >> 16) & 1) + 0x7FFF
    return ((u + r) & 0xFFFF0000).astype(np.uint32).view(np.float32)
