"""Writes the golden fixtures of this directory from the fp64 CPU oracle.

    python tests/golden/make_fixtures.py

The reference holds no golden vectors for the delta-rule ops (its tests check
chunk == recurrent self-consistency only), so these files freeze the values of
the token-by-token fp64 restatement (``oracle.recurrent``: delta_net.py:162-213,
gated_deltanet.py:165-229, kda.py:215-283) and of its reverse recurrence
(``oracle.adjoint``).  Inputs and expected outputs are stored as fp32 ``.npz``
archives (no pickled objects).  Cases:

  deltanet / gated / kda   B1 H1 T80 (one full chunk + a 16-token tail), dk=dv=64,
                           random initial state, gradients for dO and dS_T
  deltanet_varlen          three packed sequences (20, 64 and 16 tokens), H1,
                           dk=dv=64, per-sequence initial states, gradients
  steps                    one decode token of each variant (B1 H2 dk=dv=64)

Inputs are pre-normalised (q, k unit rows), so every case is computed with
``use_qk_l2norm=False``.
"""
from __future__ import annotations

import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import adjoint, recurrent  # noqa: E402
from oracle.inputs import make_inputs  # noqa: E402

F = np.float32
CASES = {"deltanet": ("none", 101), "gated": ("scalar", 102), "kda": ("vector", 103)}


def _forward(gate, x, S0):
    if gate == "none":
        return recurrent.delta_rule_recurrent(x["q"], x["k"], x["v"], x["beta"], S0)
    fn = recurrent.gated_delta_rule_recurrent if gate == "scalar" else recurrent.kda_recurrent
    return fn(x["q"], x["k"], x["v"], x["g"], x["beta"], None, S0, False)


def dense_case(gate, seed, B=1, H=1, T=80, d=64):
    x = make_inputs(seed, B, H, T, d, d, gate=gate, with_state=True, with_grad=True)
    o, S = _forward(gate, x, x["S0"])
    gr = adjoint.delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], g=x.get("g"), dS_T=x["dS"],
                                    initial_state=x["S0"], use_qk_l2norm=False)
    out = {f"in_{n}": np.asarray(a, F) for n, a in x.items()}
    out.update(o=o.astype(F), S_T=S.astype(F))
    out.update({n: a.astype(F) for n, a in gr.items() if a is not None})
    return out


def varlen_case(seed=104, H=1, d=64, lens=(20, 64, 16)):
    cu = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
    T, nseq = int(cu[-1]), len(lens)
    x = make_inputs(seed, 1, H, T, d, d, gate="none", with_grad=True)
    rng = np.random.default_rng(seed + 1000)
    S0 = (rng.standard_normal((nseq, H, d, d)) * 0.02).astype(F)
    dS = (rng.standard_normal((nseq, H, d, d)) * 0.1).astype(F)
    o, S = recurrent.varlen(recurrent.delta_rule_recurrent, cu, x["q"], x["k"], x["v"], x["beta"], initial_state=S0)
    g = {n: [] for n in ("dq", "dk", "dv", "dbeta", "dS0")}
    for s in range(nseq):
        a, b = int(cu[s]), int(cu[s + 1])
        r = adjoint.delta_rule_adjoint(x["q"][:, :, a:b], x["k"][:, :, a:b], x["v"][:, :, a:b], x["beta"][:, :, a:b],
                                       x["dO"][:, :, a:b], dS_T=dS[s:s + 1], initial_state=S0[s:s + 1])
        for n in g:
            g[n].append(r[n])
    out = {f"in_{n}": np.asarray(x[n], F) for n in ("q", "k", "v", "beta", "dO")}
    out.update(in_S0=S0, in_dS=dS, in_cu_seqlens=cu, o=o.astype(F), S_T=S.astype(F))
    for n in ("dq", "dk", "dv", "dbeta"):
        out[n] = np.concatenate(g[n], axis=2).astype(F)
    out["dS0"] = np.concatenate(g["dS0"], axis=0).astype(F)
    return out


def step_case(seed=105, B=1, H=2, d=64):
    out = {}
    for name, (gate, _) in CASES.items():
        x = make_inputs(seed, B, H, 1, d, d, gate=gate, with_state=True)
        q, k, v, beta = x["q"][:, :, 0], x["k"][:, :, 0], x["v"][:, :, 0], x["beta"][:, :, 0]
        if gate == "none":
            o, S = recurrent.delta_rule_step(q, k, v, beta, x["S0"])
        else:
            fn = recurrent.gated_delta_rule_step if gate == "scalar" else recurrent.kda_step
            o, S = fn(q, k, v, x["g"][:, :, 0], beta, x["S0"], None, False)
            out[f"{name}_in_g"] = x["g"][:, :, 0].astype(F)
        out.update({f"{name}_in_q": q, f"{name}_in_k": k, f"{name}_in_v": v, f"{name}_in_beta": beta,
                    f"{name}_in_S0": x["S0"], f"{name}_o": o.astype(F), f"{name}_S": S.astype(F)})
    return out


def main():
    for name, (gate, seed) in CASES.items():
        np.savez(os.path.join(HERE, f"{name}_B1H1T80d64.npz"), **dense_case(gate, seed))
    np.savez(os.path.join(HERE, "deltanet_varlen_3seq_T100d64.npz"), **varlen_case())
    np.savez(os.path.join(HERE, "steps_B1H2d64.npz"), **step_case())
    for f in sorted(os.listdir(HERE)):
        if f.endswith(".npz"):
            print(f, os.path.getsize(os.path.join(HERE, f)), "bytes")


if __name__ == "__main__":
    main()
