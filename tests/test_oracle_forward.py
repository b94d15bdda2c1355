"""Pins the forward oracle without the reference: closed forms, brute-force matrix
products, reductions between variants, chunk == recurrent, invariances.

Each check is chosen so that a plausible slip (dropped decay, beta applied twice, wrong
mask, transposed state) breaks it.  Reference tests these extend are cited inline.
"""
import numpy as np
import pytest

from oracle import chunkwise as ch
from oracle import recurrent as rc
from oracle.inputs import make_inputs
from conftest import max_rel


def _brute_states(q, k, v, beta, alpha, S0, scale):
    """S_t = (I - beta k k^T) diag(alpha) S_{t-1} + beta k v^T  (delta_net.py:28-29,
    gated_deltanet.py:31-32), written with explicit matrices for one head."""
    T, dk = k.shape
    S = S0.copy()
    outs = []
    for t in range(T):
        kt = k[t][:, None]
        S = (np.eye(dk) - beta[t] * kt @ kt.T) @ (np.diag(alpha[t]) @ S) + beta[t] * kt @ v[t][None, :]
        outs.append((scale * q[t][None, :] @ S)[0])
    return np.array(outs), S


@pytest.mark.parametrize("gate", ["none", "scalar", "vector"])
def test_recurrent_matches_explicit_matrix_form(gate):
    rng = np.random.default_rng(0)
    T, dk, dv = 7, 4, 3
    q, k, v = rng.standard_normal((T, dk)), rng.standard_normal((T, dk)), rng.standard_normal((T, dv))
    beta = rng.uniform(0.1, 0.9, T)
    S0 = rng.standard_normal((dk, dv))
    if gate == "none":
        alpha = np.ones((T, dk))
        o, S = rc.delta_rule_recurrent(q[None, None], k[None, None], v[None, None], beta[None, None], S0[None, None])
    elif gate == "scalar":
        g = -rng.uniform(0, 1, T)
        alpha = np.exp(g)[:, None] * np.ones((T, dk))
        o, S = rc.gated_delta_rule_recurrent(q[None, None], k[None, None], v[None, None], g[None, None],
                                              beta[None, None], None, S0[None, None], use_qk_l2norm=False)
    else:
        g = -rng.uniform(0, 1, (T, dk))
        alpha = np.exp(g)
        o, S = rc.kda_recurrent(q[None, None], k[None, None], v[None, None], g[None, None], beta[None, None],
                                None, S0[None, None], use_qk_l2norm=False)
    o_ref, S_ref = _brute_states(q, k, v, beta, alpha, S0, dk ** -0.5)
    assert np.allclose(o[0, 0], o_ref, rtol=1e-12, atol=1e-12)
    assert np.allclose(S[0, 0], S_ref, rtol=1e-12, atol=1e-12)


def test_beta_zero_keeps_decayed_state():
    # extends tests/test_deltanet.py:281-297 (beta=0 => state stays 0) to S0 != 0 with decay
    x = make_inputs(1, 1, 2, 6, 4, 4, gate="scalar", with_state=True)
    beta = np.zeros_like(x["beta"])
    o, S = rc.gated_delta_rule_recurrent(x["q"], x["k"], x["v"], x["g"], beta, None, x["S0"], use_qk_l2norm=False)
    Gc = np.cumsum(x["g"].astype(np.float64), -1)
    assert np.allclose(S, x["S0"] * np.exp(Gc[..., -1])[..., None, None], rtol=1e-12)
    o_ref = 0.5 * np.einsum("bhtk,bhkv->bhtv", x["q"].astype(np.float64), x["S0"].astype(np.float64)) * np.exp(Gc)[..., None]
    assert np.allclose(o, o_ref, rtol=1e-10, atol=1e-14)
    o0, S0 = rc.delta_rule_recurrent(x["q"], x["k"], x["v"], beta)
    assert np.all(S0 == 0) and np.all(o0 == 0)


def test_orthonormal_keys_store_and_retrieve():
    # setup of tests/test_deltanet.py:330-346; closed form S_T = V, o_t = dk^-1/2 v_t
    dk = dv = 4
    k = np.eye(dk)[None, None]
    v = np.random.default_rng(0).standard_normal((1, 1, dk, dv))
    o, S = rc.delta_rule_recurrent(k.copy(), k, v, np.ones((1, 1, dk)))
    assert np.allclose(S[0, 0], v[0, 0], atol=1e-14)
    assert np.allclose(o, dk ** -0.5 * v, atol=1e-14)


def test_single_token_closed_form():
    # T=1, S0=0: o = scale * beta * <q,k> * v
    x = {n: a.astype(np.float64) for n, a in make_inputs(2, 2, 3, 1, 8, 5).items()}
    o, S = rc.delta_rule_recurrent(x["q"], x["k"], x["v"], x["beta"])
    qk = np.sum(x["q"].astype(np.float64) * x["k"], -1)
    assert np.allclose(o, 8 ** -0.5 * (x["beta"] * qk)[..., None] * x["v"], rtol=1e-12)
    assert np.allclose(S, np.einsum("bhk,bhv->bhkv", x["k"][:, :, 0], x["beta"][:, :, 0, None] * x["v"][:, :, 0]), rtol=1e-12)


def test_steps_equal_recurrent_T1():
    # tests/test_deltanet.py:134-157, test_gated_deltanet.py:310-339, test_kda.py:219-250
    x = make_inputs(3, 2, 4, 1, 16, 32, gate="vector", with_state=True, normalize=False)
    sq = lambda a: a[:, :, 0]
    o1, S1 = rc.kda_recurrent(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["S0"])
    o2, S2 = rc.kda_step(sq(x["q"]), sq(x["k"]), sq(x["v"]), sq(x["g"]), sq(x["beta"]), x["S0"])
    assert np.array_equal(o1[:, :, 0], o2) and np.array_equal(S1, S2)
    gs = x["g"][..., 0]
    o1, S1 = rc.gated_delta_rule_recurrent(x["q"], x["k"], x["v"], gs, x["beta"], None, x["S0"])
    o2, S2 = rc.gated_delta_rule_step(sq(x["q"]), sq(x["k"]), sq(x["v"]), sq(gs), sq(x["beta"])[..., None], x["S0"])
    assert np.array_equal(o1[:, :, 0], o2) and np.array_equal(S1, S2)
    o1, S1 = rc.delta_rule_recurrent(x["q"], x["k"], x["v"], x["beta"], x["S0"])
    o2, S2 = rc.delta_rule_step(sq(x["q"]), sq(x["k"]), sq(x["v"]), sq(x["beta"]), x["S0"])
    assert np.array_equal(o1[:, :, 0], o2) and np.array_equal(S1, S2)


def test_variant_reductions():
    """gated(g=0, no l2norm) == deltanet; kda(g constant over dk) == gated."""
    x = make_inputs(4, 2, 2, 20, 8, 6, gate="scalar", with_state=True)
    a = rc.delta_rule_recurrent(x["q"], x["k"], x["v"], x["beta"], x["S0"])
    b = rc.gated_delta_rule_recurrent(x["q"], x["k"], x["v"], np.zeros_like(x["g"]), x["beta"], None, x["S0"], False)
    assert np.allclose(a[0], b[0], rtol=1e-13) and np.allclose(a[1], b[1], rtol=1e-13)
    c = rc.gated_delta_rule_recurrent(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["S0"])
    gv = np.repeat(x["g"][..., None], 8, -1)
    d = rc.kda_recurrent(x["q"], x["k"], x["v"], gv, x["beta"], None, x["S0"])
    assert np.allclose(c[0], d[0], rtol=1e-12, atol=1e-15) and np.allclose(c[1], d[1], rtol=1e-12, atol=1e-15)


def test_l2norm_flag_equals_prenormalised_inputs():
    x = make_inputs(5, 1, 2, 9, 8, 4, gate="scalar", normalize=False)
    a = rc.gated_delta_rule_recurrent(x["q"], x["k"], x["v"], x["g"], x["beta"], use_qk_l2norm=True)
    qn, kn = rc.l2norm(x["q"].astype(np.float64)), rc.l2norm(x["k"].astype(np.float64))
    b = rc.gated_delta_rule_recurrent(qn, kn, x["v"], x["g"], x["beta"], use_qk_l2norm=False)
    assert np.allclose(a[0], b[0], rtol=1e-13) and np.allclose(a[1], b[1], rtol=1e-13)


CASES = [("none", 32, 16, 32, 8), ("none", 100, 16, 8, 32), ("scalar", 64, 16, 32, 32),
         ("scalar", 50, 8, 8, 32), ("vector", 64, 8, 8, 64), ("vector", 70, 16, 8, 16)]


@pytest.mark.parametrize("gate,T,dk,dv,C", CASES)
def test_chunk_equals_recurrent_fp64(gate, T, dk, dv, C):
    # the reference's own idea (tests/test_deltanet.py:64-90, test_kda.py:252-290) at 1e-10
    # instead of 1e-3, incl. T not a multiple of C (test_gated_deltanet.py:229-247, numeric here)
    x = make_inputs(6, 2, 2, T, dk, dv, gate=gate, with_state=True)
    if gate == "none":
        a = rc.delta_rule_recurrent(x["q"], x["k"], x["v"], x["beta"], x["S0"])
        b = ch.delta_rule_chunkwise(x["q"], x["k"], x["v"], x["beta"], x["S0"], chunk_size=C)
    elif gate == "scalar":
        a = rc.gated_delta_rule_recurrent(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["S0"])
        b = ch.gated_delta_rule_chunkwise(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["S0"], C)
    else:
        a = rc.kda_recurrent(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["S0"])
        b = ch.kda_chunkwise(x["q"], x["k"], x["v"], x["g"], x["beta"], None, x["S0"], C)
    assert max_rel(b[0], a[0]) < 1e-10 and max_rel(b[1], a[1]) < 1e-10


def test_chunk_strong_decay_is_finite_and_exact():
    # gates down to -10 per token (bench_kda_kernels.py:123-129): exp(-G) would overflow,
    # the blocked form must not
    x = make_inputs(7, 1, 2, 64, 8, 8, gate="vector")
    g = -np.random.default_rng(7).uniform(0, 10, x["g"].shape)
    a = rc.kda_recurrent(x["q"], x["k"], x["v"], g, x["beta"])
    b = ch.kda_chunkwise(x["q"], x["k"], x["v"], g, x["beta"])
    assert np.isfinite(b[0]).all() and max_rel(b[0], a[0]) < 1e-10 and max_rel(b[1], a[1]) < 1e-9


def test_chunk_fp32_close_to_fp64():
    x = make_inputs(8, 2, 2, 128, 16, 16, gate="scalar")
    a = rc.gated_delta_rule_recurrent(x["q"], x["k"], x["v"], x["g"], x["beta"])
    b = ch.gated_delta_rule_chunkwise(x["q"], x["k"], x["v"], x["g"], x["beta"], dtype=np.float32)
    assert max_rel(b[0], a[0]) < 1e-5 and max_rel(b[1], a[1]) < 1e-5


def test_split_invariance_and_varlen():
    x = make_inputs(9, 1, 2, 90, 8, 8, gate="scalar")
    full = rc.gated_delta_rule_recurrent(x["q"], x["k"], x["v"], x["g"], x["beta"])
    cut = 37
    h = lambda a, s: a[:, :, s]
    o1, S1 = rc.gated_delta_rule_recurrent(*(h(x[n], slice(0, cut)) for n in ("q", "k", "v", "g", "beta")))
    o2, S2 = rc.gated_delta_rule_recurrent(*(h(x[n], slice(cut, None)) for n in ("q", "k", "v", "g", "beta")), None, S1)
    assert np.allclose(np.concatenate([o1, o2], 2), full[0], rtol=1e-13) and np.allclose(S2, full[1], rtol=1e-13)
    cu = np.array([0, 37, 90], np.int32)
    o, S = rc.varlen(lambda q, k, v, g, b, initial_state=None: rc.gated_delta_rule_recurrent(q, k, v, g, b, None, initial_state),
                     cu, x["q"], x["k"], x["v"], x["g"], x["beta"])
    assert np.allclose(o[:, :, :37], o1) and S.shape == (2, 2, 8, 8) and np.allclose(S[0], S1[0])
    assert not np.allclose(o[:, :, 37:], o2)  # second sequence restarts from zero state


def test_chunk_size_must_divide_16():
    # gated_deltanet.py:318-320, kda.py:438-440
    x = make_inputs(10, 1, 1, 24, 8, 8, gate="scalar")
    with pytest.raises(ValueError):
        ch.gated_delta_rule_chunkwise(x["q"], x["k"], x["v"], x["g"], x["beta"], chunk_size=24)
