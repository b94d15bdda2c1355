"""Pins oracle/conv.py without the reference: a textbook FIR filter (scipy), a brute-force loop, the
reference's own incremental-equals-whole property (tests/test_comprehensive.py:57-83), finite differences
and an independent torch conv1d + autograd."""
import numpy as np
import pytest
import scipy.signal
import torch

from oracle import conv as oc


def _data(seed, B, T, D, K, with_cache=True):
    r = np.random.default_rng(seed)
    x = r.standard_normal((B, T, D))
    w = r.standard_normal((K, D)) * 0.5
    b = r.standard_normal(D) * 0.1
    c = r.standard_normal((B, K - 1, D)) if with_cache else None
    return x, w, b, c


@pytest.mark.parametrize("K", [2, 3, 4])
def test_equals_fir_filter(K):
    x, w, b, _ = _data(1, 2, 19, 5, K, False)
    y, cache = oc.depthwise_conv1d_causal(x, w, b)
    for d in range(5):  # y[t] = sum_j w[j] x[t-(K-1)+j]: an FIR filter whose taps are w reversed
        ref = scipy.signal.lfilter(w[::-1, d], [1.0], x[:, :, d], axis=1) + b[d]
        assert np.allclose(y[:, :, d], ref, atol=1e-12)
    assert cache.shape == (2, K - 1, 5)
    assert np.array_equal(cache, x[:, 19 - (K - 1):])


def test_width_one_kernel_is_identity_plus_bias():
    """conv.py:39-44 returns inputs + bias for kernel_size 1 and never reads the weight; the cache is empty."""
    x, w, b, _ = _data(1, 2, 19, 5, 1, False)
    y, cache = oc.depthwise_conv1d_causal(x, w, b)
    assert np.array_equal(y, x + b) and cache.shape == (2, 0, 5)
    dy = np.random.default_rng(9).standard_normal(x.shape)
    dx, dw, db = oc.depthwise_conv1d_causal_grad(x, w, b, dy)
    assert np.array_equal(dx, dy) and not dw.any() and np.allclose(db, dy.sum((0, 1)))


def test_cache_gradient_finite_differences():
    x, w, b, c = _data(10, 2, 5, 3, 4)
    dy = np.random.default_rng(11).standard_normal(x.shape)
    for T in (5, 2):  # also a sequence shorter than the cache
        dc = oc.depthwise_conv1d_causal_grad(x[:, :T], w, b, dy[:, :T], c, "silu", with_cache=True)[3]
        f = lambda c_: (oc.depthwise_conv1d_causal(x[:, :T], w, b, c_, "silu")[0] * dy[:, :T]).sum()
        for i in np.ndindex(c.shape):
            p, m = c.copy(), c.copy()
            p[i] += 1e-6
            m[i] -= 1e-6
            assert abs((f(p) - f(m)) / 2e-6 - dc[i]) < 1e-6


def test_packed_helper_is_one_call_per_sequence():
    x, w, b, _ = _data(12, 1, 11, 3, 3, False)
    cu = [0, 4, 4, 9, 11]
    y, = oc.packed(lambda x_: (oc.depthwise_conv1d_causal(x_, w, b, None, "silu")[0],), cu, x)
    for a, e in zip(cu[:-1], cu[1:]):
        assert np.array_equal(y[:, a:e], oc.depthwise_conv1d_causal(x[:, a:e], w, b, None, "silu")[0])


def test_brute_force_with_cache_and_silu():
    x, w, b, c = _data(2, 2, 7, 3, 4)
    y, cache = oc.depthwise_conv1d_causal(x, w, b, c, "silu")
    xin = np.concatenate([c, x], 1)
    for bb in range(2):
        for t in range(7):
            for d in range(3):
                z = b[d] + sum(w[j, d] * xin[bb, t + j, d] for j in range(4))
                assert abs(y[bb, t, d] - z / (1 + np.exp(-z))) < 1e-12
    assert np.array_equal(cache, xin[:, -3:])


@pytest.mark.parametrize("K", [2, 4])
def test_incremental_equals_whole_sequence(K):
    x, w, b, _ = _data(3, 2, 8, 6, K, False)
    full, full_cache = oc.depthwise_conv1d_causal(x, w, b, None, "silu")
    cache = np.zeros((2, K - 1, 6))
    outs = []
    for t in range(8):
        o, cache = oc.depthwise_conv1d_causal(x[:, t:t + 1], w, b, cache, "silu")
        outs.append(o)
    assert np.allclose(np.concatenate(outs, 1), full, atol=1e-13) and np.array_equal(cache, full_cache)
    # a sequence shorter than the cache keeps the tail of the old cache (conv.py:67)
    _, c2 = oc.depthwise_conv1d_causal(x[:, :1], w, b, full_cache)
    assert np.array_equal(c2, np.concatenate([full_cache, x[:, :1]], 1)[:, -(K - 1):])


def test_shape_errors():
    x, w, b, _ = _data(4, 1, 4, 2, 3, False)
    with pytest.raises(ValueError):
        oc.depthwise_conv1d_causal(x, w, b, np.zeros((1, 3, 2)))
    with pytest.raises(ValueError):
        oc.depthwise_conv1d_causal(x, np.zeros((0, 2)), b)


@pytest.mark.parametrize("act", [None, "silu"])
def test_gradient_finite_differences(act):
    x, w, b, c = _data(5, 2, 6, 3, 4)
    dy = np.random.default_rng(6).standard_normal(x.shape)
    dx, dw, db = oc.depthwise_conv1d_causal_grad(x, w, b, dy, c, act)
    f = lambda x_, w_, b_: (oc.depthwise_conv1d_causal(x_, w_, b_, c, act)[0] * dy).sum()
    eps = 1e-6
    for arr, grad, which in ((x, dx, 0), (w, dw, 1), (b, db, 2)):
        it = np.nditer(arr, flags=["multi_index"])
        for _ in it:
            i = it.multi_index
            p, m = arr.copy(), arr.copy()
            p[i] += eps
            m[i] -= eps
            args_p = [x, w, b]
            args_m = [x, w, b]
            args_p[which], args_m[which] = p, m
            assert abs((f(*args_p) - f(*args_m)) / (2 * eps) - grad[i]) < 1e-6


@pytest.mark.parametrize("act", [None, "silu"])
def test_gradient_torch_conv1d_autograd(act):
    x, w, b, _ = _data(7, 3, 33, 8, 4, False)
    dy = np.random.default_rng(8).standard_normal(x.shape)
    tx, tw, tb = (torch.tensor(a, dtype=torch.float64, requires_grad=True) for a in (x, w, b))
    z = torch.nn.functional.conv1d(torch.nn.functional.pad(tx.transpose(1, 2), (3, 0)), tw.t()[:, None, :], tb, groups=8)
    z = z.transpose(1, 2)
    y = torch.nn.functional.silu(z) if act else z
    (y * torch.tensor(dy)).sum().backward()
    y0, _ = oc.depthwise_conv1d_causal(x, w, b, None, act)
    dx, dw, db = oc.depthwise_conv1d_causal_grad(x, w, b, dy, None, act)
    assert np.allclose(y0, y.detach().numpy(), atol=1e-12)
    for got, ref in ((dx, tx.grad), (dw, tw.grad), (db, tb.grad)):
        assert np.allclose(got, ref.numpy(), atol=1e-10)
