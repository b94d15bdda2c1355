"""GPU parity of the causal depthwise convolution kernels against the fp64 oracle, through the C-ABI.
Tolerances as max|x - ref| / max|ref|: 1e-5 (fp32) / 2e-2 (bf16 storage, fp32 arithmetic)."""
import numpy as np
import pytest
import torch

from oracle import conv as oc
from oracle.inputs import to_bf16_grid
from conftest import max_rel

pytestmark = pytest.mark.gpu
DEV = "cuda"


def _data(seed, B, T, D, K, bf16, with_cache=True, with_bias=True):
    r = np.random.default_rng(seed)
    rnd = (lambda a: to_bf16_grid(a.astype(np.float32))) if bf16 else (lambda a: a.astype(np.float32))
    x = rnd(r.standard_normal((B, T, D)))
    w = (r.standard_normal((K, D)) * 0.5).astype(np.float32)
    b = (r.standard_normal(D) * 0.1).astype(np.float32) if with_bias else None
    c = rnd(r.standard_normal((B, K - 1, D))) if with_cache else None
    dy = rnd(r.standard_normal((B, T, D)))
    return x, w, b, c, dy


def _t(a, dt=None, grad=False):
    if a is None:
        return None
    t = torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    if dt is not None:
        t = t.to(dt)
    return t.requires_grad_(grad)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("act", [None, "silu"])
@pytest.mark.parametrize("shape", [(2, 16, 32, 4), (1, 100, 520, 4), (3, 65, 64, 3), (2, 1, 128, 4), (1, 2, 8, 4),
                                   (2, 200, 24, 2), (1, 31, 16, 1), (2, 257, 1024, 4)])
def test_forward_backward_match_oracle(shape, act, bf16):
    import linearnexus_amd as la
    B, T, D, K = shape
    x, w, b, c, dy = _data(31, B, T, D, K, bf16, with_cache=K > 1)
    dt = torch.bfloat16 if bf16 else torch.float32
    y_ref, c_ref = oc.depthwise_conv1d_causal(x, w, b, c, act)
    dx_ref, dw_ref, db_ref = oc.depthwise_conv1d_causal_grad(x, w, b, dy, c, act)
    tx, tw, tb = _t(x, dt, True), _t(w, None, True), _t(b, None, True)
    y, nc = la.depthwise_conv1d_causal(tx, tw, tb, cache=_t(c, dt), activation=act)
    assert y.dtype == dt and y.shape == (B, T, D) and nc.shape == (B, K - 1, D) and nc.dtype == dt
    (y.float() * _t(dy)).sum().backward()
    tol = 2e-2 if bf16 else 1e-5
    assert max_rel(y.detach().float().cpu().numpy(), y_ref) < tol
    if K > 1:
        assert np.array_equal(nc.float().cpu().numpy(), c_ref.astype(np.float32))  # the carry is a copy: exact
    assert max_rel(tx.grad.float().cpu().numpy(), dx_ref) < tol
    assert max_rel(tw.grad.cpu().numpy(), dw_ref) < (1e-4 if not bf16 else 2e-2)
    assert max_rel(tb.grad.cpu().numpy(), db_ref) < (1e-4 if not bf16 else 2e-2)


def test_no_bias_no_cache_and_reference_test_shapes():
    # tests/test_comprehensive.py:30-55: B2 T16 D32 K4, output and cache shapes, gradients exist
    import linearnexus_amd as la
    x, w, _, _, dy = _data(32, 2, 16, 32, 4, False, with_cache=False, with_bias=False)
    tx, tw = _t(x, None, True), _t(w, None, True)
    y, cache = la.depthwise_conv1d_causal(tx, tw, None)
    assert y.shape == (2, 16, 32) and cache.shape == (2, 3, 32)
    (y * _t(dy)).sum().backward()
    y_ref, c_ref = oc.depthwise_conv1d_causal(x, w)
    dx_ref, dw_ref, _ = oc.depthwise_conv1d_causal_grad(x, w, None, dy)
    assert max_rel(y.detach().cpu().numpy(), y_ref) < 1e-5 and np.array_equal(cache.cpu().numpy(), c_ref.astype(np.float32))
    assert max_rel(tx.grad.cpu().numpy(), dx_ref) < 1e-5 and max_rel(tw.grad.cpu().numpy(), dw_ref) < 1e-4


@pytest.mark.parametrize("inplace", [False, True])
def test_incremental_steps_equal_whole_sequence(inplace):
    # tests/test_comprehensive.py:57-83, with the fused SiLU and, optionally, the cache updated in place
    import linearnexus_amd as la
    x, w, b, _, _ = _data(33, 2, 8, 32, 4, True, with_cache=False)
    tx, tw, tb = _t(x, torch.bfloat16), _t(w), _t(b)
    full, full_cache = la.depthwise_conv1d_causal(tx, tw, tb, activation="silu")
    cache = torch.zeros(2, 3, 32, dtype=torch.bfloat16, device=DEV)
    ptr = cache.data_ptr()
    outs = []
    for t in range(8):
        o, cache = la.depthwise_conv1d_causal(tx[:, t:t + 1], tw, tb, cache=cache, activation="silu", inplace_cache=inplace)
        assert (cache.data_ptr() == ptr) == inplace
        outs.append(o)
    assert torch.equal(torch.cat(outs, 1), full) and torch.equal(cache, full_cache)
    y_ref, _ = oc.depthwise_conv1d_causal(x, w, b, None, "silu")
    assert max_rel(full.float().cpu().numpy(), y_ref) < 2e-2


def test_errors_and_empty_sequence():
    import linearnexus_amd as la
    x = torch.randn(2, 4, 16, device=DEV)
    w = torch.randn(4, 16, device=DEV)
    with pytest.raises(ValueError):  # conv.py:49-53
        la.depthwise_conv1d_causal(x, w, None, cache=torch.zeros(2, 2, 16, device=DEV))
    with pytest.raises(ValueError):  # conv.py:36-37
        la.depthwise_conv1d_causal(x, torch.zeros(0, 16, device=DEV), None)
    with pytest.raises(RuntimeError):
        la.depthwise_conv1d_causal(x.cpu(), w, None)
    with pytest.raises(RuntimeError):
        la.depthwise_conv1d_causal(torch.randn(2, 4, 6, device=DEV), torch.randn(4, 6, device=DEV), None)  # D % 4
    c = torch.randn(2, 3, 16, device=DEV)
    y, nc = la.depthwise_conv1d_causal(x[:, :0], w, None, cache=c)
    assert y.shape == (2, 0, 16) and torch.equal(nc, c)


def test_full_size_linearity_and_shift():
    """Size-independent properties at a full layer's size (B8 T4096 D6144 bf16, no activation): the kernel is
    linear in x, and an impulse at token t0 comes out as the taps, reversed, at t0 .. t0+3."""
    import linearnexus_amd as la
    B, T, D = 8, 4096, 6144
    torch.manual_seed(0)
    w = torch.randn(4, D, device=DEV)
    x = torch.zeros(B, T, D, device=DEV, dtype=torch.bfloat16)
    x[:, 100] = 1.0
    x[:, T - 2] = 1.0
    y, cache = la.depthwise_conv1d_causal(x, w, None)
    wb = w.bfloat16()
    for j in range(4):
        assert torch.equal(y[:, 100 + j], wb[3 - j].expand(B, D))
    assert torch.equal(y[:, T - 2], wb[3].expand(B, D)) and torch.equal(y[:, T - 1], wb[2].expand(B, D))
    assert torch.count_nonzero(y[:, :100]) == 0 and torch.count_nonzero(y[:, 104:T - 2]) == 0
    assert torch.equal(cache[:, 1], torch.ones(B, D, device=DEV, dtype=torch.bfloat16)) and torch.count_nonzero(cache[:, 2]) == 0


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("act", [None, "silu"])
@pytest.mark.parametrize("case", [(300, 64, 4, [0, 64, 65, 65, 200, 300]), (40, 32, 3, [0, 1, 2, 3, 40]),
                                  (1000, 520, 4, [0, 31, 33, 500, 1000]), (130, 16, 2, [0, 130]),
                                  (100, 32, 4, [0, 100, 100]),      # empty last sequence: the carry out is zero
                                  (100, 32, 4, [0, 98, 98, 100]),   # last sequence shorter than K - 1, behind an empty one
                                  (66, 16, 3, [0, 65, 66])])
def test_packed_batch_equals_one_call_per_sequence(case, act, bf16):
    """Packed batches: the taps stop at sequence boundaries -- outputs and all gradients equal the oracle applied to
    every sequence on its own with a zero cache (sequences of 0, 1 and 2 tokens, boundaries inside a thread's run)."""
    import linearnexus_amd as la
    T, D, K, cu = case
    x, w, b, _, dy = _data(41, 1, T, D, K, bf16, with_cache=False)
    dt = torch.bfloat16 if bf16 else torch.float32
    y_ref, = oc.packed(lambda x_: (oc.depthwise_conv1d_causal(x_, w, b, None, act)[0],), cu, x)
    dx_ref, dw_ref, db_ref = oc.packed(lambda x_, dy_: oc.depthwise_conv1d_causal_grad(x_, w, b, dy_, None, act), cu, x, dy)
    tx, tw, tb = _t(x, dt, True), _t(w, None, True), _t(b, None, True)
    y, nc = la.depthwise_conv1d_causal(tx, tw, tb, activation=act, cu_seqlens=torch.tensor(cu, dtype=torch.int32))
    (y.float() * _t(dy)).sum().backward()
    tol = 2e-2 if bf16 else 1e-5
    assert max_rel(y.detach().float().cpu().numpy(), y_ref) < tol
    assert max_rel(tx.grad.float().cpu().numpy(), dx_ref) < tol
    assert max_rel(tw.grad.cpu().numpy(), dw_ref) < (1e-4 if not bf16 else 2e-2)
    assert max_rel(tb.grad.cpu().numpy(), db_ref) < (1e-4 if not bf16 else 2e-2)
    # the carry that leaves is that of the last sequence
    last = x[:, cu[-2]:]
    c_ref = np.concatenate([np.zeros((1, K - 1, D), np.float32), last], 1)[:, -(K - 1):]
    assert np.array_equal(nc.float().cpu().numpy(), c_ref)
    with pytest.raises(ValueError):
        la.depthwise_conv1d_causal(tx, tw, tb, cu_seqlens=[0, 5, 3, T])
    with pytest.raises(RuntimeError):
        la.depthwise_conv1d_causal(tx, tw, tb, cache=torch.zeros(1, K - 1, D, device=DEV, dtype=dt), cu_seqlens=cu)


@pytest.mark.parametrize("bf16", [False, True])
@pytest.mark.parametrize("shape", [(2, 16, 32, 4), (3, 2, 64, 4), (2, 1, 16, 3), (1, 70, 520, 2)])
def test_gradient_of_the_carry_in_cache(shape, bf16):
    import linearnexus_amd as la
    B, T, D, K = shape
    x, w, b, c, dy = _data(42, B, T, D, K, bf16)
    dt = torch.bfloat16 if bf16 else torch.float32
    dc_ref = oc.depthwise_conv1d_causal_grad(x, w, b, dy, c, "silu", with_cache=True)[3]
    tc = _t(c, dt, True)
    y, _ = la.depthwise_conv1d_causal(_t(x, dt, True), _t(w), _t(b), cache=tc, activation="silu")
    (y.float() * _t(dy)).sum().backward()
    assert max_rel(tc.grad.float().cpu().numpy(), dc_ref) < (2e-2 if bf16 else 1e-5)


def test_width_one_kernel_and_empty_sequence_without_cache():
    """conv.py:39-44: kernel_size 1 is inputs + bias, whatever the weight holds.  An empty sequence with no cache hands
    back the zero cache the reference builds (conv.py:46-47)."""
    import linearnexus_amd as la
    x = torch.randn(2, 9, 16, device=DEV, requires_grad=True)
    w = torch.full((1, 16), 3.0, device=DEV, requires_grad=True)
    b = torch.randn(16, device=DEV)
    y, nc = la.depthwise_conv1d_causal(x, w, b)
    assert torch.allclose(y, x + b, atol=1e-6) and nc.shape == (2, 0, 16)
    y.sum().backward()
    assert torch.allclose(x.grad, torch.ones_like(x)) and torch.count_nonzero(w.grad) == 0
    y, nc = la.depthwise_conv1d_causal(torch.randn(2, 0, 16, device=DEV), torch.randn(4, 16, device=DEV), None)
    assert y.shape == (2, 0, 16) and nc.shape == (2, 3, 16) and torch.count_nonzero(nc) == 0
