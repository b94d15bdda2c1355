"""The chunk op saves what its backward reads only when a gradient can be asked for: leaves that require grad under
torch.no_grad() (evaluation of a model in training mode) must take the forward-only kernels."""
import torch

from linearnexus_amd import linear_attn as la


def _run(monkeypatch, grad_mode, requires_grad):
    seen = []

    def fake_forward(q, k, v, g, beta, initial_state, scale, l2norm, o_dtype, cu_seqlens, forward_only, raw_gate=None):
        seen.append(forward_only)
        B, H, T, dk = q.shape
        return q.new_zeros(B, H, T, v.shape[-1]), q.new_zeros(B, H, dk, v.shape[-1]), (), None

    monkeypatch.setattr(la, "_chunk_forward", fake_forward)
    q, k = torch.randn(1, 2, 64, 128), torch.randn(1, 2, 64, 128)
    v, beta, g = torch.randn(1, 2, 64, 64), torch.rand(1, 2, 64), -torch.rand(1, 2, 64)
    for t in (q, k, v, beta, g):
        t.requires_grad_(requires_grad)
    with torch.set_grad_enabled(grad_mode):
        la.gated_delta_rule_chunkwise(q, k, v, g, beta, None, None, 64, False)
    return seen


def test_leaves_with_grad_in_grad_mode_save_for_backward(monkeypatch):
    assert _run(monkeypatch, True, True) == [False]


def test_leaves_with_grad_under_no_grad_run_forward_only(monkeypatch):
    assert _run(monkeypatch, False, True) == [True]


def test_no_leaf_requires_grad_runs_forward_only(monkeypatch):
    assert _run(monkeypatch, True, False) == [True]
