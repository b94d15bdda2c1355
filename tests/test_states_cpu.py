"""Host-side logic that needs no GPU.  The generation caches mirror the reference's dataclasses field for field and argument for argument
(delta_net.py:81-118, gated_deltanet.py:72-128, kda.py:57-113), so a caller's ``State.zeros(...)`` lines keep working."""
import dataclasses
import inspect

import pytest
import torch

import linearnexus_amd as la


def test_deltanet_state():
    assert [f.name for f in dataclasses.fields(la.DeltaNetState)] == ["S", "conv_state"]
    names = list(inspect.signature(la.DeltaNetState.zeros).parameters)
    assert names[:6] == ["batch_size", "num_heads", "key_dim", "value_dim", "conv_channels", "conv_size"]
    s = la.DeltaNetState.zeros(2, 3, 16, 32, device="cpu")
    assert tuple(s.S.shape) == (2, 3, 16, 32) and s.S.dtype == torch.float32 and s.conv_state is None
    assert not s.S.any()
    s = la.DeltaNetState.zeros(2, 3, 16, 32, conv_channels=3 * (16 + 16 + 32), conv_size=4, device="cpu")
    assert tuple(s.conv_state.shape) == (2, 3, 192)


@pytest.mark.parametrize("cls", [la.GatedDeltaNetState, la.KDAState])
def test_gated_and_kda_states(cls):
    assert [f.name for f in dataclasses.fields(cls)] == ["S", "conv_state_q", "conv_state_k", "conv_state_v"]
    names = list(inspect.signature(cls.zeros).parameters)
    assert names[:8] == ["batch_size", "num_v_heads", "key_dim_per_head", "value_dim_per_head", "key_dim_total",
                         "value_dim", "conv_size", "use_conv"]
    s = cls.zeros(2, 4, 256, 512, device="cpu")
    assert isinstance(s, cls) and tuple(s.S.shape) == (2, 4, 256, 512) and s.S.dtype == torch.float32
    assert s.conv_state_q is None and s.conv_state_k is None and s.conv_state_v is None
    s = cls.zeros(2, 4, 256, 512, key_dim_total=1024, value_dim=2048, conv_size=4, device="cpu")
    assert tuple(s.conv_state_q.shape) == (2, 3, 1024) and tuple(s.conv_state_k.shape) == (2, 3, 1024)
    assert tuple(s.conv_state_v.shape) == (2, 3, 2048)
    s = cls.zeros(2, 4, 256, 512, key_dim_total=1024, value_dim=2048, use_conv=False, device="cpu")
    assert s.conv_state_q is None


def test_segment_count_heuristic(monkeypatch):
    from linearnexus_amd.linear_attn import _prefill_segments
    monkeypatch.delenv("LNX_PREFILL_SEGMENTS", raising=False)
    assert _prefill_segments(1, 16, 131072, 128) == 8      # 32 workgroups of 64 columns -> 8 segments of 256 chunks
    assert _prefill_segments(8, 16, 4096, 128) == 1        # configuration 2: the chip is full already
    assert _prefill_segments(1, 4, 8192, 128) == 1         # too short to pay for three times the scan work
    assert _prefill_segments(1, 2, 20000, 512) == 4        # every segment keeps at least 64 chunks
    assert _prefill_segments(2, 16, 131072, 128) == 1      # 64 workgroups: three times the scan work would not pay
    assert _prefill_segments(1, 16, 16384, 128) == 1       # 32 workgroups need 32768 tokens
    monkeypatch.setenv("LNX_PREFILL_SEGMENTS", "5")
    assert _prefill_segments(8, 16, 4096, 128) == 5
    monkeypatch.setenv("LNX_PREFILL_SEGMENTS", "0")
    assert _prefill_segments(1, 16, 131072, 128) == 1


def test_dtype_promotion_rules():
    """One kernel dtype (float32 or bfloat16) passes through; anything else is computed in float32 and cast back to q's
    dtype, like the reference's up-cast (delta_net.py:170-179, :213)."""
    from linearnexus_amd.linear_attn import _promote
    t = lambda dt: torch.zeros(1, 1, 2, 4, dtype=dt)
    for dt in (torch.float32, torch.bfloat16):
        q, k, v, back = _promote(t(dt), t(dt), t(dt))
        assert back is None and q.dtype == dt
    q, k, v, back = _promote(t(torch.float32), t(torch.float32), t(torch.bfloat16))   # the DeltaNet block's mix
    assert back == torch.float32 and {q.dtype, k.dtype, v.dtype} == {torch.float32}
    q, k, v, back = _promote(t(torch.float16), t(torch.float16), t(torch.float16))
    assert back == torch.float16 and v.dtype == torch.float32
    q, k, v, back = _promote(t(torch.bfloat16), t(torch.float32), t(torch.float64))
    assert back == torch.bfloat16 and q.dtype == torch.float32
