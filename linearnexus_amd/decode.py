"""Decode driver: the single-token step of one or many layers as ONE replayed HIP graph.

The reference generates one token per Python call of the model (linearnexus/generate.py:243-271);
each layer's step (gated_deltanet.py:539-597) is a handful of host dispatches, and at decode sizes the
kernels are shorter than the dispatches.  ``DecodeGraph`` holds fixed input buffers, the fp32 states
(updated in place, the same memory for every token) and a captured graph of the step kernels of all
layers; ``replay()`` is one host call per token.  The step entry point allocates nothing, never
synchronises and launches on the stream it is given, which is what makes it capturable.
"""
from __future__ import annotations

from typing import List, Optional

import torch

from . import linear_attn as la

Tensor = torch.Tensor
_STEP = {"delta": la.delta_rule_step, "gated": la.gated_delta_rule_step, "kda": la.kda_step}


class DecodeGraph:
    """Fixed buffers + captured graph for ``layers`` independent decode steps of one variant.

    Buffers (lists, one entry per layer; write the token's projections into them before ``replay``):
    ``q, k [B,H,dk]``, ``v [B,H,dv]``, ``beta [B,H]``, ``g [B,H]`` (gated) or ``[B,H,dk]`` (kda),
    ``state [B,H,dk,dv]`` fp32 (in place) and the outputs ``o [B,H,dv]``.
    """

    def __init__(self, variant: str, B: int, H: int, dk: int, dv: int, *, layers: int = 1,
                 dtype: torch.dtype = torch.bfloat16, scale: Optional[float] = None,
                 use_qk_l2norm: bool = True, states: Optional[List[Tensor]] = None, device="cuda"):
        if variant not in _STEP:
            raise ValueError(f"variant must be one of {sorted(_STEP)}, got {variant!r}")
        self.variant, self.layers = variant, layers
        self.scale, self.l2 = scale, use_qk_l2norm
        mk = lambda *s, dt=dtype: [torch.zeros(*s, dtype=dt, device=device) for _ in range(layers)]
        self.q, self.k, self.v = mk(B, H, dk), mk(B, H, dk), mk(B, H, dv)
        self.beta = mk(B, H, dt=torch.float32)
        self.g = None if variant == "delta" else mk(*((B, H) if variant == "gated" else (B, H, dk)), dt=torch.float32)
        if states is None:
            states = mk(B, H, dk, dv, dt=torch.float32)
        if len(states) != layers:
            raise ValueError(f"{layers} layers need {layers} states, got {len(states)}")
        for S in states:
            if tuple(S.shape) != (B, H, dk, dv) or S.dtype != torch.float32 or not S.is_contiguous() or not S.is_cuda:
                raise RuntimeError("states must be contiguous float32 [B,H,dk,dv] tensors on the GPU")
        self.state = list(states)
        self.o: List[Tensor] = []
        self._graph = torch.cuda.CUDAGraph()
        # one eager pass on a side stream first (library loading and first-use work must not be captured);
        # it runs on zero inputs, which leave every state unchanged (beta = 0)
        side = torch.cuda.Stream(device=device)
        side.wait_stream(torch.cuda.current_stream(device))
        with torch.cuda.stream(side):
            self._run()
        torch.cuda.current_stream(device).wait_stream(side)
        with torch.cuda.graph(self._graph):
            self.o = self._run()

    def _run(self) -> List[Tensor]:
        outs = []
        for i in range(self.layers):
            if self.variant == "delta":
                o, _ = la.delta_rule_step(self.q[i], self.k[i], self.v[i], self.beta[i], self.state[i],
                                          self.scale, inplace=True)
            else:
                o, _ = _STEP[self.variant](self.q[i], self.k[i], self.v[i], self.g[i], self.beta[i], self.state[i],
                                           self.scale, self.l2, inplace=True)
            outs.append(o)
        return outs

    def replay(self) -> List[Tensor]:
        """Advances every layer's state by the token in the input buffers; returns the output buffers
        (the same tensors every time: consume or copy them before the next replay)."""
        self._graph.replay()
        return self.o

    def step(self, q, k, v, beta, g=None, layer: int = 0) -> None:
        """Copies one layer's token into its buffers (asynchronous device copies on the current stream)."""
        self.q[layer].copy_(q)
        self.k[layer].copy_(k)
        self.v[layer].copy_(v)
        self.beta[layer].copy_(beta.reshape(self.beta[layer].shape))
        if self.g is not None:
            self.g[layer].copy_(g)
