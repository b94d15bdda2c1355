"""Head dimensions between the chunk kernels' sizes, through the zero-channel embedding of the Python ops: the shapes
of the reference's own chunk tests (test_deltanet.py:64-90 dk16 dv32, test_gated_deltanet.py:249-284 dk16 dv32,
test_kda.py:252-290 dk8 dv8) and a few irregular ones, forward and backward against the fp64 oracles.
Metric max|x - ref| / max|ref| <= 1e-4 (fp32 inputs) or <= 2e-2 (bf16 inputs)."""
import numpy as np
import pytest
import torch

from oracle.adjoint import delta_rule_adjoint
from oracle.inputs import make_inputs
from conftest import max_rel
from test_chunk_bwd_gpu import _prep, check, gpu_grads
from test_chunk_fwd_gpu import gpu_chunk_fwd, oracle_fwd

pytestmark = pytest.mark.gpu
CASES = [("none", (2, 4, 32, 16, 32)), ("scalar", (1, 2, 64, 16, 32)), ("vector", (2, 2, 64, 8, 8)),
         ("scalar", (1, 2, 150, 96, 80)), ("vector", (1, 1, 100, 200, 100)), ("none", (1, 2, 70, 130, 64))]


@pytest.mark.parametrize("gate,shape", CASES)
@pytest.mark.parametrize("bf16", [False, True])
def test_forward_and_backward(gate, shape, bf16):
    B, H, T, dk, dv = shape
    x = make_inputs(91, B, H, T, dk, dv, gate=gate, with_state=True, with_grad=True)
    x, dt = _prep(x, bf16)
    tol = 2e-2 if bf16 else 1e-4
    o_ref, S_ref = oracle_fwd(x, gate)
    o, S = gpu_chunk_fwd(x, gate, dt)
    assert tuple(o.shape) == (B, H, T, dv) and tuple(S.shape) == (B, H, dk, dv)
    assert max_rel(o.float().cpu().numpy(), o_ref) < tol and max_rel(S.cpu().numpy(), S_ref) < tol
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x.get("g"), x["dS"], None, x["S0"], False)
    got = gpu_grads(x, gate, dt)
    assert got["dq"].shape == x["q"].shape and got["dv"].shape == x["v"].shape and got["dS0"].shape == x["S0"].shape
    check(got, ref, tol)


def test_l2norm_with_padded_channels():
    x = make_inputs(92, 1, 2, 90, 48, 40, gate="scalar", with_state=True, with_grad=True, normalize=False)
    ref = delta_rule_adjoint(x["q"], x["k"], x["v"], x["beta"], x["dO"], x["g"], x["dS"], None, x["S0"], True)
    check(gpu_grads(x, "scalar", torch.float32, l2=True), ref, 1e-4)


def test_key_dimension_above_256_is_refused():
    import linearnexus_amd as la
    x = make_inputs(93, 1, 1, 64, 320, 64)
    t = lambda n: torch.from_numpy(x[n]).to("cuda")
    with pytest.raises(RuntimeError):
        la.delta_rule_chunkwise(t("q"), t("k"), t("v"), t("beta"))
