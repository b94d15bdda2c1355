"""MI355X-native delta-rule scan (DeltaNet / Gated DeltaNet / KDA) behind the reference's op names."""
from .backend import KernelBackend, select_kernel_backend
from .conv import depthwise_conv1d_causal
from .gate import gated_deltanet_gate, kda_gate
from .norm import rmsnorm_gated
from .rwkv7 import dplr_delta_rule_recurrent, dplr_delta_rule_step
from .linear_attn import (
    DeltaNetState,
    GatedDeltaNetState,
    KDAState,
    delta_rule_chunkwise,
    delta_rule_recurrent,
    delta_rule_step,
    gated_delta_rule_chunkwise,
    gated_delta_rule_recurrent,
    gated_delta_rule_step,
    kda_chunkwise,
    kda_chunkwise_raw_gate,
    kda_recurrent,
    kda_step,
    l2norm_rows,
)

__all__ = [
    "KernelBackend", "select_kernel_backend",
    "DeltaNetState", "GatedDeltaNetState", "KDAState",
    "delta_rule_recurrent", "delta_rule_chunkwise", "delta_rule_step",
    "gated_delta_rule_recurrent", "gated_delta_rule_chunkwise", "gated_delta_rule_step",
    "kda_recurrent", "kda_chunkwise", "kda_chunkwise_raw_gate", "kda_step", "l2norm_rows", "depthwise_conv1d_causal",
    "dplr_delta_rule_recurrent", "dplr_delta_rule_step", "rmsnorm_gated", "kda_gate", "gated_deltanet_gate",
]
