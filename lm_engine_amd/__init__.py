"""MI355X-native gated delta-rule sequence mixer: the operator lm-engine's GatedDeltaNet layer
calls, as hand-written gfx950 HIP kernels behind a C-ABI library."""

from .conv import depthwise_causal_convolution
from .fla_shim import install_as_fla, uninstall_fla_shim
from .layer import gated_deltanet_mixing
from .layer_ops import delta_rule_gates, gated_rmsnorm
from .kernels import Kernel, enable_all_kernels, enable_kernels, is_kernel_allowed
from .ops import chunk_gated_delta_rule, fused_recurrent_gated_delta_rule, gated_delta_rule


__all__ = [
    "Kernel",
    "chunk_gated_delta_rule",
    "delta_rule_gates",
    "depthwise_causal_convolution",
    "enable_all_kernels",
    "enable_kernels",
    "fused_recurrent_gated_delta_rule",
    "gated_delta_rule",
    "gated_deltanet_mixing",
    "gated_rmsnorm",
    "install_as_fla",
    "is_kernel_allowed",
    "uninstall_fla_shim",
]
