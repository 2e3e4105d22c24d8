"""MI355X-native MoE layer with the public API of SonicMoE (sonicmoe/__init__.py:5-8)."""

from .count_cumsum import count_cumsum
from .enums import ActivationType, KernelBackendMoE
from .functional import enable_fp8_backward, enable_fp8_forward, enable_quack_gemm, moe_general_routing_inputs, moe_TC_softmax_topk_layer
from .moe import MoE

__all__ = [
    "ActivationType",
    "KernelBackendMoE",
    "MoE",
    "count_cumsum",
    "enable_fp8_backward",
    "enable_fp8_forward",
    "enable_quack_gemm",
    "moe_TC_softmax_topk_layer",
    "moe_general_routing_inputs",
]
