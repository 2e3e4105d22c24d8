"""Enumerations of the public API (same names and values as the reference: sonicmoe/enums.py:8-30)."""

from enum import Enum

LIBRARY_NAME = "sonicmoe"


class KernelBackendMoE(Enum):
    scattermoe = "scattermoe"
    torch = "torch"
    sonicmoe = "sonicmoe"


class ActivationType(Enum):
    SWIGLU = "swiglu"
    GEGLU = "geglu"
    REGLU = "reglu"

    RELU_SQ = "relu_sq"
    RELU = "relu"
    GELU = "gelu"
    SILU = "silu"


_GLU = (ActivationType.SWIGLU, ActivationType.REGLU, ActivationType.GEGLU)

# integer codes of the C ABI (include/sonicmoe_hip.h: smoe_activation)
ACTIVATION_CODE = {
    ActivationType.SWIGLU: 0,
    ActivationType.GEGLU: 1,
    ActivationType.REGLU: 2,
    ActivationType.RELU_SQ: 3,
    ActivationType.RELU: 4,
    ActivationType.GELU: 5,
    ActivationType.SILU: 6,
}


def is_glu(activation_type: ActivationType) -> bool:
    return activation_type in _GLU
