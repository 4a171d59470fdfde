"""MI355X-native MXFP4 fused-MoE operator (hand-written HIP kernels behind a C ABI)."""
from .enums import ActivationType, QuantType  # noqa: F401
from .fused_moe import fused_moe, fused_moe_routed  # noqa: F401
from .moe_sorting import moe_sorting  # noqa: F401
from . import mxfp4  # noqa: F401

__all__ = ["fused_moe", "fused_moe_routed", "moe_sorting", "ActivationType", "QuantType", "mxfp4"]
