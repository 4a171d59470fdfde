"""Stand-ins for ``aiter.ActivationType`` / ``aiter.QuantType`` used in the reference signature
(src/contrib/fused_moe.py:135-136); aiter itself is not a dependency."""
import enum


class ActivationType(enum.IntEnum):
    No = -1
    Silu = 0
    Gelu = 1
    Swiglu = 2


class QuantType(enum.IntEnum):
    No = 0
    per_Tensor = 1
    per_Token = 2
    per_1x32 = 3
    per_1x128 = 4
    per_128x128 = 5
