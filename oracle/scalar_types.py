"""Integer ids of the sub-byte weight types passed to the ops as `b_q_type`.

Follows the bit packing of `ScalarType.id` (reference vllm/scalar_type.py:136-164,
C++ twin csrc/core/scalar_type.hpp:143-160): fields are packed little-end first as
exponent:8, mantissa:8, signed:1, bias:32, finite_values_only:1, nan_repr:8.

Pinned by: the three literal ids quoted for uint4 / uint4b8 / uint8b128, which were
computed by hand from the field layout (mantissa<<8 | bias<<17 | nan_repr<<50 with
nan_repr = IEEE_754 = 1).
"""
from dataclasses import dataclass


@dataclass(frozen=True)
class WType:
    name: str
    size_bits: int
    bias: int
    signed: bool = False

    @property
    def id(self) -> int:
        exponent = 0
        mantissa = self.size_bits - int(self.signed)
        nan_repr_ieee = 1
        v = exponent & 0xFF
        v |= (mantissa & 0xFF) << 8
        v |= int(self.signed) << 16
        v |= (self.bias & 0xFFFFFFFF) << 17
        v |= 0 << 49
        v |= nan_repr_ieee << 50
        return v

    def has_bias(self) -> bool:
        return self.bias != 0

    def min(self) -> int:
        return -self.bias

    def max(self) -> int:
        return (1 << self.size_bits) - 1 - self.bias


uint4 = WType("uint4", 4, 0)
uint4b8 = WType("uint4b8", 4, 8)
uint8 = WType("uint8", 8, 0)
uint8b128 = WType("uint8b128", 8, 128)
