"""Sub-byte weight types and their 64-bit ids, as the ops receive them in `b_q_type`.

Host-side mirror of the slice of `ScalarType` (reference vllm/scalar_type.py:136-164, 327-356;
C++ csrc/core/scalar_type.hpp:120-160) that this path needs: integer types with an optional
bias, and the 8- and 4-bit float types the ops name (float8_e4m3fn is implemented, float4_e2m1f is recognised).  The id packs, from bit 0 up: exponent:8, mantissa:8, signed:1, bias:32,
finite_values_only:1, nan_repr:8 — so ids produced by vLLM's own ScalarType decode here and
vice versa.
"""
from dataclasses import dataclass

_NAN_REPR_NONE = 0
_NAN_REPR_IEEE_754 = 1
_NAN_REPR_EXTD_RANGE_MAX_MIN = 2


@dataclass(frozen=True)
class ScalarType:
    exponent: int
    mantissa: int
    signed: bool
    bias: int
    _finite_values_only: bool = False
    nan_repr: int = _NAN_REPR_IEEE_754

    @property
    def size_bits(self) -> int:
        return self.exponent + self.mantissa + int(self.signed)

    @property
    def id(self) -> int:
        fields = ((self.exponent, 8), (self.mantissa, 8), (int(self.signed), 1), (self.bias, 32),
                  (int(self._finite_values_only), 1), (self.nan_repr, 8))
        val, off = 0, 0
        for member, width in fields:
            val |= (int(member) & ((1 << width) - 1)) << off
            off += width
        return val

    @classmethod
    def from_id(cls, type_id: int) -> "ScalarType":
        def take(off, width):
            return (type_id >> off) & ((1 << width) - 1)
        return cls(take(0, 8), take(8, 8), bool(take(16, 1)), take(17, 32), bool(take(49, 1)), take(50, 8))

    def is_integer(self) -> bool:
        return self.exponent == 0

    def is_signed(self) -> bool:
        return self.signed

    def has_bias(self) -> bool:
        return self.bias != 0

    def min(self) -> int:
        raw = -(1 << (self.size_bits - 1)) if self.signed else 0
        return raw - self.bias

    def max(self) -> int:
        raw = (1 << self.mantissa) - 1
        return raw - self.bias

    @classmethod
    def uint(cls, size_bits: int, bias: int | None) -> "ScalarType":
        return cls(0, size_bits, False, bias or 0)

    @classmethod
    def int_(cls, size_bits: int, bias: int | None) -> "ScalarType":
        return cls(0, size_bits - 1, True, bias or 0)

    @classmethod
    def float_(cls, exponent: int, mantissa: int, finite_values_only: bool, nan_repr: int) -> "ScalarType":
        """Non-IEEE float type (scalar_type.py:292-309)."""
        return cls(exponent, mantissa, True, 0, finite_values_only, nan_repr)

    def is_floating_point(self) -> bool:
        return self.exponent != 0

    def __str__(self) -> str:
        if self.is_floating_point():
            s = f"float{self.size_bits}_e{self.exponent}m{self.mantissa}"
            if self._finite_values_only:
                s += "f"
            if self.nan_repr == _NAN_REPR_EXTD_RANGE_MAX_MIN:
                s += "n"
            return s
        s = ("int" if self.signed else "uint") + str(self.size_bits)
        return s + (f"b{self.bias}" if self.bias else "")


class scalar_types:
    int4 = ScalarType.int_(4, None)
    uint4 = ScalarType.uint(4, None)
    int8 = ScalarType.int_(8, None)
    uint8 = ScalarType.uint(8, None)
    uint4b8 = ScalarType.uint(4, 8)
    uint8b128 = ScalarType.uint(8, 128)
    float8_e4m3fn = ScalarType.float_(4, 3, True, _NAN_REPR_EXTD_RANGE_MAX_MIN)
    float4_e2m1f = ScalarType.float_(2, 1, True, _NAN_REPR_NONE)
