"""Sub-byte scalar type descriptor whose integer id crosses the op boundary as
`b_type_id`.  Mirrors aphrodite/scalar_type.py:22-340 of the reference (id
bitfield :129-156) for the integer types this build handles and the 8-bit
floating-point weight type float8_e4m3fn, the 4-bit one float4_e2m1f and the
scale type float8_e8m0fnu."""
from __future__ import annotations

import functools
from dataclasses import dataclass

_NAN_REPR_NONE = 0
_NAN_REPR_IEEE_754 = 1
_NAN_REPR_EXTD_RANGE_MAX_MIN = 2   # NaN: exponent and mantissa all ones; no infinities


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

    def is_integer(self) -> bool:
        return self.exponent == 0

    def is_floating_point(self) -> bool:
        return self.exponent != 0

    def is_signed(self) -> bool:
        return self.signed

    def has_bias(self) -> bool:
        return self.bias != 0

    def min(self) -> int:
        assert self.is_integer()
        raw = -(1 << (self.size_bits - 1)) if self.signed else 0
        return raw - self.bias

    def max(self) -> int:
        assert self.is_integer()
        return (1 << self.mantissa) - 1 - self.bias

    @functools.cached_property
    def id(self) -> int:
        val, off = 0, 0
        for member, width in ((self.exponent, 8), (self.mantissa, 8), (int(self.signed), 1),
                              (self.bias, 32), (int(self._finite_values_only), 1), (self.nan_repr, 8)):
            val |= (int(member) & ((1 << width) - 1)) << off
            off += width
        return val

    def __str__(self) -> str:
        if self.is_floating_point():   # scalar_type.py:223-233: f = no infinities, n = non-standard NaNs
            s = f"float{self.size_bits}_e{self.exponent}m{self.mantissa}"
            if self.nan_repr != _NAN_REPR_IEEE_754 or self._finite_values_only:
                s += "f" if self._finite_values_only else ""
                s += "n" if self.nan_repr != _NAN_REPR_NONE else ""
            return s
        s = ("int" if self.signed else "uint") + str(self.size_bits)
        return s + (f"b{self.bias}" if self.bias else "")

    @classmethod
    def int_(cls, size_bits: int, bias: int | None) -> "ScalarType":
        return cls(0, size_bits - 1, True, bias or 0)

    @classmethod
    def uint(cls, size_bits: int, bias: int | None) -> "ScalarType":
        return cls(0, size_bits, False, bias or 0)

    @classmethod
    def float_(cls, exponent: int, mantissa: int, finite_values_only: bool, nan_repr: int) -> "ScalarType":
        """A floating-point type that does not follow IEEE 754 (scalar_type.py:276-289)."""
        assert mantissa > 0 and exponent > 0 and nan_repr != _NAN_REPR_IEEE_754
        return cls(exponent, mantissa, True, 0, finite_values_only, nan_repr)


class scalar_types:
    int4 = ScalarType.int_(4, None)
    uint4 = ScalarType.uint(4, None)
    int8 = ScalarType.int_(8, None)
    uint8 = ScalarType.uint(8, None)
    uint4b8 = ScalarType.uint(4, 8)
    uint8b128 = ScalarType.uint(8, 128)
    float8_e4m3fn = ScalarType.float_(4, 3, True, _NAN_REPR_EXTD_RANGE_MAX_MIN)
    float8_e8m0fnu = ScalarType(8, 0, False, 0, True, _NAN_REPR_EXTD_RANGE_MAX_MIN)
    float4_e2m1f = ScalarType.float_(2, 1, True, _NAN_REPR_NONE)
