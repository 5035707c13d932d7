"""Sub-byte / biased scalar type tags passed to the quantized GEMM as a 64-bit id.

Mirrors the reference's ``vllm/scalar_type.py`` (class :22-356, id packing :136-164, named types :327-351) for the
types the W4A16 / FP8 path touches.  Id bit layout, least significant first: exponent(8) | mantissa(8) | signed(1) |
bias(32) | finite_values_only(1) | nan_repr(8).
"""
from __future__ import annotations

import functools
import struct
from dataclasses import dataclass
from enum import Enum


class NanRepr(Enum):
    NONE = 0                # nans are not supported
    IEEE_754 = 1            # exp all 1s, mantissa not all 0s
    EXTD_RANGE_MAX_MIN = 2  # exp all 1s, mantissa all 1s


_FIELDS = (("exponent", 8), ("mantissa", 8), ("signed", 1), ("bias", 32), ("_finite_values_only", 1), ("nan_repr", 8))


@dataclass(frozen=True)
class ScalarType:
    exponent: int
    mantissa: int
    signed: bool
    bias: int
    _finite_values_only: bool = False
    nan_repr: NanRepr = NanRepr.IEEE_754

    # ------------------------------------------------------------------ id
    @functools.cached_property
    def id(self) -> int:      # (computed once per object: the GEMM op takes it on every call)
        val, off = 0, 0
        for name, width in _FIELDS:
            v = getattr(self, name)
            v = v.value if isinstance(v, NanRepr) else int(v)
            val |= (v & ((1 << width) - 1)) << off
            off += width
        return val

    @classmethod
    def from_id(cls, type_id: int) -> "ScalarType":
        vals, off = {}, 0
        for name, width in _FIELDS:
            vals[name] = (type_id >> off) & ((1 << width) - 1)
            off += width
        b = vals["bias"]
        if b >= 1 << 31:
            b -= 1 << 32
        return cls(vals["exponent"], vals["mantissa"], bool(vals["signed"]), b, bool(vals["_finite_values_only"]),
                   NanRepr(vals["nan_repr"]))

    # ------------------------------------------------------------------ properties
    @property
    def size_bits(self) -> int:
        return self.exponent + self.mantissa + int(self.signed)

    def is_floating_point(self) -> bool:
        return self.exponent != 0

    def is_integer(self) -> bool:
        return self.exponent == 0

    def is_signed(self) -> bool:
        return self.signed

    def has_bias(self) -> bool:
        return self.bias != 0

    def has_infs(self) -> bool:
        return not self._finite_values_only

    def has_nans(self) -> bool:
        return self.nan_repr != NanRepr.NONE

    def _raw_max(self) -> int | float:
        if self.is_floating_point():
            max_mantissa = (1 << self.mantissa) - 1
            if self.nan_repr == NanRepr.EXTD_RANGE_MAX_MIN:
                max_mantissa -= 1
            max_exponent = (1 << self.exponent) - 2
            if self.nan_repr in (NanRepr.EXTD_RANGE_MAX_MIN, NanRepr.NONE):
                assert self.exponent < 11
                max_exponent += 1
            # assemble an IEEE double with the same unbiased exponent and left-aligned mantissa
            exponent_bias = (1 << (self.exponent - 1)) - 1
            max_exponent_double = max_exponent - exponent_bias + 1023
            bits = (max_mantissa << (52 - self.mantissa)) | (max_exponent_double << 52)
            return struct.unpack("!d", struct.pack("!Q", bits))[0]
        return (1 << self.mantissa) - 1   # `mantissa` excludes the sign bit for integers

    def _raw_min(self) -> int | float:
        if self.is_floating_point():
            assert self.signed
            return -self._raw_max()
        if self.signed:
            return -(1 << self.mantissa)
        return 0

    def max(self) -> int | float:
        return self._raw_max() - self.bias

    def min(self) -> int | float:
        return self._raw_min() - self.bias

    # ------------------------------------------------------------------ constructors
    @classmethod
    def int_(cls, size_bits: int, bias: int | None) -> "ScalarType":
        return cls(0, size_bits - 1, True, bias or 0)

    @classmethod
    def uint(cls, size_bits: int, bias: int | None) -> "ScalarType":
        return cls(0, size_bits, False, bias or 0)

    @classmethod
    def float_IEEE754(cls, exponent: int, mantissa: int) -> "ScalarType":
        return cls(exponent, mantissa, True, 0)

    @classmethod
    def float_(cls, exponent: int, mantissa: int, finite_values_only: bool, nan_repr: NanRepr) -> "ScalarType":
        return cls(exponent, mantissa, True, 0, finite_values_only, nan_repr)

    def __str__(self) -> str:
        if self.is_floating_point():
            s = f"float{self.size_bits}_e{self.exponent}m{self.mantissa}"
            if not self.has_infs():
                s += "f"
            if self.nan_repr == NanRepr.EXTD_RANGE_MAX_MIN:
                s += "n"
            return s
        s = ("int" if self.signed else "uint") + str(self.size_bits)
        if self.has_bias():
            s += f"b{self.bias}"
        return s


class scalar_types:
    int4 = ScalarType.int_(4, None)
    uint4 = ScalarType.uint(4, None)
    int8 = ScalarType.int_(8, None)
    uint8 = ScalarType.uint(8, None)
    float8_e4m3fn = ScalarType.float_(4, 3, True, NanRepr.EXTD_RANGE_MAX_MIN)
    float8_e5m2 = ScalarType.float_IEEE754(5, 2)
    float16_e8m7 = ScalarType.float_IEEE754(8, 7)
    float16_e5m10 = ScalarType.float_IEEE754(5, 10)
    # "gptq" types: unsigned storage with a symmetric bias
    uint4b8 = ScalarType.uint(4, 8)
    uint8b128 = ScalarType.uint(8, 128)
    bfloat16 = float16_e8m7
    float16 = float16_e5m10
