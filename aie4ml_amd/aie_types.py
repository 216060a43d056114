"""Fixed-point type vocabulary of the operator IR.

Mirrors the names and meaning of the reference's ``aie4ml.aie_types`` (RoundingMode /
SaturationMode / QuantIntent / AIEDataType, src/aie4ml/aie_types.py:9-178) so that tensors built by the
reference's frontends and tensors built here are interchangeable by attribute access. The float side
(FloatFormat / FloatIntent, src/aie4ml/aie_types.py:20-25, 85-98) covers the formats of the reference's
float compute path.
"""

from __future__ import annotations

from dataclasses import dataclass
from enum import Enum


class RoundingMode(Enum):
    TRN = 'TRN'                  # toward -inf
    RND_MIN_INF = 'RND_MIN_INF'  # nearest, ties toward -inf (the reference maps it to AIE floor)
    TRN_ZERO = 'TRN_ZERO'
    RND_ZERO = 'RND_ZERO'
    RND_INF = 'RND_INF'
    RND_CONV = 'RND_CONV'
    RND = 'RND'


class SaturationMode(Enum):
    WRAP = 'WRAP'
    SAT = 'SAT'
    SAT_ZERO = 'SAT_ZERO'
    SAT_SYM = 'SAT_SYM'


class FloatFormat(Enum):
    BF16 = 'bfloat16'
    FP32 = 'float32'
    FP8_E4M3 = 'fp8_e4m3'


FLOAT_FORMATS = frozenset(f.value for f in FloatFormat)


@dataclass(frozen=True)
class FloatIntent:
    """What a tensor of the float compute path holds (no fractional-bit bookkeeping)."""

    width: int
    format: FloatFormat


@dataclass(frozen=True)
class QuantIntent:
    """What a tensor is meant to hold: `width`-bit fixed point with `frac` fractional bits."""

    width: int
    frac: int
    signed: bool
    rounding: RoundingMode = RoundingMode.RND_CONV
    saturation: SaturationMode = SaturationMode.SAT


_INT_WIDTHS = {'int8': 8, 'uint8': 8, 'int16': 16, 'uint16': 16, 'int32': 32, 'uint32': 32, 'int64': 64}
_INT_WIDTHS.update({'bfloat16': 16, 'float32': 32, 'fp8_e4m3': 8, 'accfloat': 32})
_C_TYPES = {'int8': 'int8_t', 'uint8': 'uint8_t', 'int16': 'int16_t', 'uint16': 'uint16_t', 'int32': 'int32_t',
            'uint32': 'uint32_t', 'int64': 'int64_t', 'bfloat16': 'bfloat16', 'float32': 'float', 'fp8_e4m3': 'float8',
            'accfloat': 'accfloat'}


@dataclass(frozen=True)
class AIEDataType:
    """Storage type a kernel actually reads or writes (format string + fixed-point metadata)."""

    format: str
    frac: int = 0
    rounding: RoundingMode = RoundingMode.RND
    saturation: SaturationMode = SaturationMode.SAT

    def __post_init__(self):
        if self.format not in _INT_WIDTHS:
            raise ValueError(f'Unknown AIEDataType format: {self.format!r}')

    @property
    def width(self) -> int:
        return _INT_WIDTHS[self.format]

    @property
    def signed(self) -> bool:
        return not self.format.startswith('u')

    @property
    def is_float(self) -> bool:
        return self.format in FLOAT_FORMATS or self.format == 'accfloat'

    @property
    def c_type(self) -> str:
        return _C_TYPES[self.format]


def is_float_intent(precision) -> bool:
    """True for a FloatIntent, this package's or the reference's (bf16 / fp32 / fp8 tensors)."""
    return precision is not None and not hasattr(precision, 'frac') and hasattr(precision, 'format')
