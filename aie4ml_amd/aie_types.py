"""Fixed-point type vocabulary of the operator IR.

Mirrors the names and meaning of the reference's ``aie4ml.aie_types`` (RoundingMode /
SaturationMode / QuantIntent / AIEDataType, src/aie4ml/aie_types.py:9-178) so that tensors built by the
reference's frontends and tensors built here are interchangeable by attribute access. Only the integer
formats the GPU kernels execute are modelled.
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


@dataclass(frozen=True)
class QuantIntent:
    """What a tensor is meant to hold: `width`-bit fixed point with `frac` fractional bits."""

    width: int
    frac: int
    signed: bool
    rounding: RoundingMode = RoundingMode.RND_CONV
    saturation: SaturationMode = SaturationMode.SAT


_INT_WIDTHS = {'int8': 8, 'uint8': 8, 'int16': 16, 'uint16': 16, 'int32': 32, 'uint32': 32, 'int64': 64}
_C_TYPES = {'int8': 'int8_t', 'uint8': 'uint8_t', 'int16': 'int16_t', 'uint16': 'uint16_t', 'int32': 'int32_t',
            'uint32': 'uint32_t', 'int64': 'int64_t'}


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
    def c_type(self) -> str:
        return _C_TYPES[self.format]


def is_float_intent(precision) -> bool:
    """True for the reference's FloatIntent (bf16 / fp32 / fp8 tensors): no GPU integer kernel takes them."""
    return precision is not None and not hasattr(precision, 'frac') and hasattr(precision, 'format')
