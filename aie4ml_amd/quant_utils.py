"""Host-side fixed-point helpers: how float inputs, weights and biases become integers.

Behavioural mirror of src/aie4ml/quant_utils.py:38-89 and of quantize_to_int
(src/aie4ml/op_impls/families/matmul/common.py:287-304). Note the deliberate asymmetry the
reference has: host quantisation of TRN_ZERO/RND_ZERO truncates, while the kernels round those modes
to nearest with ties toward zero.
"""

from __future__ import annotations

import numpy as np

from .aie_types import RoundingMode, SaturationMode


def dtype_for_precision(width, signed: bool):
    """Smallest numpy integer dtype that holds `width` bits (int32 when the width is unknown)."""
    if width is None:
        return np.int32
    for bits, s, u in ((8, np.int8, np.uint8), (16, np.int16, np.uint16), (32, np.int32, np.uint32)):
        if width <= bits:
            return s if signed else u
    return np.int64 if signed else np.uint64


def wrap_to_width(values, width: int, signed: bool):
    """Two's-complement wrap of integers to `width` bits."""
    span = 1 << int(width)
    out = np.mod(values, span)
    if signed:
        out = np.where(out >= span // 2, out - span, out)
    return out


_ROUNDERS = {
    RoundingMode.TRN: np.floor,
    RoundingMode.RND_MIN_INF: np.floor,
    RoundingMode.TRN_ZERO: np.trunc,
    RoundingMode.RND_ZERO: np.trunc,
    RoundingMode.RND_INF: np.ceil,
    RoundingMode.RND_CONV: np.round,  # ties to even
    RoundingMode.RND: lambda v: np.where(v >= 0, np.floor(v + 0.5), np.ceil(v - 0.5)),
}


def apply_rounding(values, mode: RoundingMode):
    """Round real values to integers under a fixed-point rounding mode."""
    try:
        return _ROUNDERS[mode](values)
    except KeyError:
        raise ValueError(f'Unsupported rounding mode {mode}') from None


def handle_overflow(values, width: int, signed: bool, mode: SaturationMode):
    """Bring integers into `width` bits under an overflow mode."""
    if mode == SaturationMode.WRAP:
        return wrap_to_width(values, width, signed)
    info = np.iinfo(dtype_for_precision(width, signed))
    if mode == SaturationMode.SAT:
        return np.clip(values, info.min, info.max)
    if mode == SaturationMode.SAT_ZERO:
        return np.clip(values, 0, info.max)
    if mode == SaturationMode.SAT_SYM:
        return np.clip(values, max(info.min, -info.max), info.max)
    raise ValueError(f'Unsupported saturation mode {mode}')


def quantize_to_int(array, frac_bits: int, target_bits: int, signed: bool = True, rounding_mode=None,
                    saturation_mode=None):
    """Float parameters -> fixed-point integers: scale by 2^frac, round, handle overflow."""
    if array is None:
        return None
    scale = (1 << int(frac_bits)) if frac_bits > 0 else 1
    rounded = apply_rounding(np.asarray(array, dtype=np.float64) * scale, rounding_mode)
    ints = handle_overflow(rounded.astype(np.int64), int(target_bits), bool(signed), saturation_mode)
    return ints.astype(dtype_for_precision(target_bits, signed), copy=False)


def quantize_input(data, dtype) -> np.ndarray:
    """Graph-input quantisation (src/aie4ml/simulation.py:260-269): integer arrays pass through with a
    dtype cast only; float arrays are scaled by 2^frac, rounded with the tensor's own rounding mode and
    overflow-handled with its saturation mode."""
    data = np.asarray(data)
    np_dtype = dtype_for_precision(dtype.width, dtype.signed)
    if np.issubdtype(data.dtype, np.integer):
        return data.astype(np_dtype, copy=False)
    scaled = data * float(1 << max(0, int(dtype.frac)))
    ints = apply_rounding(scaled, dtype.rounding).astype(np.int64, copy=False)
    return handle_overflow(ints, int(dtype.width), bool(dtype.signed), dtype.saturation).astype(np_dtype, copy=False)


def dequantize_output(arr, frac: int) -> np.ndarray:
    """Raw integer outputs -> float64 (src/aie4ml/simulation.py:248-257)."""
    frac = max(0, int(frac))
    out = np.asarray(arr).astype(np.float64, copy=False)
    return out if frac == 0 else out / float(1 << frac)
