"""Numeric resolution shared by the operator variants: storage types, rounding tokens, output shifts.

Restates src/aie4ml/op_impls/utils/precision.py:13-150 and the io_view helpers of
src/aie4ml/op_impls/utils/io.py:89-104.
"""

from __future__ import annotations

from typing import Any, List

from ..aie_types import AIEDataType, QuantIntent, RoundingMode, is_float_intent

# aie::rounding_mode the kernels run under, per tensor rounding mode
ROUNDING_TOKEN_MAP = {
    RoundingMode.TRN: 'floor',
    RoundingMode.RND_MIN_INF: 'floor',
    RoundingMode.RND_INF: 'ceil',
    RoundingMode.RND: 'symmetric_inf',
    RoundingMode.TRN_ZERO: 'symmetric_zero',
    RoundingMode.RND_ZERO: 'symmetric_zero',
    RoundingMode.RND_CONV: 'conv_even',
}


def _mode_key(mode):
    """Accept this package's RoundingMode or the reference's enum of the same member names."""
    if isinstance(mode, RoundingMode):
        return mode
    name = getattr(mode, 'name', None) or str(mode)
    return RoundingMode[name]


def to_quant_intent(precision: Any) -> QuantIntent:
    if precision is None:
        raise TypeError('missing precision')
    if is_float_intent(precision):
        raise TypeError(f'Unsupported precision representation {type(precision)}')
    return QuantIntent(width=int(precision.width), frac=int(precision.frac), signed=bool(precision.signed),
                       rounding=_mode_key(precision.rounding), saturation=precision.saturation)


def float_format_name(precision: Any) -> str:
    """'bfloat16' / 'float32' / 'fp8_e4m3' of a FloatIntent (this package's or the reference's enum)."""
    fmt = precision.format
    return str(getattr(fmt, 'value', fmt))


def resolve_exact_storage_dtype(precision: Any, *, namespace: str, layer_name: str) -> AIEDataType:
    """Round the intent's width up to a storage width (4 -> 8, 8, 16, 32), keeping signedness and frac;
    a FloatIntent maps to its own format (precision.py:64-71)."""
    if is_float_intent(precision):
        return AIEDataType(format=float_format_name(precision))
    q = to_quant_intent(precision)
    if q.width <= 0:
        raise ValueError(f'{layer_name}: invalid {namespace} width {q.width}.')
    for cand in (8, 16, 32):
        if q.width <= cand:
            return AIEDataType(format=f'{"int" if q.signed else "uint"}{cand}', frac=q.frac, rounding=q.rounding,
                               saturation=q.saturation)
    raise ValueError(f'{layer_name}: {namespace} width {q.width} exceeds supported widths (4, 8, 16, 32).')


def aie_rounding_token(source) -> str:
    mode = getattr(source, 'rounding_mode', None) or getattr(source, 'rounding', None) or RoundingMode.TRN
    try:
        return ROUNDING_TOKEN_MAP[_mode_key(mode)]
    except KeyError:
        raise ValueError(f'Unsupported rounding mode {mode} for AIE kernel.') from None


def resolve_accumulator_output_shift(lhs_precision, output_precision, rhs_precision=None) -> int:
    """Right shift from accumulator fixed point (lhs_frac + rhs_frac) to the output's."""
    lhs = to_quant_intent(lhs_precision).frac
    out = to_quant_intent(output_precision).frac
    rhs = to_quant_intent(rhs_precision).frac if rhs_precision is not None else 0
    return max(0, int(lhs + rhs - out))


def view_perm(node, tensor, direction: str):
    """Permutation a folded Transpose left on this node for `tensor`, or None."""
    trait = node.traits.get('io_view')
    if trait is None:
        return None
    entry = (trait.data.get(direction) or {}).get(tensor.name)
    if not entry:
        return None
    perm = entry.get('perm')
    return None if perm is None else [int(p) for p in perm]


def view_shape(node, tensor, direction: str) -> List[int]:
    """Shape of `tensor` as this node sees it (after its io_view permutation)."""
    logical = [int(x) for x in tensor.shape]
    perm = view_perm(node, tensor, direction)
    if perm is None:
        return logical
    if sorted(perm) != list(range(len(logical))):
        raise ValueError(f'{node.name}: invalid io_view perm {perm} for rank {len(logical)}.')
    return [logical[i] for i in perm]


def is_identity(perm) -> bool:
    return perm is None or list(perm) == list(range(len(perm)))


def is_last_two_swap(perm) -> bool:
    if perm is None or len(perm) < 2:
        return False
    want = list(range(len(perm)))
    want[-1], want[-2] = want[-2], want[-1]
    return list(perm) == want
