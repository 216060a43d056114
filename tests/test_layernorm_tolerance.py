"""How far the one float step of the reference's LayerNorm can move the outputs.

layer_norm.cpp:33-34 computes inv_std16 = to_fixed(invsqrt(float(var + eps)), 15) on the AI Engine; how that float
reciprocal square root and the conversion round cannot be read off the sources, so the oracle (and the HIP kernel)
define inv_std16 as the nearest Q15 value. This test restates the LayerNorm in int64 numpy with the reciprocal
square root pluggable, checks that the nearest form reproduces the oracle bit for bit, and then measures what the other
plausible definitions do to the int8 outputs of the C4 tensor and of the two C5 LayerNorms (768 columns):

    inv_std16 off by +1 or -1 everywhere, truncation (floor) instead of nearest, and a float32 evaluation
    (1 / sqrt in float32, scaled by 2^15, truncated and rounded).

STATED TOLERANCE (asserted below): no output moves by more than 1 LSB under any of them, and under truncation or the
float32 forms fewer than 2 % of the outputs move at all. Against silicon the LayerNorm is therefore pinned to 1 LSB, not
to the bit.
"""

from fractions import Fraction
from math import isqrt

import numpy as np
import pytest

from aie4ml_amd import workloads


def srs(acc, s, lo, hi):
    """shift-round(conv_even)-saturate on int64 arrays."""
    if s > 0:
        q = acc >> s
        r = acc & ((1 << s) - 1)
        h = 1 << (s - 1)
        q = q + ((r > h) | ((r == h) & ((q & 1) == 1)))
    else:
        q = acc
    return np.clip(q, lo, hi)


def rsqrt_q15(v, how):
    """inv_std16 for an array of positive integers v under one definition of the rounding."""
    v = np.asarray(v, dtype=np.int64)
    uniq = np.unique(v)
    table = {}
    for u in uniq.tolist():
        # floor(2^15 / sqrt(u)) exactly: the largest q with q^2 * u <= 2^30
        q = isqrt((1 << 30) // u)
        while (q + 1) * (q + 1) * u <= (1 << 30):
            q += 1
        while q * q * u > (1 << 30):
            q -= 1
        near = q + 1 if (2 * q + 1) ** 2 * u < (1 << 32) else q  # nearest: is q + 1/2 still below the exact value?
        if how == 'nearest':
            r = near
        elif how == 'plus1':
            r = near + 1
        elif how == 'minus1':
            r = near - 1
        elif how == 'floor':
            r = q
        elif how == 'float32_trunc':
            r = int(np.float32(32768.0) * (np.float32(1.0) / np.sqrt(np.float32(u))))
        elif how == 'float32_round':
            r = int(np.rint(np.float32(32768.0) * (np.float32(1.0) / np.sqrt(np.float32(u)))))
        else:
            raise ValueError(how)
        table[u] = min(max(r, 0), 32767)
    return np.vectorize(table.get, otypes=[np.int64])(v)


def layernorm_np(x, gamma, beta, out_shift, eps_q0=1, how='nearest'):
    """layer_norm.cpp:14-40, 95-119 in int64 numpy (conv_even), with the reciprocal square root pluggable."""
    x = x.astype(np.int64)
    cols = x.shape[-1]
    sx = x.sum(-1)
    sq = (x * x).sum(-1)
    mu = (sx + (cols >> 1)) // cols
    var = np.maximum((sq - 2 * mu * sx + cols * mu * mu) // cols, 0)
    inv = rsqrt_q15(var + eps_q0, how)
    fscale = srs(inv[:, None] * gamma.astype(np.int64)[None, :], 7, -32768, 32767)
    acc = (x - mu[:, None]) * fscale + beta.astype(np.int64)[None, :]
    return srs(acc, 15 - out_shift, -128, 127).astype(np.int8)


def cases():
    a, b, gamma, beta, prm = workloads.c4_add_layernorm(2048, 1024)
    s = np.clip(a.astype(np.int16) + b, -128, 127).astype(np.int8)
    yield 'c4 [2048 of 16384, 1024]', s, gamma, beta, prm['out_shift']
    # the two LayerNorms of the C5 block: 768 columns, gamma / beta drawn as the block draws them, inputs with the
    # spread of a saturating residual sum of int8 activations
    r = np.random.default_rng(17 + 5)
    for i, sigma in ((1, 28.0), (2, 40.0)):
        x = np.clip(np.rint(r.normal(0, sigma, (2048, 768))), -128, 127).astype(np.int8)
        g = r.integers(32, 128, 768).astype(np.int16)
        bt = (r.integers(-15, 16, 768).astype(np.int32) << 11).astype(np.int16)  # beta / 16 in Q15
        yield f'c5 ln{i} [2048, 768]', x, g, bt, 4


@pytest.mark.parametrize('name,x,gamma,beta,out_shift', list(cases()), ids=lambda v: v if isinstance(v, str) else '')
def test_inv_std_definition_moves_outputs_by_at_most_one_lsb(oracle, name, x, gamma, beta, out_shift):
    ref = layernorm_np(x, gamma, beta, out_shift, how='nearest')
    assert np.array_equal(ref, oracle.layernorm(x, gamma, beta, out_shift, 'conv_even')), 'numpy restatement != oracle'
    report = {}
    for how in ('plus1', 'minus1', 'floor', 'float32_trunc', 'float32_round'):
        y = layernorm_np(x, gamma, beta, out_shift, how=how)
        d = np.abs(y.astype(np.int16) - ref)
        report[how] = (int(d.max()), float((d > 0).mean()))
        assert d.max() <= 1, f'{name}: {how} moves an output by {int(d.max())} LSB'
    for how in ('floor', 'float32_trunc', 'float32_round'):
        assert report[how][1] < 0.02, f'{name}: {how} moves {report[how][1]:.2%} of the outputs'
    print(name, {k: (m, f'{f:.3%}') for k, (m, f) in report.items()})


def test_nearest_q15_against_exact_rationals():
    """The pluggable reciprocal square root itself, nearest form, against exact arithmetic on a few values."""
    for v in (1, 2, 3, 4, 5, 7, 100, 399, 400, 401, 65535, 1 << 20, (1 << 30) - 1):
        q = int(rsqrt_q15(np.array([v]), 'nearest')[0])
        if v == 1:
            assert q == 32767
            continue
        # |q - 2^15/sqrt(v)| <= 1/2  <=>  (2q - 1)^2 v <= 2^32 <= (2q + 1)^2 v
        assert Fraction((2 * q - 1) ** 2 * v) <= (1 << 32) <= Fraction((2 * q + 1) ** 2 * v)
