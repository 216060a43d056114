"""Pins the CPU oracle against what the mathematics fixes, independently of its own formulas.

Every check here uses a different formulation than the oracle's C code: exact rationals for the
rounding modes, numpy int64 matmul for the GEMMs, python big ints for the integer softmax steps,
closed forms / invariants / float references with explicit error bounds for the rest.
"""

import math
from fractions import Fraction

import numpy as np
import pytest

MODES = ['floor', 'ceil', 'positive_inf', 'negative_inf', 'symmetric_inf', 'symmetric_zero', 'conv_even',
         'conv_odd']
RANGE = {'int8': (-128, 127), 'uint8': (0, 255), 'int16': (-32768, 32767), 'int32': (-2**31, 2**31 - 1)}


def exact_round(x: Fraction, mode: str) -> int:
    """Textbook definition of each AIE rounding mode on an exact rational."""
    lo = math.floor(x)
    frac = x - lo
    if mode == 'floor':
        return lo
    if mode == 'ceil':
        return math.ceil(x)
    if frac != Fraction(1, 2):
        return lo + (1 if frac > Fraction(1, 2) else 0)
    # exact tie between lo and lo+1
    if mode == 'positive_inf':
        return lo + 1
    if mode == 'negative_inf':
        return lo
    if mode == 'symmetric_inf':
        return lo + 1 if x > 0 else lo
    if mode == 'symmetric_zero':
        return lo if x > 0 else lo + 1
    if mode == 'conv_even':
        return lo if lo % 2 == 0 else lo + 1
    if mode == 'conv_odd':
        return lo if lo % 2 != 0 else lo + 1
    raise AssertionError(mode)


def exact_srs(acc: int, shift: int, mode: str, kind: str) -> int:
    q = exact_round(Fraction(acc, 1 << shift), mode)
    lo, hi = RANGE[kind]
    return min(max(q, lo), hi)


@pytest.mark.parametrize('mode', MODES)
def test_srs_bruteforce_window(oracle, mode):
    # every accumulator in a window around zero x every shift 0..12, plus extremes
    accs = list(range(-1100, 1101)) + [2**31 - 1, -2**31, 2**31 - 2, -2**31 + 1, 2**30, -2**30, 12345678, -12345678]
    for shift in list(range(0, 13)) + [15, 20, 31]:
        for kind in ('int8', 'uint8', 'int16', 'int32'):
            got = oracle.srs(np.array(accs), shift, mode, kind)
            exp = [exact_srs(a, shift, mode, kind) for a in accs]
            assert got.tolist() == exp, (mode, shift, kind)


def test_srs_known_ties(oracle):
    # 2.5 and -2.5 and 3.5 with shift 1
    table = {
        'floor': (2, -3, 3), 'ceil': (3, -2, 4), 'positive_inf': (3, -2, 4), 'negative_inf': (2, -3, 3),
        'symmetric_inf': (3, -3, 4), 'symmetric_zero': (2, -2, 3), 'conv_even': (2, -2, 4),
        'conv_odd': (3, -3, 3),
    }
    for mode, (p, n, q) in table.items():
        assert oracle.srs(np.array([5, -5, 7]), 1, mode, 'int32').tolist() == [p, n, q], mode


def _rng(seed):
    return np.random.default_rng(seed)


@pytest.mark.parametrize('a_dtype', [np.int8, np.uint8])
@pytest.mark.parametrize('mode', ['floor', 'positive_inf', 'symmetric_inf', 'conv_even'])
def test_dense_vs_int64_matmul(oracle, a_dtype, mode):
    r = _rng(1)
    M, K, N = 37, 83, 29
    lo, hi = (0, 256) if a_dtype == np.uint8 else (-128, 128)
    A = r.integers(lo, hi, (M, K)).astype(a_dtype)
    W = r.integers(-128, 128, (K, N)).astype(np.int8)
    bias = r.integers(-2**14, 2**14, N).astype(np.int32)
    shifts = r.integers(4, 11, N).astype(np.int32)
    acc = A.astype(np.int64) @ W.astype(np.int64) + bias
    for relu in (False, True):
        for out in ('int8', 'uint8', 'int16'):
            exp = np.array([[exact_srs(int(acc[m, n]), int(shifts[n]), mode, out) for n in range(N)]
                            for m in range(M)])
            if relu:
                exp = np.maximum(exp, 0)
            got = oracle.dense(A, W, bias, shifts, mode, relu=relu, out=out)
            assert np.array_equal(got.astype(np.int64), exp)
    # scalar shift == vector of equal shifts (the per-channel extension reduces to the reference)
    a = oracle.dense(A, W, bias, 7, mode)
    b = oracle.dense(A, W, bias, np.full(N, 7), mode)
    assert np.array_equal(a, b)


def test_dense_int16_activations_vs_int64_matmul(oracle):
    """(16, 8) Dense: int64 numpy product wrapped to 32 bits, then the exact srs; includes a wrapping bias."""
    r = _rng(61)
    A = r.integers(-32768, 32768, (9, 70)).astype(np.int16)
    W = r.integers(-128, 128, (70, 11)).astype(np.int8)
    for bias in (r.integers(-2**20, 2**20, 11).astype(np.int32), np.full(11, 2**31 - 1000, dtype=np.int32)):
        acc = A.astype(np.int64) @ W.astype(np.int64) + bias.astype(np.int64)
        acc = ((acc + 2**31) % 2**32) - 2**31
        for mode, shift, kind in (('conv_even', 9, 'int16'), ('symmetric_inf', 14, 'int8'), ('floor', 0, 'int16')):
            want = np.array([[exact_srs(int(v), shift, mode, kind) for v in row] for row in acc])
            np.testing.assert_array_equal(oracle.dense(A, W, bias, shift, mode, out=kind), want)


def test_dense_special_cases(oracle):
    r = _rng(2)
    K = 16
    A = r.integers(-128, 128, (8, K)).astype(np.int8)
    eye = np.eye(K, dtype=np.int8)
    # W = I, shift 0: identity
    assert np.array_equal(oracle.dense(A, eye, None, 0, 'floor'), A)
    # W = 0: out = srs(bias)
    bias = np.array([64, -64, 63, -65, 192, -192, 2**31 - 1, -2**31] * 2, dtype=np.int32)
    got = oracle.dense(A, np.zeros((K, K), np.int8), bias, 7, 'conv_even')
    exp = [exact_srs(int(b), 7, 'conv_even', 'int8') for b in bias]
    assert (got == np.array(exp, dtype=np.int8)).all()
    # accumulator wraps modulo 2^32 (acc32), it does not saturate
    A1 = np.full((1, 4), 127, np.int8)
    W1 = np.full((4, 1), 127, np.int8)
    big = np.array([2**31 - 1], np.int32)
    wrapped = (4 * 127 * 127 + 2**31 - 1 + 2**31) % 2**32 - 2**31
    assert oracle.dense(A1, W1, big, 0, 'floor', out='int32')[0, 0] == wrapped


def test_matmul_batched_and_transposed(oracle):
    r = _rng(3)
    A = r.integers(-128, 128, (2, 3, 17, 24)).astype(np.int8)
    B = r.integers(-128, 128, (2, 3, 24, 11)).astype(np.int8)
    acc = A.astype(np.int64) @ B.astype(np.int64)
    exp = np.vectorize(lambda v: exact_srs(int(v), 6, 'conv_even', 'int8'))(acc)
    assert np.array_equal(oracle.matmul(A, B, 6, 'conv_even').astype(np.int64), exp)
    Bt = np.ascontiguousarray(np.swapaxes(B, -1, -2))
    assert np.array_equal(oracle.matmul(A, Bt, 6, 'conv_even', trans_b=True).astype(np.int64), exp)
    # unsigned lhs (probabilities) x signed rhs
    P = r.integers(0, 256, (2, 3, 17, 24)).astype(np.uint8)
    acc = P.astype(np.int64) @ B.astype(np.int64)
    exp = np.vectorize(lambda v: exact_srs(int(v), 8, 'symmetric_inf', 'int8'))(acc)
    assert np.array_equal(oracle.matmul(P, B, 8, 'symmetric_inf').astype(np.int64), exp)


def test_matmul_int16_left_operand_against_python_integers(oracle):
    """The 16-bit MatMul combinations: int16 x int8 wraps to 32 bits before the shift (acc32), int16 x int16 keeps
    64 bits (acc64); checked against exact integer matrix products and the rational rounding above."""
    r = _rng(9)
    A = r.integers(-32768, 32768, (2, 9, 40)).astype(np.int16)
    A[0, 0] = 32767
    A[1, 1] = -32768
    for b_dtype, shift, wrap in ((np.int8, 13, True), (np.int16, 21, False)):
        lo, hi = (-128, 128) if b_dtype == np.int8 else (-32768, 32768)
        B = r.integers(lo, hi, (2, 40, 7)).astype(b_dtype)
        B[0, :, 0] = hi - 1
        B[1, :, 1] = lo
        acc = A.astype(np.int64) @ B.astype(np.int64)
        if wrap:
            acc = ((acc + 2**31) % 2**32) - 2**31
        for mode, kind in (('conv_even', 'int16'), ('symmetric_inf', 'int8'), ('floor', 'int16')):
            exp = np.vectorize(lambda v: exact_srs(int(v), shift, mode, kind))(acc)
            assert np.array_equal(oracle.matmul(A, B, shift, mode, out=kind).astype(np.int64), exp), (b_dtype, mode)
            Bt = np.ascontiguousarray(np.swapaxes(B, -1, -2))
            assert np.array_equal(oracle.matmul(A, Bt, shift, mode, trans_b=True, out=kind).astype(np.int64), exp)


def test_add_is_saturating(oracle):
    a = np.arange(-128, 128, dtype=np.int8).repeat(256)
    b = np.tile(np.arange(-128, 128, dtype=np.int8), 256)
    exp = np.clip(a.astype(np.int32) + b.astype(np.int32), -128, 127).astype(np.int8)
    assert np.array_equal(oracle.add(a, b), exp)
    au, bu = a.view(np.uint8), b.view(np.uint8)
    expu = np.clip(au.astype(np.int32) + bu.astype(np.int32), 0, 255).astype(np.uint8)
    assert np.array_equal(oracle.add(au, bu), expu)
    # shift 1 halves with the requested rounding
    s = a.astype(np.int32) + b.astype(np.int32)
    exp1 = np.array([exact_srs(int(v), 1, 'conv_even', 'int8') for v in s], dtype=np.int8)
    assert np.array_equal(oracle.add(a, b, 1, 'conv_even'), exp1)


# ---- integer exp softmax ---------------------------------------------------------------------

def py_exp_score(d: int, kq: int) -> int:
    """Python big-int restatement of the reference's exp_score16 steps (softmax.cpp:252-273)."""
    z = min(d * kq, 32767)
    zi, zf = z >> 8, z & 255
    t = (zf * 2811) >> 8
    e = (((t - 11004) * zf) >> 8) + 16384
    for b in range(4):
        if zi & (1 << b):
            e >>= (1 << b)
    return 0 if zi >= 16 else e


def test_exp_score_exhaustive(oracle):
    worst = 0.0
    for kq in range(1, 129):
        for d in range(256):
            e = oracle.exp_score16(d, kq)
            assert e == py_exp_score(d, kq), (d, kq)
            # and it really is 2^(-d*kq/256) in Q14, within the 2nd-order polynomial's error
            ideal = 16384.0 * 2.0 ** (-(d * kq) / 256.0)
            worst = max(worst, abs(e - ideal))
            assert abs(e - ideal) <= 40.0, (d, kq, e, ideal)
    assert oracle.exp_score16(0, 23) == 16384
    assert worst > 0.0


def py_softmax_exp(row, kq, inv_shift=15):
    m = max(row)
    e = [py_exp_score(m - v, kq) for v in row]
    inv = (255 << inv_shift) // max(sum(e), 1)
    return [min(255, (x * inv) >> inv_shift) for x in e]


def test_softmax_exp_rows(oracle):
    r = _rng(4)
    x = np.clip(np.rint(r.normal(0, 24, (64, 96))), -128, 127).astype(np.int8)
    for kq in (1, 23, 46, 128):
        got = oracle.softmax_exp(x, kq)
        exp = np.array([py_softmax_exp(list(map(int, row)), kq) for row in x], dtype=np.uint8)
        assert np.array_equal(got, exp), kq
    # float softmax of the dequantised logits, frac 4 -> kq 23: within a few codes of 255*p
    xf = x.astype(np.float64) / 16.0
    p = np.exp(xf - xf.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    assert np.abs(oracle.softmax_exp(x, 23).astype(np.float64) - 255.0 * p).max() <= 3.0
    # invariants: uniform row of C=512 -> inv = floor(510/512) = 0 -> all-zero probabilities
    assert not oracle.softmax_exp(np.zeros((1, 512), np.int8), 23).any()
    # uniform row of 32 -> inv = floor(255*2^15/(32*16384)) = 15 -> (16384*15)>>15 = 7
    assert (oracle.softmax_exp(np.full((1, 32), 5, np.int8), 23) == 7).all()
    # one-hot dominant row -> the max gets 255
    one = np.full((1, 64), -128, np.int8)
    one[0, 7] = 127
    o = oracle.softmax_exp(one, 64)
    assert o[0, 7] == 255 and o.sum() == 255


def test_softmax_exp_int16_out(oracle):
    r = _rng(5)
    x = r.integers(-128, 128, (16, 64)).astype(np.int8)
    got = oracle.softmax_exp(x, 23, out='int16')
    for row, g in zip(x, got):
        m = int(row.max())
        e = [py_exp_score(m - int(v), 23) for v in row]
        inv = 32767 // sum(e)
        assert g.tolist() == [min(32767, v * inv) for v in e]


def py_softmax_hccs(row, B, S, Dmax, inv_shift=15, out='uint8'):
    m = max(row)
    sc = [B - S * min(m - v, Dmax) for v in row]
    if out == 'uint8':
        inv = (255 << inv_shift) // sum(sc)
        return [min(255, max(0, (s * inv) >> inv_shift)) for s in sc]
    inv = 32767 // sum(sc)
    return [min(32767, s * inv) for s in sc]


def test_softmax_hccs_rows(oracle):
    r = _rng(6)
    x = np.clip(np.rint(r.normal(0, 24, (48, 512))), -128, 127).astype(np.int8)
    for (B, S, Dmax) in [(60, 1, 59), (63, 2, 31), (40, 0, 0), (33, 1, 32)]:
        got = oracle.softmax_hccs(x, B, S, Dmax)
        exp = np.array([py_softmax_hccs(list(map(int, row)), B, S, Dmax) for row in x], dtype=np.uint8)
        assert np.array_equal(got, exp)
        got16 = oracle.softmax_hccs(x, B, S, Dmax, out='int16')
        exp16 = np.array([py_softmax_hccs(list(map(int, row)), B, S, Dmax, out='int16') for row in x],
                         dtype=np.int16)
        assert np.array_equal(got16, exp16)
    # S = 0 -> uniform: every output = floor(B * floor(255*2^15/(C*B)) / 2^15)
    o = oracle.softmax_hccs(x[:1], 40, 0, 0)
    inv = (255 << 15) // (512 * 40)
    assert (o == ((40 * inv) >> 15)).all()
    # sum of codes never exceeds 255 and is close to it for a peaked surrogate
    o = oracle.softmax_hccs(x, 60, 1, 59).astype(np.int64).sum(-1)
    assert (o <= 255).all()


# ---- LayerNorm ---------------------------------------------------------------------------------

def exact_rsqrt_q15(v: int) -> int:
    """Nearest integer to 2^15/sqrt(v), by exact comparison of squares (independent of libm)."""
    # q = floor(2^15/sqrt(v) + 1/2): largest q with (q - 1/2)^2 <= 2^30 / v
    q = math.isqrt((1 << 32) // v) // 2  # coarse start, then fix up exactly
    while Fraction(2 * q + 1, 2) ** 2 * v <= (1 << 30):
        q += 1
    while q > 0 and Fraction(2 * q - 1, 2) ** 2 * v > (1 << 30):
        q -= 1
    return min(q, 32767)


def test_rsqrt_q15(oracle):
    vals = list(range(1, 5000)) + [16384, 16385, 16383, 65535, 65536, 10**6, 2**30, 2**31 - 1]
    vals += [int(v) for v in _rng(7).integers(1, 2**31 - 1, 2000)]
    for v in vals:
        assert oracle.rsqrt_q15(v) == exact_rsqrt_q15(v), v
    assert oracle.rsqrt_q15(1) == 32767       # 32768 clamps
    assert oracle.rsqrt_q15(4) == 16384
    assert oracle.rsqrt_q15(16384) == 256


def py_layernorm_row(x, gamma, beta, out_shift, mode, eps_q0=1):
    C = len(x)
    sx, sq = sum(x), sum(v * v for v in x)
    mu = (sx + C // 2) // C
    var = max(0, (sq - 2 * mu * sx + C * mu * mu) // C)
    inv = exact_rsqrt_q15(var + eps_q0)
    out = []
    for v, g, b in zip(x, gamma, beta):
        fs = exact_srs(inv * g, 7, mode, 'int16')
        out.append(exact_srs((v - mu) * fs + b, 15 - out_shift, mode, 'int8'))
    return out


@pytest.mark.parametrize('cols', [32, 128, 1024, 768, 48])
@pytest.mark.parametrize('mode', ['conv_even', 'symmetric_inf', 'floor'])
def test_layernorm_rows(oracle, cols, mode):
    r = _rng(8)
    x = np.clip(np.rint(r.normal(3, 20, (24, cols))), -128, 127).astype(np.int8)
    gamma = r.integers(32, 128, cols).astype(np.int16)
    beta = (r.integers(-16, 17, cols) << 10).astype(np.int16)
    for out_shift in (5, 4, 7):
        got = oracle.layernorm(x, gamma, beta, out_shift, mode)
        exp = np.array([py_layernorm_row(list(map(int, row)), gamma.tolist(), beta.tolist(), out_shift, mode)
                        for row in x], dtype=np.int8)
        assert np.array_equal(got, exp)


def test_layernorm_invariants_and_float(oracle):
    r = _rng(9)
    cols = 256
    gamma = r.integers(32, 128, cols).astype(np.int16)
    beta = (r.integers(-16, 17, cols) << 10).astype(np.int16)
    # constant row -> centred value 0 -> out = srs(beta, 15 - out_shift)
    const = np.full((1, cols), 17, np.int8)
    got = oracle.layernorm(const, gamma, beta, 5, 'conv_even')
    assert got[0].tolist() == [exact_srs(int(b), 10, 'conv_even', 'int8') for b in beta]
    # mean is rounded half-up: sum = C/2 -> mu = 1; sum = -C/2 -> mu = 0 (gamma large makes mu visible)
    x = np.zeros((2, cols), np.int8)
    x[0, :cols // 2] = 1
    x[1, :cols // 2] = -1
    g1 = np.full(cols, 128, np.int16)
    b0 = np.zeros(cols, np.int16)
    o = oracle.layernorm(x, g1, b0, 5, 'conv_even').astype(np.int64)
    # row0: mu=1 -> centred {0 (x=1), -1 (x=0)}: var = (C/2)/C -> 0 -> inv = 32767 (eps=1), fs = sat16(32767)
    assert o[0, 0] == 0 and o[0, -1] == exact_srs(-32767, 10, 'conv_even', 'int8')
    assert o[1, 0] == exact_srs(-32767, 10, 'conv_even', 'int8') and o[1, -1] == 0
    # against float LayerNorm: |error| <= 1.5 output LSB for well-conditioned rows
    xs = np.clip(np.rint(r.normal(0, 25, (64, cols))), -128, 127).astype(np.int8)
    out_shift = 5
    got = oracle.layernorm(xs, gamma, beta, out_shift, 'conv_even').astype(np.float64)
    xf = xs.astype(np.float64)
    ref = (xf - xf.mean(-1, keepdims=True)) / np.sqrt(xf.var(-1, keepdims=True) + 1.0)
    ref = ref * (gamma / 128.0) + beta / 32768.0
    ref = np.clip(ref * (1 << out_shift), -128, 127)
    assert np.abs(got - ref).max() <= 1.5


def test_add_layernorm_is_composition(oracle):
    r = _rng(10)
    a = np.clip(np.rint(r.normal(0, 60, (32, 128))), -128, 127).astype(np.int8)
    b = np.clip(np.rint(r.normal(0, 60, (32, 128))), -128, 127).astype(np.int8)
    gamma = r.integers(32, 128, 128).astype(np.int16)
    beta = (r.integers(-16, 17, 128) << 10).astype(np.int16)
    s, out = oracle.add_layernorm(a, b, gamma, beta, 5, 'conv_even', return_sum=True)
    s2 = oracle.add(a, b)
    assert np.array_equal(s, s2)
    assert np.array_equal(out, oracle.layernorm(s2, gamma, beta, 5, 'conv_even'))


# ---- float path: the conversions are checked against an independent library routine (torch's CPU casts) ----------

def test_bf16_conversions_against_torch_cpu(oracle):
    torch = pytest.importorskip('torch')
    r = np.random.default_rng(3)
    x = np.concatenate([r.normal(0, 1, 20000), r.normal(0, 1e-3, 2000), r.normal(0, 1e4, 2000),
                        [0.0, -0.0, 1.0, -1.0, 3.0e38, -3.0e38, 1e-40, np.inf, -np.inf]]).astype(np.float32)
    # exact ties: odd bfloat16 neighbours' midpoints, where round-to-nearest-even and half-up differ
    base = (r.integers(0x3000, 0x4800, 4000).astype(np.uint32) << 16) | 0x8000
    x = np.concatenate([x, base.view(np.float32), (base | 0x80000000).view(np.float32)])
    want = torch.from_numpy(x).to(torch.bfloat16).float().numpy()
    assert np.array_equal(oracle.bf16_round(x).view(np.uint32), want.view(np.uint32))
    t = oracle.bf16_truncate(x)
    assert np.all((t.view(np.uint32) & 0xFFFF) == 0)
    fin = np.isfinite(x)
    assert np.all(np.abs(t[fin]) <= np.abs(x[fin]))                       # toward zero
    up = ((t.view(np.uint32) + 0x10000).view(np.float32))                  # next bfloat16 away from zero
    assert np.all(np.abs(x[fin]) < np.abs(up[fin]))                        # and less than one step away


def test_float_dense_oracle_against_float64_identity_and_linearity(oracle):
    r = np.random.default_rng(4)
    A = oracle.bf16_truncate(r.normal(0, 1, (9, 40)))
    W = oracle.bf16_truncate(r.normal(0, 1, (40, 7)))
    b = r.normal(0, 1, 7).astype(np.float32)
    y = oracle.dense_float(A, W, b, relu=False, fmt='float32')
    want = np.array([[sum(float(A[m, k]) * float(W[k, n]) for k in range(40)) + float(b[n]) for n in range(7)]
                     for m in range(9)])
    assert np.allclose(y, want, rtol=2.0 ** -23, atol=0)
    yb = oracle.dense_float(A, W, b, relu=True, fmt='bfloat16')
    assert np.array_equal(yb, oracle.bf16_round(np.maximum(want, 0).astype(np.float32)))
    assert np.array_equal(oracle.dense_float(A, np.eye(40, dtype=np.float32), None, fmt='bfloat16'), A)
    assert np.array_equal(oracle.matmul_float(A, W.T.copy(), trans_b=True, fmt='float32'),
                          oracle.matmul_float(A, W, fmt='float32'))


def test_fp8_e4m3_codec_against_torch_cpu(oracle):
    torch = pytest.importorskip('torch')
    codes = np.arange(256, dtype=np.uint8)
    want = torch.from_numpy(codes).view(torch.float8_e4m3fn).float().numpy()      # independent decoder
    got = oracle.fp8_decode(codes)
    assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(got[~np.isnan(got)], want[~np.isnan(want)])
    fin = ~np.isnan(got)
    assert np.array_equal(oracle.fp8_encode(got[fin]), codes[fin])               # every value encodes to its own code
    # away from ties and below the largest value both round to nearest: the recipe must agree with torch's cast
    r = np.random.default_rng(8)
    x = np.concatenate([r.normal(0, 1, 20000), r.normal(0, 30, 5000), r.normal(0, 0.01, 5000)]).astype(np.float32)
    x = x[np.abs(x) < 440]
    t = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
    mine = oracle.fp8_encode(x)
    lo, hi = np.minimum(oracle.fp8_decode(mine), oracle.fp8_decode(t)), np.maximum(oracle.fp8_decode(mine), oracle.fp8_decode(t))
    tie = (lo != hi) & (np.abs((lo.astype(np.float64) + hi) / 2 - x) == 0)
    assert np.all((mine == t) | tie | ((mine & 0x7F) == 0) & ((t & 0x7F) == 0))   # +-0 may differ in sign handling
    # ties go away from zero (the recipe adds half a step to the magnitude), overflow gives 0x7f
    assert oracle.fp8_encode(np.float32([1.0625, -1.0625, 464.0, 480.0, 1e9, 2.0 ** -10, 2.0 ** -9])).tolist() == \
        [0x39, 0xB9, 0x7F, 0x7F, 0x7F, 0x01, 0x01]


def test_dense_int16x16_against_python_integers(oracle):
    r = np.random.default_rng(12)
    A = r.integers(-32768, 32768, (6, 50)).astype(np.int16)
    W = r.integers(-32768, 32768, (50, 7)).astype(np.int16)
    A[0, :], W[:, 0] = -32768, -32768     # 50 * 2^30: the 64-bit accumulator must not wrap at 32 bits
    bias = r.integers(-2**31, 2**31, 7).astype(np.int32)
    for mode, s in (('floor', 20), ('conv_even', 17), ('symmetric_inf', 33), ('ceil', 0)):
        got = oracle.dense(A, W, bias, s, mode, out='int16')
        for m in range(6):
            for n in range(7):
                acc = int(bias[n]) + sum(int(A[m, k]) * int(W[k, n]) for k in range(50))
                assert got[m, n] == exact_srs(acc, s, mode, 'int16'), (mode, m, n)
