#!/usr/bin/env python3
"""Writes the golden vectors under tests/golden/ (run from the repository root: python tests/golden/make_golden.py).

Every expected output here is computed with exact Python integers and rationals from the definition of the
operation (the reference's kernels restated step by step, file:line in each function) — not with the C oracle
and not with the GPU library — so the fixtures anchor both of them independently. Inputs are seeded; sizes are
small because the arithmetic is done one Python integer at a time.
"""

import math
from fractions import Fraction
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
MODES = ['floor', 'ceil', 'positive_inf', 'negative_inf', 'symmetric_inf', 'symmetric_zero', 'conv_even', 'conv_odd']
RANGE = {'int8': (-128, 127), 'uint8': (0, 255), 'int16': (-32768, 32767)}
NPDT = {'int8': np.int8, 'uint8': np.uint8, 'int16': np.int16}


def exact_round(x: Fraction, mode: str) -> int:
    """AIE-API rounding modes on an exact rational (the tokens of op_impls/utils/precision.py:13-21)."""
    lo = math.floor(x)
    frac = x - lo
    if mode == 'floor':
        return lo
    if mode == 'ceil':
        return math.ceil(x)
    if frac != Fraction(1, 2):
        return lo + (1 if frac > Fraction(1, 2) else 0)
    return {'positive_inf': lo + 1, 'negative_inf': lo, 'symmetric_inf': lo + 1 if x > 0 else lo,
            'symmetric_zero': lo if x > 0 else lo + 1, 'conv_even': lo if lo % 2 == 0 else lo + 1,
            'conv_odd': lo if lo % 2 else lo + 1}[mode]


def srs(acc: int, shift: int, mode: str, kind: str) -> int:
    """to_vector<T>(acc, shift): shift, round, saturate (dense_bias_relu.cpp:153-163)."""
    lo, hi = RANGE[kind]
    return min(max(exact_round(Fraction(acc, 1 << shift), mode), lo), hi)


def wrap32(v: int) -> int:
    v &= 0xFFFFFFFF
    return v - (1 << 32) if v >= (1 << 31) else v


def dense(A, W, bias, shifts, mode, relu, kind, acc64=False):
    """dense_bias_relu.cpp:112-163. acc64: the (16, 16) width combination, whose accumulator does not wrap at
    32 bits (precision.py:122-123)."""
    M, K = A.shape
    N = W.shape[1]
    out = np.zeros((M, N), dtype=NPDT[kind])
    for m in range(M):
        for n in range(N):
            acc = int(bias[n]) + sum(int(A[m, k]) * int(W[k, n]) for k in range(K))
            if not acc64:
                acc = wrap32(acc)
            y = srs(acc, int(shifts[n]), mode, kind)
            out[m, n] = max(y, 0) if relu else y
    return out


def matmul(A, B, shift, mode, kind):
    """matmul.cpp:80-115, B given as [K, N]."""
    return dense(A, B, np.zeros(B.shape[1], dtype=np.int64), np.full(B.shape[1], shift), mode, False, kind)


def exp_score(d: int, kq: int) -> int:
    """softmax.cpp:252-273."""
    z = min(d * kq, 32767)
    zi, zf = z >> 8, z & 255
    t = (zf * 2811) >> 8
    e = (((t - 11004) * zf) >> 8) + 16384
    e >>= (zi & 15)
    return 0 if zi >= 16 else e


def softmax_exp_row(row, kq, kind='uint8'):
    """softmax.cpp:333-384."""
    m = max(row)
    e = [exp_score(m - v, kq) for v in row]
    if kind == 'uint8':
        inv = min((255 << 15) // max(sum(e), 1), 32767)
        return [min(255, (x * inv) >> 15) for x in e]
    inv = 32767 // max(sum(e), 1)
    return [min(32767, x * inv) for x in e]


def softmax_hccs_row(row, B, S, Dmax, kind='uint8'):
    """softmax.cpp:19-101 (default inv_shift 15, no clb). Parameters must satisfy validate_hccs_params
    (softmax/common.py:59-89): then sum >= 256 and the reciprocal fits the kernel's int16 without narrowing."""
    m = max(row)
    sc = [B - S * min(m - v, Dmax) for v in row]
    if kind == 'uint8':
        inv = (255 << 15) // sum(sc)
        return [min(255, max(0, (s * inv) >> 15)) for s in sc]
    inv = 32767 // sum(sc)
    return [min(32767, s * inv) for s in sc]


def rsqrt_q15(v: int) -> int:
    """Nearest Q15 of 1/sqrt(v) by exact comparison of squares, clamped to int16 (layer_norm.cpp:33-34; the
    rounding of the AIE's float path is this build's definition)."""
    q = math.isqrt((1 << 32) // v) // 2
    while Fraction(2 * q + 1, 2) ** 2 * v <= (1 << 30):
        q += 1
    while q > 0 and Fraction(2 * q - 1, 2) ** 2 * v > (1 << 30):
        q -= 1
    return min(q, 32767)


def layernorm_row(x, gamma, beta, out_shift, mode, eps_q0=1):
    """layer_norm.cpp:14-40, 95-119 (floor division = the reference's shifts for power-of-two widths)."""
    C = len(x)
    sx, sq = sum(x), sum(v * v for v in x)
    mu = (sx + C // 2) // C
    var = max(0, (sq - 2 * mu * sx + C * mu * mu) // C)
    inv = rsqrt_q15(var + eps_q0)
    out = []
    for v, g, b in zip(x, gamma, beta):
        fs = srs(inv * g, 7, mode, 'int16')
        out.append(srs((v - mu) * fs + b, 15 - out_shift, mode, 'int8'))
    return out


def gauss8(r, sigma, shape):
    return np.clip(np.rint(r.normal(0, sigma, shape)), -128, 127).astype(np.int8)


def main():
    r = np.random.default_rng(20240917)

    # ---- srs: a window around zero, ties, large magnitudes ------------------------------------------
    acc = np.concatenate([np.arange(-70, 71), r.integers(-2**31, 2**31, 200), [2**31 - 1, -2**31, 2**30, -2**30]]).astype(np.int64)
    srs_out = {}
    for mode in MODES:
        for shift in (0, 1, 3, 7, 12):
            for kind in ('int8', 'uint8', 'int16'):
                srs_out[f'{mode}__{shift}__{kind}'] = np.array([srs(int(a), shift, mode, kind) for a in acc], dtype=NPDT[kind])
    np.savez_compressed(HERE / 'srs.npz', acc=acc, **srs_out)

    # ---- dense ---------------------------------------------------------------------------------------
    A = gauss8(r, 40, (12, 40))
    Au = r.integers(0, 256, (12, 40)).astype(np.uint8)
    W = gauss8(r, 30, (40, 20))
    bias = r.integers(-3000, 3001, 20).astype(np.int32)
    shifts = r.integers(4, 9, 20).astype(np.int32)
    d = {'A': A, 'Au': Au, 'W': W, 'bias': bias, 'shifts': shifts}
    for mode in MODES:
        d[f'y__{mode}__relu'] = dense(A, W, bias, shifts, mode, True, 'int8')
        d[f'y__{mode}__scalar6'] = dense(A, W, bias, np.full(20, 6), mode, False, 'int8')
    d['y__u8in__conv_even'] = dense(Au, W, bias, shifts, 'conv_even', False, 'int8')
    d['y__u8out__symmetric_inf'] = dense(A, W, bias, shifts, 'symmetric_inf', True, 'uint8')
    d['y__i16out__conv_even'] = dense(A, W, bias, np.full(20, 2), 'conv_even', False, 'int16')
    big = np.full(20, 2**31 - 5, dtype=np.int64)  # accumulator wraps to negative
    d['bias_wrap'] = big.astype(np.int32)
    d['y__wrap'] = dense(np.abs(A), np.abs(W), big, np.full(20, 10), 'floor', False, 'int8')
    A16 = r.integers(-32768, 32768, (12, 40)).astype(np.int16)
    d['A16'] = A16
    d['y__i16in__conv_even__i16'] = dense(A16, W, bias, np.full(20, 9), 'conv_even', False, 'int16')
    d['y__i16in__symmetric_inf__i8relu'] = dense(A16, W, bias, shifts + 8, 'symmetric_inf', True, 'int8')
    np.savez_compressed(HERE / 'dense.npz', **d)

    # ---- dense, int16 x int16 with a 64-bit accumulator (its own generator: the vectors above stay as they are) ---
    r16 = np.random.default_rng(20250301)
    A16b = r16.integers(-32768, 32768, (10, 48)).astype(np.int16)
    W16 = r16.integers(-32768, 32768, (48, 12)).astype(np.int16)
    A16b[0, :], W16[:, 0] = -32768, -32768          # the largest products: 48 * 2^30 needs more than 32 bits
    A16b[1, :], W16[:, 1] = 32767, -32768
    bias16 = r16.integers(-2**31, 2**31, 12).astype(np.int64)
    d16 = {'A': A16b, 'W': W16, 'bias': bias16.astype(np.int32)}
    sh16 = r16.integers(14, 30, 12).astype(np.int32)
    d16['shifts'] = sh16
    for mode in MODES:
        d16[f'y__{mode}__i16'] = dense(A16b, W16, bias16, sh16, mode, False, 'int16', acc64=True)
    d16['y__conv_even__i8relu__s24'] = dense(A16b, W16, bias16, np.full(12, 24), 'conv_even', True, 'int8', acc64=True)
    d16['y__floor__i16__s36'] = dense(A16b, W16, bias16, np.full(12, 36), 'floor', False, 'int16', acc64=True)
    np.savez_compressed(HERE / 'dense16.npz', **d16)

    # ---- matmul (batched, both operand orders, uint8 left operand) -------------------------------------
    Aq = gauss8(r, 30, (2, 10, 32))
    Bk = gauss8(r, 30, (2, 12, 32))       # [N, K]: transposed right operand
    P = r.integers(0, 256, (2, 10, 32)).astype(np.uint8)
    Bv = gauss8(r, 30, (2, 32, 16))       # [K, N]
    m = {'Aq': Aq, 'Bk': Bk, 'P': P, 'Bv': Bv}
    for mode in ('conv_even', 'symmetric_inf', 'floor'):
        m[f'qk__{mode}'] = np.stack([matmul(Aq[b], Bk[b].T, 5, mode, 'int8') for b in range(2)])
        m[f'pv__{mode}'] = np.stack([matmul(P[b], Bv[b], 8, mode, 'int8') for b in range(2)])
    np.savez_compressed(HERE / 'matmul.npz', **m)

    # ---- add -------------------------------------------------------------------------------------------
    a = r.integers(-128, 128, 300).astype(np.int8)
    b = r.integers(-128, 128, 300).astype(np.int8)
    au, bu = a.view(np.uint8), b.view(np.uint8)
    np.savez_compressed(HERE / 'add.npz', a=a, b=b,
                        y_i8=np.array([srs(int(x) + int(y), 0, 'floor', 'int8') for x, y in zip(a, b)], dtype=np.int8),
                        y_u8=np.array([srs(int(x) + int(y), 0, 'floor', 'uint8') for x, y in zip(au, bu)], dtype=np.uint8),
                        y_i8_shift1_conv_even=np.array([srs(int(x) + int(y), 1, 'conv_even', 'int8') for x, y in zip(a, b)],
                                                       dtype=np.int8))

    # ---- layernorm (power-of-two and 48 columns; constant and extreme rows) ---------------------------
    ln = {}
    for cols in (64, 48):
        x = gauss8(r, 25, (6, cols))
        x[0, :] = 17                       # constant row: variance 0
        x[1, :] = np.where(np.arange(cols) % 2, 127, -128)
        gamma = r.integers(-128, 129, cols).astype(np.int16)
        beta = (r.integers(-16, 17, cols) << 10).astype(np.int16)
        ln[f'x{cols}'], ln[f'gamma{cols}'], ln[f'beta{cols}'] = x, gamma, beta
        for mode in ('conv_even', 'symmetric_inf', 'floor'):
            for out_shift in (4, 7):
                ln[f'y{cols}__{mode}__{out_shift}'] = np.array(
                    [layernorm_row([int(v) for v in row], [int(g) for g in gamma], [int(t) for t in beta], out_shift, mode)
                     for row in x], dtype=np.int8)
    np.savez_compressed(HERE / 'layernorm.npz', **ln)

    # ---- softmax ---------------------------------------------------------------------------------------
    x = gauss8(r, 35, (8, 64))
    x[0, :] = -128                         # uniform row
    x[1, :] = 127
    x[2, 5] = 127                          # one dominant element
    sm = {'x': x}
    for kq in (1, 23, 92, 128):
        sm[f'exp_u8__{kq}'] = np.array([softmax_exp_row([int(v) for v in row], kq) for row in x], dtype=np.uint8)
    sm['exp_i16__23'] = np.array([softmax_exp_row([int(v) for v in row], 23, 'int16') for row in x], dtype=np.int16)
    for (B, S, D) in ((255, 3, 80), (60, 1, 56), (500, 3, 127)):
        sm[f'hccs_u8__{B}_{S}_{D}'] = np.array([softmax_hccs_row([int(v) for v in row], B, S, D) for row in x], dtype=np.uint8)
    sm['hccs_i16__255_3_80'] = np.array([softmax_hccs_row([int(v) for v in row], 255, 3, 80, 'int16') for row in x], dtype=np.int16)
    np.savez_compressed(HERE / 'softmax.npz', **sm)

    # ---- attention core: matmul(K transposed) -> softmax -> matmul, head_dim 64, 32 keys -----------------
    q, k, v = gauss8(r, 24, (2, 20, 64)), gauss8(r, 24, (2, 32, 64)), gauss8(r, 24, (2, 32, 64))
    at = {'q': q, 'k': k, 'v': v}
    for name, fn in (('exp23', lambda row: softmax_exp_row(row, 23)), ('hccs', lambda row: softmax_hccs_row(row, 255, 4, 60))):
        outs = []
        for b in range(2):
            logits = matmul(q[b], k[b].T, 6, 'conv_even', 'int8')
            probs = np.array([fn([int(t) for t in row]) for row in logits], dtype=np.uint8)
            outs.append(matmul(probs, v[b], 7, 'conv_even', 'int8'))
        at[f'o__{name}'] = np.stack(outs)
    np.savez_compressed(HERE / 'attention.npz', **at)

    # ---- MLP 16-64-32-32-5, shift 7, ReLU on the first three layers ------------------------------------
    x = r.integers(-128, 128, (9, 16)).astype(np.int8)
    dims = [16, 64, 32, 32, 5]
    mlp = {'x': x}
    for mode in ('positive_inf', 'symmetric_inf', 'conv_even'):
        h = x
        for i in range(4):
            if f'W{i}' not in mlp:
                mlp[f'W{i}'] = r.integers(-64, 64, (dims[i], dims[i + 1])).astype(np.int8)
                mlp[f'b{i}'] = r.integers(-4096, 4097, dims[i + 1]).astype(np.int32)
            h = dense(h, mlp[f'W{i}'], mlp[f'b{i}'], np.full(dims[i + 1], 7), mode, i < 3, 'int8')
        mlp[f'y__{mode}'] = h
    np.savez_compressed(HERE / 'mlp.npz', **mlp)
    print('golden vectors written to', HERE)


if __name__ == '__main__':
    main()
