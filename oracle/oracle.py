"""ctypes binding of the CPU oracle (``liba4oracle.so``).

TEST INFRASTRUCTURE. Imported only by the tests, the smoke check and the CPU-baseline leg of the
benchmark; the product package never imports this module.
"""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB_PATH = _HERE / 'liba4oracle.so'

ROUNDING = {
    'floor': 0,
    'ceil': 1,
    'positive_inf': 2,
    'negative_inf': 3,
    'symmetric_inf': 4,
    'symmetric_zero': 5,
    'conv_even': 6,
    'conv_odd': 7,
}
KIND = {'int8': 0, 'uint8': 1, 'int16': 2, 'uint16': 3, 'int32': 4}
_NP_KIND = {np.dtype(np.int8): 0, np.dtype(np.uint8): 1, np.dtype(np.int16): 2, np.dtype(np.uint16): 3,
            np.dtype(np.int32): 4}
_KIND_NP = {v: k for k, v in _NP_KIND.items()}


def build(force: bool = False) -> Path:
    if force or not _LIB_PATH.exists():
        subprocess.run(['make', '-C', str(_HERE), '-B' if force else '-s', 'liba4oracle.so'], check=True)
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = ctypes.CDLL(str(_LIB_PATH))
        i64, i32, vp = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p
        _lib.a4o_srs.argtypes = [ctypes.c_int32, i32, i32, i32]
        _lib.a4o_srs.restype = ctypes.c_int32
        _lib.a4o_dense_i8.argtypes = [vp, i32, i64, vp, i64, vp, vp, i32, i32, i32, i32, vp, i64, i64, i64, i64]
        _lib.a4o_dense_i16x16.argtypes = [vp, i64, vp, i64, vp, vp, i32, i32, i32, i32, vp, i64, i64, i64, i64]
        _lib.a4o_matmul_i8.argtypes = [vp, i32, i64, i64, vp, i64, i64, i32, vp, i64, i64, i64, i64, i64, i64,
                                       i32, i32, i32]
        _lib.a4o_add.argtypes = [vp, vp, vp, i64, i32, i32, i32]
        _lib.a4o_rsqrt_q15.argtypes = [ctypes.c_int32]
        _lib.a4o_rsqrt_q15.restype = ctypes.c_int32
        _lib.a4o_layernorm_i8.argtypes = [vp, vp, vp, vp, i64, i64, ctypes.c_int32, i32, i32, i32]
        _lib.a4o_add_layernorm_i8.argtypes = [vp, vp, i32, i32, vp, vp, vp, vp, i64, i64, ctypes.c_int32, i32,
                                              i32, i32]
        _lib.a4o_exp_score16.argtypes = [ctypes.c_int32, ctypes.c_int32]
        _lib.a4o_exp_score16.restype = ctypes.c_int32
        _lib.a4o_softmax_exp_i8.argtypes = [vp, vp, i64, i64, i32, i32, i32]
        _lib.a4o_softmax_hccs_i8.argtypes = [vp, vp, i64, i64, i32, i32, i32, i32, i32, i32]
        _lib.a4o_num_threads.restype = i32
        _lib.a4o_set_num_threads.argtypes = [i32]
    return _lib


def _ptr(a):
    return ctypes.c_void_p(a.ctypes.data) if a is not None else None


def _c(a, dtype=None):
    a = np.ascontiguousarray(a) if dtype is None else np.ascontiguousarray(a, dtype=dtype)
    return a


def _check(rc, what):
    if rc != 0:
        raise ValueError(f'oracle {what}: status {rc}')


def _mode(mode):
    return ROUNDING[mode] if isinstance(mode, str) else int(mode)


def srs(acc, shift, mode, kind='int8'):
    """Shift-round-saturate of int32 accumulator value(s)."""
    L = lib()
    k = KIND[kind]
    m = _mode(mode)
    arr = np.asarray(acc)
    flat = [L.a4o_srs(int(np.int32(v)), int(shift), m, k) for v in arr.reshape(-1)]
    return np.array(flat, dtype=np.int64).reshape(arr.shape)


def dense(A, W, bias, shifts, mode, relu=False, out='int8'):
    """A [M,K] int8/uint8/int16, W [K,N] int8 (or int16 with int16 A: 64-bit accumulator), bias [N] int32 or None,
    shifts scalar or [N]."""
    A = _c(A)
    wide = np.asarray(W).dtype == np.int16  # (16, 16): int16 weights, 64-bit accumulator
    W = _c(W, np.int16 if wide else np.int8)
    M, K = A.shape
    K2, N = W.shape
    assert K == K2
    b = _c(bias, np.int32) if bias is not None else None
    sh = _c(np.atleast_1d(shifts), np.int32)
    Y = np.empty((M, N), dtype=_KIND_NP[KIND[out]])
    if wide:
        assert A.dtype == np.int16
        rc = lib().a4o_dense_i16x16(_ptr(A), K, _ptr(W), N, _ptr(b), _ptr(sh), sh.size, _mode(mode), int(bool(relu)),
                                    KIND[out], _ptr(Y), N, M, N, K)
        _check(rc, 'dense 16x16')
        return Y
    rc = lib().a4o_dense_i8(_ptr(A), _NP_KIND[A.dtype], K, _ptr(W), N, _ptr(b), _ptr(sh), sh.size, _mode(mode),
                            int(bool(relu)), KIND[out], _ptr(Y), N, M, N, K)
    _check(rc, 'dense')
    return Y


def matmul(A, B, shift, mode, trans_b=False, out='int8'):
    """Batched: A [..., M, K]; B [..., K, N] (or [..., N, K] when trans_b). An int16 A takes the 16-bit width
    combinations (B int8: acc32, B int16: acc64): the same accumulation as Dense without bias or ReLU
    (matmul.cpp:80-115), so each problem of the batch goes through dense()."""
    A = _c(A)
    if A.dtype == np.int16:
        B = _c(B)
        Bm = np.swapaxes(B, -1, -2) if trans_b else B
        lead = A.shape[:-2]
        A3, B3 = A.reshape((-1,) + A.shape[-2:]), Bm.reshape((-1,) + Bm.shape[-2:])
        C = np.stack([dense(A3[i], np.ascontiguousarray(B3[i]), None, int(shift), mode, out=out) for i in range(A3.shape[0])])
        return C.reshape(lead + C.shape[-2:])
    B = _c(B, np.int8)
    M, K = A.shape[-2:]
    N = B.shape[-2] if trans_b else B.shape[-1]
    assert (B.shape[-1] if trans_b else B.shape[-2]) == K
    lead = A.shape[:-2]
    assert B.shape[:-2] == lead
    batch = int(np.prod(lead, dtype=np.int64)) if lead else 1
    C = np.empty(lead + (M, N), dtype=_KIND_NP[KIND[out]])
    rc = lib().a4o_matmul_i8(_ptr(A), _NP_KIND[A.dtype], K, M * K, _ptr(B), B.shape[-1], K * N, int(bool(trans_b)),
                             _ptr(C), N, M * N, batch, M, N, K, int(shift), _mode(mode), KIND[out])
    _check(rc, 'matmul')
    return C


def add(a, b, shift=0, mode='floor'):
    a = _c(a)
    b = _c(b)
    assert a.dtype == b.dtype and a.shape == b.shape
    out = np.empty_like(a)
    _check(lib().a4o_add(_ptr(a), _ptr(b), _ptr(out), a.size, _NP_KIND[a.dtype], int(shift), _mode(mode)), 'add')
    return out


def rsqrt_q15(v):
    return int(lib().a4o_rsqrt_q15(int(v)))


def layernorm(x, gamma, beta, out_shift, mode, eps_q0=1, gamma_shift=7):
    x = _c(x, np.int8)
    g = _c(gamma, np.int16)
    b = _c(beta, np.int16)
    cols = x.shape[-1]
    rows = x.size // cols
    out = np.empty_like(x)
    rc = lib().a4o_layernorm_i8(_ptr(x), _ptr(g), _ptr(b), _ptr(out), rows, cols, int(eps_q0), int(gamma_shift),
                                int(out_shift), _mode(mode))
    _check(rc, 'layernorm')
    return out


def add_layernorm(a, b, gamma, beta, out_shift, mode, eps_q0=1, gamma_shift=7, add_shift=0, add_mode='floor',
                  return_sum=False):
    a = _c(a, np.int8)
    b2 = _c(b, np.int8)
    g = _c(gamma, np.int16)
    bt = _c(beta, np.int16)
    cols = a.shape[-1]
    rows = a.size // cols
    out = np.empty_like(a)
    s = np.empty_like(a) if return_sum else None
    rc = lib().a4o_add_layernorm_i8(_ptr(a), _ptr(b2), int(add_shift), _mode(add_mode), _ptr(g), _ptr(bt), _ptr(s),
                                    _ptr(out), rows, cols, int(eps_q0), int(gamma_shift), int(out_shift),
                                    _mode(mode))
    _check(rc, 'add_layernorm')
    return (s, out) if return_sum else out


def exp_score16(d, kq):
    return int(lib().a4o_exp_score16(int(d), int(kq)))


def softmax_exp(x, exp_kq, inv_shift=15, out='uint8'):
    x = _c(x, np.int8)
    cols = x.shape[-1]
    rows = x.size // cols
    o = np.empty(x.shape, dtype=_KIND_NP[KIND[out]])
    _check(lib().a4o_softmax_exp_i8(_ptr(x), _ptr(o), rows, cols, int(exp_kq), int(inv_shift), KIND[out]),
           'softmax_exp')
    return o


def softmax_hccs(x, B, S, Dmax, inv_shift=15, use_clb=False, out='uint8'):
    x = _c(x, np.int8)
    cols = x.shape[-1]
    rows = x.size // cols
    o = np.empty(x.shape, dtype=_KIND_NP[KIND[out]])
    rc = lib().a4o_softmax_hccs_i8(_ptr(x), _ptr(o), rows, cols, int(B), int(S), int(Dmax), int(inv_shift),
                                   int(bool(use_clb)), KIND[out])
    _check(rc, 'softmax_hccs')
    return o


def mlp(x, layers, mode):
    """Chain of dense layers: layers = [(W[K,N], bias, shift, relu, out_kind), ...]."""
    h = x
    for W, bias, shift, relu, out in layers:
        h = dense(h, W, bias, shift, mode, relu=relu, out=out)
    return h


def num_threads():
    return int(lib().a4o_num_threads())


def set_num_threads(n):
    lib().a4o_set_num_threads(int(n))


# ---- floating-point compute path ---------------------------------------------------------------------------------
# The reference's float mode multiplies bfloat16 (or float32) operands into a float32 accumulator that starts at
# the bias and rounds the result to the operand format with conv_even (dense.py:105-127,
# dense_bias_relu.cpp:112-163). The AI Engine's order of additions is not visible from the sources, so the
# restatement below accumulates exactly (float64 on operands that are exact in their format) and rounds once:
# every float32 summation order stays within the usual forward error bound of it. Parity with the AI Engine
# itself is unpinned beyond the tolerances of the reference's own test (tests/test_float_sim.py:81-87:
# rtol 1e-2 / atol 5e-2 for bfloat16, 1e-3 / 1e-3 for float32).

def bf16_truncate(x):
    """float -> nearest-toward-zero bfloat16 value, as float32 (pack_as_float, matmul/common.py:272-274,
    and _bf16_like of tests/test_float_sim.py:59-61)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u >> 16) << 16).view(np.float32)


def bf16_round(x):
    """float -> bfloat16 with round-to-nearest-even (the conv_even of the kernels' to_vector), as float32."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    out = r.astype(np.uint32).view(np.float32)
    return np.where(np.isnan(x), np.float32(np.nan), out)


def fp8_encode(x):
    """float32 -> fp8 e4m3 codes by the reference's packer recipe (_float32_to_fp8_scalar,
    matmul/common.py:262-276), one value at a time as written there."""
    flat = np.ascontiguousarray(x, dtype=np.float32).reshape(-1)
    out = np.empty(flat.size, dtype=np.uint8)
    for i, bits in enumerate(flat.view(np.uint32).tolist()):
        h = (bits + 0x00080000) & 0xFFFFFFFF
        e = (h & 0x7F800000) >> 23
        m = h & 0x007FFFFF
        sign = (h & 0x80000000) >> 24
        if e > 135:
            r = sign | 0x7F
        elif e > 120:
            r = sign | (((e - 120) << 3) & 0x78) | (m >> 20)
        elif e > 116:
            r = sign | (((0x00780000 + m) >> (140 - e)) + 1) >> 1
        else:
            r = sign
        out[i] = r & 0xFF
    return out.reshape(np.shape(x))


def fp8_decode(codes):
    """fp8 e4m3 codes -> float32: bias 7, subnormals m * 2^-9, no infinities, 0x7f / 0xff NaN."""
    c = np.asarray(codes, dtype=np.uint8).astype(np.int64)
    e, m = (c >> 3) & 0xF, c & 7
    mag = np.where(e == 0, m * 2.0 ** -9, (1.0 + m / 8.0) * np.exp2(e - 7.0))
    mag = np.where((e == 15) & (m == 7), np.nan, mag)
    return np.where(c & 0x80, -mag, mag).astype(np.float32)


def fp8_quantize(x):
    """float -> nearest fp8 e4m3 value by the packer recipe, as float32."""
    return fp8_decode(fp8_encode(np.asarray(x, dtype=np.float32)))


def to_float_format(x, fmt):
    if fmt == 'fp8_e4m3':
        return fp8_quantize(np.asarray(x, dtype=np.float64).astype(np.float32))
    if fmt == 'bfloat16':
        return bf16_round(np.asarray(x, dtype=np.float64).astype(np.float32))
    if fmt == 'float32':
        return np.asarray(x, dtype=np.float64).astype(np.float32)
    raise ValueError(f'unknown float format {fmt!r}')


def dense_float(A, W, bias, relu=False, fmt='bfloat16'):
    """A [M,K], W [K,N] (values exact in `fmt`), bias float32 [N] or None -> float32 array of `fmt` values."""
    acc = np.asarray(A, dtype=np.float64) @ np.asarray(W, dtype=np.float64)
    if bias is not None:
        acc = acc + np.asarray(bias, dtype=np.float32).astype(np.float64)
    if relu:
        acc = np.maximum(acc, 0.0)
    return to_float_format(acc, fmt)


def matmul_float(A, B, trans_b=False, fmt='bfloat16'):
    B = np.asarray(B, dtype=np.float64)
    if trans_b:
        B = np.swapaxes(B, -1, -2)
    return to_float_format(np.asarray(A, dtype=np.float64) @ B, fmt)


def add_float(a, b, fmt='bfloat16'):
    return to_float_format(np.asarray(a, dtype=np.float64) + np.asarray(b, dtype=np.float64), fmt)
