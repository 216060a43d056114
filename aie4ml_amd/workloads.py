"""Seeded synthetic inputs for the five benchmark configurations (numpy, host side).

Seeds follow the reference's ONNX checker (scripts/check_onnx_bit_exact.py:119 uses
``default_rng(17)``): config i uses ``default_rng(17 + i)``.
"""

from __future__ import annotations

import numpy as np


def _gauss8(r, sigma, shape):
    return np.clip(np.rint(r.normal(0.0, sigma, shape)), -128, 127).astype(np.int8)


def c1_mlp(batch: int = 1024):
    """int8 MLP 16->64->32->32->5, ReLU on the first three layers, shift 7 everywhere."""
    r = np.random.default_rng(17 + 1)
    widths = [16, 64, 32, 32, 5]
    x = r.integers(-128, 128, (batch, widths[0])).astype(np.int8)
    layers = []
    for i, (k, n) in enumerate(zip(widths[:-1], widths[1:])):
        W = r.integers(-64, 64, (k, n)).astype(np.int8)
        b = r.integers(-4096, 4097, n).astype(np.int32)
        layers.append((W, b, 7, i < len(widths) - 2, 'int8'))
    return x, layers


def c2_dense(M: int = 8192, K: int = 4096, N: int = 4096):
    """Single Dense with bias, per-output-channel shift in [8,12], fused ReLU."""
    r = np.random.default_rng(17 + 2)
    A = _gauss8(r, 32.0, (M, K))
    W = _gauss8(r, 16.0, (K, N))
    bias = r.integers(-(1 << 14), (1 << 14) + 1, N).astype(np.int32)
    shifts = r.integers(8, 13, N).astype(np.int32)
    return A, W, bias, shifts


def c3_attention(batch: int = 32, heads: int = 16, seq: int = 512, dim: int = 64):
    """Q, K, V for the attention core; logits shift 6; exp_kq for logits at frac 4; legal HCCS set."""
    r = np.random.default_rng(17 + 3)
    shape = (batch, heads, seq, dim)
    q, k, v = _gauss8(r, 24.0, shape), _gauss8(r, 24.0, shape), _gauss8(r, 24.0, shape)
    params = {
        'logit_shift': 6,
        'exp_kq': 23,                       # round(log2(e) * 2^-4 * 256)
        'hccs': {'B': 60, 'S': 1, 'Dmax': 59},  # C*B = 30720 <= 32767, C*(B-S*Dmax) = 512 >= 256
        'pv_shift': 8,
    }
    return q, k, v, params


def c4_add_layernorm(rows: int = 16384, cols: int = 1024):
    """Residual add + LayerNorm. beta is drawn at the output scale (frac 5) and stored as Q15."""
    r = np.random.default_rng(17 + 4)
    a, b = _gauss8(r, 20.0, (rows, cols)), _gauss8(r, 20.0, (rows, cols))
    gamma = r.integers(32, 128, cols).astype(np.int16)
    out_frac = 5
    beta = (r.integers(-16, 17, cols).astype(np.int32) << (15 - out_frac)).astype(np.int16)
    return a, b, gamma, beta, {'out_shift': out_frac, 'eps_q0': 1}
