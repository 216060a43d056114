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


def _c5_params(batch, seq, hidden, heads, ffn, seed):
    """Seeded float parameters (on their quantisation grids) and the int8 input of the encoder block."""
    r = np.random.default_rng(seed)

    def weights(k, n):
        return _gauss8(r, 16.0, (k, n)).astype(np.float64) / 128.0

    def bias(n):
        return r.integers(-(1 << 10), (1 << 10) + 1, n).astype(np.float64) / 2048.0

    p = {'qkv_w': weights(hidden, 3 * hidden), 'qkv_b': bias(3 * hidden)}
    p['out_w'], p['out_b'] = weights(hidden, hidden), bias(hidden)
    p['gamma1'] = r.integers(32, 128, hidden).astype(np.float64) / 128.0
    p['beta1'] = r.integers(-15, 16, hidden).astype(np.float64) / 16.0
    p['ffn1_w'], p['ffn1_b'] = weights(hidden, ffn), bias(ffn)
    p['ffn2_w'], p['ffn2_b'] = weights(ffn, hidden), bias(hidden)
    p['gamma2'] = r.integers(32, 128, hidden).astype(np.float64) / 128.0
    p['beta2'] = r.integers(-15, 16, hidden).astype(np.float64) / 16.0
    p['x'] = _gauss8(r, 24.0, (batch, seq, hidden))
    return p


def _c5_hccs(seq: int):
    # legal for cols = seq: seq*B <= 32767 and seq*(B - S*Dmax) >= 256
    B = min(255, 32767 // seq)
    return {'B': B, 'S': 4, 'Dmax': (B - max(1, -(-256 // seq))) // 4}


def c5_encoder_block(batch: int = 64, seq: int = 128, hidden: int = 768, heads: int = 12, ffn: int = 3072,
                     softmax: str = 'hccs', seed: int = 17 + 5):
    """Full int8 transformer encoder block as an operator graph (the structure an ONNX Q/DQ export of
    the block lowers to: no Reshape, heads expressed with Split / Transpose / Concat).

    QKV Dense hidden->3*hidden, Split, per head: Q.K^T (Transpose folded into the MatMul), integer
    Softmax, P.V; Concat; output Dense; Add + LayerNorm; FFN Dense+ReLU, Dense; Add + LayerNorm.
    Weights int8 from clipped N(0,16); every tensor has a per-tensor power-of-two scale.
    Returns (model, x_int8) with x the seeded int8 input [batch, seq, hidden].
    """
    from .frontends.builder import GraphBuilder, qint

    p = _c5_params(batch, seq, hidden, heads, ffn, seed)
    hd = hidden // heads
    act = qint(8, 4)            # activations: int8, scale 2^-4
    wq = qint(8, 7)             # weights: int8, scale 2^-7
    bq = qint(32, 11)           # bias at accumulator scale 2^-(4+7)
    prob = qint(8, 8, signed=False)  # softmax probabilities: uint8, scale 1/256

    gb = GraphBuilder(config={'Iterations': 1})
    x = gb.input('x', (batch, seq, hidden), act)
    qkv = gb.dense(x, p['qkv_w'], wq, act, bias=p['qkv_b'], bias_precision=bq, name='qkv')
    q, k, v = gb.split(qkv, -1, [hidden] * 3, name='qkv_split')
    qs = gb.split(q, -1, [hd] * heads, name='q_heads')
    ks = gb.split(k, -1, [hd] * heads, name='k_heads')
    vs = gb.split(v, -1, [hd] * heads, name='v_heads')
    ctx_heads = []
    directives = {'approximation': 'hccs', 'hccs': _c5_hccs(seq)} if softmax == 'hccs' else None
    for h in range(heads):
        kt = gb.transpose(ks[h], (0, 2, 1), name=f'k_t{h}')
        # Q.K^T has a standard deviation of a few 10^4 at these scales: keep the top bits (shift 11)
        logits = gb.matmul(qs[h], kt, qint(8, -3), name=f'qk{h}')
        if softmax == 'exp':
            # temperature 1/32, absorbed by the Softmax: EXP_KQ = round(log2(e) * 2^3 / 32 * 256) = 92
            logits = gb.scale(logits, 1.0 / 32.0, name=f'qk_scale{h}')
        pr = gb.softmax(logits, prob, name=f'softmax{h}', directives=directives)
        ctx_heads.append(gb.matmul(pr, vs[h], act, name=f'pv{h}'))
    attn = gb.concat(ctx_heads, -1, name='heads_concat')
    proj = gb.dense(attn, p['out_w'], wq, act, bias=p['out_b'], bias_precision=bq, name='attn_out')
    res1 = gb.add(x, proj, act, name='residual1')
    ln1 = gb.layer_norm(res1, p['gamma1'], p['beta1'], act, eps_q0=1, name='ln1')
    h1 = gb.dense(ln1, p['ffn1_w'], wq, act, bias=p['ffn1_b'], bias_precision=bq, relu=True, name='ffn1')
    h2 = gb.dense(h1, p['ffn2_w'], wq, act, bias=p['ffn2_b'], bias_precision=bq, name='ffn2')
    res2 = gb.add(ln1, h2, act, name='residual2')
    out = gb.layer_norm(res2, p['gamma2'], p['beta2'], act, eps_q0=1, name='ln2')
    gb.output(out)
    return gb.build(), p['x']


def c5_encoder_block_onnx(batch: int = 64, seq: int = 128, hidden: int = 768, heads: int = 12, ffn: int = 3072,
                          softmax: str = 'hccs', seed: int = 17 + 5):
    """The same block, same parameters, as an ONNX Q/DQ model: float input, int8 / int32 initializers behind
    DequantizeLinear, a QuantizeLinear / DequantizeLinear pair after every operator. Returns
    (onnx bytes, config dict with the layer directives, x_int8); the float input is x_int8 / 16."""
    from .frontends.builder import qint
    from .frontends.onnx_writer import QdqWriter

    p = _c5_params(batch, seq, hidden, heads, ffn, seed)
    hd = hidden // heads
    act, wq, bq, prob = qint(8, 4), qint(8, 7), qint(32, 11), qint(8, 8, signed=False)
    w = QdqWriter('encoder_block')

    def dense(x, name, relu=False):
        (y,) = w.node('MatMul', [x, w.weight(f'{name}_w', p[f'{name}_w'], wq)], name=name)
        (y,) = w.node('Add', [y, w.weight(f'{name}_b', p[f'{name}_b'], bq)], name=f'{name}_bias')
        y = w.qdq(y, act)
        if relu:
            (y,) = w.node('Relu', [y], name=f'{name}_relu')
            y = w.qdq(y, act)
        return y

    def layer_norm(x, i):
        g = w.const(f'gamma{i}', p[f'gamma{i}'].astype(np.float32))
        b = w.const(f'beta{i}', p[f'beta{i}'].astype(np.float32))
        (y,) = w.node('LayerNormalization', [x, g, b], name=f'ln{i}', axis=-1, epsilon=2.0 ** -8)  # = 1 at the input's scale^2
        return w.qdq(y, act)

    x = w.input('x', (batch, seq, hidden), act)
    qkv = dense(x, 'qkv')
    q, k, v = w.node('Split', [qkv, w.const('qkv_sizes', np.array([hidden] * 3, dtype=np.int64))], 3, name='qkv_split', axis=-1)
    head_sizes = w.const('head_sizes', np.array([hd] * heads, dtype=np.int64))
    qs = w.node('Split', [q, head_sizes], heads, name='q_heads', axis=2)
    ks = w.node('Split', [k, head_sizes], heads, name='k_heads', axis=2)
    vs = w.node('Split', [v, head_sizes], heads, name='v_heads', axis=2)
    directives = {}
    ctx_heads = []
    for h in range(heads):
        (kt,) = w.node('Transpose', [ks[h]], name=f'k_t{h}', perm=[0, 2, 1])
        (lg,) = w.node('MatMul', [qs[h], kt], name=f'qk{h}')
        lg = w.qdq(lg, qint(8, -3))
        if softmax == 'exp':
            (lg,) = w.node('Mul', [lg, w.const(f'temp{h}', np.array(1.0 / 32.0, dtype=np.float32))], name=f'qk_scale{h}')
        else:
            directives[f'softmax{h}'] = {'approximation': 'hccs', 'hccs': _c5_hccs(seq)}
        (pr,) = w.node('Softmax', [lg], name=f'softmax{h}', axis=-1)
        pr = w.qdq(pr, prob)
        (o,) = w.node('MatMul', [pr, vs[h]], name=f'pv{h}')
        ctx_heads.append(w.qdq(o, act))
    (attn,) = w.node('Concat', ctx_heads, name='heads_concat', axis=-1)
    proj = dense(attn, 'out')
    (res1,) = w.node('Add', [x, proj], name='residual1')
    ln1 = layer_norm(w.qdq(res1, act), 1)
    h2 = dense(dense(ln1, 'ffn1', relu=True), 'ffn2')
    (res2,) = w.node('Add', [ln1, h2], name='residual2')
    out = layer_norm(w.qdq(res2, act), 2)
    w.output(out, (batch, seq, hidden))
    return w.to_bytes(), {'Iterations': 1, 'LayerDirectives': directives}, p['x']


def c1_mlp_model(batch: int = 1024, rounding=None):
    """The C1 MLP as an operator graph (hls4ml-style: Dense + ReLU layers, shift 7 everywhere)."""
    from .aie_types import RoundingMode
    from .frontends.builder import GraphBuilder, qint

    rounding = rounding or RoundingMode.RND
    x, layers = c1_mlp(batch)
    # activations int8 frac 0; weights frac 7 -> acc frac 7 -> shift 7 to an int8 frac-0 output
    act = qint(8, 0, rounding=rounding)
    gb = GraphBuilder(config={'Iterations': 1})
    t = gb.input('x', (batch, x.shape[1]), act)
    for i, (W, b, _shift, relu, _kind) in enumerate(layers):
        t = gb.dense(t, W.astype(np.float64) / 128.0, qint(8, 7), act, bias=b.astype(np.float64) / 128.0,
                     bias_precision=qint(32, 7), relu=relu, name=f'fc{i}')
    gb.output(t)
    return gb.build(), x, layers
