"""Golden vectors (tests/golden/*.npz, written by tests/golden/make_golden.py with exact Python integers):
the CPU oracle must reproduce them (not gpu), and so must the HIP library through its C ABI (gpu)."""

from pathlib import Path

import numpy as np
import pytest

GOLD = Path(__file__).resolve().parent / 'golden'
MODES = ['floor', 'ceil', 'positive_inf', 'negative_inf', 'symmetric_inf', 'symmetric_zero', 'conv_even', 'conv_odd']


def load(name):
    return np.load(GOLD / f'{name}.npz', allow_pickle=False)


# ---- CPU: oracle against the vectors ----------------------------------------------------------------------

def test_oracle_srs():
    from oracle import oracle
    g = load('srs')
    n = 0
    for key in g.files:
        if key == 'acc':
            continue
        mode, shift, kind = key.split('__')
        # the accumulator the kernels hand to srs is an int32; the vectors hold the same values
        np.testing.assert_array_equal(oracle.srs(g['acc'].astype(np.int32), int(shift), mode, kind), g[key], err_msg=key)
        n += 1
    assert n == 8 * 5 * 3


def test_oracle_dense_matmul_add(oracle):
    g = load('dense')
    for mode in MODES:
        np.testing.assert_array_equal(oracle.dense(g['A'], g['W'], g['bias'], g['shifts'], mode, relu=True), g[f'y__{mode}__relu'])
        np.testing.assert_array_equal(oracle.dense(g['A'], g['W'], g['bias'], 6, mode), g[f'y__{mode}__scalar6'])
    np.testing.assert_array_equal(oracle.dense(g['Au'], g['W'], g['bias'], g['shifts'], 'conv_even'), g['y__u8in__conv_even'])
    np.testing.assert_array_equal(oracle.dense(g['A'], g['W'], g['bias'], g['shifts'], 'symmetric_inf', relu=True, out='uint8'),
                                  g['y__u8out__symmetric_inf'])
    np.testing.assert_array_equal(oracle.dense(g['A'], g['W'], g['bias'], 2, 'conv_even', out='int16'), g['y__i16out__conv_even'])
    np.testing.assert_array_equal(oracle.dense(np.abs(g['A']), np.abs(g['W']), g['bias_wrap'], 10, 'floor'), g['y__wrap'])
    np.testing.assert_array_equal(oracle.dense(g['A16'], g['W'], g['bias'], 9, 'conv_even', out='int16'), g['y__i16in__conv_even__i16'])
    np.testing.assert_array_equal(oracle.dense(g['A16'], g['W'], g['bias'], g['shifts'] + 8, 'symmetric_inf', relu=True),
                                  g['y__i16in__symmetric_inf__i8relu'])
    g16 = load('dense16')
    for mode in MODES:
        np.testing.assert_array_equal(oracle.dense(g16['A'], g16['W'], g16['bias'], g16['shifts'], mode, out='int16'),
                                      g16[f'y__{mode}__i16'])
    np.testing.assert_array_equal(oracle.dense(g16['A'], g16['W'], g16['bias'], 24, 'conv_even', relu=True), g16['y__conv_even__i8relu__s24'])
    np.testing.assert_array_equal(oracle.dense(g16['A'], g16['W'], g16['bias'], 36, 'floor', out='int16'), g16['y__floor__i16__s36'])
    m = load('matmul')
    for mode in ('conv_even', 'symmetric_inf', 'floor'):
        np.testing.assert_array_equal(oracle.matmul(m['Aq'], m['Bk'], 5, mode, trans_b=True), m[f'qk__{mode}'])
        np.testing.assert_array_equal(oracle.matmul(m['P'], m['Bv'], 8, mode), m[f'pv__{mode}'])
    a = load('add')
    np.testing.assert_array_equal(oracle.add(a['a'], a['b']), a['y_i8'])
    np.testing.assert_array_equal(oracle.add(a['a'].view(np.uint8), a['b'].view(np.uint8)), a['y_u8'])
    np.testing.assert_array_equal(oracle.add(a['a'], a['b'], 1, 'conv_even'), a['y_i8_shift1_conv_even'])


def test_oracle_layernorm_softmax_attention_mlp(oracle):
    g = load('layernorm')
    for cols in (64, 48):
        for mode in ('conv_even', 'symmetric_inf', 'floor'):
            for s in (4, 7):
                got = oracle.layernorm(g[f'x{cols}'], g[f'gamma{cols}'], g[f'beta{cols}'], s, mode)
                np.testing.assert_array_equal(got, g[f'y{cols}__{mode}__{s}'], err_msg=f'{cols} {mode} {s}')
    sm = load('softmax')
    for kq in (1, 23, 92, 128):
        np.testing.assert_array_equal(oracle.softmax_exp(sm['x'], kq), sm[f'exp_u8__{kq}'])
    np.testing.assert_array_equal(oracle.softmax_exp(sm['x'], 23, out='int16'), sm['exp_i16__23'])
    for (B, S, D) in ((255, 3, 80), (60, 1, 56), (500, 3, 127)):
        np.testing.assert_array_equal(oracle.softmax_hccs(sm['x'], B, S, D), sm[f'hccs_u8__{B}_{S}_{D}'])
    np.testing.assert_array_equal(oracle.softmax_hccs(sm['x'], 255, 3, 80, out='int16'), sm['hccs_i16__255_3_80'])
    at = load('attention')
    lg = oracle.matmul(at['q'], at['k'], 6, 'conv_even', trans_b=True)
    np.testing.assert_array_equal(oracle.matmul(oracle.softmax_exp(lg, 23), at['v'], 7, 'conv_even'), at['o__exp23'])
    np.testing.assert_array_equal(oracle.matmul(oracle.softmax_hccs(lg, 255, 4, 60), at['v'], 7, 'conv_even'), at['o__hccs'])
    ml = load('mlp')
    layers = [(ml[f'W{i}'], ml[f'b{i}'], 7, i < 3, 'int8') for i in range(4)]
    for mode in ('positive_inf', 'symmetric_inf', 'conv_even'):
        np.testing.assert_array_equal(oracle.mlp(ml['x'], layers, mode), ml[f'y__{mode}'])


# ---- GPU: the HIP library against the same vectors ----------------------------------------------------------

def _dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def _host(t):
    return t.cpu().numpy()


@pytest.mark.gpu
def test_gpu_dense_matmul_add():
    from aie4ml_amd import ops
    g = load('dense')
    W, bias = _dev(g['W']), _dev(g['bias'])
    per_channel = ops.pack_dense(W, bias, g['shifts'])
    scalar6 = ops.pack_dense(W, bias, 6)
    for mode in MODES:
        np.testing.assert_array_equal(_host(ops.dense(_dev(g['A']), per_channel, mode, relu=True)), g[f'y__{mode}__relu'])
        np.testing.assert_array_equal(_host(ops.dense(_dev(g['A']), scalar6, mode)), g[f'y__{mode}__scalar6'])
    np.testing.assert_array_equal(_host(ops.dense(_dev(g['Au']), per_channel, 'conv_even')), g['y__u8in__conv_even'])
    np.testing.assert_array_equal(_host(ops.dense(_dev(g['A']), per_channel, 'symmetric_inf', relu=True, out_kind='uint8')),
                                  g['y__u8out__symmetric_inf'])
    np.testing.assert_array_equal(_host(ops.dense(_dev(g['A']), ops.pack_dense(W, bias, 2), 'conv_even', out_kind='int16')),
                                  g['y__i16out__conv_even'])
    wrap = ops.pack_dense(_dev(np.abs(g['W'])), _dev(g['bias_wrap']), 10)
    np.testing.assert_array_equal(_host(ops.dense(_dev(np.abs(g['A'])), wrap, 'floor')), g['y__wrap'])
    np.testing.assert_array_equal(_host(ops.dense(_dev(g['A16']), ops.pack_dense(W, bias, 9), 'conv_even', out_kind='int16')),
                                  g['y__i16in__conv_even__i16'])
    np.testing.assert_array_equal(_host(ops.dense(_dev(g['A16']), ops.pack_dense(W, bias, g['shifts'] + 8), 'symmetric_inf', relu=True)),
                                  g['y__i16in__symmetric_inf__i8relu'])
    g16 = load('dense16')
    for mode in MODES:
        p16 = ops.pack_dense(_dev(g16['W']), _dev(g16['bias']), g16['shifts'])
        np.testing.assert_array_equal(_host(ops.dense(_dev(g16['A']), p16, mode, out_kind='int16')), g16[f'y__{mode}__i16'])
    np.testing.assert_array_equal(_host(ops.dense(_dev(g16['A']), ops.pack_dense(_dev(g16['W']), _dev(g16['bias']), 24), 'conv_even',
                                                  relu=True)), g16['y__conv_even__i8relu__s24'])
    np.testing.assert_array_equal(_host(ops.dense(_dev(g16['A']), ops.pack_dense(_dev(g16['W']), _dev(g16['bias']), 36), 'floor',
                                                  out_kind='int16')), g16['y__floor__i16__s36'])
    m = load('matmul')
    for mode in ('conv_even', 'symmetric_inf', 'floor'):
        np.testing.assert_array_equal(_host(ops.matmul(_dev(m['Aq']), _dev(m['Bk']), 5, mode, trans_b=True)), m[f'qk__{mode}'])
        np.testing.assert_array_equal(_host(ops.matmul(_dev(m['P']), _dev(m['Bv']), 8, mode)), m[f'pv__{mode}'])
    a = load('add')
    np.testing.assert_array_equal(_host(ops.add(_dev(a['a']), _dev(a['b']))), a['y_i8'])
    np.testing.assert_array_equal(_host(ops.add(_dev(a['a'].view(np.uint8)), _dev(a['b'].view(np.uint8)))), a['y_u8'])
    np.testing.assert_array_equal(_host(ops.add(_dev(a['a']), _dev(a['b']), 1, 'conv_even')), a['y_i8_shift1_conv_even'])


@pytest.mark.gpu
def test_gpu_layernorm_softmax_attention_mlp():
    from aie4ml_amd import ops
    g = load('layernorm')
    for cols in (64, 48):
        for mode in ('conv_even', 'symmetric_inf', 'floor'):
            for s in (4, 7):
                got = _host(ops.layernorm(_dev(g[f'x{cols}']), _dev(g[f'gamma{cols}']), _dev(g[f'beta{cols}']), s, mode))
                np.testing.assert_array_equal(got, g[f'y{cols}__{mode}__{s}'], err_msg=f'{cols} {mode} {s}')
    sm = load('softmax')
    x = _dev(sm['x'])
    for kq in (1, 23, 92, 128):
        np.testing.assert_array_equal(_host(ops.softmax_exp(x, kq)), sm[f'exp_u8__{kq}'])
    np.testing.assert_array_equal(_host(ops.softmax_exp(x, 23, out_kind='int16')), sm['exp_i16__23'])
    for (B, S, D) in ((255, 3, 80), (60, 1, 56), (500, 3, 127)):
        np.testing.assert_array_equal(_host(ops.softmax_hccs(x, B, S, D)), sm[f'hccs_u8__{B}_{S}_{D}'])
    np.testing.assert_array_equal(_host(ops.softmax_hccs(x, 255, 3, 80, out_kind='int16')), sm['hccs_i16__255_3_80'])
    at = load('attention')
    q, k, v = _dev(at['q']), _dev(at['k']), _dev(at['v'])
    got = ops.attention(q, k, v, 6, 'conv_even', {'kind': 'exp', 'exp_kq': 23}, 7, 'conv_even')
    np.testing.assert_array_equal(_host(got), at['o__exp23'])
    got = ops.attention(q, k, v, 6, 'conv_even', {'kind': 'hccs', 'B': 255, 'S': 4, 'Dmax': 60}, 7, 'conv_even')
    np.testing.assert_array_equal(_host(got), at['o__hccs'])
    lg = ops.matmul(q, k, 6, 'conv_even', trans_b=True)
    np.testing.assert_array_equal(_host(ops.matmul(ops.softmax_exp(lg, 23), v, 7, 'conv_even')), at['o__exp23'])
    ml = load('mlp')
    for mode in ('positive_inf', 'symmetric_inf', 'conv_even'):
        specs = [ops.MlpLayerSpec(ops.pack_dense(_dev(ml[f'W{i}']), _dev(ml[f'b{i}']), 7), 7, i < 3, 'int8') for i in range(4)]
        np.testing.assert_array_equal(_host(ops.mlp(_dev(ml['x']), specs, mode)), ml[f'y__{mode}'])
