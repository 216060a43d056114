"""Float-simulation check of imported ONNX Q/DQ graphs: the semantics of the reference's
scripts/check_onnx_bit_exact.py:128-136. The same .onnx bytes go (a) through `from_onnx` -> passes -> resolve -> the
integer executor and (b) through tests/onnx_float_eval.py, a float64 evaluation of the ONNX operator definitions that
shares nothing with the package. The float outputs are put on the output tensor's integer grid (round half to even,
saturate) and compared.

Tolerances, stated here and measured by these tests:
  * graphs of Dense / MatMul / Add / ReLU (with folded power-of-two scales, folded biases, transposed operands):
    the reference's checker accepts 1 LSB because onnxruntime accumulates in float32; a float64 evaluation is exact on
    these graphs (every product and sum is an integer times a power of two below 2^53), so the bar here is 0 LSB;
  * graphs with the integer Softmax (2nd-order exp, floor reciprocal, floor product) or the integer LayerNorm: the
    operators approximate exp / 1/sqrt, so the distance to the float graph is a property of the reference's
    arithmetic, not of this implementation: see SOFTMAX_ATOL, LAYERNORM_ATOL, ENCODER_ATOL below.

The same comparisons run on the CPU against the oracle's graph interpreter (`-m "not gpu"`) and on the GPU against
`predict()` (`-m gpu`): a wrong shift, fold or scale in the importer, the passes or the resolution moves the integer
side away from the ONNX semantics in both.
"""

import numpy as np
import pytest

import onnx_float_eval as ofe
from aie4ml_amd import from_onnx, qint, workloads
from aie4ml_amd.frontends.onnx_writer import QdqWriter

# Measured distances (max |dq| in LSB of the output tensor) with the seeds below; the bounds sit just above them.
SOFTMAX_ATOL = 1     # uint8 probabilities (scale 1/256), accurate integer exp with a folded temperature: measured 1
HCCS_ATOL = 32       # the clipped-linear surrogate is a different function from exp by design: measured 31
LAYERNORM_ATOL = 1   # int8 output of one integer LayerNorm on exact inputs: measured 1
ENCODER_ATOL = 4     # whole encoder block with the accurate Softmax, small shape: measured 3
ENCODER_C5_ATOL = 5  # the same block at the C5 shape (hidden 768, 12 heads, FFN 3072, seq 128, LayerNorm over 768
                     # columns), 4 sequences: measured 4 (79.7 % of the outputs equal, 18.6 % off by 1, 1.7 % by more)


def _grid(r, shape, intent, lo=None, hi=None):
    """Random values on the grid of `intent` (so that the graph-input QuantizeLinear is exact or not, as we like)."""
    info_lo = -(1 << (intent.width - 1)) if intent.signed else 0
    info_hi = (1 << (intent.width - 1)) - 1 if intent.signed else (1 << intent.width) - 1
    return r.integers(info_lo if lo is None else lo, (info_hi if hi is None else hi) + 1, shape).astype(np.float64) / 2.0 ** intent.frac


def _dense(w, x, name, W, wq, out_q, bias=None, bq=None, relu=False, gemm=False):
    if gemm:   # Gemm(A, B^T, C) with transB = 1
        ins = [x, w.weight(f'{name}_w', np.ascontiguousarray(W.T), wq)]
        if bias is not None:
            ins.append(w.weight(f'{name}_b', bias, bq))
        (y,) = w.node('Gemm', ins, name=name, transB=1)
    else:
        (y,) = w.node('MatMul', [x, w.weight(f'{name}_w', W, wq)], name=name)
        if bias is not None:
            (y,) = w.node('Add', [y, w.weight(f'{name}_b', bias, bq)], name=f'{name}_bias')
    y = w.qdq(y, out_q)   # exporters put a Q/DQ pair behind every operator, the Relu included
    if relu:
        (y,) = w.node('Relu', [y], name=f'{name}_relu')
        y = w.qdq(y, out_q)
    return y


def mlp_graph(seed=1, batch=96):
    """Gemm(transB) + bias, MatMul + Add + Relu, different scales on every tensor, float inputs off the grid."""
    r = np.random.default_rng(seed)
    a0, a1, a2, a3 = qint(8, 5), qint(8, 3), qint(8, 4), qint(8, 2)
    w = QdqWriter('mlp')
    x = w.input('x', (batch, 24), a0)
    h = _dense(w, x, 'fc0', _grid(r, (24, 40), qint(8, 6)), qint(8, 6), a1, _grid(r, 40, qint(32, 11), -3000, 3000), qint(32, 11), gemm=True)
    h = _dense(w, h, 'fc1', _grid(r, (40, 32), qint(8, 7)), qint(8, 7), a2, _grid(r, 32, qint(32, 10), -2000, 2000), qint(32, 10), relu=True)
    h = _dense(w, h, 'fc2', _grid(r, (32, 7), qint(8, 5)), qint(8, 5), a3)
    w.output(h, (batch, 7))
    feeds = {'x': r.uniform(-4.2, 4.2, (batch, 24))}   # saturates and rounds at the input quantiser
    return w.to_bytes(), {'Iterations': 1}, feeds


def attention_no_softmax_graph(seed=2, batch=3, seq=48, hidden=64, heads=2, transposed_input=False):
    """QKV projection, Split, per-head Transpose(K), Q.K^T, a power-of-two Mul folded into the MatMul's shift, then
    (logits).V, Concat, output projection, residual Add. With `transposed_input` the graph input arrives as
    [batch, hidden, seq] and a Transpose feeds the projection (a transposed left operand)."""
    r = np.random.default_rng(seed)
    act, wq, bq = qint(8, 4), qint(8, 7), qint(32, 11)
    hd = hidden // heads
    w = QdqWriter('attn')
    if transposed_input:
        xt = w.input('x', (batch, hidden, seq), act)
        (x,) = w.node('Transpose', [xt], name='x_t', perm=[0, 2, 1])
    else:
        x = w.input('x', (batch, seq, hidden), act)
    qkv = _dense(w, x, 'qkv', _grid(r, (hidden, 3 * hidden), wq, -40, 40), wq, act, _grid(r, 3 * hidden, bq, -4000, 4000), bq)
    q, k, v = w.node('Split', [qkv, w.const('sizes', np.array([hidden] * 3, dtype=np.int64))], 3, name='qkv_split', axis=-1)
    hs = w.const('head_sizes', np.array([hd] * heads, dtype=np.int64))
    qs, ks, vs = (w.node('Split', [t, hs], heads, name=f'{n}_heads', axis=2) for t, n in ((q, 'q'), (k, 'k'), (v, 'v')))
    outs = []
    for h in range(heads):
        (kt,) = w.node('Transpose', [ks[h]], name=f'kt{h}', perm=[0, 2, 1])
        (lg,) = w.node('MatMul', [qs[h], kt], name=f'qk{h}')
        if h % 2 == 0:   # Mul by 2^-3 before the quantiser: folds into the MatMul's output shift
            (lg,) = w.node('Mul', [lg, w.const(f'c{h}', np.array(0.125, dtype=np.float32))], name=f'qk_scale{h}')
            lg = w.qdq(lg, qint(8, 1))
        else:            # Div by 4
            (lg,) = w.node('Div', [lg, w.const(f'c{h}', np.array(4.0, dtype=np.float32))], name=f'qk_scale{h}')
            lg = w.qdq(lg, qint(8, 0))
        (o,) = w.node('MatMul', [lg, vs[h]], name=f'pv{h}')
        outs.append(w.qdq(o, qint(8, -1)))
    (cat,) = w.node('Concat', outs, name='concat', axis=-1)
    proj = _dense(w, cat, 'proj', _grid(r, (hidden, hidden), wq, -40, 40), wq, act)
    if not transposed_input:
        (res,) = w.node('Add', [x, proj], name='residual')
        proj = w.qdq(res, act)
    w.output(proj, (batch, seq, hidden))
    shape = (batch, hidden, seq) if transposed_input else (batch, seq, hidden)
    return w.to_bytes(), {'Iterations': 1}, {'x': _grid(r, shape, act)}


def ffn_graph(seed=3, rows=80, hidden=64, ffn=192):
    """Dense + ReLU, Dense, residual Add (saturating), one output."""
    r = np.random.default_rng(seed)
    act, wq, bq = qint(8, 4), qint(8, 7), qint(32, 11)
    w = QdqWriter('ffn')
    x = w.input('x', (rows, hidden), act)
    h = _dense(w, x, 'up', _grid(r, (hidden, ffn), wq), wq, qint(8, 3), _grid(r, ffn, bq, -9000, 9000), bq, relu=True)
    # a bias lives on the accumulator's grid (input scale x weight scale), as exporters write it: 2^-(3+7) here
    y = _dense(w, h, 'down', _grid(r, (ffn, hidden), wq), wq, act, _grid(r, hidden, qint(32, 10), -9000, 9000), qint(32, 10))
    (res,) = w.node('Add', [x, y], name='residual')
    w.output(w.qdq(res, act), (rows, hidden))
    return w.to_bytes(), {'Iterations': 1}, {'x': _grid(r, (rows, hidden), act)}


def softmax_graph(seed=4, rows=64, cols=128, approx='exp'):
    """Quantised logits -> (temperature Mul) -> Softmax -> uint8 probabilities."""
    r = np.random.default_rng(seed)
    lq, prob = qint(8, 3), qint(8, 8, signed=False)
    w = QdqWriter('softmax')
    x = w.input('x', (rows, cols), lq)
    cfg = {'Iterations': 1}
    if approx == 'exp':
        (x,) = w.node('Mul', [x, w.const('temp', np.array(0.5, dtype=np.float32))], name='temperature')
    else:
        cfg['LayerDirectives'] = {'sm': {'approximation': 'hccs', 'hccs': {'B': 255, 'S': 8, 'Dmax': 31}}}
    (p,) = w.node('Softmax', [x], name='sm', axis=-1)
    w.output(w.qdq(p, prob), (rows, cols))
    return w.to_bytes(), cfg, {'x': _grid(r, (rows, cols), lq, -60, 60)}


def layernorm_graph(seed=5, rows=64, cols=256):
    r = np.random.default_rng(seed)
    act = qint(8, 4)
    w = QdqWriter('ln')
    x = w.input('x', (rows, cols), act)
    g = w.const('gamma', (r.integers(32, 128, cols) / 128.0).astype(np.float32))
    b = w.const('beta', (r.integers(-15, 16, cols) / 16.0).astype(np.float32))
    (y,) = w.node('LayerNormalization', [x, g, b], name='ln', axis=-1, epsilon=2.0 ** -8)
    w.output(w.qdq(y, act), (rows, cols))
    return w.to_bytes(), {'Iterations': 1}, {'x': _grid(r, (rows, cols), act, -100, 100)}


def encoder_graph(softmax='exp', shape=(2, 64, 128, 2, 256)):
    data, cfg, x = workloads.c5_encoder_block_onnx(*shape, softmax=softmax)
    return data, cfg, {'x': x.astype(np.float64) / 16.0}


# ---- the two integer executors ----------------------------------------------------------------------------------

def _integer_outputs(model, feeds, executor):
    """Raw integer outputs, name -> int64 array, with float graph inputs quantised at the boundary."""
    graph = model.context.ir.logical
    names = list(graph.output_tensor_names)
    if executor == 'gpu':
        got = model.predict(feeds if len(feeds) > 1 else next(iter(feeds.values())), quantize_in=True, dequantize_out=False)
        return got if isinstance(got, dict) else {names[0]: got}
    from oracle import oracle
    from oracle.graph import run_graph

    prepared = model.prepare_inputs(feeds if len(feeds) > 1 else next(iter(feeds.values())), quantize=True)
    ints = {k: np.asarray(v)[0] if np.asarray(v).ndim > len(graph.tensors[k].shape) else np.asarray(v) for k, v in prepared.items()}
    vals = run_graph(model, oracle, ints)
    return {n: np.asarray(vals[n]).astype(np.int64) for n in names}


def _compare(build, executor, atol):
    data, cfg, feeds = build()
    model = from_onnx(data, cfg)
    if executor == 'gpu':
        model.compile()
    else:   # everything up to the resolved constants; packing uploads to the device and is not needed by the oracle
        from aie4ml_amd.passes import GPU_PIPELINE, PackKernelArtifacts, run_aie_passes

        run_aie_passes(model.context, [cls() for cls in GPU_PIPELINE if cls is not PackKernelArtifacts])
    got = _integer_outputs(model, feeds, executor)
    ref = ofe.run(data, feeds)
    assert len(ref) == len(got)
    worst = 0
    for (fname, fval), (iname, ival) in zip(ref.items(), got.items()):
        t = model.context.ir.logical.tensors[iname]
        dt = model._io_dtype(t, 'output')
        ref_q = ofe.requantize_output(fval, dt.width, dt.signed, dt.frac)
        ival = np.asarray(ival).reshape(ref_q.shape)
        diff = np.abs(ref_q - ival)
        worst = max(worst, int(diff.max()))
        assert diff.max() <= atol, f'{fname}: max |dq| = {int(diff.max())} > {atol} ({int((diff > atol).sum())} of {diff.size})'
        assert ival.std() > 0, f'{iname}: degenerate output, the check would be vacuous'
    return worst


EXACT = {
    'mlp': mlp_graph,
    'attention_no_softmax': attention_no_softmax_graph,
    'attention_transposed_input': lambda: attention_no_softmax_graph(seed=7, transposed_input=True),
    'ffn': ffn_graph,
}
APPROX = {
    'softmax_exp': (lambda: softmax_graph(approx='exp'), SOFTMAX_ATOL),
    'softmax_hccs': (lambda: softmax_graph(approx='hccs'), HCCS_ATOL),
    'layernorm': (layernorm_graph, LAYERNORM_ATOL),
    'encoder_exp': (lambda: encoder_graph('exp'), ENCODER_ATOL),
}


@pytest.mark.parametrize('name', sorted(EXACT))
def test_linear_graphs_match_the_float_graph_exactly_cpu(name):
    assert _compare(EXACT[name], 'oracle', 0) == 0


@pytest.mark.parametrize('name', sorted(APPROX))
def test_softmax_layernorm_graphs_within_stated_tolerance_cpu(name):
    build, atol = APPROX[name]
    _compare(build, 'oracle', atol)


@pytest.mark.gpu
@pytest.mark.parametrize('name', sorted(EXACT))
def test_linear_graphs_match_the_float_graph_exactly_gpu(name):
    assert _compare(EXACT[name], 'gpu', 0) == 0


@pytest.mark.gpu
@pytest.mark.parametrize('name', sorted(APPROX))
def test_softmax_layernorm_graphs_within_stated_tolerance_gpu(name):
    build, atol = APPROX[name]
    _compare(build, 'gpu', atol)


@pytest.mark.gpu
def test_encoder_block_at_the_c5_shape_within_stated_tolerance_gpu():
    _compare(lambda: encoder_graph('exp', (4, 128, 768, 12, 3072)), 'gpu', ENCODER_C5_ATOL)


def test_a_wrong_shift_is_caught(monkeypatch):
    """The check has teeth: an output shift that is off by one in the Dense resolution fails it."""
    from aie4ml_amd.op_impls import precision

    real = precision.resolve_accumulator_output_shift

    def off_by_one(*a, **k):
        return real(*a, **k) + 1

    import aie4ml_amd.op_impls.dense as dense_mod

    for mod in (precision, dense_mod):
        if hasattr(mod, 'resolve_accumulator_output_shift'):
            monkeypatch.setattr(mod, 'resolve_accumulator_output_shift', off_by_one)
    with pytest.raises(AssertionError, match='max .dq.'):
        _compare(ffn_graph, 'oracle', 0)


def test_evaluator_reads_what_other_writers_emit():
    """The evaluator's own protobuf reader against hand-assembled bytes (typed repeated fields instead of raw_data)."""
    import struct

    def key(num, wt):
        return bytes([(num << 3) | wt])

    def ld(num, payload):
        assert len(payload) < 128
        return key(num, 2) + bytes([len(payload)]) + payload

    scale = key(2, 0) + bytes([1]) + ld(8, b's') + ld(4, struct.pack('<f', 0.25))          # float_data, rank 0
    zp = key(2, 0) + bytes([3]) + ld(8, b'z') + key(5, 0) + bytes([0])                      # int32_data, int8
    node = ld(1, b'x') + ld(1, b's') + ld(1, b'z') + ld(2, b'y') + ld(4, b'QuantizeLinear')
    graph = ld(1, node) + ld(5, scale) + ld(5, zp) + ld(11, ld(1, b'x')) + ld(12, ld(1, b'y'))
    out = ofe.run(ld(7, graph), {'x': np.array([0.125, 0.375, -0.125, 100.0, -0.625])})
    assert out['y'].dtype == np.int8 and out['y'].tolist() == [0, 2, 0, 127, -2]            # ties to even, saturation
