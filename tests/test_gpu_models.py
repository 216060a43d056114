"""GPU tests of the operator-graph executor: graphs built through the front end, lowered by the pass
pipeline, run with GPUModel.predict on the MI355X and compared bit for bit with the CPU oracle evaluating
the same resolved graph node by node."""

import numpy as np
import pytest

from aie4ml_amd import GraphBuilder, qint, workloads
from aie4ml_amd.aie_types import RoundingMode

from oracle.graph import run_graph

pytestmark = pytest.mark.gpu


def _graph_check(model, oracle, inputs):
    model.compile()
    got = model.predict(inputs if len(inputs) > 1 else next(iter(inputs.values())), simulator='gpu',
                        quantize_in=False, dequantize_out=False)
    vals = run_graph(model, oracle, inputs)
    outs = model.context.ir.logical.output_tensor_names
    if len(outs) == 1:
        got = {outs[0]: got}
    for name in outs:
        want = vals[name].astype(np.int64)
        assert got[name].shape[-want.ndim:] == want.shape or got[name].size == want.size
        np.testing.assert_array_equal(got[name].reshape(want.shape), want, err_msg=name)
    return got


@pytest.mark.parametrize('rounding', [RoundingMode.RND, RoundingMode.RND_CONV, RoundingMode.TRN])
def test_c1_mlp_graph(oracle, rounding):
    model, x, layers = workloads.c1_mlp_model(batch=256, rounding=rounding)
    model.compile()
    assert model.context.config['gpu_fusion_plan']['mlp_chains'] == [['fc0_aie', 'fc1_aie', 'fc2_aie', 'fc3_aie']]
    y = model.predict(x, quantize_in=False, dequantize_out=False)
    mode = {RoundingMode.RND: 'symmetric_inf', RoundingMode.RND_CONV: 'conv_even', RoundingMode.TRN: 'floor'}[rounding]
    want = x
    for W, b, shift, relu, kind in layers:
        want = oracle.dense(want, W, b, shift, mode, relu=relu, out=kind)
    np.testing.assert_array_equal(y, want.astype(np.int64))
    # float inputs on the grid quantise to the same integers; dequantised output is value / 2^frac
    yf = model.predict(x.astype(np.float64))
    np.testing.assert_array_equal(yf, want.astype(np.float64))
    assert yf.dtype == np.float64


def test_mlp_graph_unfused_matches_fused(oracle):
    model, x, layers = workloads.c1_mlp_model(batch=128)
    model.compile()
    fused = model.predict(x, quantize_in=False, dequantize_out=False)
    model.context.config['gpu_fusion_plan'] = {'add_layernorm': {}, 'mlp_chains': []}
    unfused = model.predict(x, quantize_in=False, dequantize_out=False)
    np.testing.assert_array_equal(fused, unfused)


def test_wide_mlp_picks_its_form_by_batch(oracle):
    """A fusable chain of wide layers (57-200-200-200-3, rows of 57 bytes): planned as one chain; on 32 768 samples the
    fused launch runs on the matrix units and is taken, on 3000 samples the executor's cost model prefers one GEMM per
    layer to the small-batch form of the fused launch, on 64 samples it takes that form. The oracle's integers in all."""
    import torch
    from aie4ml_amd.model import _mlp_layers_are_faster
    r = np.random.default_rng(31)
    dims = [57, 200, 200, 200, 3]
    for batch, kinds in ((32768, ['mlp']), (64, ['mlp'])):
        gb = GraphBuilder()
        t = gb.input('x', (batch, dims[0]), qint(8, 4))
        for i in range(4):
            W = r.integers(-100, 100, (dims[i], dims[i + 1])) / 128.0
            b = r.integers(-512, 512, dims[i + 1]) / 2048.0
            t = gb.dense(t, W, qint(8, 7), qint(8, 4), bias=b, bias_precision=qint(32, 11), relu=i < 3, name=f'fc{i}')
        gb.output(t)
        model = gb.build()
        model.compile()
        assert len(model.context.config['gpu_fusion_plan']['mlp_chains']) == 1
        x = np.clip(np.rint(r.normal(0, 30, (batch, dims[0]))), -128, 127).astype(np.int8)
        trace = []
        model.execute({'x': torch.from_numpy(x).cuda()}, trace=trace)
        assert [t['kind'] for t in trace] == kinds
        _graph_check(model, oracle, {'x': x})
    shapes = list(zip(dims[:-1], dims[1:]))
    assert _mlp_layers_are_faster(32768, shapes) and not _mlp_layers_are_faster(64, shapes)


def test_wide_mlp_with_aligned_rows_on_a_large_batch_stays_fused(oracle):
    """The same widths behind 64 inputs (rows that can be fetched in 16-byte pieces): from 4096 samples the fused launch
    runs on the matrix units and the executor keeps it, whatever the per-layer model says."""
    import torch

    r = np.random.default_rng(33)
    dims = [64, 200, 200, 200, 3]
    batch = 8192 + 40
    gb = GraphBuilder()
    t = gb.input('x', (batch, dims[0]), qint(8, 4))
    for i in range(4):
        W = r.integers(-100, 100, (dims[i], dims[i + 1])) / 128.0
        b = r.integers(-512, 512, dims[i + 1]) / 2048.0
        t = gb.dense(t, W, qint(8, 7), qint(8, 4), bias=b, bias_precision=qint(32, 11), relu=i < 3, name=f'fc{i}')
    gb.output(t)
    model = gb.build()
    model.compile()
    x = np.clip(np.rint(r.normal(0, 30, (batch, dims[0]))), -128, 127).astype(np.int8)
    trace = []
    model.execute({'x': torch.from_numpy(x).cuda()}, trace=trace)
    assert [t['kind'] for t in trace] == ['mlp']
    _graph_check(model, oracle, {'x': x})


def test_iteration_axis_folds_into_batch(oracle):
    model, x, layers = workloads.c1_mlp_model(batch=64)
    xs = np.stack([x, x[::-1], x])                      # (iterations, batch, features)
    y = model.predict(xs, quantize_in=False, dequantize_out=False)
    assert y.shape == (3 * 64, layers[-1][0].shape[1])
    one = model.predict(x, quantize_in=False, dequantize_out=False)
    np.testing.assert_array_equal(y[:64], one)
    np.testing.assert_array_equal(y[64:128], one[::-1])


def test_float_quantisation_at_the_boundary(oracle):
    gb = GraphBuilder()
    x = gb.input('x', (32, 64), qint(8, 4, rounding=RoundingMode.RND_CONV))
    r = np.random.default_rng(3)
    W = r.integers(-100, 100, (64, 48)) / 128.0
    bias = r.integers(-64, 64, 48) / 8.0
    y = gb.dense(x, W, qint(8, 7), qint(8, 2, rounding=RoundingMode.RND), bias=bias, bias_precision=qint(32, 11),
                 name='fc')
    gb.output(y)
    model = gb.build()
    xf = r.normal(0, 3, (32, 64))                        # off-grid floats, some beyond +-8 (saturate)
    got = model.predict(xf)
    xq = np.clip(np.round(xf * 16), -128, 127)           # numpy's round is ties-to-even = RND_CONV
    want = oracle.dense(xq.astype(np.int8), np.round(W * 128).astype(np.int8), np.round(bias * 2048).astype(np.int32),
                        4 + 7 - 2, 'symmetric_inf')
    np.testing.assert_array_equal(got, want / 4.0)


@pytest.mark.parametrize('probs_out', [True, False])
@pytest.mark.parametrize('approx', ['exp', 'hccs'])
def test_attention_core_graph(oracle, approx, probs_out):
    r = np.random.default_rng(11)
    gb = GraphBuilder()
    q = gb.input('q', (3, 128, 64), qint(8, 4))
    k = gb.input('k', (3, 128, 64), qint(8, 4))
    v = gb.input('v', (3, 128, 64), qint(8, 4))
    kt = gb.transpose(k, (0, 2, 1))
    logits = gb.matmul(q, kt, qint(8, 0), name='qk')
    d = None
    if approx == 'exp':
        logits = gb.scale(logits, 0.125, name='temp')
    else:
        d = {'approximation': 'hccs', 'hccs': {'B': 255, 'S': 3, 'Dmax': 84}}
    p = gb.softmax(logits, qint(8, 8, signed=False), name='sm', directives=d)
    o = gb.matmul(p, v, qint(8, 4), name='pv')
    gb.output(o)
    if probs_out:
        gb.output(p)
    model = gb.build()
    model.compile()
    # with the probabilities as a graph output the three operators run separately, otherwise as one launch
    assert (len(model.context.config['gpu_fusion_plan']['attention']) == 0) is probs_out
    ins = {n: np.clip(r.normal(0, 20, (3, 128, 64)), -128, 127).astype(np.int8) for n in 'qkv'}
    got = _graph_check(model, oracle, ins)
    assert len(got) == (2 if probs_out else 1)           # several outputs come back as a dict by name


@pytest.mark.parametrize('keep_sum', [False, True])
def test_add_layernorm_graph(oracle, keep_sum):
    r = np.random.default_rng(5)
    gb = GraphBuilder()
    a = gb.input('a', (4, 96, 768), qint(8, 4))
    b = gb.input('b', (4, 96, 768), qint(8, 4))
    s = gb.add(a, b, qint(8, 4), name='res')
    y = gb.layer_norm(s, r.integers(32, 128, 768) / 128.0, r.integers(-15, 16, 768) / 16.0, qint(8, 4), eps_q0=1,
                      name='ln')
    gb.output(y)
    if keep_sum:
        gb.output(s)
    model = gb.build()
    model.compile()
    assert model.context.config['gpu_fusion_plan']['add_layernorm']['res_aie']['keep_sum'] is keep_sum
    ins = {n: np.clip(r.normal(0, 30, (4, 96, 768)), -128, 127).astype(np.int8) for n in 'ab'}
    _graph_check(model, oracle, ins)


@pytest.mark.parametrize('softmax', ['exp', 'hccs'])
def test_encoder_block_small(oracle, softmax):
    model, x = workloads.c5_encoder_block(batch=2, seq=64, hidden=128, heads=2, ffn=256, softmax=softmax)
    model.compile()
    (grp,) = model.context.config['gpu_fusion_plan']['attention']
    assert len(grp['heads']) == 2 and grp['concat']     # both heads in one fused-attention launch
    got = _graph_check(model, oracle, {'x': x})
    model.context.config['gpu_fusion_plan'] = {}        # and the same graph operator by operator
    _graph_check(model, oracle, {'x': x})
    out = next(iter(got.values()))
    assert len(np.unique(out)) > 32        # a live signal, not a saturated or constant tensor


@pytest.mark.parametrize('seq', [100, 197])
def test_encoder_block_with_a_sequence_off_the_tile_grid(oracle, seq):
    """A vision transformer's token counts (196 patches + 1, or 100): the heads still go to the fused attention
    launch, which masks the keys that its tiles of 32 have too many."""
    model, x = workloads.c5_encoder_block(batch=2, seq=seq, hidden=128, heads=2, ffn=256, softmax='exp')
    model.compile()
    (grp,) = model.context.config['gpu_fusion_plan']['attention']
    assert len(grp['heads']) == 2 and grp['concat']
    import torch

    trace = []
    dx = {'x': torch.from_numpy(x).cuda()}
    model.execute(dx, trace=trace)
    assert [t['kind'] for t in trace].count('attention') == 1 and not any(t['kind'] in ('matmul', 'softmax') for t in trace)
    got = _graph_check(model, oracle, {'x': x})
    model.context.config['gpu_fusion_plan'] = {}        # and the same graph operator by operator
    _graph_check(model, oracle, {'x': x})
    assert len(np.unique(next(iter(got.values())))) > 32


@pytest.mark.parametrize('batch,taken', [(16, True), (2, True), (16, False)])
def test_narrow_encoder_block_runs_in_four_launches(oracle, batch, taken, monkeypatch):
    """64 features, 4 heads of 16, feed-forward width 256: the Q/K/V projection, the attention, the output projection
    with its Add and LayerNorm, and the feed-forward pair with theirs. Where the chain kernel refuses at launch, the last
    two run as their parts."""
    import torch

    from aie4ml_amd import ops

    model, x = workloads.c5_encoder_block(batch=batch, seq=64, hidden=64, heads=4, ffn=256, softmax='exp')
    model.compile()
    plan = model.context.config['gpu_fusion_plan']
    assert [len(v['chain']) for v in plan['mlp_add_layernorm'].values()] == [1, 2]
    if not taken:
        monkeypatch.setattr(ops, 'mlp_add_layernorm_applicable', lambda x, layers: False)
    trace = []
    model.execute({'x': torch.from_numpy(x).cuda()}, trace=trace)
    assert [t['kind'] for t in trace] == ['dense', 'attention', 'mlp_add_layer_norm', 'mlp_add_layer_norm']
    got = _graph_check(model, oracle, {'x': x})
    model.context.config['gpu_fusion_plan'] = {}        # and the same graph operator by operator
    _graph_check(model, oracle, {'x': x})
    assert len(np.unique(next(iter(got.values())))) > 32


def test_encoder_block_c5_shape(oracle):
    """BERT-base geometry (hidden 768, 12 heads of 64, FFN 3072, seq 128) on a batch the oracle finishes
    in seconds; the full batch of 64 differs only in the number of independent sequences."""
    model, x = workloads.c5_encoder_block(batch=2, seq=128, hidden=768, heads=12, ffn=3072, softmax='hccs')
    got = _graph_check(model, oracle, {'x': x})
    out = next(iter(got.values()))
    assert out.shape[-1] == 768 and len(np.unique(out)) > 64


@pytest.mark.parametrize('softmax', ['exp', 'hccs'])
def test_encoder_block_from_onnx_file(oracle, softmax, tmp_path):
    """The block written as an ONNX Q/DQ file, read back without the onnx package, run on float inputs: equals the
    builder-made graph on the same parameters, and the oracle evaluating the imported graph."""
    from aie4ml_amd import from_onnx

    shape = (2, 64, 128, 2, 256)
    data, cfg, x = workloads.c5_encoder_block_onnx(*shape, softmax=softmax)
    path = tmp_path / 'encoder_block.onnx'
    path.write_bytes(data)
    model = from_onnx(str(path), cfg)
    y = model.predict(x.astype(np.float32) / 16.0)                       # float in, float out (value / 2^4)
    ref_model, x2 = workloads.c5_encoder_block(*shape, softmax=softmax)
    want = ref_model.predict(x2, quantize_in=False, dequantize_out=False)
    np.testing.assert_array_equal(y * 16.0, want)
    name = model.context.ir.logical.output_tensor_names[0]
    np.testing.assert_array_equal(want, run_graph(model, oracle, {'x': x})[name].astype(np.int64))
    assert len(model.context.config['gpu_fusion_plan']['attention']) == 1


def test_captured_execution_replays_match_eager(oracle):
    """The whole encoder block recorded into a HIP graph: every replay, with eager work and synchronisations in
    between and fresh inputs each time, equals the eager result."""
    import torch

    model, x = workloads.c5_encoder_block(4, 64, 128, 2, 256, softmax='exp')
    model.compile()
    name = model.context.ir.logical.output_tensor_names[0]
    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    captured = model.capture({'x': dev(x)})
    r = np.random.default_rng(2)
    for i in range(4):
        xi = np.roll(x, i, axis=0) if i < 3 else np.clip(np.rint(r.normal(0, 30, x.shape)), -128, 127).astype(np.int8)
        eager = model.execute({'x': dev(xi)})[name].clone()
        torch.cuda.synchronize()
        junk = torch.randint(-128, 127, (1 << 20,), dtype=torch.int8, device='cuda').add_(1)   # unrelated eager work
        replay = captured({'x': dev(xi)})[name]
        torch.cuda.synchronize()
        assert torch.equal(replay, eager), f'replay {i}'
        del junk
    with pytest.raises(ValueError, match='captured for'):
        captured({'x': dev(x[:2])})


def test_int16_activation_mlp_graph(oracle):
    """An MLP with 16-bit activations and 8-bit weights (the (16, 8) combination hls4ml models use): the dense
    variant accepts it, the fused-MLP kernel (8-bit only) is not chosen, results equal the oracle."""
    r = np.random.default_rng(23)
    gb = GraphBuilder()
    t = gb.input('x', (64, 48), qint(16, 8))
    dims = [48, 96, 64, 10]
    for i in range(3):
        W = r.integers(-100, 100, (dims[i], dims[i + 1])) / 128.0
        b = r.integers(-512, 512, dims[i + 1]) / 32768.0
        t = gb.dense(t, W, qint(8, 7), qint(16, 8), bias=b, bias_precision=qint(32, 15), relu=i < 2, name=f'fc{i}')
    gb.output(t)
    model = gb.build()
    model.compile()
    assert model.context.config['gpu_fusion_plan']['mlp_chains'] == []
    x = r.integers(-32768, 32768, (64, 48)).astype(np.int16)
    _graph_check(model, oracle, {'x': x})


def test_int16_weight_mlp_graph(oracle):
    """16-bit activations and 16-bit weights (hls4ml's default ap_fixed<16, 6> everywhere): the (16, 16)
    combination with its 64-bit accumulator, through the graph executor."""
    r = np.random.default_rng(29)
    gb = GraphBuilder()
    t = gb.input('x', (32, 48), qint(16, 10))
    dims = [48, 80, 10]
    for i in range(2):
        W = r.integers(-32768, 32768, (dims[i], dims[i + 1])) / 2.0 ** 14
        b = r.integers(-2 ** 20, 2 ** 20, dims[i + 1]) / 2.0 ** 24
        t = gb.dense(t, W, qint(16, 14), qint(16, 10), bias=b, bias_precision=qint(32, 24), relu=i < 1, name=f'fc{i}')
    gb.output(t)
    model = gb.build()
    model.compile()
    cfg = model.context.ir.execution.get('fc0_aie').config
    assert cfg.accumulator_tag == 'acc64' and cfg.shift == 14
    assert model.context.config['gpu_fusion_plan']['mlp_chains'] == []
    x = r.integers(-32768, 32768, (32, 48)).astype(np.int16)
    _graph_check(model, oracle, {'x': x})


@pytest.mark.parametrize('rhs_bits', [8, 16])
def test_int16_matmul_graph(oracle, rhs_bits):
    """Dynamic MatMul with a 16-bit left operand inside a graph: transposed right operand (folded Transpose),
    then a second MatMul on the result, as the attention score / context pair does."""
    r = np.random.default_rng(rhs_bits)
    gb = GraphBuilder()
    q = gb.input('q', (2, 3, 40, 32), qint(16, 12))
    k = gb.input('k', (2, 3, 40, 32), qint(rhs_bits, rhs_bits - 2))
    v = gb.input('v', (2, 3, 40, 32), qint(rhs_bits, rhs_bits - 2))
    s = gb.matmul(q, gb.transpose(k, (0, 1, 3, 2)), qint(16, 9), name='qk')
    gb.output(gb.matmul(s, v, qint(16, 8), name='pv'))
    model = gb.build()
    model.compile()
    cfg = model.context.ir.execution.get('qk_aie').config
    assert cfg.accumulator_tag == ('acc64' if rhs_bits == 16 else 'acc32') and cfg.flags.transpose_rhs
    lo, hi = -(1 << (rhs_bits - 1)), 1 << (rhs_bits - 1)
    dt = np.int16 if rhs_bits == 16 else np.int8
    feeds = {'q': r.integers(-32768, 32768, (2, 3, 40, 32)).astype(np.int16),
             'k': r.integers(lo, hi, (2, 3, 40, 32)).astype(dt), 'v': r.integers(lo, hi, (2, 3, 40, 32)).astype(dt)}
    _graph_check(model, oracle, feeds)


# ---- float compute path through the graph executor ----------------------------------------------------------------

def _float_net(compute_dtype, batch, n_in=32, n_h=32, n_out=16, seed=0):
    r = np.random.default_rng(seed)
    q = qint(16, 13)
    w0, b0 = r.normal(0, 0.05, (n_in, n_h)), r.normal(0, 0.05, n_h)
    w1, b1 = r.normal(0, 0.05, (n_h, n_out)), r.normal(0, 0.05, n_out)
    gb = GraphBuilder({'ComputeDtype': compute_dtype})
    x = gb.input('x', (batch, n_in), q)
    h = gb.dense(x, w0, q, q, bias=b0, bias_precision=q, relu=True, name='dense0')
    gb.output(gb.dense(h, w1, q, q, bias=b1, bias_precision=q, name='dense1'))
    return gb.build(), (w0, b0, w1, b1)


@pytest.mark.parametrize('compute_dtype,rtol,atol', [('bfloat16', 1e-2, 5e-2), ('float', 1e-3, 1e-3)])
@pytest.mark.parametrize('batch,width', [(4, 32), (512, 256)])
def test_forced_float_mode_mlp(oracle, compute_dtype, rtol, atol, batch, width):
    """The reference's float test (tests/test_float_sim.py:113-149): a quantised two-layer network forced into
    float mode must match the plain float network within rtol / atol. The comparison model is that test's
    _float_reference: bfloat16 by truncation of the input, the weights and the hidden activations, float32
    bias, float32 matmuls. Width 256 takes the tiled matrix-core kernel, width 32 the generic one."""
    model, (w0, b0, w1, b1) = _float_net(compute_dtype, batch, n_in=width, n_h=width)
    x = np.random.default_rng(42).uniform(-2.0, 2.0, (batch, width)).astype(np.float32)
    y = model.predict(x)
    assert y.dtype == np.float64 and y.shape == (batch, 16)
    cast = oracle.bf16_truncate if compute_dtype == 'bfloat16' else (lambda a: np.asarray(a, dtype=np.float32))
    h = cast(x) @ cast(w0) + b0.astype(np.float32)
    h = np.maximum(h, 0.0).astype(np.float32)
    ref = cast(h) @ cast(w1) + b1.astype(np.float32)
    np.testing.assert_allclose(y, ref, rtol=rtol, atol=atol)
    # and against the layer-by-layer oracle (exact accumulation, one rounding per layer): at most one unit in
    # the last place of the output format per layer, carried through the second layer
    fmt = 'bfloat16' if compute_dtype == 'bfloat16' else 'float32'
    h_o = oracle.dense_float(cast(x), cast(w0), b0, relu=True, fmt=fmt)
    y_o = oracle.dense_float(h_o, cast(w1), b1, fmt=fmt)
    ulp = 2.0 ** -7 if fmt == 'bfloat16' else 2.0 ** -22
    slack = ulp * (np.abs(h_o).astype(np.float64) @ np.abs(cast(w1)).astype(np.float64) + np.abs(y_o) + np.abs(b1))
    assert np.all(np.abs(y - y_o) <= slack)


def test_float_graph_with_matmul_and_add(oracle):
    from aie4ml_amd.aie_types import FloatFormat, FloatIntent

    bf = FloatIntent(16, FloatFormat.BF16)
    r = np.random.default_rng(7)
    gb = GraphBuilder()
    a = gb.input('a', (2, 64, 32), bf)
    b = gb.input('b', (2, 64, 32), bf)
    s = gb.add(a, b, bf, name='sum')
    gb.output(gb.matmul(s, gb.transpose(b, (0, 2, 1)), bf, name='mm'))
    model = gb.build()
    A = oracle.bf16_truncate(r.normal(0, 1, (2, 64, 32)))
    B = oracle.bf16_truncate(r.normal(0, 1, (2, 64, 32)))
    y = model.predict({'a': A, 'b': B})
    s_o = oracle.add_float(A, B, 'bfloat16')
    y_o = oracle.matmul_float(s_o, B, trans_b=True, fmt='bfloat16')
    bound = 2.0 ** -7 * np.abs(y_o) + 34 * 2.0 ** -24 * (np.abs(s_o).astype(np.float64) @ np.abs(np.swapaxes(B, -1, -2)))
    assert np.all(np.abs(y - y_o) <= bound)


@pytest.mark.parametrize('bf', [False, True])
def test_float_onnx_model_predicts(oracle, bf):
    from aie4ml_amd import from_onnx
    from aie4ml_amd.frontends import onnx_proto as op

    r = np.random.default_rng(1)
    cast = oracle.bf16_truncate if bf else (lambda a: np.asarray(a, dtype=np.float32))
    elem = op.BFLOAT16 if bf else op.FLOAT
    w0, b0, w1 = cast(r.normal(0, 0.1, (64, 128))), cast(r.normal(0, 0.1, 128)), cast(r.normal(0, 0.1, (128, 32)))
    g = op.Graph(name='float_mlp')
    g.inputs.append(op.ValueInfo('x', elem, (8, 64)))
    g.initializers += [op.Tensor('w0', w0, bfloat16=bf), op.Tensor('b0', b0, bfloat16=bf), op.Tensor('w1', w1, bfloat16=bf)]
    g.nodes += [op.Node('Gemm', ['x', 'w0', 'b0'], ['h'], 'fc0', {}), op.Node('Relu', ['h'], ['hr'], 'relu0', {}),
                op.Node('MatMul', ['hr', 'w1'], ['y'], 'fc1', {})]
    g.outputs.append(op.ValueInfo('y', elem, (8, 32)))
    model = from_onnx(op.serialize_model(op.Model(graph=g, opset={'': 17}, producer_name='test')))
    x = cast(r.uniform(-2, 2, (8, 64)))
    y = model.predict(x)
    fmt = 'bfloat16' if bf else 'float32'
    h_o = oracle.dense_float(x, w0, b0, relu=True, fmt=fmt)
    y_o = oracle.dense_float(h_o, w1, None, fmt=fmt)
    rtol, atol = (1e-2, 5e-2) if bf else (1e-3, 1e-3)  # the reference's float tolerances (tests/test_float_sim.py:81-87)
    np.testing.assert_allclose(y, y_o, rtol=rtol, atol=atol)


def test_report_times_every_launch(oracle):
    """report(): one entry per launch group of the executor, operation count by the reference's convention
    (2 * n_in * n_out per row, dense and matmul only; src/aie4ml/report.py:133-155)."""
    model, x, _layers = workloads.c1_mlp_model(batch=256)
    rep = model.report(x, repeats=3)
    assert rep['design']['launches'] == 1 and rep['kernels'][0]['kind'] == 'mlp'      # four dense nodes, one fused launch
    assert rep['design']['ops'] == 2 * 256 * (16 * 64 + 64 * 32 + 32 * 32 + 32 * 5)
    assert rep['latency']['graph_replay_us'] > 0 and rep['bottleneck']['name'] == rep['kernels'][0]['name']
    text = str(rep)
    assert 'GPU execution report' in text and 'Bottleneck' in text

    onnx_bytes, config, x_int = workloads.c5_encoder_block_onnx(batch=2, seq=32, hidden=128, heads=2, ffn=256, softmax='hccs')
    from aie4ml_amd import from_onnx

    enc = from_onnx(onnx_bytes, config)
    rep = enc.report(repeats=3)
    kinds = [k['kind'] for k in rep['kernels']]
    # the QKV projection, all heads in one attention launch, and layers this narrow carry the residual add and the
    # LayerNorm behind them: the output projection in one launch, the FFN pair in another
    assert kinds == ['dense', 'attention', 'mlp_add_layer_norm', 'mlp_add_layer_norm']
    assert abs(sum(k['pct'] for k in rep['kernels']) - 100.0) < 1.0
    assert all(k['time_us'] > 0 for k in rep['kernels'])


def test_predict_with_hip_graph_replay(oracle):
    """Config key 'HipGraph': predict() records one HIP graph per input signature and replays it; every call must
    equal the eager result, also after a call with another batch size in between."""
    data, cfg, x = workloads.c5_encoder_block_onnx(batch=4, seq=32, hidden=128, heads=2, ffn=256, softmax='exp')
    from aie4ml_amd import from_onnx

    eager = from_onnx(data, cfg)
    graphed = from_onnx(data, dict(cfg, HipGraph=True))
    r = np.random.default_rng(3)
    for i in range(4):
        xi = r.integers(-128, 128, x.shape).astype(np.int8)
        want = eager.predict(xi, quantize_in=False, dequantize_out=False)
        got = graphed.predict(xi, quantize_in=False, dequantize_out=False)
        assert np.array_equal(got, want), i
    assert len(graphed._captured) == 1


# ---- hls4ml model graphs --------------------------------------------------------------------------------------------

def test_hls4ml_mlp_matches_the_quantised_network(oracle):
    """The network of the reference's hls4ml test (tests/test_hls4ml_dense.py: QDense + quantized_relu layers, 8 bits),
    presented as hls4ml presents it (stand-in objects), must predict what the quantised network itself computes:
    exact fixed-point products, round-to-nearest-even and saturation at every activation quantiser."""
    from aie4ml_amd import from_hls4ml
    from tests.hls4ml_standin import qkeras_mlp

    dims, batch = [16, 64, 32, 32, 5], 256
    hls_model, weights = qkeras_mlp(dims, batch)
    model = from_hls4ml(hls_model)
    r = np.random.default_rng(11)
    x = r.uniform(-4, 4, (batch, dims[0]))
    y = model.predict(x)
    assert y.shape == (batch, 5) and y.dtype == np.float64

    def quant(v, frac, lo, hi):  # numpy's rint is round-half-even
        return np.clip(np.rint(v * 2.0 ** frac), lo, hi) / 2.0 ** frac

    h = quant(x, 5, -128, 127)
    for i, (W, b) in enumerate(weights):
        z = h @ W + b                                   # exact: every operand is a small dyadic rational
        h = quant(np.maximum(z, 0), 8, 0, 255) if i < len(weights) - 1 else quant(z, 5, -128, 127)
    assert np.array_equal(y, h)
    # and bit for bit against the oracle's graph interpreter
    _graph_check(model, oracle, {'input_layer': np.rint(quant(x, 5, -128, 127) * 32).astype(np.int8)})


@pytest.mark.parametrize('mode', ['io', 'internal'])
@pytest.mark.parametrize('in_shape', [(384,), (8, 16, 384)])
def test_fanout_graph_with_two_outputs(oracle, mode, in_shape):
    """The graphs of the reference's fan-out test (tests/test_hls4ml_fanout.py:28-68): the input ('io') or a shared
    Dense + ReLU ('internal') feeds two Dense branches, each a graph output; batch 1, five iterations; also with the
    multi-dimensional input of its nd cases. predict() returns a dict keyed by output tensor name."""
    r = np.random.default_rng(len(in_shape) + (mode == 'io'))
    hidden, act, wq, relu6 = 256, qint(8, 5), qint(8, 5), qint(8, 2, signed=False)
    gb = GraphBuilder({'Iterations': 5})
    t = gb.input('input_layer', (1,) + in_shape, act)

    def dense(src, name, out_prec, relu):
        W = r.integers(-128, 128, (int(src.shape[-1]), hidden)) / 32.0
        b = r.integers(-128, 128, hidden) / 32.0
        return gb.dense(src, W, wq, out_prec, bias=b, bias_precision=wq, relu=relu, name=name)

    if mode == 'internal':
        t = dense(t, 'shared_internal_dense', qint(8, 8, signed=False), True)
    y1 = gb.output(dense(t, 'branch1', relu6, True))
    y2 = gb.output(dense(t, 'branch2', relu6, True))
    model = gb.build()
    x = r.integers(-128, 128, (5, 1) + in_shape).astype(np.int8)
    got = model.predict(x, quantize_in=False, dequantize_out=False)
    assert list(got) == [y1.name, y2.name] and got[y1.name].shape == (5,) + in_shape[:-1] + (hidden,)
    assert not np.array_equal(got[y1.name], got[y2.name])
    flat = x.reshape((5,) + in_shape)
    want = run_graph(model, oracle, {'input_layer': flat})
    for name in (y1.name, y2.name):
        np.testing.assert_array_equal(got[name].reshape(want[name].shape), want[name].astype(np.int64))
    deq = model.predict(x.astype(np.float64) / 32.0)
    np.testing.assert_array_equal(deq[y1.name], got[y1.name] / 4.0)


def test_int16_input_with_8bit_layers_is_not_planned_as_fused_mlp(oracle):
    """int16 activations x int8 weights accumulate in acc32 like the 8-bit case, but the fused MLP launch only reads
    8-bit inputs: a chain whose head takes an int16 tensor and whose layers write int8 runs layer by layer."""
    r = np.random.default_rng(31)
    gb = GraphBuilder()
    t = gb.input('x', (48, 40), qint(16, 8))
    dims = [40, 64, 32, 6]
    for i in range(3):
        W = r.integers(-100, 100, (dims[i], dims[i + 1])) / 128.0
        b = r.integers(-512, 512, dims[i + 1]) / 2.0 ** (15 if i == 0 else 11)
        t = gb.dense(t, W, qint(8, 7), qint(8, 4), bias=b, bias_precision=qint(32, 15 if i == 0 else 11), relu=i < 2, name=f'fc{i}')
    gb.output(t)
    model = gb.build()
    model.compile()
    chains = model.context.config['gpu_fusion_plan']['mlp_chains']
    assert all('fc0_aie' not in c for c in chains)
    x = r.integers(-3000, 3000, (48, 40)).astype(np.int16)
    _graph_check(model, oracle, {'x': x})


def test_attention_with_unaligned_head_slices_runs_unfused(oracle):
    """Heads cut from a packed projection at offsets that are not multiples of 16 bytes (an 8-column prefix in front of
    Q): the fused attention launch needs 16-byte aligned head slices, so the planner must leave these heads to the
    separate MatMul / Softmax / MatMul launches (decided at run time, on the views' addresses); a logit shift above
    24 must do the same (decided by the planner)."""
    r = np.random.default_rng(37)
    batch, seq, heads, d = 2, 64, 2, 64
    width = 8 + 3 * heads * d
    for shift_case in ('unaligned', 'deep_shift'):
        gb = GraphBuilder()
        x = gb.input('x', (batch, seq, width), qint(8, 4))
        if shift_case == 'unaligned':
            _pad, q, k, v = gb.split(x, -1, [8, heads * d, heads * d, heads * d], name='qkv_split')
        else:
            q, k, v, _pad = gb.split(x, -1, [heads * d, heads * d, heads * d, 8], name='qkv_split')
        qs, ks, vs = (gb.split(t, -1, [d] * heads, name=f'{n}_heads') for t, n in ((q, 'q'), (k, 'k'), (v, 'v')))
        outs = []
        for h in range(heads):
            kt = gb.transpose(ks[h], (0, 2, 1), name=f'kt{h}')
            # acc frac 8; deep_shift: output frac -17 -> shift 25, beyond what the fused kernel takes
            lg = gb.matmul(qs[h], kt, qint(8, -3 if shift_case == 'unaligned' else -17), name=f'qk{h}')
            lg = gb.scale(lg, 2.0 ** (-5 if shift_case == 'unaligned' else -19), name=f'temp{h}')  # EXP_KQ = 92
            pr = gb.softmax(lg, qint(8, 8, signed=False), name=f'sm{h}')
            outs.append(gb.matmul(pr, vs[h], qint(8, 4), name=f'pv{h}'))
        gb.output(gb.concat(outs, -1, name='cat'))
        model = gb.build()
        model.compile()
        plan = model.context.config['gpu_fusion_plan']['attention']
        if shift_case == 'deep_shift':
            assert plan == []
        # 'unaligned': the planner sees head offsets inside the nearest source tensor only (0, 64 of a 128-wide slice);
        # that the slice itself starts 8 bytes into rows of 392 bytes shows at run time, where the executor falls back
        xin = np.clip(np.rint(r.normal(0, 24, (batch, seq, width))), -128, 127).astype(np.int8)
        _graph_check(model, oracle, {'x': xin})
