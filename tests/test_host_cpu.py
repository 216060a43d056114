"""CPU tests of the host side: fixed-point helpers, graph passes, numeric resolution, error behaviour.
No kernels run; the pipeline is driven up to Resolve (packing uploads to the GPU)."""

import numpy as np
import pytest

from aie4ml_amd import GraphBuilder, qint
from aie4ml_amd.aie_types import AIEDataType, RoundingMode, SaturationMode
from aie4ml_amd.ir import get_backend_context
from aie4ml_amd.passes import (FoldBias, FoldScale, FoldViewOps, FuseActivationCasts, PlanGpuFusion, Resolve,
                               run_aie_passes)
from aie4ml_amd.quant_utils import (apply_rounding, dequantize_output, handle_overflow, quantize_input,
                                    quantize_to_int, wrap_to_width)

FRONT = (FoldBias, FoldScale, FuseActivationCasts, FoldViewOps, Resolve)


def lower(gb, passes=FRONT):
    ctx = gb.ctx
    run_aie_passes(ctx, [p() for p in passes])
    return ctx


# ---- fixed-point helpers (values fixed by the definition of each mode) ---------------------------------

def test_apply_rounding_ties():
    v = np.array([-2.5, -1.5, -0.5, 0.5, 1.5, 2.5, 2.4, -2.6])
    assert apply_rounding(v, RoundingMode.TRN).tolist() == [-3, -2, -1, 0, 1, 2, 2, -3]
    assert apply_rounding(v, RoundingMode.RND_MIN_INF).tolist() == [-3, -2, -1, 0, 1, 2, 2, -3]
    assert apply_rounding(v, RoundingMode.TRN_ZERO).tolist() == [-2, -1, -0.0, 0, 1, 2, 2, -2]
    assert apply_rounding(v, RoundingMode.RND_INF).tolist() == [-2, -1, -0.0, 1, 2, 3, 3, -2]
    assert apply_rounding(v, RoundingMode.RND_CONV).tolist() == [-2, -2, -0.0, 0, 2, 2, 2, -3]
    assert apply_rounding(v, RoundingMode.RND).tolist() == [-3, -2, -1, 1, 2, 3, 2, -3]


def test_overflow_modes():
    v = np.array([-300, -129, -128, 127, 128, 300])
    assert handle_overflow(v, 8, True, SaturationMode.SAT).tolist() == [-128, -128, -128, 127, 127, 127]
    assert handle_overflow(v, 8, True, SaturationMode.SAT_SYM).tolist() == [-127, -127, -127, 127, 127, 127]
    assert handle_overflow(v, 8, True, SaturationMode.SAT_ZERO).tolist() == [0, 0, 0, 127, 127, 127]
    assert handle_overflow(v, 8, True, SaturationMode.WRAP).tolist() == [-44, 127, -128, 127, -128, 44]
    assert handle_overflow(v, 8, False, SaturationMode.SAT).tolist() == [0, 0, 0, 127, 128, 255]
    assert wrap_to_width(np.array([256, 255, -1]), 8, False).tolist() == [0, 255, 255]


def test_quantize_input_and_dequantize():
    dt = AIEDataType('int8', frac=4, rounding=RoundingMode.RND_CONV, saturation=SaturationMode.SAT)
    x = np.array([0.03125, 0.09375, -0.09375, 7.99, -9.0, 1.0])
    assert quantize_input(x, dt).tolist() == [0, 2, -2, 127, -128, 16]   # 0.5 -> 0, 1.5 -> 2 (ties to even)
    assert quantize_input(x, dt).dtype == np.int8
    # integer arrays pass through untouched (cast only)
    assert quantize_input(np.array([300, -5], dtype=np.int64), dt).tolist() == [44, -5]
    du = AIEDataType('uint8', frac=8, rounding=RoundingMode.TRN, saturation=SaturationMode.WRAP)
    assert quantize_input(np.array([0.999, 1.0, -1 / 256]), du).tolist() == [255, 0, 255]
    assert dequantize_output(np.array([16, -8]), 4).tolist() == [1.0, -0.5]
    assert dequantize_output(np.array([3]), 0).dtype == np.float64
    w = quantize_to_int(np.array([0.5, -1.0, 0.996]), 7, 8, True, RoundingMode.RND, SaturationMode.SAT)
    assert w.tolist() == [64, -128, 127] and w.dtype == np.int8


# ---- passes ---------------------------------------------------------------------------------------------

def small_mlp(relu_on_last=False):
    gb = GraphBuilder()
    x = gb.input('x', (4, 16), qint(8, 4))
    r = np.random.default_rng(0)
    h = gb.dense(x, r.integers(-64, 64, (16, 32)) / 128.0, qint(8, 7), qint(8, 4), bias=r.integers(-8, 8, 32) / 16.0,
                 bias_precision=qint(32, 11), relu=True, name='fc0')
    y = gb.dense(h, r.integers(-64, 64, (32, 8)) / 128.0, qint(8, 7), qint(8, 3), bias=np.zeros(8),
                 bias_precision=qint(32, 11), relu=relu_on_last, name='fc1')
    gb.output(y)
    return gb


def test_fold_bias_fuse_relu_and_resolve_constants():
    gb = small_mlp()
    assert [n.op_type for n in gb.graph.nodes] == ['dense', 'add', 'activation', 'dense', 'add']
    ctx = lower(gb)
    assert [n.op_type for n in ctx.ir.logical.nodes] == ['dense', 'dense']
    fc0, fc1 = ctx.ir.logical.nodes
    assert fc0.metadata['use_bias'] and fc0.roles[fc0.inputs[2].name] == 'bias'
    assert fc0.traits['fused_activation'].data == {'activation': 'relu'}
    c0, c1 = ctx.ir.execution.get(fc0.name).config, ctx.ir.execution.get(fc1.name).config
    assert c0.shift == 4 + 7 - 4 and c1.shift == 4 + 7 - 3
    assert c0.rounding_mode == 'conv_even' and c0.accumulator_tag == 'acc32'
    assert c0.flags.use_relu and c0.flags.use_bias and not c1.flags.use_relu
    assert c0.precision['bias'].format == 'int32' and c0.precision['bias'].frac == 11
    assert c0.precision['acc'].frac == 11 and c0.precision['output'].format == 'int8'
    # weights and bias quantise exactly as the reference packs them: bias at 2^(in_frac + w_frac)
    inst = ctx.ir.execution.get(fc0.name)
    W, b = inst.variant.quantize_weight_bias(inst)
    r = np.random.default_rng(0)
    assert np.array_equal(W, r.integers(-64, 64, (16, 32)))
    assert np.array_equal(b, r.integers(-8, 8, 32) * 128) and b.dtype == np.int32


def test_rounding_token_map():
    from aie4ml_amd.op_impls.precision import aie_rounding_token

    want = {RoundingMode.TRN: 'floor', RoundingMode.RND_MIN_INF: 'floor', RoundingMode.RND_INF: 'ceil',
            RoundingMode.RND: 'symmetric_inf', RoundingMode.TRN_ZERO: 'symmetric_zero',
            RoundingMode.RND_ZERO: 'symmetric_zero', RoundingMode.RND_CONV: 'conv_even'}
    for mode, token in want.items():
        assert aie_rounding_token(qint(8, 0, rounding=mode)) == token


def test_relu_without_dense_has_no_kernel():
    gb = GraphBuilder()
    a = gb.input('a', (4, 32), qint(8, 4))
    b = gb.input('b', (4, 32), qint(8, 4))
    s = gb.add(a, b, qint(8, 4))
    (y,) = gb._emit('activation', 'lonely_relu', [s], [('y', s.shape, qint(8, 4))], ['lhs'], {'activation': 'relu'})
    gb.output(y)
    with pytest.raises(NotImplementedError, match='No family resolver'):
        lower(gb)


def attention_graph(scale=0.125, approx=None, hccs=None, frac=4):
    gb = GraphBuilder()
    q = gb.input('q', (2, 64, 32), qint(8, frac))
    k = gb.input('k', (2, 64, 32), qint(8, frac))
    v = gb.input('v', (2, 64, 32), qint(8, frac))
    kt = gb.transpose(k, (0, 2, 1))
    logits = gb.matmul(q, kt, qint(8, frac), name='qk')
    if scale is not None:
        logits = gb.scale(logits, scale, qint(8, frac), name='qk_scale')
    d = {}
    if approx:
        d['approximation'] = approx
    if hccs:
        d['hccs'] = hccs
    p = gb.softmax(logits, qint(8, 8, signed=False), name='sm', directives=d or None)
    o = gb.matmul(p, v, qint(8, frac), name='pv')
    gb.output(o)
    return gb


def test_transpose_folds_into_matmul_and_scale_prefers_softmax():
    # a Scale between MatMul and Softmax is absorbed by the Softmax (as in the reference: the consumer
    # is tried first), so the MatMul keeps its plain alignment shift and EXP_KQ carries the 1/8
    ctx = lower(attention_graph())
    kinds = [n.op_type for n in ctx.ir.logical.nodes]
    assert kinds == ['matmul', 'softmax', 'matmul']
    qk, sm, pv = ctx.ir.logical.nodes
    assert qk.traits['io_view'].data['inputs']['k'] == {'perm': [0, 2, 1]}
    assert 'output_scale' not in qk.traits and sm.traits['input_scale'].data['scale'] == 0.125
    c = ctx.ir.execution.get(qk.name).config
    assert c.flags.transpose_rhs and not c.flags.transpose_lhs
    assert c.shift == 4 + 4 - 4
    cs = ctx.ir.execution.get(sm.name).config
    assert cs.approximation == 'exp' and cs.exp_kq == 3    # round(log2(e) * 2^-4 / 8 * 256)
    assert cs.inv_shift == 15 and cs.rounding_mode == 'floor' and cs.precision['output'].format == 'uint8'
    cp = ctx.ir.execution.get(pv.name).config
    assert cp.precision['lhs'].format == 'uint8' and cp.shift == 8 + 4 - 4
    assert ctx.ir.execution.get('sm_aie') is not None
    assert lower(attention_graph(scale=None)).ir.execution.get('sm_aie').config.exp_kq == 23


def test_scale_after_matmul_folds_into_its_shift():
    gb = GraphBuilder()
    a = gb.input('a', (2, 16, 32), qint(8, 4))
    b = gb.input('b', (2, 32, 16), qint(8, 4))
    y = gb.scale(gb.matmul(a, b, qint(8, 4), name='mm'), 0.125, qint(8, 4))
    gb.output(y)
    ctx = lower(gb)
    (mm,) = ctx.ir.logical.nodes
    assert mm.traits['output_scale'].data['scale'] == 0.125
    c = ctx.ir.execution.get(mm.name).config
    assert c.shift == (4 + 4 - 4) + 3 and not c.flags.transpose_rhs   # alignment + log2(1/scale)


def test_scale_before_softmax_becomes_temperature():
    gb = GraphBuilder()
    x = gb.input('x', (8, 64), qint(8, 4))
    s = gb.scale(x, 0.5, qint(8, 4))
    p = gb.softmax(s, qint(8, 8, signed=False), name='sm')
    gb.output(p)
    ctx = lower(gb)
    (sm,) = ctx.ir.logical.nodes
    assert sm.traits['input_scale'].data['scale'] == 0.5
    assert ctx.ir.execution.get(sm.name).config.exp_kq == round(1.4426950408889634 * 2 ** -4 * 0.5 * 256)


def matmul_scale_graph(scale):
    gb = GraphBuilder()
    a = gb.input('a', (2, 16, 32), qint(8, 4))
    b = gb.input('b', (2, 32, 16), qint(8, 4))
    gb.output(gb.scale(gb.matmul(a, b, qint(8, 4), name='mm'), scale, qint(8, 4)))
    return gb


def test_scale_errors():
    with pytest.raises(NotImplementedError, match='not a power of two'):
        lower(matmul_scale_graph(0.3))
    with pytest.raises(ValueError, match=r'range \(0, 1\]'):
        lower(matmul_scale_graph(2.0))
    gb = GraphBuilder()
    x = gb.input('x', (4, 32), qint(8, 4))
    y = gb.scale(x, 0.5)
    gb.output(gb.add(y, x, qint(8, 4)))
    with pytest.raises(NotImplementedError, match='no adjacent op absorbs this scale'):
        lower(gb)


def test_softmax_variants_and_hccs_validation():
    ok = {'B': 100, 'S': 1, 'Dmax': 90}
    ctx = lower(attention_graph(scale=None, approx='hccs', hccs=ok))
    cfg = ctx.ir.execution.get('sm_aie').config
    assert cfg.approximation == 'hccs' and cfg.hccs == ok and cfg.param_sets == 1 and not cfg.use_clb
    with pytest.raises(ValueError, match='directives missing S, Dmax'):
        lower(attention_graph(scale=None, approx='hccs', hccs={'B': 10}))
    with pytest.raises(ValueError, match=r'cols \* B <= 32767'):
        lower(attention_graph(scale=None, approx='hccs', hccs={'B': 600, 'S': 1, 'Dmax': 5}))
    with pytest.raises(ValueError, match=r'B - S\*Dmax >= 0'):
        lower(attention_graph(scale=None, approx='hccs', hccs={'B': 50, 'S': 1, 'Dmax': 60}))
    with pytest.raises(ValueError, match='>= 256 for reciprocal range'):
        lower(attention_graph(scale=None, approx='hccs', hccs={'B': 60, 'S': 1, 'Dmax': 59}))  # 64 * 1 < 256
    with pytest.raises(ValueError, match="'S' must be in"):
        lower(attention_graph(scale=None, approx='hccs', hccs={'B': 300, 'S': 200, 'Dmax': 1}))
    with pytest.raises(ValueError, match='cannot apply a runtime input_scale'):
        gb = GraphBuilder()
        x = gb.input('x', (8, 64), qint(8, 4))
        gb.output(gb.softmax(gb.scale(x, 0.5), qint(8, 8, signed=False), name='sm',
                             directives={'approximation': 'hccs', 'hccs': ok}))
        lower(gb)
    # exp needs the logit scale in range: frac 12 -> KQ rounds to 0
    with pytest.raises(ValueError, match='1 <= EXP_KQ'):
        lower(attention_graph(scale=None, frac=12))
    # int8 output is not a softmax output type
    gb = GraphBuilder()
    x = gb.input('x', (8, 64), qint(8, 4))
    gb.output(gb.softmax(x, qint(8, 7), name='sm'))
    with pytest.raises(ValueError, match='requires uint8 or int16 output'):
        lower(gb)


def test_matmul_rules():
    gb = GraphBuilder()
    a = gb.input('a', (2, 16, 32), qint(8, 4))
    b = gb.input('b', (2, 32, 16), qint(8, 4, signed=False))
    gb.output(gb.matmul(a, b, qint(8, 4)))
    with pytest.raises(ValueError, match='RHS must use a signed integer precision'):
        lower(gb)
    gb = GraphBuilder()
    a = gb.input('a', (2, 16, 32), qint(8, 4))
    b = gb.input('b', (2, 16, 32), qint(8, 4))
    bt = gb.transpose(b, (1, 0, 2))
    gb.output(gb.matmul(a, bt, qint(8, 4)))
    with pytest.raises(ValueError):
        lower(gb)
    gb = GraphBuilder()
    a = gb.input('a', (2, 16, 32), qint(32, 4))
    gb.output(gb.dense(a, np.zeros((32, 8)), qint(8, 7), qint(8, 4)))
    with pytest.raises(ValueError, match='no dense variant matches'):
        lower(gb)
    # 16-bit activations with 8-bit weights are a Dense combination (acc32), not a MatMul one
    gb = GraphBuilder()
    a = gb.input('a', (2, 16, 32), qint(16, 8))
    gb.output(gb.dense(a, np.zeros((32, 8)), qint(8, 7), qint(16, 8), name='fc'))
    cfg = lower(gb).ir.execution.get('fc_aie').config
    assert cfg.precision['lhs'].format == 'int16' and cfg.shift == 8 + 7 - 8 and cfg.accumulator_tag == 'acc32'
    # 16 x 16 accumulates in 64 bits (precision.py:122-123); 8-bit activations with 16-bit weights have no variant
    gb = GraphBuilder()
    a = gb.input('a', (2, 16, 32), qint(16, 8))
    gb.output(gb.dense(a, np.zeros((32, 8)), qint(16, 14), qint(16, 8), name='fc'))
    cfg = lower(gb).ir.execution.get('fc_aie').config
    assert cfg.precision['rhs'].format == 'int16' and cfg.accumulator_tag == 'acc64' and cfg.shift == 14
    assert cfg.precision['acc'].format == 'int64' and cfg.precision['bias'].format == 'int32'
    gb = GraphBuilder()
    a = gb.input('a', (2, 16, 32), qint(8, 4))
    gb.output(gb.dense(a, np.zeros((32, 8)), qint(16, 14), qint(16, 8), name='fc'))
    with pytest.raises((RuntimeError, ValueError)):
        lower(gb)
    # the dynamic MatMul takes the same width combinations (matmul/common.py:52-66)
    for rhs_bits, tag in ((8, 'acc32'), (16, 'acc64')):
        gb = GraphBuilder()
        a = gb.input('a', (2, 16, 32), qint(16, 8))
        b = gb.input('b', (2, 32, 16), qint(rhs_bits, 4))
        gb.output(gb.matmul(a, b, qint(8, 4), name='mm'))
        cfg = lower(gb).ir.execution.get('mm_aie').config
        assert cfg.accumulator_tag == tag and cfg.shift == 8 + 4 - 4 and cfg.precision['lhs'].format == 'int16'
    gb = GraphBuilder()
    a = gb.input('a', (2, 16, 32), qint(8, 4))
    b = gb.input('b', (2, 32, 16), qint(16, 4))
    gb.output(gb.matmul(a, b, qint(8, 4)))
    with pytest.raises((RuntimeError, ValueError)):
        lower(gb)


def ln_graph(cols=64, eps=None, eps_q0=None, gamma=None, out_frac=5):
    gb = GraphBuilder()
    a = gb.input('a', (8, cols), qint(8, 4))
    b = gb.input('b', (8, cols), qint(8, 4))
    s = gb.add(a, b, qint(8, 4), name='res')
    y = gb.layer_norm(s, np.ones(cols) * 0.75 if gamma is None else gamma, np.zeros(cols), qint(8, out_frac), epsilon=eps,
                      eps_q0=eps_q0, name='ln')
    gb.output(y)
    return gb


def test_layernorm_resolution_and_errors():
    ctx = lower(ln_graph(eps=2.0 ** -8))
    cfg = ctx.ir.execution.get('ln_aie').config
    assert cfg.eps_q0 == 1 and cfg.out_shift == 5 and cfg.gamma_shift == 7 and cfg.cols == 64 and cfg.rows == 8
    assert cfg.precision['gamma'].frac == 7 and cfg.precision['beta'].frac == 15 and cfg.power_of_two_cols
    assert ctx.ir.execution.get('res_aie').config.shift == 0
    assert lower(ln_graph(eps_q0=3)).ir.execution.get('ln_aie').config.eps_q0 == 3
    assert not lower(ln_graph(cols=48)).ir.execution.get('ln_aie').config.power_of_two_cols  # extension
    with pytest.raises(ValueError, match='not exactly representable'):
        lower(ln_graph(eps=1e-5))
    with pytest.raises(ValueError, match='positive variance floor'):
        lower(ln_graph(eps=0.0))
    with pytest.raises(ValueError, match=r'out_shift=20 must be in \[0, 15\]'):
        lower(ln_graph(out_frac=20))
    from aie4ml_amd.op_impls.layernorm import pack_layernorm_param

    assert pack_layernorm_param([0.5, -1.0, 0.996], name='gamma', full_inner=3, frac=7).tolist() == [64, -128, 127]
    with pytest.raises(ValueError, match='cannot be represented as signed int16 Q7'):
        pack_layernorm_param([300.0], name='gamma', full_inner=1, frac=7)
    with pytest.raises(ValueError, match='does not match full_inner'):
        pack_layernorm_param([1.0, 2.0], name='beta', full_inner=3, frac=15)


def test_add_requires_one_storage_type():
    gb = GraphBuilder()
    a = gb.input('a', (8, 64), qint(8, 4))
    b = gb.input('b', (8, 64), qint(8, 5))
    gb.output(gb.add(a, b, qint(8, 4)))
    with pytest.raises(ValueError, match='same storage type'):
        lower(gb)
    gb = GraphBuilder()
    a = gb.input('a', (8, 64), qint(8, 4))
    b = gb.input('b', (8, 32), qint(8, 4))
    gb.output(gb.add(a, b, qint(8, 4)))
    with pytest.raises(ValueError, match='exact-shape inputs'):
        lower(gb)


def test_split_concat_become_view_placeholders():
    gb = GraphBuilder()
    x = gb.input('x', (4, 8, 96), qint(8, 4))
    a, b, c = gb.split(x, -1, [32, 32, 32], name='sp')
    y = gb.concat([c, a], -1, name='cat')
    gb.output(gb.add(y, gb.concat([a, b], -1, name='cat2'), qint(8, 4)))
    ctx = lower(gb)
    sp = next(n for n in ctx.ir.logical.nodes if n.name == 'sp_aie')
    assert sp.is_placeholder and sp.traits['slice_view'].data['axis'] == 2
    assert [s['start'] for s in sp.traits['slice_view'].data['slices']] == [0, 32, 64]
    cat = next(n for n in ctx.ir.logical.nodes if n.name == 'cat_aie')
    assert cat.is_placeholder and [s['start'] for s in cat.traits['concat_view'].data['slices']] == [0, 32]
    assert ctx.ir.execution.get('sp_aie') is None


def test_gpu_fusion_plan():
    ctx = lower(small_mlp(), FRONT + (PlanGpuFusion,))
    assert ctx.config['gpu_fusion_plan']['mlp_chains'] == [['fc0_aie', 'fc1_aie']]
    ctx = lower(ln_graph(), FRONT + (PlanGpuFusion,))
    assert ctx.config['gpu_fusion_plan']['add_layernorm'] == {'res_aie': {'layer_norm': 'ln_aie', 'keep_sum': False}}


def test_encoder_block_graph_lowers():
    from aie4ml_amd import workloads

    model, x = workloads.c5_encoder_block(batch=2, seq=32, hidden=64, heads=2, ffn=128)
    ctx = lower(GraphHolder(model), FRONT + (PlanGpuFusion,))
    kinds = [n.op_type for n in ctx.ir.logical.nodes if not n.is_placeholder]
    assert kinds.count('dense') == 4 and kinds.count('matmul') == 4 and kinds.count('softmax') == 2
    assert kinds.count('layer_norm') == 2 and kinds.count('add') == 2
    plan = ctx.config['gpu_fusion_plan']
    assert plan['add_layernorm']['residual1_aie'] == {'layer_norm': 'ln1_aie', 'keep_sum': False}
    assert plan['mlp_chains'] == [['ffn1_aie', 'ffn2_aie']]   # widths 64/128/64 fit the fused-MLP kernel
    assert x.shape == (2, 32, 64) and x.dtype == np.int8
    (grp,) = plan['attention']              # head_dim 32: both heads in one fused launch, Q / K / V slices 32 apart
    assert len(grp['heads']) == 2 and grp['concat'] == 'heads_concat_aie'
    assert plan['dense_add_layernorm'] == {}  # 64 outputs: too narrow for the projection that normalises its own rows


def test_plan_joins_narrow_layers_with_the_add_and_layernorm_behind_them():
    from aie4ml_amd import workloads

    model, _ = workloads.c5_encoder_block(batch=2, seq=32, hidden=64, heads=2, ffn=128)
    plan = lower(GraphHolder(model), FRONT + (PlanGpuFusion,)).config['gpu_fusion_plan']
    # the attention output projection (64 -> 64) is a chain of one; the feed-forward pair is a chain of two
    assert plan['mlp_add_layernorm'] == {
        'residual1_aie': {'chain': ['attn_out_aie'], 'layer_norm': 'ln1_aie', 'residual': 'x'},
        'residual2_aie': {'chain': ['ffn1_aie', 'ffn2_aie'], 'layer_norm': 'ln2_aie', 'residual': 'ln1_out'}}
    assert plan['dense_add_layernorm'] == {}
    # layers wider than the chain kernel's 256 columns stay out of it
    model, _ = workloads.c5_encoder_block(batch=1, seq=32, hidden=768, heads=12, ffn=3072)
    assert lower(GraphHolder(model), FRONT + (PlanGpuFusion,)).config['gpu_fusion_plan']['mlp_add_layernorm'] == {}


def test_plan_marks_projections_that_can_normalise_their_rows():
    from aie4ml_amd import workloads

    model, _ = workloads.c5_encoder_block(batch=1, seq=32, hidden=768, heads=12, ffn=3072)
    ctx = lower(GraphHolder(model), FRONT + (PlanGpuFusion,))
    plan = ctx.config['gpu_fusion_plan']
    # the attention output projection (768 -> 768) feeds only the residual add in front of a LayerNorm whose input nobody
    # else reads; the second feed-forward projection has 3072 inputs, past what that kernel is used for
    assert plan['dense_add_layernorm'] == {'residual1_aie': {'dense': 'attn_out_aie', 'layer_norm': 'ln1_aie', 'residual': 'x'}}
    assert set(plan['add_layernorm']) == {'residual1_aie', 'residual2_aie'}


def test_attention_plan_merges_heads():
    from aie4ml_amd import workloads

    model, _ = workloads.c5_encoder_block(batch=2, seq=32, hidden=192, heads=3, ffn=128)
    ctx = lower(GraphHolder(model), FRONT + (PlanGpuFusion,))
    (grp,) = ctx.config['gpu_fusion_plan']['attention']
    assert [tr['qk'] for tr in grp['heads']] == ['qk0_aie', 'qk1_aie', 'qk2_aie']
    assert grp['concat'] == 'heads_concat_aie' and (grp['q_base'], grp['k_base'], grp['v_base']) == (0, 0, 0)
    # a lone triple (its probabilities are also a graph output in the second graph: not fusable)
    gb = attention_graph(scale=None)
    ctx = lower(gb, FRONT + (PlanGpuFusion,))
    (grp,) = ctx.config['gpu_fusion_plan']['attention']         # head_dim 32 has a fused kernel of its own
    assert grp['concat'] is None
    gb = GraphBuilder()                                         # head_dim 40 has none (48 would run padded to 64)
    q = gb.input('q', (2, 64, 40), qint(8, 4))
    k = gb.input('k', (2, 64, 40), qint(8, 4))
    v = gb.input('v', (2, 64, 40), qint(8, 4))
    p = gb.softmax(gb.matmul(q, gb.transpose(k, (0, 2, 1)), qint(8, 4), name='qk'), qint(8, 8, signed=False), name='sm')
    gb.output(gb.matmul(p, v, qint(8, 4), name='pv'))
    assert lower(gb, FRONT + (PlanGpuFusion,)).config['gpu_fusion_plan']['attention'] == []
    gb = GraphBuilder()
    q = gb.input('q', (2, 64, 64), qint(8, 4))
    k = gb.input('k', (2, 64, 64), qint(8, 4))
    v = gb.input('v', (2, 64, 64), qint(8, 4))
    p = gb.softmax(gb.matmul(q, gb.transpose(k, (0, 2, 1)), qint(8, 4), name='qk'), qint(8, 8, signed=False), name='sm')
    gb.output(gb.matmul(p, v, qint(8, 4), name='pv'))
    ctx = lower(gb, FRONT + (PlanGpuFusion,))
    (grp,) = ctx.config['gpu_fusion_plan']['attention']
    assert grp['concat'] is None and grp['heads'][0]['softmax'] == 'sm_aie'
    gb.output(p)
    ctx = lower(gb, FRONT + (PlanGpuFusion,))
    assert ctx.config['gpu_fusion_plan']['attention'] == []


class GraphHolder:
    """Adapts a model to the `gb.ctx` attribute lower() expects."""

    def __init__(self, model):
        self.ctx = get_backend_context(model)


def test_predict_input_contract_without_gpu():
    gb = small_mlp()
    model = gb.build()
    with pytest.raises(ValueError, match='Unknown simulator'):
        model.predict(np.zeros((4, 16)), simulator='x86')
    good = model.prepare_inputs(np.zeros((4, 16)))
    assert good['x'].shape == (1, 4, 16) and good['x'].dtype == np.int8
    assert model.prepare_inputs(np.zeros((3, 4, 16)))['x'].shape == (3, 4, 16)
    assert model.prepare_inputs({'x': np.zeros((1, 4, 16))})['x'].shape == (1, 4, 16)
    with pytest.raises(ValueError, match='expected shape'):
        model.prepare_inputs(np.zeros((4, 15)))
    with pytest.raises(ValueError, match='quantize=False requires integer inputs'):
        model.prepare_inputs(np.zeros((4, 16)), quantize=False)
    assert model.prepare_inputs(np.full((4, 16), 1.0))['x'][0, 0, 0] == 16   # 1.0 * 2^4


# ---- float compute path (host side) -----------------------------------------------------------------------

def _float_mlp(config=None, in_prec=None, w_prec=None):
    # the network of the reference's float test (tests/test_float_sim.py:77-78: 32 -> 32 -> 16, batch 4)
    r = np.random.default_rng(0)
    q = qint(16, 13)
    gb = GraphBuilder(config or {})
    x = gb.input('x', (4, 32), in_prec or q)
    h = gb.dense(x, r.normal(0, 0.05, (32, 32)), w_prec or q, in_prec or q, bias=r.normal(0, 0.05, 32),
                 bias_precision=w_prec or q, relu=True, name='dense0')
    y = gb.dense(h, r.normal(0, 0.05, (32, 16)), w_prec or q, in_prec or q, bias=r.normal(0, 0.05, 16),
                 bias_precision=w_prec or q, name='dense1')
    gb.output(y)
    return gb


@pytest.mark.parametrize('compute_dtype,fmt', [('bfloat16', 'bfloat16'), ('float', 'float32'), ('float32', 'float32')])
def test_force_float_mode_resolves_float_variants(compute_dtype, fmt):
    from aie4ml_amd.passes import ForceFloatMode

    gb = _float_mlp({'ComputeDtype': compute_dtype})
    ctx = lower(gb, (ForceFloatMode,) + FRONT)
    for name, relu in (('dense0_aie', True), ('dense1_aie', False)):
        inst = ctx.ir.execution.get(name)
        assert inst.variant.variant_id == 'dense.b.r.float.gfx950.v1'
        cfg = inst.config
        assert cfg.shift == 0 and cfg.accumulator_tag == 'accfloat' and cfg.rounding_mode == 'conv_even'
        assert cfg.flags.use_relu is relu and cfg.flags.use_bias is True
        assert {cfg.precision[k].format for k in ('lhs', 'rhs', 'output')} == {fmt}
        assert cfg.precision['bias'].format == 'float32' and cfg.precision['acc'].format == 'accfloat'
    assert [n.op_type for n in ctx.ir.logical.nodes] == ['dense', 'dense']  # bias and ReLU folded as in integer mode
    # the fused int8 MLP kernel must not claim a float chain
    PlanGpuFusion().transform(ctx)
    assert ctx.config['gpu_fusion_plan']['mlp_chains'] == []


def test_float_mode_rules():
    from aie4ml_amd.aie_types import FloatFormat, FloatIntent
    from aie4ml_amd.op_impls.float_ops import pack_as_float
    from aie4ml_amd.passes import ForceFloatMode

    with pytest.raises(ValueError, match='is not recognised'):
        lower(_float_mlp({'ComputeDtype': 'float16'}), (ForceFloatMode,) + FRONT)
    bf, f32 = FloatIntent(16, FloatFormat.BF16), FloatIntent(32, FloatFormat.FP32)
    # mixed float / fixed point, and mixed float formats, are rejected as in the reference's _resolve_numeric
    with pytest.raises(ValueError):
        lower(_float_mlp(in_prec=bf, w_prec=qint(8, 6)))
    with pytest.raises(ValueError, match='share float precision'):
        lower(_float_mlp(in_prec=bf, w_prec=f32))
    f8 = FloatIntent(8, FloatFormat.FP8_E4M3)
    cfg = lower(_float_mlp(in_prec=f8, w_prec=f8)).ir.execution.get('dense0_aie').config
    assert cfg.precision['lhs'].format == 'fp8_e4m3' and cfg.precision['bias'].format == 'float32'
    # the fp8 packer: ties away from zero, bias 7, 0x7f from 480 up (matmul/common.py:262-276)
    from aie4ml_amd.op_impls.float_ops import float32_to_fp8_codes, fp8_codes_to_float32
    assert float32_to_fp8_codes([0.0, 1.0, -1.0, 1.0625, 448.0, 464.0, 2.0 ** -9, 0.3]).tolist() == \
        [0x00, 0x38, 0xB8, 0x39, 0x7E, 0x7F, 0x01, 0x2A]
    assert fp8_codes_to_float32([0x38, 0x7E, 0x01, 0x2A, 0xB9]).tolist() == [1.0, 448.0, 2.0 ** -9, 0.3125, -1.125]
    # a power-of-two scale cannot fold into a float dense
    gb = GraphBuilder()
    x = gb.input('x', (4, 32), bf)
    gb.output(gb.scale(gb.dense(x, np.zeros((32, 8)), bf, bf, name='fc'), 0.5, bf))
    with pytest.raises(NotImplementedError, match='not implemented for float'):
        lower(gb)
    # LayerNorm and Softmax have no float variant
    gb = GraphBuilder()
    x = gb.input('x', (4, 32), bf)
    gb.output(gb.softmax(x, bf))
    with pytest.raises((ValueError, NotImplementedError)):
        lower(gb)
    # parameters reach bfloat16 by truncation
    v = np.array([1.0, 1.00390625, 1.0078125, -1.00390625, 3.14159], dtype=np.float32)
    assert pack_as_float(v, 'bfloat16').tolist() == [1.0, 1.0, 1.0078125, -1.0, 3.140625]
    assert pack_as_float(v, 'float32').tolist() == v.tolist()


# ---- hls4ml model graphs (read by attribute access; stand-in objects, hls4ml is not installed) ----------------

def test_hls4ml_lowering_gives_the_reference_graph():
    from aie4ml_amd.frontends.hls4ml_lower import lower_hls4ml_model
    from aie4ml_amd.passes import FoldApplyAlpha
    from tests.hls4ml_standin import qkeras_mlp

    model, weights = qkeras_mlp([16, 64, 32, 5], batch=8)
    ctx = lower_hls4ml_model(model)
    g = ctx.ir.logical
    assert [n.op_type for n in g.nodes] == ['input', 'dense', 'activation', 'dense', 'activation', 'dense', 'activation']
    assert g.nodes[0].is_placeholder and g.input_tensor_names == ['input_layer'] and g.output_tensor_names == ['act2_out']
    d0 = g.nodes[1]
    assert d0.metadata['n_in'] == 16 and d0.metadata['n_out'] == 64 and d0.metadata['use_bias'] is True
    assert [d0.roles[t.name] for t in d0.inputs] == ['lhs', 'rhs', 'bias']
    assert g.tensors['dense0_out'].shape == (8, 64) and g.tensors['input_layer'].shape == (8, 16)
    w = g.tensors['dense0_weight']
    assert (w.precision.width, w.precision.frac, w.precision.rounding) == (8, 5, RoundingMode.RND_CONV)
    assert np.array_equal(w.data, weights[0][0])
    # through the passes: activations fold away, relu fuses, every dense resolves with the post-activation type
    run_aie_passes(ctx, [p() for p in (FoldApplyAlpha,) + FRONT])
    assert [n.op_type for n in g.nodes if not n.is_placeholder] == ['dense', 'dense', 'dense']
    cfgs = [ctx.ir.execution.get(f'dense{i}_aie').config for i in range(3)]
    assert [c.flags.use_relu for c in cfgs] == [True, True, False]
    assert cfgs[0].precision['output'].format == 'uint8' and cfgs[2].precision['output'].format == 'int8'
    assert cfgs[0].shift == 5 + 5 - 8 and cfgs[1].shift == 8 + 5 - 8 and cfgs[2].shift == 8 + 5 - 5
    assert cfgs[0].rounding_mode == 'conv_even'


def test_hls4ml_apply_alpha_folds_into_the_dense():
    from aie4ml_amd.frontends.hls4ml_lower import lower_hls4ml_model
    from aie4ml_amd.passes import FoldApplyAlpha
    from tests.hls4ml_standin import qkeras_mlp

    model, weights = qkeras_mlp([16, 32, 8], batch=4, alpha=0.25)
    ctx = lower_hls4ml_model(model)
    assert 'applyalpha' in [n.op_type for n in ctx.ir.logical.nodes]
    run_aie_passes(ctx, [p() for p in (FoldApplyAlpha,) + FRONT])
    assert [n.op_type for n in ctx.ir.logical.nodes if not n.is_placeholder] == ['dense', 'dense']
    w = ctx.ir.logical.tensors['dense0_weight']
    assert w.precision.frac == 5 + 2                                     # scale 2^-2 moves the binary point
    assert np.allclose(ctx.ir.logical.tensors['dense0_bias'].data, weights[0][1] * 0.25)
    assert ctx.ir.execution.get('dense0_aie').config.shift == 5 + 7 - 8


def test_hls4ml_lowering_errors():
    from aie4ml_amd.frontends.hls4ml_lower import lower_hls4ml_model
    from tests.hls4ml_standin import Layer, qkeras_mlp

    model, _ = qkeras_mlp([16, 8], batch=4)
    with pytest.raises(KeyError, match='BatchSize'):
        lower_hls4ml_model(type(model)(model.get_layers(), model.output_vars, {}))
    model._layers[1].weights.pop('weight')
    with pytest.raises(RuntimeError, match='no weight variable'):
        lower_hls4ml_model(model)
    conv = Layer('pw', 'Conv1D', ['input'], {'filt_width': 3, 'stride_width': 1, 'pad_left': 0, 'pad_right': 0, 'in_width': 8,
                                            'out_width': 8})
    model2, _ = qkeras_mlp([16, 8], batch=4)
    model2._layers[1] = conv
    model2.output_vars['pw'] = model2.output_vars['dense0']
    with pytest.raises(ValueError, match='not true pointwise'):
        lower_hls4ml_model(model2)
