"""CPU tests of the ONNX path: the protobuf reader/writer, the Q/DQ lowering, its error behaviour."""

import struct

import numpy as np
import pytest

from aie4ml_amd import qint, workloads
from aie4ml_amd.frontends import onnx_proto as op
from aie4ml_amd.frontends.onnx_import import lower_onnx_model
from aie4ml_amd.frontends.onnx_writer import QdqWriter
from aie4ml_amd.ir import get_backend_context
from aie4ml_amd.passes import (FoldBias, FoldScale, FoldViewOps, FuseActivationCasts, PlanGpuFusion, Resolve,
                               run_aie_passes)

FRONT = (FoldBias, FoldScale, FuseActivationCasts, FoldViewOps, Resolve, PlanGpuFusion)


def test_proto_round_trip_and_typed_fields():
    data, _, _ = workloads.c5_encoder_block_onnx(2, 32, 128, 2, 256, softmax='exp')
    m = op.parse_model(data)
    assert op.serialize_model(m) == data                      # every field we write is read back
    assert m.opset == {'': 17} and m.graph.name == 'encoder_block' and m.producer_name == 'aie4ml_amd'
    w = next(t for t in m.graph.initializers if t.name == 'qkv_w')
    assert w.array.dtype == np.int8 and w.array.shape == (128, 384)
    node = next(n for n in m.graph.nodes if n.op_type == 'Transpose')
    assert node.attrs == {'perm': [0, 2, 1]}
    ln = next(n for n in m.graph.nodes if n.op_type == 'LayerNormalization')
    assert ln.attrs['axis'] == -1 and ln.attrs['epsilon'] == 2.0 ** -8

    # what other writers emit: unpacked repeated dims, int32_data / float_data / int64_data instead of raw_data
    def ld(num, payload):
        return op._key(num, 2) + op._enc_varint(len(payload)) + payload
    t_i8 = op._vi(1, 2) + op._vi(1, 2) + op._vi(2, op.INT8) + ld(8, b'a') + b''.join(op._vi(5, v & 0xFFFFFFFFFFFFFFFF) for v in (1, -2, 3, -128))
    t_f = ld(1, op._enc_varint(3)) + op._vi(2, op.FLOAT) + ld(8, b'f') + ld(4, struct.pack('<3f', 0.5, -1.0, 2.0))
    t_i64 = op._vi(2, op.INT64) + ld(8, b's') + ld(7, op._enc_varint(7))
    graph = ld(5, t_i8) + ld(5, t_f) + ld(5, t_i64) + ld(2, b'g')
    m2 = op.parse_model(op._vi(1, 7) + ld(7, graph) + ld(99, b'ignored'))
    got = {t.name: t.array for t in m2.graph.initializers}
    assert got['a'].tolist() == [[1, -2], [3, -128]] and got['a'].dtype == np.int8
    assert got['f'].tolist() == [0.5, -1.0, 2.0] and got['s'].shape == () and int(got['s']) == 7
    with pytest.raises(ValueError, match='no graph field'):
        op.parse_model(op._vi(1, 7))
    with pytest.raises(ValueError, match='truncated'):
        op.parse_model(data[:-3])


def lowered(source, cfg=None):
    ctx = lower_onnx_model(source, cfg)
    run_aie_passes(ctx, [p() for p in FRONT])
    return ctx


@pytest.mark.parametrize('softmax', ['exp', 'hccs'])
def test_imported_encoder_resolves_like_the_builder_graph(softmax):
    shape = (2, 32, 128, 2, 256)
    data, cfg, x = workloads.c5_encoder_block_onnx(*shape, softmax=softmax)
    ctx = lowered(data, cfg)
    model, x2 = workloads.c5_encoder_block(*shape, softmax=softmax)
    ref = get_backend_context(model)
    run_aie_passes(ref, [p() for p in FRONT])
    assert np.array_equal(x, x2)
    a = [n for n in ctx.ir.logical.nodes if not n.is_placeholder]
    b = [n for n in ref.ir.logical.nodes if not n.is_placeholder]
    assert [n.op_type for n in a] == [n.op_type for n in b]
    for na, nb in zip(a, b):
        ca, cb = ctx.ir.execution.get(na.name).config, ref.ir.execution.get(nb.name).config
        for field in ('shift', 'rounding_mode', 'exp_kq', 'approximation', 'hccs', 'inv_shift', 'out_shift', 'eps_q0', 'cols', 'rows'):
            assert getattr(ca, field, None) == getattr(cb, field, None), (na.name, field)
        assert {k: (v.format, v.frac) for k, v in ca.precision.items()} == {k: (v.format, v.frac) for k, v in cb.precision.items()}
        if na.op_type == 'dense':
            ia, ib = ctx.ir.execution.get(na.name), ref.ir.execution.get(nb.name)
            for u, v in zip(ia.variant.quantize_weight_bias(ia), ib.variant.quantize_weight_bias(ib)):
                assert np.array_equal(u, v)
    (grp,) = ctx.config['gpu_fusion_plan']['attention']
    assert len(grp['heads']) == 2 and grp['concat'] == 'heads_concat_aie'
    assert len(ctx.config['gpu_fusion_plan']['add_layernorm']) == 2


def small_graph(scale=0.0625, zero=0, w_scale=2.0 ** -7, op_type='MatMul', per_axis=False):
    w = QdqWriter('small')
    x = w.input('x', (4, 16), qint(8, 4))
    wt = w.const('W', np.ones((16, 8), dtype=np.int8))
    ws = w.const('W_scale', np.array([w_scale] * (8 if per_axis else 1), dtype=np.float32).reshape(-1 if per_axis else ()))
    wz = w.const('W_zp', np.array(zero, dtype=np.int8))
    (wd,) = w.node('DequantizeLinear', [wt, ws, wz], name='W_dq')
    (y,) = w.node(op_type, [x, wd], name='fc')
    ys = w.const('y_scale', np.array(scale, dtype=np.float32))
    yz = w.const('y_zp', np.zeros((), dtype=np.int8))
    (q,) = w.node('QuantizeLinear', [y, ys, yz], name='yq')
    (d,) = w.node('DequantizeLinear', [q, ys, yz], name='ydq')
    w.output(d, (4, 8))
    return w


def test_import_errors():
    ctx = lowered(small_graph().to_bytes())
    (fc,) = ctx.ir.logical.nodes
    assert fc.op_type == 'dense' and ctx.ir.execution.get(fc.name).config.shift == 4 + 7 - 4
    assert ctx.ir.logical.output_tensor_names == ['ydq_out']
    with pytest.raises(ValueError, match='is not a power of two'):
        lower_onnx_model(small_graph(scale=0.3).to_bytes())
    with pytest.raises(ValueError, match='zero_point must be 0'):
        lower_onnx_model(small_graph(zero=3).to_bytes())
    with pytest.raises(ValueError, match='per-axis quantization is not supported'):
        lower_onnx_model(small_graph(per_axis=True).to_bytes())
    with pytest.raises(ValueError, match='fc: unsupported ONNX op Conv'):
        lower_onnx_model(small_graph(op_type='Conv').to_bytes())
    with pytest.raises(ValueError, match='Unused LayerDirectives entries: nosuch'):
        lower_onnx_model(small_graph().to_bytes(), {'LayerDirectives': {'nosuch': {'approximation': 'hccs'}}})
    # an operator whose result never meets a QuantizeLinear has no storage type
    w = QdqWriter('noq')
    x = w.input('x', (4, 16), qint(8, 4))
    (y,) = w.node('Relu', [x], name='r')
    (y2,) = w.node('Softmax', [y], name='sm')
    w.output(y2, (4, 16))
    with pytest.raises(ValueError, match='missing quantization intent after ONNX QDQ lowering'):
        lower_onnx_model(w.to_bytes())
    # dynamic and missing input shapes
    m = op.parse_model(small_graph().to_bytes())
    m.graph.inputs[0].shape = (None, 16)
    with pytest.raises(ValueError, match='dynamic shapes are not supported'):
        lower_onnx_model(m)
    m.graph.inputs[0].shape = None
    with pytest.raises(ValueError, match='tensor shape is missing'):
        lower_onnx_model(m)


def test_gemm_bias_relu_and_slice():
    w = QdqWriter('gemm')
    x = w.input('x', (8, 32), qint(8, 4))
    (g,) = w.node('Gemm', [x, w.weight('W', np.full((16, 32), 0.25), qint(8, 7)), w.weight('b', np.arange(16) / 2048.0, qint(32, 11))],
                  name='fc', transB=1)
    (r,) = w.node('Relu', [g], name='relu')
    y = w.qdq(r, qint(8, 5, signed=False))
    (s,) = w.node('Slice', [y, w.const('st', np.array([4], dtype=np.int64)), w.const('en', np.array([12], dtype=np.int64)),
                            w.const('ax', np.array([1], dtype=np.int64))], name='cut')
    w.output(s, (8, 8))
    ctx = lowered(w.to_bytes())
    fc = next(n for n in ctx.ir.logical.nodes if n.op_type == 'dense')
    cfg = ctx.ir.execution.get(fc.name).config
    assert cfg.flags.use_bias and cfg.flags.use_relu and cfg.shift == 4 + 7 - 5
    assert cfg.precision['output'].format == 'uint8'
    inst = ctx.ir.execution.get(fc.name)
    W, b = inst.variant.quantize_weight_bias(inst)
    assert W.shape == (32, 16) and np.all(W == 32) and b.tolist() == list(range(16))
    cut = next(n for n in ctx.ir.logical.nodes if n.is_placeholder)
    assert cut.traits['slice_view'].data['slices'] == [{'output': 'cut_out', 'start': 4, 'extent': 8}]


def test_float_onnx_graph_imports_with_float_intents():
    """A graph without Q/DQ nodes is a float graph: bare FLOAT / BFLOAT16 inputs and initializers carry a
    FloatIntent (frontends/onnx/context.py:18-24, utils.py:229-241) and matmul-family outputs inherit it."""
    from aie4ml_amd.aie_types import FloatFormat, is_float_intent
    from aie4ml_amd.frontends import onnx_proto as op
    from aie4ml_amd.frontends.onnx_import import lower_onnx_model
    from aie4ml_amd.passes import FoldBias, FoldScale, FoldViewOps, FuseActivationCasts, Resolve, run_aie_passes

    r = np.random.default_rng(0)
    for elem, bf in ((op.FLOAT, False), (op.BFLOAT16, True)):
        def cast(a):
            a = np.ascontiguousarray(a, dtype=np.float32)
            return ((a.view(np.uint32) >> 16) << 16).view(np.float32) if bf else a

        g = op.Graph(name='float_mlp')
        g.inputs.append(op.ValueInfo('x', elem, (4, 32)))
        g.initializers += [op.Tensor('w0', cast(r.normal(0, 0.1, (32, 32))), bfloat16=bf),
                           op.Tensor('b0', cast(r.normal(0, 0.1, 32)), bfloat16=bf),
                           op.Tensor('w1', cast(r.normal(0, 0.1, (32, 16))), bfloat16=bf)]
        g.nodes += [op.Node('Gemm', ['x', 'w0', 'b0'], ['h'], 'fc0', {}), op.Node('Relu', ['h'], ['hr'], 'relu0', {}),
                    op.Node('MatMul', ['hr', 'w1'], ['y'], 'fc1', {})]
        g.outputs.append(op.ValueInfo('y', elem, (4, 16)))
        blob = op.serialize_model(op.Model(graph=g, opset={'': 17}, producer_name='test'))
        back = op.parse_model(blob)
        assert [t.bfloat16 for t in back.graph.initializers] == [bf] * 3
        assert np.array_equal(back.graph.initializers[0].array, g.initializers[0].array)
        ctx = lower_onnx_model(blob, {})
        fmt = FloatFormat.BF16 if bf else FloatFormat.FP32
        assert all(is_float_intent(t.precision) and t.precision.format is fmt for t in ctx.ir.logical.tensors.values())
        run_aie_passes(ctx, [p() for p in (FoldBias, FoldScale, FuseActivationCasts, FoldViewOps, Resolve)])
        assert [n.op_type for n in ctx.ir.logical.nodes] == ['dense', 'dense']
        cfg = ctx.ir.execution.get(ctx.ir.logical.nodes[0].name).config
        assert cfg.accumulator_tag == 'accfloat' and cfg.flags.use_relu and cfg.flags.use_bias


def test_float8_onnx_tensors_round_trip_and_import():
    from aie4ml_amd.aie_types import FloatFormat
    from aie4ml_amd.frontends import onnx_proto as op
    from aie4ml_amd.frontends.onnx_import import lower_onnx_model
    from aie4ml_amd.op_impls.float_ops import pack_as_float

    w = pack_as_float(np.random.default_rng(2).normal(0, 0.5, (16, 8)), 'fp8_e4m3')
    g = op.Graph(name='f8')
    g.inputs.append(op.ValueInfo('x', op.FLOAT8E4M3FN, (4, 16)))
    g.initializers.append(op.Tensor('w', w, float8=True))
    g.nodes.append(op.Node('MatMul', ['x', 'w'], ['y'], 'fc', {}))
    g.outputs.append(op.ValueInfo('y', op.FLOAT8E4M3FN, (4, 8)))
    blob = op.serialize_model(op.Model(graph=g, opset={'': 19}, producer_name='test'))
    back = op.parse_model(blob).graph.initializers[0]
    assert back.float8 and np.array_equal(back.array, w)
    ctx = lower_onnx_model(blob, {})
    assert {t.precision.format for t in ctx.ir.logical.tensors.values()} == {FloatFormat.FP8_E4M3}
    with pytest.raises(ValueError, match='not exact in float8'):
        op.serialize_model(op.Model(graph=op.Graph(name='bad', initializers=[op.Tensor('w', np.float32([0.3]), float8=True)]),
                                    opset={'': 19}, producer_name='test'))
