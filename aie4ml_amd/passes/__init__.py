"""Graph passes of the GPU backend.

The fold / fuse passes decide what each kernel fuses and restate the reference's passes of the same
names (src/aie4ml/passes/fold_bias.py, fold_scale.py, fuse_activation.py, fold_views.py); Resolve and
PackKernelArtifacts restate passes/resolve.py:48-95 and passes/pack.py:20-37 without the AIE contract /
staging propagation. Everything the reference runs after packing (transport, placement, memory plan)
is AIE-physical and has no counterpart here. PlanGpuFusion is the GPU-only addition; ForceFloatMode restates
passes/force_float_mode.py.
"""

from __future__ import annotations

from typing import Iterable

import numpy as np

from ..aie_types import FloatFormat, FloatIntent, QuantIntent, is_float_intent
from ..ir import TraitInstance, get_backend_context, input_tensor_for_role
from ..op_impls import get_family_resolver_registry
from ..op_impls.base import OpImplVariant


class AIEPass:
    """Base class: transform(model_or_ctx) -> True when the IR changed."""

    name: str = ''

    def transform(self, model_or_ctx) -> bool:
        raise NotImplementedError


def run_aie_passes(ctx, passes: Iterable[AIEPass]) -> None:
    ctx.ir.logical.verify()
    for p in passes:
        p.transform(ctx)


class ForceFloatMode(AIEPass):
    """Replace every QuantIntent of the logical IR with a FloatIntent when the run configuration names a
    ComputeDtype ('bfloat16', 'float32' or 'float'): the reference's way of exercising its float path on a
    quantised model (src/aie4ml/passes/force_float_mode.py:15-46)."""

    name = 'force_float_mode'
    FORMATS = {'bfloat16': (FloatFormat.BF16, 16), 'float32': (FloatFormat.FP32, 32), 'float': (FloatFormat.FP32, 32)}

    def transform(self, model_or_ctx) -> bool:
        ctx = get_backend_context(model_or_ctx)
        fmt_str = str(ctx.config.get('ComputeDtype') or '').lower()
        if not fmt_str:
            return False
        if fmt_str not in self.FORMATS:
            raise ValueError(f'ComputeDtype={fmt_str!r} is not recognised. Use one of: {list(self.FORMATS)}')
        fmt, width = self.FORMATS[fmt_str]
        intent = FloatIntent(width=width, format=fmt)
        changed = False
        for tv in ctx.ir.logical.tensors.values():
            if tv.precision is not None and not is_float_intent(tv.precision):
                tv.precision = intent
                changed = True
        return changed


class FoldApplyAlpha(AIEPass):
    """Fold a per-channel power-of-two output scale (hls4ml's ApplyAlpha after a Dense) into the Dense: the weight
    intent gains round(-log2(max scale)) fractional bits, the bias is multiplied by the scale, the node goes
    (src/aie4ml/passes/fold_apply_alpha.py:13-60). Float graphs are left alone, as there."""

    name = 'fold_apply_alpha'

    def transform(self, model_or_ctx) -> bool:
        graph = get_backend_context(model_or_ctx).ir.logical
        changed = False
        for node in list(graph.nodes):
            if node.op_type != 'applyalpha':
                continue
            scale = np.asarray(node.metadata['scale'], dtype=np.float64)
            p_min = int(np.round(-np.log2(scale.max())))
            dense = node.inputs[0].producer
            weight = dense.inputs[1]
            old = weight.precision
            if is_float_intent(old):
                continue
            weight.precision = QuantIntent(width=old.width, frac=old.frac + p_min, signed=old.signed, rounding=old.rounding,
                                           saturation=old.saturation)
            if dense.metadata.get('use_bias') and len(dense.inputs) > 2:
                dense.inputs[2].data = np.asarray(dense.inputs[2].data, dtype=np.float64) * scale
            graph.remove_node(node, mode='contract')
            changed = True
        return changed


class FoldBias(AIEPass):
    """add(dense_output, constant) -> the dense's bias input."""

    name = 'fold_bias'

    def transform(self, model_or_ctx) -> bool:
        graph = get_backend_context(model_or_ctx).ir.logical
        changed = False
        for add in list(graph.nodes):
            if add.op_type != 'add' or len(add.inputs) != 2 or len(add.outputs) != 1:
                continue
            a, b = add.inputs
            if self._biasless_dense(a) and b.is_parameter:
                dense_out, bias = a, b
            elif self._biasless_dense(b) and a.is_parameter:
                dense_out, bias = b, a
            else:
                continue
            dense = dense_out.producer
            n_out = int(dense.metadata['n_out'])
            size = int(np.asarray(bias.data).size)
            if size != n_out:
                raise ValueError(f'{add.name}: dense bias Add requires exactly {n_out} elements, got {size}.')
            if len(dense_out.consumers) != 1:
                raise ValueError(f'{add.name}: cannot fold bias because dense output {dense_out.name!r} '
                                 f'has {len(dense_out.consumers)} consumers.')
            y = add.outputs[0]
            dense.inputs.append(bias)
            bias.consumers = [c for c in bias.consumers if c is not add] + [dense]
            dense.metadata['use_bias'] = True
            dense.metadata['input_roles'] = ['lhs', 'rhs', 'bias']
            dense.roles[bias.name] = 'bias'
            dense.outputs = [y]
            y.producer = dense
            graph.tensors.pop(dense_out.name, None)
            graph.nodes.remove(add)
            add.inputs, add.outputs = [], []
            changed = True
        return changed

    @staticmethod
    def _biasless_dense(t) -> bool:
        p = t.producer
        return p is not None and p.op_type == 'dense' and not p.metadata.get('use_bias')


# which op absorbs a constant scale, and on which side
_SCALE_ABSORBERS = {'dense': 'output_scale', 'matmul': 'output_scale', 'softmax': 'input_scale'}


class FoldScale(AIEPass):
    """Constant `scale` nodes fold into a following softmax (temperature) or a preceding dense / matmul
    (extra output shift). There is no standalone scale kernel."""

    name = 'fold_scale'

    def transform(self, model_or_ctx) -> bool:
        graph = get_backend_context(model_or_ctx).ir.logical
        changed = False
        for node in list(graph.nodes):
            if node.op_type != 'scale':
                continue
            if len(node.inputs) != 1 or len(node.outputs) != 1:
                raise ValueError(f'{node.name}: scale must have exactly one input and one output.')
            scale = float(node.metadata['scale'])
            if scale <= 0.0:
                raise ValueError(f'{node.name}: scale must be positive, got {scale}.')
            src = node.inputs[0]
            consumers = list(node.outputs[0].consumers)
            producer = src.producer
            consumer = consumers[0] if len(consumers) == 1 else None
            if consumer is not None and _SCALE_ABSORBERS.get(consumer.op_type) == 'input_scale':
                self._accumulate(consumer, 'input_scale', scale)
                graph.remove_node(node, mode='bypass')
            elif producer is not None and _SCALE_ABSORBERS.get(producer.op_type) == 'output_scale':
                if len(src.consumers) != 1:
                    raise NotImplementedError(f'{node.name}: cannot fold output scale because {src.name!r} '
                                              f'has {len(src.consumers)} consumers.')
                self._accumulate(producer, 'output_scale', scale)
                graph.remove_node(node, mode='contract')
            else:
                raise NotImplementedError(
                    f'{node.name}: no adjacent op absorbs this scale (producer='
                    f'{producer.op_type if producer else None}, consumers={[c.op_type for c in consumers]}); '
                    'there is no standalone scale kernel.')
            changed = True
        return changed

    @staticmethod
    def _accumulate(node, trait_name: str, scale: float) -> None:
        prev = node.traits.get(trait_name)
        node.add_trait(TraitInstance(trait_name, {'scale': scale * float(prev.data['scale']) if prev else scale}))


class FuseActivationCasts(AIEPass):
    """relu after a dense becomes the dense's fused_activation trait; linear activations disappear."""

    name = 'fuse_activation_casts'

    def transform(self, model_or_ctx) -> bool:
        graph = get_backend_context(model_or_ctx).ir.logical
        changed = False
        for act in list(graph.nodes):
            if act.op_type != 'activation' or len(act.inputs) != 1 or len(act.outputs) != 1:
                continue
            kind = (act.metadata.get('activation', '') or '').lower()
            if kind == 'relu':
                producer = act.inputs[0].producer
                if producer is None or producer.op_type != 'dense' or len(producer.outputs) != 1:
                    continue  # stays an activation node: Resolve will refuse it (no standalone kernel)
                producer.add_trait(TraitInstance('fused_activation', {'activation': 'relu'}))
                graph.remove_node(act, mode='contract')
                changed = True
            elif kind in ('linear', ''):
                graph.remove_node(act, mode='contract')
                changed = True
        return changed


class FoldViewOps(AIEPass):
    """Transpose -> io_view permutation on its consumers; Split / Slice / Concat -> placeholder nodes
    carrying slice_view / concat_view traits."""

    name = 'fold_view_ops'

    def transform(self, model_or_ctx) -> bool:
        graph = get_backend_context(model_or_ctx).ir.logical
        changed = False
        for node in list(graph.nodes):
            if node.op_type == 'transpose':
                changed = self._transpose(graph, node) or changed
            elif node.op_type == 'concat':
                changed = self._concat(node) or changed
            elif node.op_type in ('slice', 'split'):
                changed = self._slice(node) or changed
        return changed

    @staticmethod
    def _view(node):
        trait = node.traits.get('io_view')
        if trait is None:
            trait = TraitInstance('io_view', {'inputs': {}, 'outputs': {}})
            node.add_trait(trait)
        trait.data.setdefault('inputs', {})
        trait.data.setdefault('outputs', {})
        return trait.data

    def _transpose(self, graph, node) -> bool:
        src, dst = node.inputs[0], node.outputs[0]
        perm = node.metadata.get('perm')
        if perm is None:
            raise ValueError(f'{node.name}: missing transpose permutation metadata.')
        perm = [int(p) for p in perm]
        rank = len(src.shape)
        if len(dst.shape) != rank:
            raise ValueError(f'{node.name}: transpose rank mismatch between input and output.')
        if sorted(perm) != list(range(rank)):
            raise ValueError(f'{node.name}: invalid permutation {perm} for rank {rank}.')
        for consumer in dst.consumers:
            view = self._view(consumer)
            view['inputs'][src.name] = {'perm': list(perm)}
            view['inputs'].pop(dst.name, None)
        graph.remove_node(node, mode='bypass')
        return True

    @staticmethod
    def _concat(node) -> bool:
        if len(node.outputs) != 1:
            raise ValueError(f'{node.name}: concat must have exactly one output.')
        if not node.inputs:
            raise ValueError(f'{node.name}: concat must have at least one input.')
        out = node.outputs[0]
        rank = len(out.shape)
        axis = int(node.metadata.get('axis', -1))
        axis = axis + rank if axis < 0 else axis
        if not 0 <= axis < rank:
            raise ValueError(f'{node.name}: concat axis {node.metadata.get("axis")} is out of range for rank {rank}.')
        offset, slices = 0, []
        for t in node.inputs:
            if len(t.shape) != rank:
                raise ValueError(f'{node.name}: concat input {t.name!r} rank does not match output rank.')
            extent = int(t.shape[axis])
            slices.append({'input': t.name, 'start': offset, 'extent': extent})
            offset += extent
        if int(out.shape[axis]) != offset:
            raise ValueError(f'{node.name}: concat output axis extent {out.shape[axis]} does not match input sum {offset}.')
        node.add_trait(TraitInstance('concat_view', {'kind': 'concat', 'axis': axis, 'output': out.name, 'slices': slices}))
        node.is_placeholder = True
        return True

    @staticmethod
    def _slice(node) -> bool:
        if len(node.inputs) != 1:
            raise ValueError(f'{node.name}: {node.op_type} view must have exactly one input.')
        if not node.outputs:
            raise ValueError(f'{node.name}: {node.op_type} view must have at least one output.')
        src = node.inputs[0]
        rank = len(src.shape)
        axis = int(node.metadata['axis'])
        axis = axis + rank if axis < 0 else axis
        if not 0 <= axis < rank:
            raise ValueError(f'{node.name}: {node.op_type} axis {axis} is out of range for rank {rank}.')
        items = list(node.metadata.get('slices', ()))
        if len(items) != len(node.outputs):
            raise ValueError(f'{node.name}: {node.op_type} slice metadata does not match output count.')
        norm = []
        for out, item in zip(node.outputs, items):
            start, extent = int(item['start']), int(item['extent'])
            if start < 0 or extent <= 0 or start + extent > int(src.shape[axis]):
                raise ValueError(f'{node.name}: invalid {node.op_type} range [{start}, {start + extent}).')
            if int(out.shape[axis]) != extent:
                raise ValueError(f'{node.name}: {node.op_type} output {out.name!r} extent mismatch.')
            norm.append({'output': out.name, 'start': start, 'extent': extent})
        node.add_trait(TraitInstance('slice_view', {'kind': node.op_type, 'axis': axis, 'source': src.name, 'slices': norm}))
        node.is_placeholder = True
        return True


class Resolve(AIEPass):
    """Bind every non-placeholder node to an operator variant and its resolved constants."""

    name = 'resolve'

    def transform(self, model_or_ctx) -> bool:
        ctx = get_backend_context(model_or_ctx)
        ctx.ir.logical.verify()
        registry = get_family_resolver_registry()
        changed, visited = False, set()
        for node in ctx.ir.logical:
            if node.is_placeholder:
                continue
            resolver = registry.get(node.op_type)  # NotImplementedError for e.g. a stray activation
            config, variant = resolver.resolve(node, ctx.device, dict(node.directives or {}))
            variant.validate_config(node, config, ctx.device)
            inst = ctx.ir.execution.get(node.name)
            if inst is None or inst.variant is not variant or inst.config != config:
                ctx.ir.execution.register(node, variant, config)
                changed = True
            visited.add(node.name)
        return ctx.ir.execution.prune(visited) or changed


class PackKernelArtifacts(AIEPass):
    """Quantise and upload kernel-resident parameters (weights, bias, gamma, beta)."""

    name = 'pack_kernel_artifacts'

    def transform(self, model_or_ctx) -> bool:
        ctx = get_backend_context(model_or_ctx)
        changed = False
        for inst in ctx.ir.execution:
            if type(inst.variant).pack is OpImplVariant.pack or inst.artifacts:
                continue
            packed = inst.variant.pack(inst)
            if packed:
                inst.artifacts.update(packed)
                changed = True
        return changed


class PlanGpuFusion(AIEPass):
    """GPU-only: mark node groups the executor runs as one launch.

    * add -> layer_norm: the residual add is computed inside the LayerNorm kernel (the sum is written out
      only if something else reads it).
    * a chain of dense nodes whose whole weight set fits LDS: one fused-MLP launch.
    * dense -> add -> layer_norm where nothing else reads the dense output or the sum: one launch whose workgroups
      compute whole rows (the dense must fit the limits of that kernel).
    * matmul(Q, K^T) -> softmax -> matmul(P, V) whose logits and probabilities have no other reader: one
      fused-attention launch; triples that read per-head slices of the same three tensors and feed one
      concat are merged into a single launch over all heads that writes the concat's output directly.
    All are exact: the fused kernels perform the same integer operations in the same order.
    """

    name = 'plan_gpu_fusion'
    MLP_MAX_WIDTH = 256
    MLP_MAX_WEIGHT_BYTES = 96 * 1024

    def transform(self, model_or_ctx) -> bool:
        ctx = get_backend_context(model_or_ctx)
        graph, execution = ctx.ir.logical, ctx.ir.execution
        plan = {'add_layernorm': {}, 'mlp_chains': [], 'attention': []}
        outputs = set(graph.output_tensor_names)
        plan['attention'] = self._plan_attention(graph, execution, outputs)
        for node in graph.nodes:
            if node.op_type != 'add' or execution.get(node.name) is None:
                continue
            cfg = execution.get(node.name).config
            s = node.outputs[0]
            lns = [c for c in s.consumers if c.op_type == 'layer_norm']
            if len(lns) == 1 and cfg.shift == 0 and cfg.precision['output'].format == 'int8' \
                    and not lns[0].traits.get('io_view'):
                keep_sum = len(s.consumers) > 1 or s.name in outputs
                plan['add_layernorm'][node.name] = {'layer_norm': lns[0].name, 'keep_sum': keep_sum}
        # dense chains: every link a dense with a single consumer that is the next dense
        used = set()
        for node in graph.nodes:
            if node.op_type != 'dense' or node.name in used or execution.get(node.name) is None:
                continue
            prev = node.inputs[0].producer
            if prev is not None and prev.op_type == 'dense' and len(node.inputs[0].consumers) == 1 \
                    and node.inputs[0].name not in outputs:
                continue  # not a chain head
            chain, cur = [node], node
            while True:
                out = cur.outputs[0]
                nxt = out.consumers[0] if len(out.consumers) == 1 and out.name not in outputs else None
                if nxt is None or nxt.op_type != 'dense' or nxt.inputs[0] is not out or execution.get(nxt.name) is None:
                    break
                chain.append(nxt)
                cur = nxt
            if len(chain) >= 2 and self._fits(chain, execution):
                plan['mlp_chains'].append([n.name for n in chain])
                used.update(n.name for n in chain)
        # dense -> add -> layer_norm: the dense computes whole rows and normalises them itself
        plan['dense_add_layernorm'] = {}
        for add_name, info in plan['add_layernorm'].items():
            if info['keep_sum']:
                continue
            add_node = next(n for n in graph.nodes if n.name == add_name)
            for t in add_node.inputs:
                d = t.producer
                if d is None or d.op_type != 'dense' or d.name in used or execution.get(d.name) is None:
                    continue
                if len(t.consumers) != 1 or t.name in outputs or d.traits.get('io_view') or add_node.traits.get('io_view'):
                    continue
                if self._rows_complete(execution.get(d.name).config):
                    other = [u for u in add_node.inputs if u is not t]
                    if len(other) == 1 and not other[0].is_parameter:
                        plan['dense_add_layernorm'][add_name] = {'dense': d.name, 'layer_norm': info['layer_norm'],
                                                                 'residual': other[0].name}
                        break
        # (chain of) narrow dense -> add -> layer_norm: the chain kernel normalises the rows itself
        plan['mlp_add_layernorm'] = {}
        by_name = {n.name: n for n in graph.nodes}
        chain_of_tail = {c[-1]: c for c in plan['mlp_chains']}
        for add_name, info in plan['add_layernorm'].items():
            add_node = by_name[add_name]
            if info['keep_sum'] or add_node.traits.get('io_view') or add_name in plan['dense_add_layernorm']:
                continue
            for t in add_node.inputs:
                d = t.producer
                if d is None or d.op_type != 'dense' or execution.get(d.name) is None or len(t.consumers) != 1 or t.name in outputs:
                    continue
                chain = chain_of_tail.get(d.name)
                if chain is None:
                    if d.name in used or not self._fits([d], execution):
                        continue
                    chain = [d.name]
                cfg = execution.get(chain[-1]).config
                other = [u for u in add_node.inputs if u is not t]
                if cfg.precision['output'].format == 'int8' and cfg.n_out % 16 == 0 and len(other) == 1 and not other[0].is_parameter:
                    plan['mlp_add_layernorm'][add_name] = {'chain': list(chain), 'layer_norm': info['layer_norm'],
                                                           'residual': other[0].name}
                    break
        changed = ctx.config.get('gpu_fusion_plan') != plan
        ctx.config['gpu_fusion_plan'] = plan
        return changed

    # Dense layers the row-complete kernel takes (the limits of a4g_dense_add_layernorm_i8) and can win on; whether it
    # does depends on the number of rows, which the executor knows at launch (ops.dense_add_layernorm_pays).
    ROWLN_MAX_K = 1536

    def _rows_complete(self, cfg) -> bool:
        return (cfg.accumulator_tag == 'acc32' and cfg.precision['lhs'].format in ('int8', 'uint8')
                and cfg.precision['output'].format == 'int8' and cfg.shift_per_channel is None
                and not cfg.flags.transpose_lhs and cfg.n_out % 32 == 0 and cfg.n_out <= 768 and cfg.n_in % 128 == 0
                and cfg.n_in <= self.ROWLN_MAX_K and cfg.n_out >= 384)

    # ---- attention -------------------------------------------------------------------------------------
    # head dimension -> keys the fused kernel takes (16, 48, 80, 96, 112 run padded to 32, 64, 128)
    ATTN_MAX_KEYS = {16: 512, 32: 512, 48: 512, 64: 512, 80: 256, 96: 256, 112: 256, 128: 256}
    ATTN_MAX_SHIFT = 24

    def _plan_attention(self, graph, execution, outputs):
        triples = []
        for qk in graph.nodes:
            if qk.op_type != 'matmul' or execution.get(qk.name) is None:
                continue
            c1 = execution.get(qk.name).config
            logits = qk.outputs[0]
            if not c1.flags.transpose_rhs or c1.flags.transpose_lhs or logits.name in outputs or len(logits.consumers) != 1:
                continue
            sm = logits.consumers[0]
            if sm.op_type != 'softmax' or execution.get(sm.name) is None or sm.traits.get('io_view'):
                continue
            probs = sm.outputs[0]
            if probs.name in outputs or len(probs.consumers) != 1:
                continue
            pv = probs.consumers[0]
            if pv.op_type != 'matmul' or execution.get(pv.name) is None or input_tensor_for_role(pv, 'lhs') is not probs:
                continue
            c2, c3 = execution.get(sm.name).config, execution.get(pv.name).config
            q, k = input_tensor_for_role(qk, 'lhs'), input_tensor_for_role(qk, 'rhs')
            v = input_tensor_for_role(pv, 'rhs')
            if k.is_parameter or v.is_parameter or c3.flags.transpose_rhs or c3.flags.transpose_lhs:
                continue
            if c1.precision['output'].format != 'int8' or c2.precision['output'].format != 'uint8' \
                    or c3.precision['output'].format != 'int8' or c1.precision['lhs'].format != 'int8':
                continue
            if len(q.shape) != len(k.shape) or len(k.shape) != len(v.shape) or tuple(k.shape) != tuple(v.shape) \
                    or tuple(q.shape[:-2]) != tuple(k.shape[:-2]) or len(q.shape) not in (2, 3, 4):
                continue
            if not 1 <= int(k.shape[-2]) <= self.ATTN_MAX_KEYS.get(int(q.shape[-1]), 0):
                continue
            if c1.shift > self.ATTN_MAX_SHIFT or c3.shift > self.ATTN_MAX_SHIFT:
                continue  # the fused kernel takes shifts up to 24, the MatMul kernels up to 31
            triples.append({'qk': qk.name, 'softmax': sm.name, 'pv': pv.name, 'q': q.name, 'k': k.name, 'v': v.name,
                            'out': pv.outputs[0].name})
        groups, used = [], set()
        by_name = {n.name: n for n in graph.nodes}
        # merge per-head triples: operands are last-axis slices of three common tensors, results feed one concat
        def slice_of(tname):
            prod = None
            for n in graph.nodes:
                if n.is_placeholder and n.traits.get('slice_view') is not None:
                    for it in n.traits['slice_view'].data['slices']:
                        if it['output'] == tname:
                            prod = (n, it)
            if prod is None:
                return None
            n, it = prod
            sv = n.traits['slice_view'].data
            src = n.inputs[0]
            ax = int(sv['axis'])
            if ax not in (-1, len(src.shape) - 1):
                return None
            return sv['source'], int(it['start']), int(it['extent'])

        cand = {}
        for tr in triples:
            out_t = by_name[tr['pv']].outputs[0]
            if out_t.name in outputs or len(out_t.consumers) != 1:
                continue
            cat = out_t.consumers[0]
            cv = cat.traits.get('concat_view')
            if not cat.is_placeholder or cv is None:
                continue
            cat_out = cat.outputs[0]
            if int(cv.data['axis']) not in (-1, len(cat_out.shape) - 1) or len(cat_out.shape) != 3:
                continue
            sq, sk_, sv_ = slice_of(tr['q']), slice_of(tr['k']), slice_of(tr['v'])
            if not (sq and sk_ and sv_):
                continue
            o_start = next(int(it['start']) for it in cv.data['slices'] if it['input'] == out_t.name)
            key = (sq[0], sk_[0], sv_[0], cat.name)
            cand.setdefault(key, []).append((o_start, sq[1], sk_[1], sv_[1], tr))
        for (qs, ks, vs, cat_name), items in cand.items():
            items.sort(key=lambda x: x[0])
            d = int(graph.tensors[items[0][4]['q']].shape[-1])  # head dimension
            cat = by_name[cat_name]
            regular = len(items) == len(cat.traits['concat_view'].data['slices']) and len(items) >= 2
            for h, (o, a, b, c, tr) in enumerate(items):
                regular = regular and o == h * d and a == items[0][1] + h * d and b == items[0][2] + h * d \
                    and c == items[0][3] + h * d
            ref = [self._attn_signature(execution, items[0][4])]
            regular = regular and all(self._attn_signature(execution, it[4]) == ref[0] for it in items)
            # the fused kernel reads 16-byte chunks: head slices must start on 16-byte boundaries of 16-byte aligned rows
            srcs = [graph.tensors[t] for t in (qs, ks, vs)]
            regular = regular and all(b % 16 == 0 for b in items[0][1:4]) and all(int(t.shape[-1]) % 16 == 0 for t in srcs)
            if not regular:
                continue
            groups.append({'heads': [it[4] for it in items], 'q_src': qs, 'k_src': ks, 'v_src': vs,
                           'q_base': items[0][1], 'k_base': items[0][2], 'v_base': items[0][3], 'concat': cat_name,
                           'out': cat.outputs[0].name})
            used.update(it[4]['qk'] for it in items)
        for tr in triples:
            if tr['qk'] not in used:
                groups.append({'heads': [tr], 'concat': None, 'out': tr['out']})
        return groups

    @staticmethod
    def _attn_signature(execution, tr):
        c1, c2, c3 = (execution.get(tr[k]).config for k in ('qk', 'softmax', 'pv'))
        return (c1.shift, c1.rounding_mode, c2.approximation, c2.exp_kq, tuple(sorted((c2.hccs or {}).items())), c2.inv_shift,
                c2.use_clb, c3.shift, c3.rounding_mode)

    def _fits(self, chain, execution) -> bool:
        if len(chain) > 8:
            return False
        if any(execution.get(n.name).config.accumulator_tag != 'acc32' for n in chain):
            return False  # the fused MLP kernel is the int8 one
        if execution.get(chain[0].name).config.precision['lhs'].format not in ('int8', 'uint8'):
            return False  # acc32 also covers int16 activations x int8 weights: those layers run one by one
        total, mode = 0, None
        for i, n in enumerate(chain):
            cfg = execution.get(n.name).config
            if cfg.n_in > self.MLP_MAX_WIDTH or cfg.n_out > self.MLP_MAX_WIDTH or cfg.flags.transpose_lhs:
                return False
            if cfg.shift_per_channel is not None or n.traits.get('io_view'):
                return False
            last = i + 1 == len(chain)
            fmt = cfg.precision['output'].format
            if fmt not in ('int8', 'uint8') and not (last and fmt == 'int16'):
                return False
            mode = mode or cfg.rounding_mode
            if cfg.rounding_mode != mode:
                return False
            total += cfg.n_out * ((cfg.n_in + 15) // 16 * 16)
        return total <= self.MLP_MAX_WEIGHT_BYTES


GPU_PIPELINE = (ForceFloatMode, FoldApplyAlpha, FoldBias, FoldScale, FuseActivationCasts, FoldViewOps, Resolve, PackKernelArtifacts, PlanGpuFusion)
