"""Runtime object of the GPU backend: the counterpart of the reference's AIEModel
(src/aie4ml/model.py:29-153) whose predict() runs the graph on the MI355X instead of writing text
files and shelling out to the Vitis simulator.

I/O contract of predict() (src/aie4ml/simulation.py:157-196, 248-269; model.py:137-147):
  * X is an array (single graph input) or a dict tensor-name -> array;
  * each array has the input tensor's shape, or (1, *shape), or (iterations, *shape);
  * quantize_in=True: floats are scaled by 2^frac, rounded with the tensor's rounding mode and
    overflow-handled with its saturation mode; integer arrays pass through with a dtype cast;
    quantize_in=False requires integer arrays;
  * the result is int64 raw values, or float64 value / 2^frac with dequantize_out=True; a leading
    iteration axis is folded into the batch axis; one output -> ndarray, several -> dict by name;
  * with the run-configuration key 'HipGraph' set, predict() records the whole graph into a HIP graph per input
    signature and replays it on later calls (one launch on the host instead of one per operator);
  * tensors of the float compute path (FloatIntent) take float32 arrays as they are (simulation.py:184-185)
    and come back as float64 (simulation.py:235, 253-254), whatever the two flags say.
"""

from __future__ import annotations

import logging
from typing import Any, Dict, List, Optional

import numpy as np

from .ir import CONTEXT_ATTR, BackendContext, get_backend_context, input_tensor_for_role
from .op_impls.float_ops import pack_as_float, to_device_float
from .op_impls.precision import resolve_exact_storage_dtype
from .passes import GPU_PIPELINE, run_aie_passes
from .quant_utils import dequantize_output, dtype_for_precision, quantize_input

log = logging.getLogger(__name__)


class GPUModel:
    """Owns a backend context; compile() resolves + packs, predict() executes."""

    def __init__(self, ctx: BackendContext, source_model: Optional[Any] = None):
        setattr(self, CONTEXT_ATTR, ctx)
        self.source_model = source_model
        self._compiled = False
        self._captured: Dict[Any, Any] = {}  # input signature -> CapturedExecution (config key 'HipGraph')

    @classmethod
    def from_context(cls, ctx: BackendContext, source_model: Optional[Any] = None) -> 'GPUModel':
        return cls(ctx, source_model=source_model)

    @property
    def context(self) -> BackendContext:
        return get_backend_context(self)

    def run_pipeline(self) -> 'GPUModel':
        run_aie_passes(self.context, [cls() for cls in GPU_PIPELINE])
        return self

    def write(self) -> 'GPUModel':
        """Nothing is emitted for the GPU (no firmware project); kept so call sites written for the
        reference's write() / compile() / predict() sequence work unchanged."""
        return self.run_pipeline()

    def compile(self) -> int:
        """Load the HIP library (raises if it was never built), resolve every node, upload parameters."""
        from . import _lib

        _lib.load()
        self.run_pipeline()
        self._compiled = True
        return 0

    build = compile

    # ---- I/O boundary -------------------------------------------------------------------------------
    def _io_dtype(self, tensor, namespace: str):
        if tensor.precision is None:
            raise RuntimeError(f'{tensor.name}: graph {namespace} has no precision; every activation must carry a '
                               'QuantIntent.')
        return resolve_exact_storage_dtype(tensor.precision, namespace=namespace, layer_name=tensor.name)

    def prepare_inputs(self, X, quantize: bool = True) -> Dict[str, np.ndarray]:
        graph = self.context.ir.logical
        inputs = graph.graph_inputs()
        iterations = int(self.context.config.get('Iterations', 1))
        if len(inputs) == 1 and not isinstance(X, dict):
            X = {inputs[0].name: X}
        prepared = {}
        for t in inputs:
            expected = tuple(int(d) for d in t.shape)
            if t.name not in X:
                raise KeyError(f'{t.name}: missing graph input.')
            arr = np.asarray(X[t.name])
            if tuple(arr.shape) == expected:
                arr = arr[np.newaxis, ...]
            elif not (arr.ndim == len(expected) + 1 and tuple(arr.shape[1:]) == expected):
                raise ValueError(f'{t.name}: expected shape {expected}, (1, *{expected}) or ({iterations}, *{expected}); '
                                 f'got {tuple(arr.shape)}')
            dtype = self._io_dtype(t, 'input')
            if dtype.is_float:
                prepared[t.name] = np.asarray(arr, dtype=np.float32)  # simulation.py:184-185
            elif quantize:
                prepared[t.name] = quantize_input(arr, dtype)
            else:
                if not np.issubdtype(arr.dtype, np.integer):
                    raise ValueError(f'{t.name}: quantize=False requires integer inputs')
                prepared[t.name] = arr.astype(dtype_for_precision(dtype.width, dtype.signed), copy=False)
        return prepared

    def to_device(self, prepared: Dict[str, np.ndarray]) -> Dict[str, Any]:
        """Prepared host arrays -> device tensors; the iteration axis and the tensors' own leading (batch)
        axis become one batch axis on the GPU."""
        import torch

        graph = self.context.ir.logical
        dev_inputs = {}
        for name, arr in prepared.items():
            merged = arr.reshape((arr.shape[0] * arr.shape[1],) + tuple(arr.shape[2:])) if arr.ndim >= 2 else arr
            dtype = self._io_dtype(graph.tensors[name], 'input')
            if dtype.is_float:
                # float32 values enter the device format the way parameters do (pack_as_float truncates to bfloat16)
                dev_inputs[name] = to_device_float(pack_as_float(merged, dtype.format), dtype.format)
            else:
                dev_inputs[name] = torch.from_numpy(np.ascontiguousarray(merged)).cuda()
        return dev_inputs

    def report(self, X=None, repeats: int = 10):
        """Per-launch timing report on the GPU (the counterpart of the reference's report())."""
        from .report import report

        return report(self, X=X, repeats=repeats)

    def predict(self, X, simulator: str = 'gpu', *, quantize_in: bool = True, dequantize_out: bool = True):
        if simulator.lower() not in ('gpu', 'mi355x', 'gfx950'):
            raise ValueError(f'Unknown simulator "{simulator}". Expected one of: gpu.')
        if not self._compiled:
            self.compile()
        import torch

        prepared = self.prepare_inputs(X, quantize=quantize_in)
        graph = self.context.ir.logical
        dev_inputs = self.to_device(prepared)
        iters = next(iter(prepared.values())).shape[0]
        if self.context.config.get('HipGraph'):
            # serving loops: one HIP graph per input signature, recorded at the first call and replayed afterwards
            key = tuple((n, tuple(t.shape), str(t.dtype)) for n, t in sorted(dev_inputs.items()))
            captured = self._captured.get(key)
            if captured is None:
                captured = self._captured[key] = CapturedExecution(self, dev_inputs)
            dev_out = captured(dev_inputs)
        else:
            dev_out = self.execute(dev_inputs, batch_scale=iters)
        torch.cuda.synchronize()
        results = {}
        for t in graph.graph_outputs():
            dtype = self._io_dtype(t, 'output')
            if dtype.is_float:
                results[t.name] = dev_out[t.name].float().cpu().numpy().astype(np.float64)  # simulation.py:235, 253-254
                continue
            raw = dev_out[t.name].cpu().numpy().astype(np.int64)
            results[t.name] = dequantize_output(raw, dtype.frac) if dequantize_out else raw
        if len(results) == 1:
            return next(iter(results.values()))
        return results

    # ---- executor -------------------------------------------------------------------------------------
    def execute(self, inputs: Dict[str, Any], batch_scale: int = 1, trace: Optional[List[dict]] = None) -> Dict[str, Any]:
        """Run the resolved graph on device tensors. `inputs`: graph-input name -> integer device tensor
        whose leading axis may be `batch_scale` times the declared one. Returns every graph output.
        With `trace` (a list), every launch group is bracketed by two events and appended to it as
        {'name', 'kind', 'nodes', 'events'} (used by report())."""
        from . import ops

        ctx = self.context
        graph, execution = ctx.ir.logical, ctx.ir.execution
        plan = ctx.config.get('gpu_fusion_plan') or {}
        plan = {'add_layernorm': plan.get('add_layernorm', {}), 'mlp_chains': plan.get('mlp_chains', []),
                'attention': plan.get('attention', []), 'dense_add_layernorm': plan.get('dense_add_layernorm', {}),
                'mlp_add_layernorm': plan.get('mlp_add_layernorm', {})}
        values: Dict[str, Any] = dict(inputs)
        fused_ln = {v['layer_norm'] for v in plan['add_layernorm'].values()}
        fused_ln |= {v['layer_norm'] for v in plan['dense_add_layernorm'].values()}
        fused_ln |= {v['layer_norm'] for v in plan['mlp_add_layernorm'].values()}
        fused_dense = {v['dense'] for v in plan['dense_add_layernorm'].values()}
        fused_dense |= {n for v in plan['mlp_add_layernorm'].values() for n in v['chain']}  # run at the add's position
        chain_head = {c[0]: c for c in plan['mlp_chains']}
        chain_rest = {n for c in plan['mlp_chains'] for n in c[1:]}
        attn_at, attn_skip = {}, set()
        order = {n.name: i for i, n in enumerate(graph.nodes)}
        for grp in plan['attention']:
            members = [tr[k] for tr in grp['heads'] for k in ('qk', 'softmax', 'pv')]
            first = min((tr['qk'] for tr in grp['heads']), key=order.get)
            attn_at[first] = grp
            attn_skip.update(m for m in members if m != first)
            if grp.get('concat'):
                attn_skip.add(grp['concat'])

        def launch(label, kind, members, fn):
            if trace is None:
                fn()
                return
            import torch

            ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            ev0.record()
            fn()
            ev1.record()
            trace.append({'name': label, 'kind': kind, 'nodes': list(members), 'events': (ev0, ev1)})

        for node in graph.nodes:
            if node.name in attn_skip:
                continue
            if node.is_placeholder:
                self._run_view(node, values)
                continue
            if node.name in fused_ln or node.name in fused_dense or node.name in chain_rest:
                continue  # executed as part of a fused launch
            if node.name in attn_at:
                grp = attn_at[node.name]
                members = [tr[k] for tr in grp['heads'] for k in ('qk', 'softmax', 'pv')]
                launch(node.name, 'attention', members, lambda: self._run_attention(grp, values, ops))
                continue
            inst = execution.get(node.name)
            if inst is None:
                raise RuntimeError(f'{node.name}: node was never resolved; run compile() first.')
            if node.name in chain_head:
                chain = chain_head[node.name]
                launch(node.name, 'mlp', chain, lambda: self._run_mlp(chain, values, ops))
            elif node.name in plan['mlp_add_layernorm']:
                info = plan['mlp_add_layernorm'][node.name]
                launch(info['chain'][0], 'mlp_add_layer_norm', [*info['chain'], node.name, info['layer_norm']],
                       lambda: self._run_mlp_add_layernorm(info, values, ops))
            elif node.name in plan['dense_add_layernorm']:
                # launched at the add's position: the residual may be computed after the dense's own input
                info = plan['dense_add_layernorm'][node.name]
                launch(info['dense'], 'dense_add_layer_norm', [info['dense'], node.name, info['layer_norm']],
                       lambda: self._run_dense_add_layernorm(info, values, ops))
            elif node.name in plan['add_layernorm']:
                # launched at the add's position: everything that reads the sum comes later in the order
                info = plan['add_layernorm'][node.name]
                launch(node.name, 'add_layer_norm', [node.name, info['layer_norm']],
                       lambda: self._run_add_layernorm((node.name, info), execution.get(info['layer_norm']), values, ops))
            else:
                args = {t.name: values[t.name] for t in node.inputs if not t.is_parameter}
                launch(node.name, node.op_type, [node.name], lambda: values.update(inst.variant.run(inst, args)))
        return {name: values[name] for name in graph.output_tensor_names}

    def _run_view(self, node, values) -> None:
        from . import ops

        sv, cv = node.traits.get('slice_view'), node.traits.get('concat_view')
        if sv is not None:
            src = values[sv.data['source']]
            for item in sv.data['slices']:
                values[item['output']] = src.narrow(int(sv.data['axis']), int(item['start']), int(item['extent']))
        elif cv is not None:
            values[cv.data['output']] = ops.concat([values[i['input']] for i in cv.data['slices']], int(cv.data['axis']))
        elif node.op_type == 'input':
            pass  # hls4ml-style input placeholder
        else:
            raise NotImplementedError(f'{node.name}: placeholder of type {node.op_type!r} has no view trait.')

    def _run_add_layernorm(self, fused, ln_inst, values, ops) -> None:
        add_name, info = fused
        add_inst = self.context.ir.execution.get(add_name)
        add_node, ln_node, cfg = add_inst.node, ln_inst.node, ln_inst.config
        a = values[input_tensor_for_role(add_node, 'lhs').name]
        b = values[input_tensor_for_role(add_node, 'rhs').name]
        res = ops.add_layernorm(a, b, ln_inst.artifacts['packed_gamma'], ln_inst.artifacts['packed_beta'], cfg.out_shift,
                                cfg.rounding_mode, eps_q0=cfg.eps_q0, gamma_shift=cfg.gamma_shift,
                                add_shift=add_inst.config.shift, add_rounding=add_inst.config.rounding_mode,
                                return_sum=bool(info['keep_sum']))
        if info['keep_sum']:
            values[add_node.outputs[0].name], values[ln_node.outputs[0].name] = res
        else:
            values[ln_node.outputs[0].name] = res

    def _run_dense_add_layernorm(self, info, values, ops) -> None:
        execution = self.context.ir.execution
        d_inst, ln_inst = execution.get(info['dense']), execution.get(info['layer_norm'])
        dcfg, cfg = d_inst.config, ln_inst.config
        x = values[input_tensor_for_role(d_inst.node, 'lhs').name]
        packed = d_inst.artifacts['packed_weights']
        rows = x.numel() // int(x.shape[-1]) if x.numel() else 0
        if ops.dense_add_layernorm_applicable(x, packed) and ops.dense_add_layernorm_pays(rows, packed):
            values[ln_inst.node.outputs[0].name] = ops.dense_add_layernorm(
                x, packed, values[info['residual']], ln_inst.artifacts['packed_gamma'], ln_inst.artifacts['packed_beta'],
                cfg.out_shift, dense_rounding=dcfg.rounding_mode, relu=dcfg.flags.use_relu, rounding=cfg.rounding_mode,
                eps_q0=cfg.eps_q0, gamma_shift=cfg.gamma_shift)
            return
        # batch sizes at which the one-launch form does not pay: the same integers from two launches
        y = ops.dense(x, packed, dcfg.rounding_mode, relu=dcfg.flags.use_relu, out_kind='int8')
        values[ln_inst.node.outputs[0].name] = ops.add_layernorm(
            y, values[info['residual']], ln_inst.artifacts['packed_gamma'], ln_inst.artifacts['packed_beta'], cfg.out_shift,
            cfg.rounding_mode, eps_q0=cfg.eps_q0, gamma_shift=cfg.gamma_shift)

    def _run_mlp_add_layernorm(self, info, values, ops) -> None:
        execution = self.context.ir.execution
        insts = [execution.get(n) for n in info['chain']]
        ln_inst = execution.get(info['layer_norm'])
        cfg = ln_inst.config
        specs = [ops.MlpLayerSpec(i.artifacts['packed_weights'], i.config.shift, i.config.flags.use_relu,
                                  i.config.precision['output'].format) for i in insts]
        x = values[input_tensor_for_role(insts[0].node, 'lhs').name]
        same_mode = all(i.config.rounding_mode == insts[0].config.rounding_mode for i in insts)
        rows = x.numel() // max(1, int(x.shape[-1]))
        shapes = [(s.params.K, s.params.N) for s in specs]
        if same_mode and ops.mlp_add_layernorm_applicable(x, specs) and ops.mlp_add_layernorm_pays(rows, shapes):
            values[ln_inst.node.outputs[0].name] = ops.mlp_add_layernorm(
                x, specs, values[info['residual']], ln_inst.artifacts['packed_gamma'], ln_inst.artifacts['packed_beta'],
                cfg.out_shift, rounding=insts[0].config.rounding_mode, ln_rounding=cfg.rounding_mode, eps_q0=cfg.eps_q0,
                gamma_shift=cfg.gamma_shift)
            return
        # outside the fused launch's limits: the chain (or the single layer) as planned without it, then Add + LayerNorm
        if len(insts) > 1:
            self._run_mlp(info['chain'], values, ops)
        else:
            name = input_tensor_for_role(insts[0].node, 'lhs').name
            values.update(insts[0].variant.run(insts[0], {name: values[name]}))
        y = values[insts[-1].node.outputs[0].name]
        values[ln_inst.node.outputs[0].name] = ops.add_layernorm(
            y, values[info['residual']], ln_inst.artifacts['packed_gamma'], ln_inst.artifacts['packed_beta'], cfg.out_shift,
            cfg.rounding_mode, eps_q0=cfg.eps_q0, gamma_shift=cfg.gamma_shift)

    def _run_attention(self, grp, values, ops) -> None:
        """One fused launch for a matmul -> softmax -> matmul triple, or for all heads of a merged group
        (operands become [batch, heads, seq, head_dim] strided views, the result lands in the concat output)."""
        import torch

        execution = self.context.ir.execution
        tr0 = grp['heads'][0]
        c1, c2, c3 = (execution.get(tr0[k]).config for k in ('qk', 'softmax', 'pv'))
        if c2.approximation == 'exp':
            sm = {'kind': 'exp', 'exp_kq': c2.exp_kq, 'inv_shift': c2.inv_shift}
        else:
            sm = {'kind': 'hccs', 'B': int(c2.hccs['B']), 'S': int(c2.hccs['S']), 'Dmax': int(c2.hccs['Dmax']),
                  'inv_shift': c2.inv_shift, 'use_clb': c2.use_clb}
        if grp.get('concat'):
            nh, d = len(grp['heads']), int(self.context.ir.logical.tensors[tr0['q']].shape[-1])

            def heads_view(t, base):  # [batch, seq, H*d] slice -> [batch, H, seq, d] view
                t = t.narrow(-1, base, nh * d)
                return t.unflatten(-1, (nh, d)).permute(0, 2, 1, 3)

            q = heads_view(values[grp['q_src']], grp['q_base'])
            k = heads_view(values[grp['k_src']], grp['k_base'])
            v = heads_view(values[grp['v_src']], grp['v_base'])
            if not _views_are_16_byte_aligned(q, k, v):
                # slices of slices can start anywhere: the planner sees offsets within the nearest source only
                self._run_attention_unfused(grp, values, heads_view=(q, k, v))
                return
            out = torch.empty((q.shape[0], q.shape[2], nh * d), dtype=torch.int8, device=q.device)
            ops.attention(q, k, v, c1.shift, c1.rounding_mode, sm, c3.shift, c3.rounding_mode,
                          out=out.unflatten(-1, (nh, d)).permute(0, 2, 1, 3))
            values[grp['out']] = out
        elif not _views_are_16_byte_aligned(values[tr0['q']], values[tr0['k']], values[tr0['v']]):
            self._run_attention_unfused(grp, values)
        else:
            values[grp['out']] = ops.attention(values[tr0['q']], values[tr0['k']], values[tr0['v']], c1.shift, c1.rounding_mode,
                                               sm, c3.shift, c3.rounding_mode)

    def _run_attention_unfused(self, grp, values, heads_view=None) -> None:
        """The members of a planned attention group one operator at a time: MatMul, Softmax, MatMul per head, then the
        concat. Taken when the operands turn out not to be 16-byte aligned views at run time."""
        execution, graph = self.context.ir.execution, self.context.ir.logical
        for h, tr in enumerate(grp['heads']):
            if heads_view is not None:  # head h of the [batch, heads, seq, d] views, should its slice node come later
                for key, view in zip(('q', 'k', 'v'), heads_view):
                    values.setdefault(tr[key], view[:, h])
            for key in ('qk', 'softmax', 'pv'):
                inst = execution.get(tr[key])
                args = {t.name: values[t.name] for t in inst.node.inputs if not t.is_parameter}
                values.update(inst.variant.run(inst, args))
        if grp.get('concat'):
            self._run_view(next(n for n in graph.nodes if n.name == grp['concat']), values)

    def _run_mlp(self, chain: List[str], values, ops) -> None:
        execution = self.context.ir.execution
        insts = [execution.get(n) for n in chain]
        specs = [ops.MlpLayerSpec(i.artifacts['packed_weights'], i.config.shift, i.config.flags.use_relu,
                                  i.config.precision['output'].format) for i in insts]
        x = values[input_tensor_for_role(insts[0].node, 'lhs').name]
        lead = tuple(x.shape[:-1])
        rows = 1
        for d in lead:
            rows *= int(d)
        shapes = [(s.params.K, s.params.N) for s in specs]
        x_pitch = int(x.shape[-1]) if x.is_contiguous() else 0
        if _mlp_layers_are_faster(rows, shapes, ops.mlp_runs_on_matrix_units(rows, x_pitch, shapes, specs[-1].out_kind)):
            for inst in insts:  # wide layers on a large batch: one GEMM per layer beats the launch that keeps weights in LDS
                values.update(inst.variant.run(inst, {input_tensor_for_role(inst.node, 'lhs').name:
                                                      values[input_tensor_for_role(inst.node, 'lhs').name]}))
            return
        y = ops.mlp(x.reshape(-1, x.shape[-1]), specs, insts[0].config.rounding_mode)
        values[insts[-1].node.outputs[0].name] = y.reshape(lead + (y.shape[-1],))


def _views_are_16_byte_aligned(*tensors) -> bool:
    """What the fused attention launch asks of its operands: 16-byte aligned base addresses and row / head / batch
    pitches (int8 tensors, so elements are bytes)."""
    return all(t.data_ptr() % 16 == 0 and all(int(st) % 16 == 0 for st in t.stride()[:-1]) for t in tensors)


def _mlp_layers_are_faster(rows: int, layers, on_matrix_units: bool = False) -> bool:
    """Whether a chain of Dense layers should run as one GEMM per layer instead of the fused launch, where that launch
    takes its small-batch form (its large-batch form, on the matrix units, is ahead of the per-layer GEMMs wherever it
    applies: 16-64-32-32-5 on 1 048 576 rows 44 us against 479 us, 64-200-200-200-3 on 65 536 rows 33 against 114 us).
    A model of the two,
    fitted to measurements: the fused kernel (weights in LDS, dot products on the vector units) sustains about
    46 TOP/s after staging its weights (8 us + 1 us per 3 KB); a GEMM launch costs about 17 us at least and sustains
    about 200 TOP/s on its tiles, which are 128 wide in N and 64 deep in K at least (256 for wide layers).
    Measured: 57-200-200-200-3 on 65 536 rows 299 us fused / 139 us per layer; on 8192 rows 65 / 70 us;
    16-64-32-32-5 on 1 000 000 rows 190 / 478 us. The per-layer form must be ahead by a quarter to be chosen."""
    if on_matrix_units:
        # ahead of the per-layer GEMMs except for layers that suit the weights-in-registers GEMM (reductions in whole
        # 128-byte tiles, 128 outputs or more) on a batch that gives a CU only a few units of 32 samples:
        # 128-256-128, fused / per layer: 13.4 / 9.3 us on 4096 rows, 14.0 / 10.8 on 16 384, 15.8 / 17.8 on 65 536
        return rows < 32768 and all(k % 128 == 0 and n >= 128 for k, n in layers)

    def up(v, m):
        return (v + m - 1) // m * m
    macs = sum(k * n for k, n in layers)
    weight_bytes = sum(up(k, 16) * n for k, n in layers)
    fused_us = 8.0 + weight_bytes / 3000.0 + 2.0 * macs * rows / 46e6
    per_layer_us = sum(max(17.0, 2.0 * rows * up(k, 64) * up(n, 128) / 200e6) for k, n in layers)
    return per_layer_us < 0.75 * fused_us


class CapturedExecution:
    """A whole-graph execution recorded once into a HIP graph: replaying it costs one launch on the host
    instead of one Python round trip per operator. Inputs are copied into fixed device buffers, outputs live
    in fixed device buffers that the next call overwrites."""

    def __init__(self, model: 'GPUModel', example_inputs: Dict[str, Any]):
        import torch

        self._inputs = {k: v.clone() for k, v in example_inputs.items()}
        # warm up on a side stream (allocator pools, lazily built kernel attributes), then record
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            model.execute(self._inputs)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        self._graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self._graph):
            self._outputs = model.execute(self._inputs)

    def __call__(self, inputs: Dict[str, Any]) -> Dict[str, Any]:
        for name, buf in self._inputs.items():
            src = inputs[name]
            if tuple(src.shape) != tuple(buf.shape) or src.dtype != buf.dtype:
                raise ValueError(f'{name}: captured for {tuple(buf.shape)} {buf.dtype}, got {tuple(src.shape)} {src.dtype}')
            buf.copy_(src)
        self._graph.replay()
        return self._outputs


def _capture(self: GPUModel, example_inputs: Dict[str, Any]) -> CapturedExecution:
    """Record execute() on inputs of these shapes into a HIP graph; see CapturedExecution."""
    if not self._compiled:
        self.compile()
    return CapturedExecution(self, example_inputs)


GPUModel.capture = _capture


def from_context(ctx: BackendContext) -> GPUModel:
    return GPUModel.from_context(ctx)
