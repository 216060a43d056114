"""Checker-only graph interpreter (test infrastructure, never on the product path): walks a resolved operator graph and evaluates every node with the CPU
oracle. It shares the graph and the resolved constants with the GPU executor, but none of its arithmetic."""

import numpy as np

from aie4ml_amd.ir import input_tensor_for_role


def run_graph(model, oracle, inputs):
    """inputs: graph-input name -> integer numpy array. Returns name -> numpy array for every tensor."""
    ctx = model.context
    graph, execution = ctx.ir.logical, ctx.ir.execution
    vals = dict(inputs)
    for node in graph.nodes:
        if node.is_placeholder:
            sv, cv = node.traits.get('slice_view'), node.traits.get('concat_view')
            if sv is not None:
                src, ax = vals[sv.data['source']], int(sv.data['axis'])
                for it in sv.data['slices']:
                    idx = [slice(None)] * src.ndim
                    idx[ax] = slice(int(it['start']), int(it['start']) + int(it['extent']))
                    vals[it['output']] = np.ascontiguousarray(src[tuple(idx)])
            elif cv is not None:
                vals[cv.data['output']] = np.concatenate([vals[i['input']] for i in cv.data['slices']],
                                                         axis=int(cv.data['axis']))
            continue
        inst = execution.get(node.name)
        cfg = inst.config
        out = node.outputs[0].name
        if node.op_type == 'dense':
            W, bias = inst.variant.quantize_weight_bias(inst)
            x = vals[input_tensor_for_role(node, 'lhs').name]
            if cfg.flags.transpose_lhs:  # the operand is consumed through a last-two-axes transpose view
                x = np.ascontiguousarray(np.swapaxes(x, -1, -2))
            x2 = x.reshape(-1, x.shape[-1])
            shifts = np.array(cfg.shift_per_channel) if cfg.shift_per_channel is not None else cfg.shift
            y = oracle.dense(x2, W, bias, shifts, cfg.rounding_mode, relu=cfg.flags.use_relu,
                             out=cfg.precision['output'].format)
            vals[out] = y.reshape(x.shape[:-1] + (y.shape[-1],))
        elif node.op_type == 'matmul':
            a = vals[input_tensor_for_role(node, 'lhs').name]
            if cfg.flags.transpose_lhs:
                a = np.ascontiguousarray(np.swapaxes(a, -1, -2))
            b = vals[input_tensor_for_role(node, 'rhs').name]
            vals[out] = oracle.matmul(a, b, cfg.shift, cfg.rounding_mode, trans_b=cfg.flags.transpose_rhs,
                                      out=cfg.precision['output'].format)
        elif node.op_type == 'add':
            vals[out] = oracle.add(vals[input_tensor_for_role(node, 'lhs').name],
                                   vals[input_tensor_for_role(node, 'rhs').name], cfg.shift, cfg.rounding_mode)
        elif node.op_type == 'layer_norm':
            from aie4ml_amd.op_impls.layernorm import BETA_FRAC_BITS, GAMMA_FRAC_BITS, pack_layernorm_param

            g = pack_layernorm_param(input_tensor_for_role(node, 'gamma').data, name='gamma', full_inner=cfg.cols,
                                     frac=GAMMA_FRAC_BITS)
            b = pack_layernorm_param(input_tensor_for_role(node, 'beta').data, name='beta', full_inner=cfg.cols,
                                     frac=BETA_FRAC_BITS)
            vals[out] = oracle.layernorm(vals[input_tensor_for_role(node, 'lhs').name], g, b, cfg.out_shift,
                                         cfg.rounding_mode, eps_q0=cfg.eps_q0, gamma_shift=cfg.gamma_shift)
        elif node.op_type == 'softmax':
            x = vals[input_tensor_for_role(node, 'lhs').name]
            fmt = cfg.precision['output'].format
            if cfg.approximation == 'exp':
                vals[out] = oracle.softmax_exp(x, cfg.exp_kq, cfg.inv_shift, out=fmt)
            else:
                h = cfg.hccs
                vals[out] = oracle.softmax_hccs(x, int(h['B']), int(h['S']), int(h['Dmax']), cfg.inv_shift, cfg.use_clb,
                                                out=fmt)
        else:
            raise NotImplementedError(node.op_type)
    return vals
