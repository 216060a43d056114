"""Per-launch timing report of a compiled GPUModel: the counterpart of the reference's report()
(src/aie4ml/report.py:475-560), which gathers tiles, latency and per-kernel cycles from the artifacts of the
AMD toolchain. Here the numbers come from the GPU itself: every launch group of the executor is bracketed by
events on the launch stream, the whole graph is timed as one replayed HIP graph, and the operation count
follows the reference's convention (report.py:133-155: 2 * n_in * n_out per independent row, dense and matmul
only).

    from aie4ml_amd.report import report
    print(report(model))                 # tables; report(model)['bottleneck'] etc. index the raw dict
"""

from __future__ import annotations

from typing import Any, Dict, List

import numpy as np

from .ir import get_backend_context, input_tensor_for_role


class Report(dict):
    """Prints as the rendered report and indexes as the raw dict (as the reference's Report does)."""

    def __str__(self) -> str:
        return format_report(self)

    __repr__ = __str__


def _node_ops(node, batch_scale: int) -> int:
    """2 * n_in * n_out * (elements outside the feature axis) for dense / matmul, else 0."""
    if node.op_type not in ('dense', 'matmul') or 'n_in' not in node.metadata:
        return 0
    independent = 1
    for dim in node.outputs[0].shape[:-1]:
        independent *= int(dim)
    rhs = input_tensor_for_role(node, 'rhs')
    n_in = int(node.metadata['n_in'])
    if node.op_type == 'matmul' and rhs is not None:  # the contraction length as this node sees its operands
        lhs = input_tensor_for_role(node, 'lhs')
        n_in = int(lhs.shape[-1])
    return 2 * n_in * int(node.outputs[0].shape[-1]) * independent * int(batch_scale)


def _node_bytes(node, batch_scale: int) -> int:
    """Bytes an operator has to read and write once: activations in + out (parameters are negligible)."""
    total = 0
    for t in list(node.inputs) + list(node.outputs):
        if t.is_parameter or t.precision is None:
            continue
        total += int(np.prod(t.shape)) * max(1, int(getattr(t.precision, 'width', 8)) // 8)
    return total * int(batch_scale)


def collect_report(model, X=None, repeats: int = 10) -> Report:
    """Run the model `repeats` times with event brackets around every launch group and once more as a replayed
    HIP graph. X: inputs as for predict() (quantised like predict does); default: zeros of the declared shapes."""
    import torch

    if not getattr(model, '_compiled', False):
        model.compile()
    ctx = get_backend_context(model)
    graph = ctx.ir.logical
    if X is None:
        X = {t.name: np.zeros(tuple(int(d) for d in t.shape), dtype=np.float32) for t in graph.graph_inputs()}
    prepared = model.prepare_inputs(X, quantize=True)
    iters = next(iter(prepared.values())).shape[0]
    dev_inputs = model.to_device(prepared)

    import time

    model.execute(dev_inputs, batch_scale=iters)  # warm-up: lazily set kernel attributes, allocator pools
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    model.execute(dev_inputs, batch_scale=iters)
    host_s = time.perf_counter() - t0  # what the interpreter needs to issue one pass
    torch.cuda.synchronize()
    runs: List[List[dict]] = []
    for _ in range(max(1, int(repeats))):
        trace: List[dict] = []
        # keep the GPU busy while the pass is being issued, so that the event pairs bracket kernels that run back
        # to back instead of the gaps in which the GPU waits for the interpreter
        try:
            torch.cuda._sleep(int(host_s * 2.5e9 * 2) + 200_000)
        except (AttributeError, RuntimeError):
            pass
        model.execute(dev_inputs, batch_scale=iters, trace=trace)
        torch.cuda.synchronize()
        for item in trace:
            ev0, ev1 = item.pop('events')
            item['us'] = ev0.elapsed_time(ev1) * 1e3
        runs.append(trace)

    nodes = {n.name: n for n in graph.nodes}
    kernels = []
    for i, item in enumerate(runs[0]):
        us = float(np.median([r[i]['us'] for r in runs]))
        members = [nodes[m] for m in item['nodes'] if m in nodes]
        ops = sum(_node_ops(n, iters) for n in members)
        moved = sum(_node_bytes(n, iters) for n in members)
        kernels.append({'name': item['name'], 'kind': item['kind'], 'nodes': item['nodes'], 'time_us': round(us, 2),
                        'ops': int(ops), 'tops': round(ops / us / 1e6, 2) if ops else None,
                        'bytes': int(moved), 'gbs': round(moved / us / 1e3, 1) if moved else None})
    total = sum(k['time_us'] for k in kernels) or 1.0
    for k in kernels:
        k['pct'] = round(100.0 * k['time_us'] / total, 1)

    # the whole graph as one replayed HIP graph: what a serving loop would see per batch
    captured = model.capture(dev_inputs)
    captured(dev_inputs)
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    reps = max(3, int(repeats))
    ev0.record()
    for _ in range(reps):
        captured._graph.replay()
    ev1.record()
    torch.cuda.synchronize()
    graph_us = ev0.elapsed_time(ev1) * 1e3 / reps

    batch = int(next(iter(dev_inputs.values())).shape[0]) if dev_inputs else 0
    ops_total = sum(k['ops'] for k in kernels)
    props = torch.cuda.get_device_properties(0)
    worst = max(kernels, key=lambda k: k['time_us']) if kernels else None
    return Report({
        'device': {'name': props.name, 'compute_units': int(props.multi_processor_count),
                   'memory_gib': round(props.total_memory / 2 ** 30, 1)},
        'design': {'nodes': len([n for n in graph.nodes if not n.is_placeholder]), 'launches': len(kernels),
                   'ops': int(ops_total), 'batch': batch},
        'kernels': kernels,
        'latency': {'graph_replay_us': round(graph_us, 2), 'sum_of_launches_us': round(total, 2)},
        'throughput': {'samples_per_s': round(batch / (graph_us * 1e-6), 1) if batch else None,
                       'tops': round(ops_total / graph_us / 1e6, 2) if ops_total else None},
        'bottleneck': {'name': worst['name'], 'kind': worst['kind'], 'time_us': worst['time_us'], 'pct': worst['pct']}
        if worst else {},
    })


def report(model, X=None, repeats: int = 10) -> Report:
    """Collect the timing report of a model on the GPU (see collect_report)."""
    return collect_report(model, X=X, repeats=repeats)


def format_report(rep: Dict[str, Any]) -> str:
    out: List[str] = []
    add = out.append
    dev, design = rep.get('device') or {}, rep.get('design') or {}
    add('=' * 100)
    add('  aie4ml_amd  |  GPU execution report')
    add(f'  {dev.get("name", "?")}, {dev.get("compute_units", "?")} CUs, {dev.get("memory_gib", "?")} GiB')
    add('=' * 100)
    add(f'  {design.get("nodes", 0)} operator nodes in {design.get("launches", 0)} launches, '
        f'{design.get("ops", 0):,} ops per batch of {design.get("batch", 0)} (dense / matmul, 2 per multiply-add)')
    lat, thr = rep.get('latency') or {}, rep.get('throughput') or {}
    add('')
    add('Latency  (one batch, inputs resident on the device)')
    add(f'    whole graph, replayed as one HIP graph   {lat.get("graph_replay_us", 0):12,.1f} us')
    add(f'    sum of the launches, timed one by one    {lat.get("sum_of_launches_us", 0):12,.1f} us')
    if thr.get('samples_per_s'):
        line = f'    throughput                               {thr["samples_per_s"]:12,.0f} samples/s'
        if thr.get('tops'):
            line += f'   {thr["tops"]:,.1f} TOP/s'
        add(line)
    add('')
    add('Launches')
    add(f'    {"name":40s} {"kind":16s} {"time us":>10s} {"share":>7s} {"TOP/s":>9s} {"GB/s":>9s}')
    for k in rep.get('kernels') or []:
        name = k['name'] if len(k['name']) <= 40 else k['name'][:37] + '...'
        tops = f'{k["tops"]:9,.1f}' if k.get('tops') else f'{"-":>9s}'
        gbs = f'{k["gbs"]:9,.0f}' if k.get('gbs') else f'{"-":>9s}'
        add(f'    {name:40s} {k["kind"]:16s} {k["time_us"]:10,.1f} {k["pct"]:6.1f}% {tops} {gbs}')
    b = rep.get('bottleneck') or {}
    if b:
        add('')
        add(f'Bottleneck: {b["name"]} ({b["kind"]}), {b["time_us"]:,.1f} us, {b["pct"]}% of the launch time')
    return '\n'.join(out)
