#!/usr/bin/env python3
"""Benchmark of the quantized-operator hot path on one MI355X.

Default workload: the single quantized Dense of the baseline configuration
(M=8192 rows x K=4096 -> N=4096, int32 bias, per-output-channel shift in [8,12], round-to-nearest-even,
saturate to int8, fused ReLU). One step = one pass of the operator over the whole synthetic batch,
inputs already resident in HBM. Prints ONE JSON line.

The default run also times, after the headline workload, the matrix-core calibration loop (`roofline.calibrated_peak`,
`frac_of_calibrated`, the clock under matrix load) and every other baseline configuration with the same method
(`workloads`: value, ms_per_step, bit_exact, roofline per configuration; no CPU leg). `--only` skips both.
The HBM-bound workloads are timed twice: on one set of buffers like every other workload (`value`, `roofline.frac`:
operands that fit the 256 MB memory-side cache are found there by the next launch), and over a ring of operand copies
of 1 GiB (`roofline.frac_operands_from_hbm`: every operand comes from HBM).

Other workloads (--workload c2_dense_i16 | c2_dense_i16x16 | c2_dense_bf16 | c2_dense_fp8 | c1_mlp | c1_mlp_stream | c3_softmax_exp | c3_softmax_hccs | c3_qk | c3_pv |
c3_attention_exp | c3_attention_hccs | c4_add_layernorm | c4_layernorm | c4_add | c5_encoder) print the same line for that operator or graph;
--workload calib_copy runs a plain 256 MiB elementwise copy, the known-size kernel the HBM traffic
counters are scaled against; --workload calib_mfma runs the register-resident int8 MFMA loop alone.
"""

from __future__ import annotations

import argparse
import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, TOP/s
PEAK_BF16_TFLOPS = 2500.0  # MI355X dense bf16 MFMA, TFLOP/s
PEAK_FP8_TFLOPS = 5000.0   # MI355X dense fp8 MFMA, TFLOP/s
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, GB/s
COLD_RING_BYTES = 1 << 30  # operand copies the cold leg of the HBM-bound workloads cycles through: 4 x the 256 MB memory-side cache

# HBM bytes per launch of each workload's dominant kernel come from hardware counters (FETCH_SIZE and WRITE_SIZE, one
# counter run each, scaled by what the same counter reads for calib_copy). The summaries of those runs are the text
# files under profiles/, named <kernel>__<workload>.txt; the figure is read from their line "traffic = X MB per launch"
# so that it cannot outlive the profile it came from. None = no profile for this kernel and workload.
def measured_traffic(kernel, wl):
    import re

    path = ROOT / 'profiles' / f'{kernel}__{wl}.txt'
    if not path.exists():
        return None, None
    m = re.search(r'^\s*traffic = ([0-9.]+) MB per launch', path.read_text(), flags=re.M)
    return (int(float(m.group(1)) * 1e6), f'profiles/{path.name}') if m else (None, None)


def _time_gpu(torch, fn, steps, warmup, use_graph=True):
    """Times exactly `steps` launches between two events on the launch stream, synchronised on both
    sides. The launches are recorded once into a HIP graph and replayed, so that the interval holds
    back-to-back kernels rather than the Python interpreter's per-call cost (which exceeds the run time
    of the small row kernels); falls back to eager launches if capture is not possible. Besides the `warmup`
    eager launches the recorded graph is replayed three times untimed: per-launch times keep falling over the
    first few hundred launches while the clocks settle."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    graph = None
    if use_graph:
        try:
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):
                fn()
            torch.cuda.current_stream().wait_stream(side)
            torch.cuda.synchronize()
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph):
                for _ in range(steps):
                    fn()
            for _ in range(3):  # untimed replays: the first uploads the graph, the others let the clocks settle
                graph.replay()
            torch.cuda.synchronize()
        except Exception as exc:  # noqa: BLE001
            print(f'bench.py: graph capture failed ({exc}); timing eager launches', file=sys.stderr)
            graph = None
            torch.cuda.synchronize()
    ev0 = torch.cuda.Event(enable_timing=True)
    ev1 = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev0.record()
    if graph is not None:
        graph.replay()
    else:
        for _ in range(steps):
            fn()
    ev1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return wall_ms / steps, ev0.elapsed_time(ev1) / steps, graph is not None


def _time_cpu(fn, budget_s=12.0, min_runs=2):
    fn()  # warm
    times = []
    t_start = time.perf_counter()
    while len(times) < min_runs or (time.perf_counter() - t_start < budget_s and len(times) < 7):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return float(np.median(times))


# The four projections of the c5 encoder block as Dense workloads of their own (rows = batch 64 x seq 128): shape,
# the kernel that runs them, and which projection it is.
ENCODER_PROJECTIONS = {
    'c5_proj_qkv': (8192, 768, 2304, 'gemm_wrow_kernel', 'fused Q/K/V projection'),
    'c5_proj_out': (8192, 768, 768, 'gemm_wrow_kernel', 'attention output projection'),
    'c5_ffn_up': (8192, 768, 3072, 'gemm_wrow_kernel', 'first feed-forward projection'),
    'c5_ffn_down': (8192, 3072, 768, 'gemm_sk_kernel', 'second feed-forward projection'),
}


def prepare(wl, torch):
    """Builds one workload on the GPU, runs it once and checks it against the oracle. Returns a dict with the step
    function `fn`, the algorithmic work per step, the roofline that bounds it and what the CPU leg needs."""
    from aie4ml_amd import ops, workloads
    from oracle import oracle

    dev = lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()  # noqa: E731
    extra = {}
    fn_cold = None

    def rotating(call, tensors, bytes_per_launch):
        """`call(*tensors)` over a ring of copies of the tensors that holds COLD_RING_BYTES in all: by the time a copy's
        turn comes again, four times the memory-side cache's capacity has passed through it, so every launch fetches its
        operands from HBM. The plain step function works on one set of buffers, which a replayed graph finds in that
        cache again where they fit (the C4 tensors do)."""
        nsets = max(2, -(-COLD_RING_BYTES // int(bytes_per_launch)))
        ring = []  # made on the first call: a run that skips this leg allocates and copies nothing for it
        turn = [0]

        def step():
            if not ring:
                ring.extend(tuple(t.clone() for t in tensors) for _ in range(nsets))
            ts = ring[turn[0] % nsets]
            turn[0] += 1
            call(*ts)

        step.bytes_per_launch = int(bytes_per_launch)
        return step
    cpu_fn = None
    cpu_samples = None
    cpu_work = cpu_desc = None
    peak_mfma, mfma_unit = PEAK_INT8_TOPS, 'TOP/s'

    if wl in ('c2_dense', 'c2_dense_zero') or wl in ENCODER_PROJECTIONS:
        M, K, N = ENCODER_PROJECTIONS[wl][:3] if wl in ENCODER_PROJECTIONS else (8192, 4096, 4096)
        A, W, bias, shifts = workloads.c2_dense(M, K, N)
        if wl == 'c2_dense_zero':  # power-limit probe: see main()
            A, W = np.zeros_like(A), np.zeros_like(W)
        p = ops.pack_dense(dev(W), dev(bias), shifts)
        dA = dev(A)
        out = torch.empty((M, N), dtype=torch.int8, device='cuda')
        fn = lambda: ops.dense(dA, p, 'conv_even', relu=True, out=out)  # noqa: E731
        fn()
        # bit-exact gate on a row subset (rows are independent)
        rows = np.random.default_rng(0).choice(M, 96, replace=False)
        exp = oracle.dense(A[rows], W, bias, shifts, 'conv_even', relu=True)
        torch.cuda.synchronize()
        bit_exact = bool(np.array_equal(out[torch.from_numpy(rows).cuda()].cpu().numpy(), exp))
        work, unit_work, bound = 2.0 * M * N * K, 'op', 'mfma'
        samples = M
        config = {'workload': f'{wl}: Dense {M}x{K} -> {N}, int8, bias, per-channel shift 8..12, conv_even, '
                              'sat int8, ReLU' + (' (all-zero operands)' if wl == 'c2_dense_zero' else '') +
                              (f' (the {ENCODER_PROJECTIONS[wl][4]} of the c5 encoder block, alone)' if wl in ENCODER_PROJECTIONS else '')}
        sample_rows = 2048  # about 1 s per pass on 16 host threads, 10 s with the repeats
        cpu_desc = f'oracle Dense on the first {sample_rows} of {M} rows (same W/bias/shifts), scaled per op'
        cpu_fn = lambda: oracle.dense(A[:sample_rows], W, bias, shifts, 'conv_even', relu=True)  # noqa: E731
        cpu_work = 2.0 * sample_rows * N * K
        metric, unit = 'int8_dense_tops', 'TOP/s'
        kernel = ENCODER_PROJECTIONS[wl][3] if wl in ENCODER_PROJECTIONS else 'gemm_rs_kernel'
    elif wl == 'c5_proj_out_ln':
        # the attention output projection of the c5 block together with the residual add and the LayerNorm behind it,
        # as the graph executor launches them at this batch size: one kernel whose workgroups own whole rows
        M, K, N = 8192, 768, 768
        A, W, bias, _ = workloads.c2_dense(M, K, N)
        r = np.random.default_rng(23)
        res = np.clip(np.rint(r.normal(0, 30, (M, N))), -128, 127).astype(np.int8)
        gamma = r.integers(32, 128, N).astype(np.int16)
        beta = (r.integers(-16, 17, N).astype(np.int32) << 10).astype(np.int16)
        p = ops.pack_dense(dev(W), dev(bias), np.array([9], np.int32))
        dA, dres, dg, dbt = dev(A), dev(res), dev(gamma), dev(beta)
        out = torch.empty((M, N), dtype=torch.int8, device='cuda')
        fn = lambda: ops.dense_add_layernorm(dA, p, dres, dg, dbt, 5, 'conv_even', False, 'conv_even', out=out)  # noqa: E731
        fn()
        rows = np.random.default_rng(0).choice(M, 96, replace=False)
        ref = lambda sel: oracle.add_layernorm(oracle.dense(A[sel], W, bias, 9, 'conv_even', out='int8'), res[sel], gamma,  # noqa: E731
                                               beta, 5, 'conv_even')
        exp = ref(rows)
        torch.cuda.synchronize()
        bit_exact = bool(np.array_equal(out[torch.from_numpy(rows).cuda()].cpu().numpy(), exp))
        work, bound = 2.0 * M * N * K, 'mfma'
        samples = M
        config = {'workload': f'c5_proj_out_ln: Dense {M}x{K} -> {N} (int8, bias, shift 9, conv_even) + residual add + LayerNorm '
                              f'over {N} columns in one launch (the tail of the attention half of the c5 encoder block)'}
        sample_rows = 2048
        cpu_desc = f'oracle dense -> add -> layernorm on the first {sample_rows} of {M} rows, scaled per op'
        cpu_fn = lambda: ref(slice(0, sample_rows))  # noqa: E731
        cpu_work = 2.0 * sample_rows * N * K
        metric, unit = 'int8_dense_tops', 'TOP/s'
        kernel = 'gemm_rowln_kernel'
    elif wl == 'c2_dense_i16':
        # the (16, 8) width combination on the C2 shape: int16 activations, int8 weights, int16 output
        M, K, N = 8192, 4096, 4096
        _, W, bias, shifts = workloads.c2_dense(M, K, N)
        A = np.random.default_rng(19).integers(-32768, 32768, (M, K)).astype(np.int16)
        shifts = shifts + 6
        p = ops.pack_dense(dev(W), dev(bias), shifts)
        dA = dev(A)
        out = torch.empty((M, N), dtype=torch.int16, device='cuda')
        fn = lambda: ops.dense(dA, p, 'conv_even', relu=True, out_kind='int16', out=out)  # noqa: E731
        fn()
        rows = np.random.default_rng(0).choice(M, 64, replace=False)
        exp = oracle.dense(A[rows], W, bias, shifts, 'conv_even', relu=True, out='int16')
        torch.cuda.synchronize()
        bit_exact = bool(np.array_equal(out[torch.from_numpy(rows).cuda()].cpu().numpy(), exp))
        work, bound = 2.0 * M * N * K, 'mfma'
        samples = M
        config = {'workload': 'c2_dense_i16: Dense 8192x4096 -> 4096, int16 activations x int8 weights (acc32), bias, '
                              'per-channel shift, conv_even, sat int16, ReLU'}
        sample_rows = 256
        cpu_desc = f'oracle Dense (int16 activations) on the first {sample_rows} of {M} rows, scaled per op'
        cpu_fn = lambda: oracle.dense(A[:sample_rows], W, bias, shifts, 'conv_even', relu=True, out='int16')  # noqa: E731
        cpu_work = 2.0 * sample_rows * N * K
        metric, unit = 'int16x8_dense_tops', 'TOP/s'
        kernel = 'gemm_rs_kernel'
    elif wl == 'c2_dense_i16x16':
        # the (16, 16) width combination on the C2 shape: int16 activations and weights, 64-bit accumulator, int16 output
        M, K, N = 8192, 4096, 4096
        r = np.random.default_rng(29)
        A = r.integers(-32768, 32768, (M, K)).astype(np.int16)
        W = r.integers(-32768, 32768, (K, N)).astype(np.int16)
        bias = r.integers(-2**30, 2**30, N).astype(np.int32)
        shifts = r.integers(25, 29, N).astype(np.int32)
        p = ops.pack_dense(dev(W), dev(bias), shifts)
        dA = dev(A)
        out = torch.empty((M, N), dtype=torch.int16, device='cuda')
        fn = lambda: ops.dense(dA, p, 'conv_even', relu=True, out_kind='int16', out=out)  # noqa: E731
        fn()
        rows = np.random.default_rng(0).choice(M, 64, replace=False)
        exp = oracle.dense(A[rows], W, bias, shifts, 'conv_even', relu=True, out='int16')
        torch.cuda.synchronize()
        bit_exact = bool(np.array_equal(out[torch.from_numpy(rows).cuda()].cpu().numpy(), exp))
        work, bound = 2.0 * M * N * K, 'mfma'
        samples = M
        config = {'workload': 'c2_dense_i16x16: Dense 8192x4096 -> 4096, int16 activations x int16 weights (acc64), bias, '
                              'per-channel shift, conv_even, sat int16, ReLU'}
        sample_rows = 256
        cpu_desc = f'oracle Dense (int16 x int16) on the first {sample_rows} of {M} rows, scaled per op'
        cpu_fn = lambda: oracle.dense(A[:sample_rows], W, bias, shifts, 'conv_even', relu=True, out='int16')  # noqa: E731
        cpu_work = 2.0 * sample_rows * N * K
        metric, unit = 'int16x16_dense_tops', 'TOP/s'
        kernel = 'gemm_rs_kernel'
    elif wl in ('c2_dense_bf16', 'c2_dense_fp8'):
        # the reference's float compute path on the C2 shape: bfloat16 / fp8 e4m3 operands, float32 accumulation and bias
        M, K, N = 8192, 4096, 4096
        fp8 = wl == 'c2_dense_fp8'
        fmt, tdt = ('fp8_e4m3', torch.float8_e4m3fn) if fp8 else ('bfloat16', torch.bfloat16)
        r = np.random.default_rng(23)
        A32 = r.normal(0, 1.0, (M, K)).astype(np.float32)
        W32 = r.normal(0, 0.02, (K, N)).astype(np.float32)
        bias = r.normal(0, 0.1, N).astype(np.float32)
        if fp8:  # the library's device cast makes the operands (round to nearest even); what it made is what both sides use
            dA = torch.from_numpy(A32).cuda().to(tdt)
            dW = torch.from_numpy(W32).cuda().to(tdt)
            A, W = dA.float().cpu().numpy(), dW.float().cpu().numpy()
        else:
            A, W = oracle.bf16_truncate(A32), oracle.bf16_truncate(W32)
            dA, dW = torch.from_numpy(A).cuda().to(tdt), torch.from_numpy(W).cuda().to(tdt)
        p = ops.pack_dense_float(dW, torch.from_numpy(bias).cuda())
        out = torch.empty((M, N), dtype=tdt, device='cuda')
        fn = lambda: ops.dense_float(dA, p, relu=True, out=out)  # noqa: E731
        fn()
        rows = r.choice(M, 16 if fp8 else 64, replace=False)
        exp = oracle.dense_float(A[rows], W, bias, relu=True, fmt=fmt)
        torch.cuda.synchronize()
        got = out[torch.from_numpy(rows).cuda()].float().cpu().numpy()
        # float path: no bit-exactness across summation orders. bfloat16: the reference's own tolerance; fp8 (no
        # reference test): one unit in the last place of the output format
        rtol, atol = (2.0 ** -3, 2.0 ** -9) if fp8 else (1e-2, 5e-2)
        bit_exact = bool(np.allclose(got, exp, rtol=rtol, atol=atol))
        extra['parity'] = f'within rtol {rtol:g} / atol {atol:g} of the exact-accumulation oracle (float path)'
        extra['max_abs_err'] = float(np.max(np.abs(got - exp)))
        work, bound = 2.0 * M * N * K, 'mfma'
        peak_mfma, mfma_unit = (PEAK_FP8_TFLOPS if fp8 else PEAK_BF16_TFLOPS), 'TFLOP/s'
        samples = M
        config = {'workload': f'{wl}: Dense 8192x4096 -> 4096, {fmt} operands, float32 accumulate + bias, ReLU, {fmt} out'}
        sample_rows = 64 if fp8 else 256
        cpu_desc = f'oracle float Dense (float64 numpy matmul) on the first {sample_rows} of {M} rows, scaled per op'
        cpu_fn = lambda: oracle.dense_float(A[:sample_rows], W, bias, relu=True, fmt=fmt)  # noqa: E731
        cpu_work = 2.0 * sample_rows * N * K
        metric, unit = ('fp8_dense_tflops' if fp8 else 'bf16_dense_tflops'), 'TFLOP/s'
        kernel = 'gemm_rs_kernel'
    elif wl == 'c1_mlp':
        x, layers = workloads.c1_mlp(1024)
        specs = [ops.MlpLayerSpec(ops.pack_dense(dev(Wl), dev(b), s), s, relu, o) for (Wl, b, s, relu, o) in layers]
        dx = dev(x)
        out = torch.empty((1024, 5), dtype=torch.int8, device='cuda')
        fn = lambda: ops.mlp(dx, specs, 'positive_inf', out=out)  # noqa: E731
        fn()
        torch.cuda.synchronize()
        bit_exact = bool(np.array_equal(out.cpu().numpy(), oracle.mlp(x, layers, 'positive_inf')))
        work, bound = 8512.0 * 1024, 'mfma'
        samples = 1024
        config = {'workload': 'c1_mlp: int8 MLP 16-64-32-32-5, batch 1024, shift 7, round half up, fused single launch'}
        cpu_desc = 'oracle MLP (layer by layer) on the full batch of 1024'
        cpu_fn = lambda: oracle.mlp(x, layers, 'positive_inf')  # noqa: E731
        cpu_work = work
        metric, unit = 'int8_mlp_samples_per_s', 'samples/s'
        kernel = 'mlp_mfma_kernel'
    elif wl == 'c1_mlp_stream':
        # the same network on a stream of samples: what a trigger or a tagging farm asks of it (throughput, not latency)
        nb = 1 << 20
        x, layers = workloads.c1_mlp(nb)
        specs = [ops.MlpLayerSpec(ops.pack_dense(dev(Wl), dev(b), s), s, relu, o) for (Wl, b, s, relu, o) in layers]
        dx = dev(x)
        out = torch.empty((nb, 5), dtype=torch.int8, device='cuda')
        fn = lambda: ops.mlp(dx, specs, 'positive_inf', out=out)  # noqa: E731
        fn()
        torch.cuda.synchronize()
        got = out.cpu().numpy()
        sl = slice(0, 65536)
        bit_exact = bool(np.array_equal(got[sl], oracle.mlp(x[sl], layers, 'positive_inf'))
                         and np.array_equal(got[-4099:], oracle.mlp(x[-4099:], layers, 'positive_inf')))
        work, bound = 21.0 * nb, 'hbm'  # 16 bytes in, 5 out per sample
        samples = nb
        config = {'workload': 'c1_mlp_stream: int8 MLP 16-64-32-32-5, batch 1048576, shift 7, round half up, fused single '
                              'launch on the matrix units'}
        cpu_desc = 'oracle MLP (layer by layer) on 65536 samples'
        cpu_fn = lambda: oracle.mlp(x[sl], layers, 'positive_inf')  # noqa: E731
        cpu_work = 21.0 * 65536
        cpu_samples = 65536
        metric, unit = 'int8_mlp_samples_per_s', 'samples/s'
        kernel = 'mlp_mfma_kernel'
    elif wl in ('c4_add_layernorm', 'c4_layernorm', 'c4_add'):
        rows, cols = 16384, 1024
        a, b, gamma, beta, prm = workloads.c4_add_layernorm(rows, cols)
        da, db, dg, dbt = dev(a), dev(b), dev(gamma), dev(beta)
        sub = slice(0, 512)
        dout = torch.empty_like(da)
        if wl == 'c4_add_layernorm':
            fn = lambda: ops.add_layernorm(da, db, dg, dbt, prm['out_shift'], 'conv_even', out=dout)  # noqa: E731
            got = fn()
            exp = oracle.add_layernorm(a[sub], b[sub], gamma, beta, prm['out_shift'], 'conv_even')
            work = 3.0 * rows * cols
            cpu_fn = lambda: oracle.add_layernorm(a, b, gamma, beta, prm['out_shift'], 'conv_even')  # noqa: E731
            kernel = 'layernorm_rows_kernel'
            fn_cold = rotating(lambda a_, b_, o_: ops.add_layernorm(a_, b_, dg, dbt, prm['out_shift'], 'conv_even', out=o_),
                               (da, db, dout), work)
        elif wl == 'c4_layernorm':
            fn = lambda: ops.layernorm(da, dg, dbt, prm['out_shift'], 'conv_even', out=dout)  # noqa: E731
            got = fn()
            exp = oracle.layernorm(a[sub], gamma, beta, prm['out_shift'], 'conv_even')
            work = 2.0 * rows * cols
            cpu_fn = lambda: oracle.layernorm(a, gamma, beta, prm['out_shift'], 'conv_even')  # noqa: E731
            kernel = 'layernorm_rows_kernel'
            fn_cold = rotating(lambda a_, o_: ops.layernorm(a_, dg, dbt, prm['out_shift'], 'conv_even', out=o_), (da, dout), work)
        else:
            fn = lambda: ops.add(da, db, out=dout)  # noqa: E731
            got = fn()
            exp = oracle.add(a[sub], b[sub])
            work = 3.0 * rows * cols
            cpu_fn = lambda: oracle.add(a, b)  # noqa: E731
            kernel = 'add_sat8_kernel'
            fn_cold = rotating(lambda a_, b_, o_: ops.add(a_, b_, out=o_), (da, db, dout), work)
        torch.cuda.synchronize()
        bit_exact = bool(np.array_equal(got[sub].cpu().numpy(), exp))
        bound, samples = 'hbm', rows
        cpu_work = work
        cpu_desc = f'oracle {wl} on the full [{rows},{cols}] tensor'
        config = {'workload': f'{wl}: [{rows},{cols}] int8, conv_even, out frac 5'}
        metric, unit = f'{wl}_gbs', 'GB/s'
    elif wl in ('c3_softmax_exp', 'c3_softmax_hccs', 'c3_qk', 'c3_pv'):
        Bt, H, S, D = 32, 16, 512, 64
        q, k, v, prm = workloads.c3_attention(Bt, H, S, D)
        dq, dk, dv = dev(q), dev(k), dev(v)
        logits = ops.matmul(dq, dk, prm['logit_shift'], 'conv_even', trans_b=True)
        probs = ops.softmax_exp(logits, prm['exp_kq'])
        torch.cuda.synchronize()
        hb = (0, 3)  # one (batch, head) slice for the bit-exact gate
        l_ref = oracle.matmul(q[hb], k[hb], prm['logit_shift'], 'conv_even', trans_b=True)
        if wl == 'c3_qk':
            out = torch.empty_like(logits)
            fn = lambda: ops.matmul(dq, dk, prm['logit_shift'], 'conv_even', trans_b=True, out=out)  # noqa: E731
            fn()
            torch.cuda.synchronize()
            bit_exact = bool(np.array_equal(out[hb].cpu().numpy(), l_ref))
            work, bound = 2.0 * Bt * H * S * S * D, 'hbm'
            bytes_ = Bt * H * (2 * S * D + S * S)
            extra['tops'] = None
            cpu_fn = lambda: oracle.matmul(q[0, :4], k[0, :4], prm['logit_shift'], 'conv_even', trans_b=True)  # noqa: E731
            cpu_work = bytes_ * 4 / (Bt * H)
            cpu_desc = 'oracle MatMul on 4 of 512 (batch, head) slices'
            work = float(bytes_)
            kernel = 'matmul_lean_nt_kernel'
            fn_cold = rotating(lambda q_, k_, o_: ops.matmul(q_, k_, prm['logit_shift'], 'conv_even', trans_b=True, out=o_),
                               (dq, dk, out), bytes_)
        elif wl == 'c3_pv':
            ws = torch.empty((ops._lib.load().a4g_matmul_i8_workspace_bytes(Bt * H, S, D, S, 0, 1),), dtype=torch.uint8,
                             device='cuda')
            out = torch.empty((Bt, H, S, D), dtype=torch.int8, device='cuda')
            fn = lambda: ops.matmul(probs, dv, prm['pv_shift'], 'conv_even', out=out, workspace=ws)  # noqa: E731
            fn()
            torch.cuda.synchronize()
            p_ref = oracle.softmax_exp(l_ref, prm['exp_kq'])
            bit_exact = bool(np.array_equal(out[hb].cpu().numpy(), oracle.matmul(p_ref, v[hb], prm['pv_shift'], 'conv_even')))
            bytes_ = Bt * H * (S * S + 2 * S * D)
            work, bound = float(bytes_), 'hbm'
            pl = probs[0, :4].cpu().numpy()
            cpu_fn = lambda: oracle.matmul(pl, v[0, :4], prm['pv_shift'], 'conv_even')  # noqa: E731
            cpu_work = bytes_ * 4 / (Bt * H)
            cpu_desc = 'oracle MatMul (uint8 x int8) on 4 of 512 (batch, head) slices'
            kernel = 'matmul_lean_nn_kernel'
            fn_cold = rotating(lambda p_, v_, o_: ops.matmul(p_, v_, prm['pv_shift'], 'conv_even', out=o_, workspace=ws),
                               (probs, dv, out), bytes_)
        else:
            out = torch.empty(logits.shape, dtype=torch.uint8, device='cuda')
            hc = prm['hccs']
            if wl == 'c3_softmax_exp':
                fn = lambda: ops.softmax_exp(logits, prm['exp_kq'], out=out)  # noqa: E731
                fn_cold = rotating(lambda x_, o_: ops.softmax_exp(x_, prm['exp_kq'], out=o_), (logits, out), 2.0 * Bt * H * S * S)
                ref = oracle.softmax_exp(l_ref, prm['exp_kq'])
                cpu1 = lambda x_: oracle.softmax_exp(x_, prm['exp_kq'])  # noqa: E731
            else:
                fn = lambda: ops.softmax_hccs(logits, hc['B'], hc['S'], hc['Dmax'], out=out)  # noqa: E731
                fn_cold = rotating(lambda x_, o_: ops.softmax_hccs(x_, hc['B'], hc['S'], hc['Dmax'], out=o_), (logits, out),
                                   2.0 * Bt * H * S * S)
                ref = oracle.softmax_hccs(l_ref, hc['B'], hc['S'], hc['Dmax'])
                cpu1 = lambda x_: oracle.softmax_hccs(x_, hc['B'], hc['S'], hc['Dmax'])  # noqa: E731
            fn()
            torch.cuda.synchronize()
            bit_exact = bool(np.array_equal(out[hb].cpu().numpy(), ref))
            work, bound = 2.0 * Bt * H * S * S, 'hbm'
            lsub = logits[:2].cpu().numpy()
            cpu_fn = lambda: cpu1(lsub)  # noqa: E731
            cpu_work = 2.0 * 2 * H * S * S
            cpu_desc = 'oracle softmax on 2 of 32 batches (16384 of 262144 rows)'
            kernel = 'softmax_lut_kernel'
        samples = Bt
        config = {'workload': f'{wl}: attention core batch 32 x 16 heads, seq 512, head_dim 64'}
        metric, unit = f'{wl}_gbs', 'GB/s'
    elif wl in ('c3_attention_exp', 'c3_attention_hccs'):
        Bt, H, S, D = 32, 16, 512, 64
        q, k, v, prm = workloads.c3_attention(Bt, H, S, D)
        dq, dk, dv = dev(q), dev(k), dev(v)
        if wl.endswith('exp'):
            sm = {'kind': 'exp', 'exp_kq': prm['exp_kq']}
            sm_ref = lambda x_: oracle.softmax_exp(x_, prm['exp_kq'])  # noqa: E731
        else:
            sm = dict(prm['hccs'], kind='hccs')
            sm_ref = lambda x_: oracle.softmax_hccs(x_, sm['B'], sm['S'], sm['Dmax'])  # noqa: E731
        out = torch.empty_like(dq)
        fn = lambda: ops.attention(dq, dk, dv, prm['logit_shift'], 'conv_even', sm, prm['pv_shift'], 'conv_even',  # noqa: E731
                                   out=out)
        fn()
        torch.cuda.synchronize()

        def ref_heads(qs, ks, vs):
            lg = oracle.matmul(qs, ks, prm['logit_shift'], 'conv_even', trans_b=True)
            return oracle.matmul(sm_ref(lg), vs, prm['pv_shift'], 'conv_even')

        hb = (5, slice(2, 6))
        bit_exact = bool(np.array_equal(out[hb].cpu().numpy(), ref_heads(q[hb], k[hb], v[hb])))
        work, bound = 2 * 2.0 * Bt * H * S * S * D, 'mfma'
        samples = Bt
        config = {'workload': f'{wl}: fused attention core (QK^T shift {prm["logit_shift"]} -> softmax -> PV), batch 32 x 16 '
                              'heads, seq 512, head_dim 64, one launch'}
        cpu_fn = lambda: ref_heads(q[0, :4], k[0, :4], v[0, :4])  # noqa: E731
        cpu_work = work * 4 / (Bt * H)
        cpu_samples = 4 / H
        cpu_desc = 'oracle MatMul -> Softmax -> MatMul on 4 of 512 (batch, head) slices'
        metric, unit = 'int8_attention_tops', 'TOP/s'
        kernel = 'attention_kernel'
    elif wl == 'c5_encoder':
        from oracle.graph import run_graph

        batch, seq, hidden, heads, ffn = 64, 128, 768, 12, 3072
        from aie4ml_amd import from_onnx

        onnx_bytes, onnx_cfg, x = workloads.c5_encoder_block_onnx(batch, seq, hidden, heads, ffn, softmax='hccs')
        model = from_onnx(onnx_bytes, onnx_cfg)   # the block as an ONNX Q/DQ model, read by the built-in importer
        model.compile()
        dx = {'x': dev(x)}
        out_name = model.context.ir.logical.output_tensor_names[0]
        fn = lambda: model.execute(dx)  # noqa: E731
        got = fn()[out_name]
        torch.cuda.synchronize()
        nsub = 2
        ref = run_graph(model, oracle, {'x': x[:nsub]})[out_name]
        bit_exact = bool(np.array_equal(got[:nsub].cpu().numpy(), ref))
        rows = batch * seq
        gemm_ops = 2.0 * rows * (hidden * 3 * hidden + hidden * hidden + 2 * hidden * ffn)
        attn_ops = 2 * 2.0 * batch * heads * seq * seq * (hidden // heads)
        work, bound = gemm_ops + attn_ops, 'mfma'
        samples = batch
        config = {'workload': f'c5_encoder: int8 encoder block, hidden {hidden}, {heads} heads, FFN {ffn}, seq {seq}, '
                              f'batch {batch}, HCCS softmax, LayerNorm over {hidden} columns, imported from ONNX Q/DQ, through the graph executor'}
        cpu_fn = lambda: run_graph(model, oracle, {'x': x[:nsub]})  # noqa: E731
        cpu_work = work * nsub / batch
        cpu_desc = f'oracle graph interpreter on {nsub} of {batch} sequences'
        metric, unit = 'int8_encoder_sequences_per_s', 'samples/s'
        kernel = 'whole graph (GEMM kernels dominate)'
        cpu_samples = nsub
    elif wl == 'calib_copy':
        n = 256 << 20
        src = torch.randint(-128, 127, (n,), dtype=torch.int8, device='cuda')
        dst = torch.empty_like(src)
        fn = lambda: torch.add(src, 0, out=dst)  # noqa: E731
        fn()
        torch.cuda.synchronize()
        bit_exact = bool(torch.equal(src, dst))
        work, bound, samples = 2.0 * n, 'hbm', 1
        config = {'workload': 'calib_copy: 256 MiB read + 256 MiB write, one elementwise kernel'}
        metric, unit = 'copy_gbs', 'GB/s'
        kernel = 'elementwise_kernel'
    else:
        sys.exit(f'unknown workload {wl}')


    return dict(wl=wl, fn=fn, fn_cold=fn_cold, bit_exact=bit_exact, work=work, bound=bound, samples=samples, config=config, metric=metric,
                unit=unit, kernel=kernel, extra=extra, cpu_fn=cpu_fn, cpu_work=cpu_work, cpu_desc=cpu_desc,
                cpu_samples=cpu_samples, peak_mfma=peak_mfma, mfma_unit=mfma_unit)


KERNEL_FILE = {'whole graph (GEMM kernels dominate)': 'graph_executor'}


def measure(torch, w, steps, warmup, eager=False, cold_leg=True):
    """Times `steps` launches of a prepared workload; returns (ms per step, value in the workload's unit, roofline)."""
    ms_wall, ms_ev, graphed = _time_gpu(torch, w['fn'], steps, warmup, use_graph=not eager)
    ms = max(ms_wall, ms_ev)
    work, unit = w['work'], w['unit']
    traffic, source = measured_traffic(KERNEL_FILE.get(w['kernel'], w['kernel']), w['wl'])
    if w['bound'] == 'mfma':
        achieved = work / (ms_ev * 1e-3) / 1e12
        roof = {'bound': 'mfma', 'achieved': round(achieved, 3), 'peak': w['peak_mfma'], 'unit': w['mfma_unit'],
                'frac': round(achieved / w['peak_mfma'], 4)}
    else:
        achieved = work / (ms_ev * 1e-3) / 1e9
        roof = {'bound': 'hbm', 'achieved': round(achieved, 2), 'peak': PEAK_HBM_GBS, 'unit': 'GB/s',
                'frac': round(achieved / PEAK_HBM_GBS, 4)}
    roof.update({'traffic': traffic, 'traffic_source': source, 'kernel': w['kernel'], 'kernel_ms': round(ms_ev, 5)})
    cold = w.get('fn_cold')
    if cold_leg and cold is not None and w['bound'] == 'hbm' and steps * cold.bytes_per_launch >= COLD_RING_BYTES // 2:
        # the same launches over a ring of operand copies four times the size of the memory-side cache: nothing is found there
        _, ms_cold, _ = _time_gpu(torch, cold, steps, warmup, use_graph=not eager)
        roof.update({'achieved_operands_from_hbm': round(work / (ms_cold * 1e-3) / 1e9, 2),
                     'frac_operands_from_hbm': round(work / (ms_cold * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                     'kernel_ms_operands_from_hbm': round(ms_cold, 5)})
    if unit in ('TOP/s', 'TFLOP/s'):
        value = work / (ms * 1e-3) / 1e12
    elif unit == 'GB/s':
        value = work / (ms * 1e-3) / 1e9
    else:
        value = w['samples'] / (ms * 1e-3)
    return ms, value, roof, graphed


_BENCH_LIB = None


def _bench_lib():
    """The measurement-aid library (the matrix-core calibration loop), built beside the product library."""
    global _BENCH_LIB
    if _BENCH_LIB is None:
        import ctypes

        from aie4ml_amd import _lib
        from aie4ml_amd.build import BENCH_LIB_PATH

        _lib.load()  # the HIP runtime torch owns is in the process before this library binds to it
        L = ctypes.CDLL(str(BENCH_LIB_PATH))
        L.a4g_calib_mfma_i8_ops.restype = ctypes.c_int64
        L.a4g_calib_mfma_i8_ops.argtypes = [ctypes.c_int, ctypes.c_int]
        L.a4g_calib_mfma_i8.restype = ctypes.c_int
        L.a4g_calib_mfma_i8.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p]
        _BENCH_LIB = L
    return _BENCH_LIB


def calibrate_mfma(torch, blocks_per_cu=2, iters=4096, zero=False):
    """The int8 matrix-core rate this GPU sustains with register-resident operands (no memory traffic), and the clock
    it holds meanwhile: (TOP/s, GHz). ``zero``: all-zero operands, i.e. the same instruction stream at the power the
    multipliers draw when nothing toggles."""
    L = _bench_lib()
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    blocks = cus * blocks_per_cu
    sink = torch.zeros(4, dtype=torch.int32, device='cuda')
    clocks = torch.zeros(2 * blocks, dtype=torch.int64, device='cuda')
    def fn():
        rc = L.a4g_calib_mfma_i8(blocks, iters, int(zero), sink.data_ptr(), clocks.data_ptr(),
                                 torch.cuda.current_stream().cuda_stream)  # the capture stream, when capturing
        if rc != 0:
            raise RuntimeError(f'a4g_calib_mfma_i8 failed with {rc}')

    _, ms_ev, _ = _time_gpu(torch, fn, 20, 5)
    ops_ = int(L.a4g_calib_mfma_i8_ops(blocks, iters))
    c = clocks.cpu().numpy().reshape(-1, 2).astype(np.float64)
    ghz = float(np.median(c[:, 0] / np.maximum(c[:, 1], 1.0)) * 0.1)  # shader ticks per 10 ns tick of the 100 MHz counter
    return ops_ / (ms_ev * 1e-3) / 1e12, ghz, ms_ev, blocks, iters


# the other configurations, timed in the default run after the headline workload (same steps, no CPU leg)
ALSO = ('c1_mlp', 'c1_mlp_stream', 'c3_qk', 'c3_softmax_exp', 'c3_softmax_hccs', 'c3_pv', 'c3_attention_exp', 'c4_add', 'c4_layernorm',
        'c4_add_layernorm', 'c5_encoder', 'c5_proj_qkv', 'c5_proj_out', 'c5_ffn_up', 'c5_ffn_down', 'c5_proj_out_ln')


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument('--gpus', type=int, default=1)
    ap.add_argument('--steps', type=int, default=50)
    ap.add_argument('--warmup', type=int, default=10)
    ap.add_argument('--workload', default='c2_dense')
    ap.add_argument('--no-cpu-baseline', action='store_true')
    ap.add_argument('--only', action='store_true', help='time the named workload alone (the default run of c2_dense '
                    'also times the other configurations and the matrix-core calibration loop)')
    ap.add_argument('--eager', action='store_true', help='time eager launches instead of a replayed HIP graph')
    ap.add_argument('--one-buffer-set', action='store_true', help='skip the second timing of the HBM-bound workloads over a ring '
                    'of operand copies (for a profiler run, whose kernel table should hold one kind of launch)')
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit('bench.py: this build runs on exactly one GPU (every operator is row-independent, so more GPUs '
                 'would each take a slice of the batch with the weights replicated). Use --gpus 1.')

    import torch

    if not torch.cuda.is_available():
        sys.exit('bench.py: no GPU visible')
    from oracle import oracle

    wl = args.workload
    if wl in ('calib_mfma', 'calib_mfma_zero'):
        tops, ghz, ms_ev, blocks, iters = calibrate_mfma(torch, zero=wl == 'calib_mfma_zero')
        print(json.dumps({
            'metric': 'int8_mfma_calibration_tops', 'value': float(f'{tops:.6g}'), 'unit': 'TOP/s', 'n_gpus': 1, 'steps': 20,
            'warmup': 5, 'ms_per_step': round(ms_ev, 5), 'higher_is_better': True, 'scaling': 'weak', 'vs_baseline': None,
            'dtype': 'int8', 'data': 'synthetic',
            'config': {'workload': f'{wl}: {blocks} workgroups x 4 waves x {iters} x 16 v_mfma_i32_32x32x32_i8 on '
                                   f'register-resident {"all-zero" if wl == "calib_mfma_zero" else "pseudo-random"} operands, no memory traffic'},
            'roofline': {'bound': 'mfma', 'achieved': round(tops, 3), 'peak': PEAK_INT8_TOPS, 'unit': 'TOP/s',
                         'frac': round(tops / PEAK_INT8_TOPS, 4), 'traffic': None, 'kernel': 'calib_mfma_i8_kernel',
                         'kernel_ms': round(ms_ev, 5)},
            'clock_ghz_under_mfma_load': round(ghz, 3), 'cpu_baseline': None}), flush=True)
        return

    w = prepare(wl, torch)
    ms, value, roof, graphed = measure(torch, w, args.steps, args.warmup, args.eager, not args.one_buffer_set)
    unit, samples, bit_exact = w['unit'], w['samples'], w['bit_exact']

    cpu = None
    if w['cpu_fn'] is not None and not args.no_cpu_baseline:
        t = _time_cpu(w['cpu_fn'])
        if unit in ('TOP/s', 'TFLOP/s'):
            v = w['cpu_work'] / t / 1e12
        elif unit == 'GB/s':
            v = w['cpu_work'] / t / 1e9
        else:
            v = (w['cpu_samples'] or samples) / t
        cpu = {'value': float(f'{v:.6g}'), 'unit': unit, 'cores': oracle.num_threads(), 'kind': 'port',
               'sample': w['cpu_desc'], 'host_cpus': os.cpu_count()}

    line = {
        'metric': w['metric'], 'value': float(f'{value:.6g}'), 'unit': unit, 'n_gpus': 1, 'steps': args.steps,
        'warmup': args.warmup, 'ms_per_step': round(ms, 5), 'higher_is_better': True, 'scaling': 'weak',
        'vs_baseline': None, 'dtype': {'c2_dense_i16': 'int16', 'c2_dense_i16x16': 'int16', 'c2_dense_bf16': 'bf16', 'c2_dense_fp8': 'fp8'}.get(wl, 'int8'), 'data': 'synthetic', 'config': w['config'],
        'samples_per_s': float(f'{samples / (ms * 1e-3):.6g}'), 'bit_exact': bit_exact,
        'roofline': roof, 'cpu_baseline': cpu, 'launch': 'hip_graph' if graphed else 'eager',
    }
    line.update(w['extra'])
    all_exact = bit_exact

    if wl == 'c2_dense' and not args.only:
        # what this box's matrix cores sustain with no memory traffic, next to the data-sheet peak
        tops, ghz, _, _, _ = calibrate_mfma(torch)
        roof['calibrated_peak'] = round(tops, 1)
        roof['frac_of_calibrated'] = round(roof['achieved'] / tops, 4)
        roof['clock_ghz_under_mfma_load'] = round(ghz, 3)
        # the control: the same register-only loop on all-zero operands (nothing toggles in the multipliers)
        ztops, zghz, _, _, _ = calibrate_mfma(torch, zero=True)
        roof['calibrated_peak_zero_operands'] = round(ztops, 1)
        roof['clock_ghz_zero_operands'] = round(zghz, 3)
        # The same kernel, same shape, all-zero operands: identical instruction stream and memory traffic, but the
        # multipliers do not toggle. The difference to the headline is what the board's power limit takes for
        # full-entropy int8 operands (the clock drops under load; the schedule itself sustains the zero-operand rate).
        z = prepare('c2_dense_zero', torch)
        _, z_value, z_roof, _ = measure(torch, z, args.steps, args.warmup, args.eager)
        roof['zero_operand_tops'] = round(z_roof['achieved'], 1)
        roof['zero_operand_frac'] = z_roof['frac']
        all_exact = all_exact and z['bit_exact']
        del z
        # the other configurations: same timing method and step count, no CPU leg
        del w
        others = {}
        for name in ALSO:
            torch.cuda.empty_cache()
            try:
                o = prepare(name, torch)
                o_ms, o_value, o_roof, _ = measure(torch, o, args.steps, args.warmup, args.eager, not args.one_buffer_set)
                others[name] = {'value': float(f'{o_value:.6g}'), 'unit': o['unit'], 'ms_per_step': round(o_ms, 5),
                                'bit_exact': o['bit_exact'], 'roofline': {k: o_roof[k] for k in ('bound', 'achieved', 'peak', 'unit', 'frac', 'traffic', 'traffic_source', 'kernel',
                                                                   'achieved_operands_from_hbm', 'frac_operands_from_hbm',
                                                                   'kernel_ms_operands_from_hbm') if k in o_roof}}
                all_exact = all_exact and o['bit_exact']
                del o
            except Exception as exc:  # noqa: BLE001
                others[name] = {'error': f'{type(exc).__name__}: {exc}'}
                all_exact = False
        line['workloads'] = others

    print(json.dumps(line), flush=True)
    if not all_exact:
        sys.exit('bench.py: a GPU result differs from the oracle (or a workload failed) — throughput above is INVALID')


if __name__ == '__main__':
    main()
