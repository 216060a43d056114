"""The five baseline configurations at their full sizes. The oracle checks a slice it finishes in seconds; the
rest of each tensor is covered by properties that do not depend on size: independence of rows (a split run equals
the whole run), equality of the fused and the operator-by-operator paths, column-permutation equivariance of
Softmax, shift invariance of LayerNorm."""

import numpy as np
import pytest
import torch

from aie4ml_amd import ops, workloads

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def test_c1_mlp_full_batch(oracle):
    x, layers = workloads.c1_mlp(1024)
    specs = [ops.MlpLayerSpec(ops.pack_dense(dev(W), dev(b), s), s, relu, o) for (W, b, s, relu, o) in layers]
    for mode in ('positive_inf', 'symmetric_inf', 'conv_even'):
        got = ops.mlp(dev(x), specs, mode)
        np.testing.assert_array_equal(got.cpu().numpy(), oracle.mlp(x, layers, mode))
        h = dev(x)
        for (W, b, s, relu, o), sp in zip(layers, specs):       # layer by layer through the GEMM path
            h = ops.dense(h, sp.params, mode, relu=relu, out_kind=o)
        assert torch.equal(h, got)


def test_c2_dense_full_size(oracle):
    M, K, N = 8192, 4096, 4096
    A, W, bias, shifts = workloads.c2_dense(M, K, N)
    p = ops.pack_dense(dev(W), dev(bias), shifts)
    dA = dev(A)
    full = ops.dense(dA, p, 'conv_even', relu=True)
    rows = np.random.default_rng(1).choice(M, 64, replace=False)
    want = oracle.dense(A[rows], W, bias, shifts, 'conv_even', relu=True)
    np.testing.assert_array_equal(full[torch.from_numpy(rows).cuda()].cpu().numpy(), want)
    # rows are independent: ragged pieces (other tile shapes, other kernels) reproduce the whole
    cuts = [0, 100, 1379, 4096, 8191, 8192]
    pieces = [ops.dense(dA[a:b].contiguous(), p, 'conv_even', relu=True) for a, b in zip(cuts[:-1], cuts[1:])]
    assert torch.equal(torch.cat(pieces), full)
    assert int(full.min()) == 0 and int(full.max()) == 127 and len(torch.unique(full)) == 128   # live, ReLU'd, saturating


def test_c3_attention_full_size(oracle):
    B, H, S, D = 32, 16, 512, 64
    q, k, v, prm = workloads.c3_attention(B, H, S, D)
    dq, dk, dv = dev(q), dev(k), dev(v)
    logits = ops.matmul(dq, dk, prm['logit_shift'], 'conv_even', trans_b=True)
    hc = prm['hccs']
    for kind in ('exp', 'hccs'):
        if kind == 'exp':
            probs = ops.softmax_exp(logits, prm['exp_kq'])
            sm = {'kind': 'exp', 'exp_kq': prm['exp_kq']}
            ref_sm = lambda x: oracle.softmax_exp(x, prm['exp_kq'])  # noqa: E731
        else:
            probs = ops.softmax_hccs(logits, hc['B'], hc['S'], hc['Dmax'])
            sm = dict(hc, kind='hccs')
            ref_sm = lambda x: oracle.softmax_hccs(x, hc['B'], hc['S'], hc['Dmax'])  # noqa: E731
        out = ops.matmul(probs, dv, prm['pv_shift'], 'conv_even')
        fused = ops.attention(dq, dk, dv, prm['logit_shift'], 'conv_even', sm, prm['pv_shift'], 'conv_even')
        assert torch.equal(fused, out), kind                                     # one launch == three launches
        hb = (7, slice(3, 5))
        lg = oracle.matmul(q[hb], k[hb], prm['logit_shift'], 'conv_even', trans_b=True)
        np.testing.assert_array_equal(logits[hb].cpu().numpy(), lg)
        np.testing.assert_array_equal(probs[hb].cpu().numpy(), ref_sm(lg))
        np.testing.assert_array_equal(out[hb].cpu().numpy(), oracle.matmul(ref_sm(lg), v[hb], prm['pv_shift'], 'conv_even'))
        # Softmax does not care about the order of a row's columns
        perm = torch.randperm(S, device='cuda', generator=torch.Generator(device='cuda').manual_seed(3))
        sub = logits[:4]
        shuffled = sub[..., perm].contiguous()
        p2 = ops.softmax_exp(shuffled, prm['exp_kq']) if kind == 'exp' else ops.softmax_hccs(shuffled, hc['B'], hc['S'], hc['Dmax'])
        assert torch.equal(p2, probs[:4][..., perm])
        assert int(probs.max()) <= 255 and int(probs.to(torch.int32).sum(-1).max()) <= 255 + S   # floor never overshoots much


def test_c4_add_layernorm_full_size(oracle):
    rows, cols = 16384, 1024
    a, b, gamma, beta, prm = workloads.c4_add_layernorm(rows, cols)
    da, db, dg, dbt = dev(a), dev(b), dev(gamma), dev(beta)
    s = ops.add(da, db)
    y = ops.layernorm(s, dg, dbt, prm['out_shift'], 'conv_even')
    s2, y2 = ops.add_layernorm(da, db, dg, dbt, prm['out_shift'], 'conv_even', return_sum=True)
    assert torch.equal(s, s2) and torch.equal(y, y2)                               # fused == add then LayerNorm
    sub = slice(5000, 5256)
    np.testing.assert_array_equal(s[sub].cpu().numpy(), oracle.add(a[sub], b[sub]))
    np.testing.assert_array_equal(y[sub].cpu().numpy(), oracle.layernorm(oracle.add(a[sub], b[sub]), gamma, beta,
                                                                         prm['out_shift'], 'conv_even'))
    # a row shifted by a constant (no saturation) has the same mean-removed values, variance and output
    small = torch.clamp(da, -100, 100)
    y0 = ops.layernorm(small, dg, dbt, prm['out_shift'], 'conv_even')
    y1 = ops.layernorm(small + 20, dg, dbt, prm['out_shift'], 'conv_even')
    assert torch.equal(y0, y1)
    assert len(torch.unique(y)) > 64


def test_c5_encoder_block_full_batch(oracle):
    from oracle.graph import run_graph

    model, x = workloads.c5_encoder_block(64, 128, 768, 12, 3072, softmax='hccs')
    model.compile()
    name = model.context.ir.logical.output_tensor_names[0]
    fused = model.execute({'x': dev(x)})[name]
    plan = model.context.config['gpu_fusion_plan']
    assert len(plan['attention']) == 1 and len(plan['attention'][0]['heads']) == 12 and len(plan['add_layernorm']) == 2
    # the attention output projection (768 inputs) can normalise its own rows; the second feed-forward projection (3072
    # inputs) is beyond what that kernel wins on and keeps its launches
    assert len(plan['dense_add_layernorm']) == 1
    np.testing.assert_array_equal(fused[:1].cpu().numpy(), run_graph(model, oracle, {'x': x[:1]})[name])
    model.context.config['gpu_fusion_plan'] = {}
    assert torch.equal(model.execute({'x': dev(x)})[name], fused)                   # operator by operator, all 64 sequences
    model.context.config['gpu_fusion_plan'] = plan
    halves = [model.execute({'x': dev(x[i:i + 32])})[name] for i in (0, 32)]
    assert torch.equal(torch.cat(halves), fused)                                      # sequences are independent
    # two sequences are too few rows for the row-complete projection to pay: the executor runs its two launches instead
    assert torch.equal(model.execute({'x': dev(x[:2])})[name], fused[:2])
