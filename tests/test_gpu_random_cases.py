"""Seeded random cases through the C ABI against the CPU oracle: shapes drawn around the tile sizes of every kernel
family (so that each dispatch branch is met with ragged edges), pitched and misaligned views, every rounding mode,
operand width and output kind. Bit-exact, like every integer test here."""

import os

import numpy as np
import pytest

torch = pytest.importorskip('torch')

pytestmark = pytest.mark.gpu

MODES = ['floor', 'ceil', 'positive_inf', 'negative_inf', 'symmetric_inf', 'symmetric_zero', 'conv_even', 'conv_odd']
M_CHOICES = [1, 7, 31, 64, 127, 128, 129, 255, 300, 513, 1000, 2049]
N_CHOICES = [1, 17, 32, 64, 96, 128, 192, 200, 256, 384, 768, 1000]
K_CHOICES = [1, 15, 16, 48, 64, 100, 128, 192, 256, 384, 1000, 1024, 512, 640, 768]
EXTRA = int(os.environ.get('A4G_RANDOM_EXTRA', '0'))  # more seeds for a longer hunt


@pytest.fixture(scope='module')
def ops():
    if not torch.cuda.is_available():
        pytest.skip('no GPU')
    from aie4ml_amd import ops as _ops

    return _ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def draw(r, dtype, shape):
    info = np.iinfo(dtype)
    if r.random() < 0.5:   # full range, else a narrow bell (more ties, less saturation)
        return r.integers(info.min, info.max + 1, shape).astype(dtype)
    sigma = (info.max - info.min) / 12.0
    return np.clip(np.rint(r.normal(0, sigma, shape)), info.min, info.max).astype(dtype)


def pitched(t, r):
    """A 2-d tensor as a view into a wider buffer: row pitch and start offset that may break 16-byte alignment."""
    rows, cols = t.shape
    pad, off = int(r.choice([0, 0, 16, 3])), int(r.choice([0, 0, 16, 5]))
    if pad == 0 and off == 0:
        return t
    big = torch.zeros((rows, cols + pad + off), dtype=t.dtype, device=t.device)
    big[:, off:off + cols] = t
    return big[:, off:off + cols]


@pytest.mark.parametrize('seed', range(40 + EXTRA))
def test_dense_random_case(ops, oracle, seed):
    r = np.random.default_rng(1000 + seed)
    a_dtype = [np.int8, np.uint8, np.int16][seed % 3]
    w_dtype = np.int16 if (a_dtype == np.int16 and r.random() < 0.5) else np.int8
    M, N, K = int(r.choice(M_CHOICES)), int(r.choice(N_CHOICES)), int(r.choice(K_CHOICES))
    if seed % 10 == 9:  # large enough for the pipelined kernels of every width
        M, N, K = int(r.choice([2100, 4096])), int(r.choice([3100, 2048])), int(r.choice([256, 384]))
    wide = w_dtype == np.int16
    A, W = draw(r, a_dtype, (M, K)), draw(r, w_dtype, (K, N))
    bias = None if r.random() < 0.2 else r.integers(-2**31 if wide else -2**24, 2**31 if wide else 2**24, N).astype(np.int32)
    top = 40 if wide else 20
    shifts = int(r.integers(0, top)) if r.random() < 0.4 else r.integers(0, top, N).astype(np.int32)
    mode, relu = str(r.choice(MODES)), bool(r.random() < 0.5)
    kind = str(r.choice(['int8', 'uint8', 'int16']))
    p = ops.pack_dense(dev(W), None if bias is None else dev(bias), shifts)
    x = pitched(dev(A), r)
    out_full = torch.full((M, N + 16), 77, dtype={'int8': torch.int8, 'uint8': torch.uint8, 'int16': torch.int16}[kind],
                          device='cuda')
    out = out_full[:, :N] if r.random() < 0.5 else None
    got = ops.dense(x, p, mode, relu=relu, out_kind=kind, out=out)
    exp = oracle.dense(A, W, bias, shifts, mode, relu=relu, out=kind)
    assert np.array_equal(host(got), exp), (seed, a_dtype, w_dtype, M, N, K, mode, kind)
    if out is not None:
        assert bool((out_full[:, N:] == 77).all()), 'wrote beyond the output columns'


@pytest.mark.parametrize('seed', range(30 + EXTRA))
def test_matmul_random_case(ops, oracle, seed):
    r = np.random.default_rng(2000 + seed)
    a_dtype = [np.int8, np.uint8, np.int16][seed % 3]
    b_dtype = np.int16 if (a_dtype == np.int16 and r.random() < 0.5) else np.int8
    lead = [(), (3,), (2, 2)][int(r.integers(0, 3))]
    M, N, K = int(r.choice(M_CHOICES[:9])), int(r.choice(N_CHOICES[:10])), int(r.choice(K_CHOICES[:10]))
    if seed % 10 == 9:
        lead, M, N, K = (2,), 1500, 2048, 256
    trans_b = bool(r.random() < 0.5)
    A = draw(r, a_dtype, lead + (M, K))
    B = draw(r, b_dtype, lead + ((N, K) if trans_b else (K, N)))
    shift = int(r.integers(0, 30 if b_dtype == np.int16 else 20))
    mode, kind = str(r.choice(MODES)), str(r.choice(['int8', 'uint8', 'int16']))
    got = host(ops.matmul(dev(A), dev(B), shift, mode, trans_b=trans_b, out_kind=kind))
    exp = oracle.matmul(A, B, shift, mode, trans_b=trans_b, out=kind)
    assert np.array_equal(got, exp), (seed, a_dtype, b_dtype, lead, M, N, K, trans_b, mode, kind)


@pytest.mark.parametrize('seed', range(24 + EXTRA))
def test_row_operator_random_case(ops, oracle, seed):
    r = np.random.default_rng(3000 + seed)
    rows = int(r.choice([1, 5, 63, 64, 100, 257, 1000]))
    cols = int(r.choice([16, 48, 64, 100, 128, 256, 512, 768, 1024, 2048, 4096, 5000]))
    x = draw(r, np.int8, (rows, cols))
    y = draw(r, np.int8, (rows, cols))
    mode = str(r.choice(MODES))
    which = seed % 4
    if which == 0:
        gmax = int(r.choice([100, 511, 600, 32767]))
        gamma = r.integers(-gmax, gmax + 1, cols).astype(np.int16)
        beta = r.integers(-32768, 32768, cols).astype(np.int16)
        out_shift, gamma_shift, eps = int(r.integers(0, 16)), int(r.integers(0, 16)), int(r.integers(1, 50))
        got = host(ops.layernorm(dev(x), dev(gamma), dev(beta), out_shift, mode, eps_q0=eps, gamma_shift=gamma_shift))
        exp = oracle.layernorm(x, gamma, beta, out_shift, mode, eps_q0=eps, gamma_shift=gamma_shift)
    elif which == 1:
        gamma = r.integers(-300, 301, cols).astype(np.int16)
        beta = r.integers(-32768, 32768, cols).astype(np.int16)
        out_shift = int(r.integers(0, 16))
        got = host(ops.add_layernorm(dev(x), dev(y), dev(gamma), dev(beta), out_shift, mode))
        exp = oracle.add_layernorm(x, y, gamma, beta, out_shift, mode)
    elif which == 2:
        kq = int(r.integers(1, 129))
        kind = str(r.choice(['uint8', 'int16']))
        got = host(ops.softmax_exp(dev(x), kq, out_kind=kind))
        exp = oracle.softmax_exp(x, kq, out=kind)
    else:
        shift = int(r.integers(0, 4))
        got = host(ops.add(dev(x), dev(y), shift, mode))
        exp = oracle.add(x, y, shift, mode)
    assert np.array_equal(got, exp), (seed, which, rows, cols, mode)


HCCS = {32: (255, 4, 60), 64: (255, 3, 80), 128: (255, 2, 126), 256: (127, 1, 126), 512: (60, 1, 59)}


@pytest.mark.parametrize('seed', range(20 + EXTRA // 8))
def test_attention_random_case(ops, oracle, seed):
    """The fused attention core against the oracle's three separate operators."""
    r = np.random.default_rng(4000 + seed)
    sk = int(r.choice([32, 64, 128, 256, 512]))
    sq = int(r.choice([1, 33, 128, 200, 256, 512, 700]))
    lead = [(1, 1), (2, 3), (5, 2)][int(r.integers(0, 3))]
    if sq >= 256 and r.random() < 0.5:
        lead = (16, 16)  # enough work for the 256-row workgroups with the bank-replicated score table
    sigma = float(r.choice([8.0, 24.0, 60.0]))
    g = lambda s: np.clip(np.rint(r.normal(0, sigma, s)), -128, 127).astype(np.int8)  # noqa: E731
    q, k, v = g(lead + (sq, 64)), g(lead + (sk, 64)), g(lead + (sk, 64))
    lshift, oshift = int(r.integers(0, 17)), int(r.integers(0, 12))
    lmode, omode = str(r.choice(MODES)), str(r.choice(MODES))
    if r.random() < 0.5:
        lmode = 'conv_even'
    if seed % 2 == 0:
        sm = {'kind': 'exp', 'exp_kq': int(r.integers(1, 129))}
        logits = oracle.matmul(q, k, lshift, lmode, trans_b=True)
        p = oracle.softmax_exp(logits, sm['exp_kq'])
    else:
        B, S, Dmax = HCCS[sk]
        sm = {'kind': 'hccs', 'B': B, 'S': S, 'Dmax': Dmax}
        logits = oracle.matmul(q, k, lshift, lmode, trans_b=True)
        p = oracle.softmax_hccs(logits, B, S, Dmax, 15, False)
    exp = oracle.matmul(p, v, oshift, omode)
    got = host(ops.attention(dev(q), dev(k), dev(v), lshift, lmode, sm, oshift, omode))
    assert np.array_equal(got, exp), (seed, lead, sq, sk, lshift, lmode, oshift, omode, sm)


@pytest.mark.parametrize('seed', range(24 + EXTRA // 4))
def test_attention_any_key_count_and_head_dimension_random_case(ops, oracle, seed):
    """Head dimensions 16, 32, 64 and 128, any number of keys the fused kernel takes for them, any number of queries."""
    r = np.random.default_rng(4500 + seed)
    d = int(r.choice([16, 32, 64, 128]))
    sk = int(r.integers(1, (256 if d == 128 else 512) + 1))
    if r.random() < 0.3:
        sk = int(r.choice([31, 33, 64, 100, 197, 255, 256]))
    sq = int(r.choice([1, 33, 100, sk, 197, 300]))
    lead = [(1, 1), (2, 3), (5, 2), (3,)][int(r.integers(0, 4))]
    sigma = float(r.choice([8.0, 24.0, 60.0])) * (0.6 if d == 128 else 1.0)
    g = lambda s: np.clip(np.rint(r.normal(0, sigma, s)), -128, 127).astype(np.int8)  # noqa: E731
    q, k, v = g(lead + (sq, d)), g(lead + (sk, d)), g(lead + (sk, d))
    lshift, oshift = int(r.integers(0, 17)), int(r.integers(0, 12))
    lmode, omode = str(r.choice(MODES)), str(r.choice(MODES))
    if r.random() < 0.5:
        lmode = 'conv_even'
    logits = oracle.matmul(q, k, lshift, lmode, trans_b=True)
    B = min(255, 32767 // sk)
    dmax = min(126, B - (256 + sk - 1) // sk)
    if seed % 2 == 0 or dmax < 1:
        sm = {'kind': 'exp', 'exp_kq': int(r.integers(1, 129))}
        p = oracle.softmax_exp(logits, sm['exp_kq'])
    else:
        sm = {'kind': 'hccs', 'B': B, 'S': 1, 'Dmax': dmax}
        p = oracle.softmax_hccs(logits, B, 1, dmax, 15, False)
    exp = oracle.matmul(p, v, oshift, omode)
    got = host(ops.attention(dev(q), dev(k), dev(v), lshift, lmode, sm, oshift, omode))
    assert np.array_equal(got, exp), (seed, lead, sq, sk, d, lshift, lmode, oshift, omode, sm)


@pytest.mark.parametrize('seed', range(24 + EXTRA // 4))
def test_mlp_chain_on_a_long_batch_random_case(ops, oracle, seed):
    """Chains of one to five layers of random widths up to 256 on 4096 samples or more (the matrix-unit form where the
    fragments fit the LDS, the dot-product form otherwise): random shifts, ReLU, signed and unsigned activations, rows at
    random byte offsets, biases that sometimes reach the int32 limits."""
    r = np.random.default_rng(4700 + seed)
    n_layers = int(r.integers(1, 6))
    widths = [int(r.choice([1, 5, 16, 17, 32, 48, 57, 64, 100, 128, 200, 256])) for _ in range(n_layers + 1)]
    batch = 4096 + int(r.integers(0, 200))
    mode = str(r.choice(MODES))
    x_unsigned = bool(r.random() < 0.3)
    x = r.integers(0, 256, (batch, widths[0])).astype(np.uint8) if x_unsigned else r.integers(-128, 128, (batch, widths[0])).astype(np.int8)
    big_bias = r.random() < 0.15
    layers_np, specs = [], []
    for i, (k, n) in enumerate(zip(widths[:-1], widths[1:])):
        W = r.integers(-64, 64, (k, n)).astype(np.int8)
        span = 2**31 - 2**23 if big_bias else 2**13
        b = r.integers(-span, span + 1, n).astype(np.int32) if r.random() < 0.9 else None
        sh = int(r.integers(0, 13)) if r.random() < 0.85 else int(r.integers(13, 32))
        relu = bool(r.random() < 0.6)
        last = i == n_layers - 1
        out = str(r.choice(['int8', 'uint8', 'int16'])) if last else str(r.choice(['int8', 'uint8']))
        layers_np.append((W, b, sh, relu, out))
        specs.append(ops.MlpLayerSpec(ops.pack_dense(dev(W), dev(b) if b is not None else None, sh), sh, relu, out))
    off = int(r.choice([0, 0, 1, 2, 3, 16]))
    buf = torch.zeros(batch * widths[0] + 32, dtype=torch.uint8 if x_unsigned else torch.int8, device='cuda')
    xv = buf[off:off + batch * widths[0]].view(batch, widths[0])
    xv.copy_(torch.from_numpy(x))
    try:
        got = host(ops.mlp(xv, specs, mode))
    except NotImplementedError:
        return  # more weights than the fused kernels hold
    assert np.array_equal(got, oracle.mlp(x, layers_np, mode)), (seed, widths, batch, mode, off, [(l[2], l[3], l[4]) for l in layers_np])


@pytest.mark.parametrize('seed', range(24 + EXTRA // 4))
def test_mlp_chain_with_add_and_layernorm_random_case(ops, oracle, seed):
    """Chains of one to four layers that end in 16 to 256 int8 columns, then the residual Add and the LayerNorm, in one
    launch: random widths, shifts, ReLU, hidden activation signs, batches from one sample to thousands, both rounding
    modes, the LayerNorm's two shifts and its variance floor; the residual is sometimes absent and sometimes a window of
    a wider matrix (16-byte aligned, as the entry point asks)."""
    r = np.random.default_rng(9100 + seed)
    n_layers = int(r.integers(1, 5))
    widths = [int(r.choice([5, 16, 17, 32, 48, 57, 64, 100, 128, 200, 256])) for _ in range(n_layers)]
    widths.append(int(r.choice([16, 32, 48, 64, 80, 128, 144, 256])))
    batch = int(r.choice([1, 31, 32, 33, 500, 1000, 4096 + int(r.integers(0, 100))]))
    mode, lmode = str(r.choice(MODES)), str(r.choice(MODES))
    x = draw(r, np.int8, (batch, widths[0]))
    layers_np, specs = [], []
    for i, (k, n) in enumerate(zip(widths[:-1], widths[1:])):
        W = r.integers(-64, 64, (k, n)).astype(np.int8)
        b = r.integers(-2**13, 2**13 + 1, n).astype(np.int32) if r.random() < 0.9 else None
        sh = int(r.integers(4, 12))
        last = i == n_layers - 1
        relu = bool(r.random() < 0.6) and not last
        out = 'int8' if last else str(r.choice(['int8', 'uint8']))
        layers_np.append((W, b, sh, relu, out))
        specs.append(ops.MlpLayerSpec(ops.pack_dense(dev(W), dev(b) if b is not None else None, sh), sh, relu, out))
    N = widths[-1]
    res = draw(r, np.int8, (batch, N)) if r.random() < 0.8 else None
    dres = None
    if res is not None:
        pad = int(r.choice([0, 16, 48]))
        wide = torch.zeros((batch, N + pad), dtype=torch.int8, device='cuda')
        dres = wide[:, pad:]
        dres.copy_(torch.from_numpy(res))
    gamma = r.integers(-700, 700, N).astype(np.int16) if r.random() < 0.5 else r.integers(-32768, 32768, N).astype(np.int16)
    beta = r.integers(-32768, 32768, N).astype(np.int16)
    out_shift, gamma_shift, eps = int(r.integers(0, 16)), int(r.integers(0, 16)), int(r.choice([1, 3, 100, 1 << 20]))
    try:
        got = host(ops.mlp_add_layernorm(dev(x), specs, dres, dev(gamma), dev(beta), out_shift, mode, lmode, eps_q0=eps,
                                         gamma_shift=gamma_shift))
    except NotImplementedError:
        return  # more weights than the kernel holds
    y = oracle.mlp(x, layers_np, mode)
    if res is not None:
        want = oracle.add_layernorm(y, res, gamma, beta, out_shift, lmode, eps_q0=eps, gamma_shift=gamma_shift)
    else:
        want = oracle.layernorm(y, gamma, beta, out_shift, lmode, eps_q0=eps, gamma_shift=gamma_shift)
    assert np.array_equal(got, want), (seed, widths, batch, mode, lmode, out_shift, gamma_shift, eps, res is not None)


@pytest.mark.parametrize('seed', range(16 + EXTRA // 4))
def test_long_row_operator_random_case(ops, oracle, seed):
    """LayerNorm, fused Add + LayerNorm and both Softmax forms on rows of 4112 to 20 000 columns."""
    r = np.random.default_rng(4900 + seed)
    cols = int(r.choice([4112, 4608, 5120, 6144, 7168, 8192, 8208, 10240, 12288, 16384, 16400, 20000]))
    rows = int(r.integers(1, 80))
    mode = str(r.choice(MODES))
    x = np.clip(np.rint(r.normal(float(r.integers(-20, 20)), float(r.choice([5.0, 25.0, 70.0])), (rows, cols))), -128, 127).astype(np.int8)
    gamma = r.integers(-600, 600, cols).astype(np.int16)
    beta = r.integers(-20000, 20000, cols).astype(np.int16)
    oshift, eps = int(r.integers(0, 9)), int(r.integers(1, 50))
    which = seed % 4
    if which == 0:
        got = host(ops.layernorm(dev(x), dev(gamma), dev(beta), oshift, mode, eps_q0=eps))
        assert np.array_equal(got, oracle.layernorm(x, gamma, beta, oshift, mode, eps_q0=eps)), (seed, cols, rows, mode)
    elif which == 1:
        x2 = np.clip(np.rint(r.normal(0, 40, (rows, cols))), -128, 127).astype(np.int8)
        s_, o_ = ops.add_layernorm(dev(x), dev(x2), dev(gamma), dev(beta), oshift, mode, eps_q0=eps, return_sum=True)
        es, eo = oracle.add_layernorm(x, x2, gamma, beta, oshift, mode, eps_q0=eps, return_sum=True)
        assert np.array_equal(host(s_), es) and np.array_equal(host(o_), eo), (seed, cols, rows, mode)
    elif which == 2:
        kq, out = int(r.integers(1, 129)), str(r.choice(['uint8', 'int16']))
        got = host(ops.softmax_exp(dev(x), kq, out_kind=out))
        assert np.array_equal(got, oracle.softmax_exp(x, kq, out=out)), (seed, cols, rows, kq, out)
    else:
        B = max(2, 32767 // cols)
        if cols * B > 32767:
            return
        got = host(ops.softmax_hccs(dev(x), B, 1, B - 1))
        assert np.array_equal(got, oracle.softmax_hccs(x, B, 1, B - 1)), (seed, cols, rows)


@pytest.mark.parametrize('seed', range(24 + EXTRA))
def test_transposed_lhs_random_case(ops, oracle, seed):
    """MatMul and Dense whose left operand is stored [K][M] (transposed inside the kernel): shapes around the tile
    sizes, M off the dword grid (byte loads), every rounding mode, signed and unsigned operands."""
    r = np.random.default_rng(7000 + seed)
    M, N, K = int(r.choice(M_CHOICES[:10])), int(r.choice(N_CHOICES)), int(r.choice(K_CHOICES))
    a_dtype = np.uint8 if seed % 3 == 2 else np.int8
    mode = str(r.choice(MODES))
    kind = str(r.choice(['int8', 'uint8', 'int16']))
    batch = int(r.choice([1, 2, 3]))
    At = draw(r, a_dtype, (batch, K, M))
    A = np.ascontiguousarray(np.swapaxes(At, -1, -2))
    if seed % 2 == 0:
        trans_b = bool(r.random() < 0.5)
        B = draw(r, np.int8, (batch, N, K) if trans_b else (batch, K, N))
        shift = int(r.integers(0, 20))
        got = ops.matmul(dev(At), dev(B), shift, mode, trans_b=trans_b, out_kind=kind, trans_a=True)
        exp = oracle.matmul(A, B, shift, mode, trans_b=trans_b, out=kind)
    else:
        W = draw(r, np.int8, (K, N))
        bias = r.integers(-2**24, 2**24, N).astype(np.int32)
        shifts = r.integers(0, 20, N).astype(np.int32)
        relu = bool(r.random() < 0.5)
        p = ops.pack_dense(dev(W), dev(bias), shifts)
        got = ops.dense(dev(At), p, mode, relu=relu, out_kind=kind, trans_a=True)
        exp = oracle.dense(A.reshape(-1, K), W, bias, shifts, mode, relu=relu, out=kind).reshape(batch, M, N)
    assert np.array_equal(host(got), exp), (seed, a_dtype, batch, M, N, K, mode, kind)
