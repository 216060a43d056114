"""GPU parity of the floating-point compute path (bfloat16 / float32 Dense, MatMul, Add) through the C ABI.

The oracle accumulates exactly and rounds once; the kernels accumulate in float32 in matrix-core order. Two
bars, both written out below: the tolerances of the reference's own float test (tests/test_float_sim.py:81-87:
rtol 1e-2 / atol 5e-2 for bfloat16, rtol 1e-3 / atol 1e-3 for float32), and the tighter forward error bound
of a float32 dot product plus one rounding to the output format.
"""

import numpy as np
import pytest

torch = pytest.importorskip('torch')

pytestmark = pytest.mark.gpu

# fp8: the reference has no fp8 test; the bar is one unit in the last place (relative 2^-3) of the output format
REF_TOL = {'bfloat16': (1e-2, 5e-2), 'float32': (1e-3, 1e-3), 'fp8_e4m3': (2.0 ** -3, 2.0 ** -9)}
TORCH_DT = {'bfloat16': torch.bfloat16, 'float32': torch.float32, 'fp8_e4m3': torch.float8_e4m3fn}
HALF_ULP = {'bfloat16': 2.0 ** -8, 'float32': 2.0 ** -24, 'fp8_e4m3': 2.0 ** -4}
FORMATS = ['bfloat16', 'float32', 'fp8_e4m3']


@pytest.fixture(scope='module')
def ops():
    if not torch.cuda.is_available():
        pytest.skip('no GPU')
    from aie4ml_amd import ops as _ops

    return _ops


def operand(r, shape, fmt, oracle, scale=1.0):
    x = (r.normal(0, scale, shape)).astype(np.float32)
    if fmt == 'fp8_e4m3':
        return oracle.fp8_quantize(x)
    return oracle.bf16_truncate(x) if fmt == 'bfloat16' else x


def dev(a, fmt):
    if fmt == 'fp8_e4m3':  # by code: the values are exact in the format, the codes are the oracle's
        from oracle import oracle as o
        return torch.from_numpy(o.fp8_encode(np.ascontiguousarray(a, dtype=np.float32))).cuda().view(torch.float8_e4m3fn)
    return torch.from_numpy(np.ascontiguousarray(a, dtype=np.float32)).cuda().to(TORCH_DT[fmt])


def host(t):
    torch.cuda.synchronize()
    return t.float().cpu().numpy()


def check(got, exp, fmt, k, abs_products):
    rtol, atol = REF_TOL[fmt]
    np.testing.assert_allclose(got, exp, rtol=rtol, atol=atol)
    # float32 accumulation of k terms, any order: |err| <= k * 2^-24 * sum|a||w|; then one rounding of the
    # result (half an ulp), which can land on the neighbouring value when the two sums straddle a tie
    bound = 2.0 * HALF_ULP[fmt] * np.abs(exp) + (k + 2) * 2.0 ** -24 * abs_products + 1e-30
    if fmt == 'fp8_e4m3':
        bound = bound + 2.0 ** -9  # one step of the subnormal range
    assert np.all(np.abs(got.astype(np.float64) - exp.astype(np.float64)) <= bound)


@pytest.mark.parametrize('fmt', FORMATS)
@pytest.mark.parametrize('shape', [(4, 32, 32), (4, 32, 16), (7, 19, 5), (130, 96, 70), (256, 256, 256), (300, 128, 260),
                                   (512, 1024, 384), (1024, 64, 64)])
def test_dense_float(ops, oracle, fmt, shape):
    M, K, N = shape
    r = np.random.default_rng(M + K + N)
    A = operand(r, (M, K), fmt, oracle, 2.0)
    W = operand(r, (K, N), fmt, oracle, 0.1)
    b = r.normal(0, 0.05, N).astype(np.float32)
    absprod = np.abs(A).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(b)
    p = ops.pack_dense_float(dev(W, fmt), torch.from_numpy(b).cuda())
    for relu in (False, True):
        got = host(ops.dense_float(dev(A, fmt), p, relu=relu))
        check(got, oracle.dense_float(A, W, b, relu=relu, fmt=fmt), fmt, K, absprod)
    p0 = ops.pack_dense_float(dev(W, fmt), None)
    check(host(ops.dense_float(dev(A, fmt), p0)), oracle.dense_float(A, W, None, fmt=fmt), fmt, K, absprod)


@pytest.mark.parametrize('fmt', FORMATS)
def test_dense_float_exact_cases(ops, oracle, fmt):
    # small integers: every product and partial sum is exact in float32, so any order gives the same bits
    r = np.random.default_rng(5)
    amax, wmax = (2, 1) if fmt == 'fp8_e4m3' else (8, 4)  # fp8: keep every sum below the largest value, 448
    A = r.integers(-amax, amax + 1, (200, 128)).astype(np.float32)
    W = r.integers(-wmax, wmax + 1, (128, 192)).astype(np.float32)
    b = r.integers(-16, 17, 192).astype(np.float32)
    p = ops.pack_dense_float(dev(W, fmt), torch.from_numpy(b).cuda())
    got = host(ops.dense_float(dev(A, fmt), p, relu=True))
    assert np.array_equal(got, oracle.dense_float(A, W, b, relu=True, fmt=fmt))
    # identity weights return the input; empty batch
    eye = np.eye(64, dtype=np.float32)
    X = operand(r, (33, 64), fmt, oracle)
    pe = ops.pack_dense_float(dev(eye, fmt), None)
    assert np.array_equal(host(ops.dense_float(dev(X, fmt), pe)), X)
    empty = ops.dense_float(torch.empty((0, 64), dtype=TORCH_DT[fmt], device='cuda'), pe)
    assert tuple(empty.shape) == (0, 64)


@pytest.mark.parametrize('fmt', FORMATS)
@pytest.mark.parametrize('trans_b', [True, False])
@pytest.mark.parametrize('shape', [((2, 3), 64, 64, 64), ((4,), 128, 96, 32), ((), 130, 70, 48), ((2,), 50, 17, 24),
                                   ((3,), 256, 128, 256)])
def test_matmul_float(ops, oracle, fmt, trans_b, shape):
    lead, M, K, N = shape
    r = np.random.default_rng(M * 3 + K + N)
    A = operand(r, lead + (M, K), fmt, oracle)
    B = operand(r, lead + ((N, K) if trans_b else (K, N)), fmt, oracle)
    got = host(ops.matmul_float(dev(A, fmt), dev(B, fmt), trans_b=trans_b))
    Bm = np.swapaxes(B, -1, -2) if trans_b else B
    absprod = np.abs(A).astype(np.float64) @ np.abs(Bm).astype(np.float64)
    check(got, oracle.matmul_float(A, B, trans_b=trans_b, fmt=fmt), fmt, K, absprod)


@pytest.mark.parametrize('fmt', FORMATS)
@pytest.mark.parametrize('shape', [((), 64, 64, 64), ((3,), 130, 70, 48), ((2,), 50, 17, 24), ((), 300, 256, 128)])
def test_transposed_lhs_in_kernel_float(ops, oracle, fmt, shape):
    """Float Dense and MatMul read a left operand stored as [..., K, M] themselves (TRANSPOSE_A, matmul.cpp:60-66,
    dense_bias_relu.cpp:95-101); same tolerances as the untransposed operand, against the oracle on the materialised
    transpose."""
    lead, M, K, N = shape
    r = np.random.default_rng(M * 5 + K + N)
    At = operand(r, lead + (K, M), fmt, oracle)
    A = np.ascontiguousarray(np.swapaxes(At, -1, -2))
    W = operand(r, (K, N), fmt, oracle, 0.1)
    b = r.normal(0, 0.05, N).astype(np.float32)
    p = ops.pack_dense_float(dev(W, fmt), torch.from_numpy(b).cuda())
    got = host(ops.dense_float(dev(At, fmt), p, relu=True, trans_a=True))
    absprod = np.abs(A).astype(np.float64) @ np.abs(W).astype(np.float64) + np.abs(b)
    want = oracle.dense_float(A.reshape(-1, K), W, b, relu=True, fmt=fmt).reshape(lead + (M, N))
    check(got, want, fmt, K, absprod)
    for trans_b in (True, False):
        B = operand(r, lead + ((N, K) if trans_b else (K, N)), fmt, oracle)
        got = host(ops.matmul_float(dev(At, fmt), dev(B, fmt), trans_b=trans_b, trans_a=True))
        Bm = np.swapaxes(B, -1, -2) if trans_b else B
        absprod = np.abs(A).astype(np.float64) @ np.abs(Bm).astype(np.float64)
        check(got, oracle.matmul_float(A, B, trans_b=trans_b, fmt=fmt), fmt, K, absprod)


@pytest.mark.parametrize('fmt', FORMATS)
def test_add_float(ops, oracle, fmt):
    r = np.random.default_rng(9)
    a = operand(r, (5, 1001), fmt, oracle, 3.0)
    b = operand(r, (5, 1001), fmt, oracle, 3.0)
    got = host(ops.add_float(dev(a, fmt), dev(b, fmt)))
    assert np.array_equal(got, oracle.add_float(a, b, fmt))  # one exact sum, one rounding: bit-exact


def test_float_argument_errors(ops):
    w = torch.zeros((8, 8), dtype=torch.float16, device='cuda')
    with pytest.raises(NotImplementedError):
        ops.pack_dense_float(w, None)
    p = ops.pack_dense_float(torch.zeros((8, 8), dtype=torch.bfloat16, device='cuda'), None)
    with pytest.raises(ValueError, match='share float precision'):
        ops.dense_float(torch.zeros((2, 8), dtype=torch.float32, device='cuda'), p)
    with pytest.raises(ValueError, match='features'):
        ops.dense_float(torch.zeros((2, 9), dtype=torch.bfloat16, device='cuda'), p)
