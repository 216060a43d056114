"""GPU parity: every operator, through the C ABI, bit-exact against the CPU oracle on seeded inputs.

Sizes are chosen so the oracle finishes in seconds; the full benchmark shapes are covered by row
subsets (every operator is row-independent) in test_gpu_configs.py.
"""

import numpy as np
import pytest

torch = pytest.importorskip('torch')

pytestmark = pytest.mark.gpu

MODES = ['floor', 'ceil', 'positive_inf', 'negative_inf', 'symmetric_inf', 'symmetric_zero', 'conv_even',
         'conv_odd']
REF_MODES = ['floor', 'symmetric_inf', 'conv_even', 'positive_inf']


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


def rng(seed):
    return np.random.default_rng(seed)


def gauss8(r, sigma, shape):
    return np.clip(np.rint(r.normal(0, sigma, shape)), -128, 127).astype(np.int8)


# ---- Add ------------------------------------------------------------------------------------------------

@pytest.mark.parametrize('n', [0, 1, 15, 16, 4096 + 3, 1 << 20])
@pytest.mark.parametrize('dtype', [np.int8, np.uint8])
def test_add_saturating(ops, oracle, n, dtype):
    r = rng(n + 1)
    lo, hi = (0, 256) if dtype == np.uint8 else (-128, 128)
    a = r.integers(lo, hi, n).astype(dtype)
    b = r.integers(lo, hi, n).astype(dtype)
    got = host(ops.add(dev(a), dev(b)))
    assert np.array_equal(got, oracle.add(a, b))


def test_add_exhaustive_pairs(ops, oracle):
    a = np.arange(-128, 128, dtype=np.int8).repeat(256)
    b = np.tile(np.arange(-128, 128, dtype=np.int8), 256)
    assert np.array_equal(host(ops.add(dev(a), dev(b))), oracle.add(a, b))
    au, bu = a.view(np.uint8), b.view(np.uint8)
    assert np.array_equal(host(ops.add(dev(au), dev(bu))), oracle.add(au, bu))


@pytest.mark.parametrize('mode', MODES)
def test_add_shift_and_modes(ops, oracle, mode):
    r = rng(3)
    a = r.integers(-128, 128, 5000).astype(np.int8)
    b = r.integers(-128, 128, 5000).astype(np.int8)
    for shift in (1, 2):
        assert np.array_equal(host(ops.add(dev(a), dev(b), shift, mode)), oracle.add(a, b, shift, mode))
    a16 = r.integers(-32768, 32768, 3001).astype(np.int16)
    b16 = r.integers(-32768, 32768, 3001).astype(np.int16)
    assert np.array_equal(host(ops.add(dev(a16), dev(b16), 0, mode)), oracle.add(a16, b16, 0, mode))


@pytest.mark.parametrize('mode', MODES)
def test_add_every_pair_at_every_shift(ops, oracle, mode):
    """All 65 536 pairs of 8-bit operands, signed and unsigned, at shifts 0 to 9 (the 16-byte-per-lane kernel), and 16-bit
    operands at the ends of their range at shifts 0 to 15."""
    a = np.arange(-128, 128, dtype=np.int8).repeat(256)
    b = np.tile(np.arange(-128, 128, dtype=np.int8), 256)
    au, bu = a.view(np.uint8), b.view(np.uint8)
    for shift in range(0, 10):
        assert np.array_equal(host(ops.add(dev(a), dev(b), shift, mode)), oracle.add(a, b, shift, mode)), (mode, shift)
        assert np.array_equal(host(ops.add(dev(au), dev(bu), shift, mode)), oracle.add(au, bu, shift, mode)), (mode, shift)
    r = rng(5)
    edge = np.array([-32768, -32767, -16385, -16384, -3, -2, -1, 0, 1, 2, 3, 16383, 16384, 32766, 32767], dtype=np.int16)
    a16 = np.concatenate([edge.repeat(len(edge)), r.integers(-32768, 32768, 4001).astype(np.int16)])
    b16 = np.concatenate([np.tile(edge, len(edge)), r.integers(-32768, 32768, 4001).astype(np.int16)])
    for shift in range(0, 16):
        assert np.array_equal(host(ops.add(dev(a16), dev(b16), shift, mode)), oracle.add(a16, b16, shift, mode)), (mode, shift)


def test_add_unaligned_views(ops, oracle):
    r = rng(4)
    a = r.integers(-128, 128, 10007).astype(np.int8)
    b = r.integers(-128, 128, 10007).astype(np.int8)
    ta, tb = dev(a)[3:10003], dev(b)[5:10005]
    got = host(ops.add(ta, tb))
    assert np.array_equal(got, oracle.add(a[3:10003], b[5:10005]))


# ---- transposes ------------------------------------------------------------------------------------------

@pytest.mark.parametrize('dtype', [np.int8, np.int16, np.float32])
@pytest.mark.parametrize('shape', [(1, 1, 1), (3, 64, 64), (2, 5, 300), (1, 129, 65), (7, 100, 1), (1, 1000, 257)])
def test_transpose_entry_point(ops, dtype, shape):
    r = rng(sum(shape))
    x = (r.standard_normal(shape) * 100).astype(dtype)
    got = host(ops.transpose_last2(dev(x)))
    assert got.shape == (shape[0], shape[2], shape[1])
    assert np.array_equal(got, np.swapaxes(x, -1, -2))


def test_transpose_pitched_through_the_c_abi(ops):
    # source rows and destination rows that are slices of wider buffers, batch stride larger than the matrix
    import ctypes
    from aie4ml_amd import _lib
    L = _lib.load()
    r = rng(77)
    src = torch.from_numpy(r.integers(-30000, 30000, (3, 40, 100)).astype(np.int16)).cuda()
    dst = torch.zeros((3, 70, 64), dtype=torch.int16, device='cuda')
    R, C = 33, 61
    rc = L.a4g_transpose(ctypes.c_void_p(src.data_ptr()), 2, 100, 40 * 100, ctypes.c_void_p(dst.data_ptr()), 64, 70 * 64, 3, R, C,
                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    got, s = dst.cpu().numpy(), src.cpu().numpy()
    assert np.array_equal(got[:, :C, :R], np.swapaxes(s[:, :R, :C], -1, -2))
    assert not got[:, C:, :].any() and not got[:, :, R:].any()


# ---- Dense ----------------------------------------------------------------------------------------------

def run_dense(ops, oracle, M, K, N, mode, a_dtype=np.int8, relu=True, per_channel=True, out='int8', bias=True,
              seed=0):
    r = rng(seed)
    if a_dtype == np.uint8:
        A = r.integers(0, 256, (M, K)).astype(np.uint8)
    else:
        A = gauss8(r, 40, (M, K))
    W = gauss8(r, 30, (K, N))
    b = r.integers(-2**14, 2**14, N).astype(np.int32) if bias else None
    if per_channel:
        shifts = r.integers(5, 11, N).astype(np.int32)
    else:
        shifts = np.array([7], dtype=np.int32)
    p = ops.pack_dense(dev(W), dev(b) if bias else None, shifts)
    got = host(ops.dense(dev(A), p, mode, relu=relu, out_kind=out))
    exp = oracle.dense(A, W, b, shifts if per_channel else 7, mode, relu=relu, out=out)
    assert got.dtype == exp.dtype
    assert np.array_equal(got, exp), f'mismatch at {np.argwhere(got != exp)[:5]}'


@pytest.mark.parametrize('shape', [(1, 16, 1), (7, 16, 5), (64, 64, 64), (130, 96, 70), (256, 256, 256),
                                   (300, 128, 260), (33, 1024, 17), (512, 80, 384), (1024, 16, 64)])
def test_dense_shapes_mfma_path(ops, oracle, shape):
    M, K, N = shape
    run_dense(ops, oracle, M, K, N, 'conv_even', seed=M + K + N)


@pytest.mark.parametrize('shape', [(5000, 16, 64), (4096, 64, 32), (4100, 32, 5), (6000, 48, 200), (4500, 192, 256),
                                   (4097, 80, 33), (5000, 20, 64), (5000, 16, 300), (5000, 128, 10), (600, 256, 3)])
@pytest.mark.parametrize('mode', ['conv_even', 'positive_inf', 'symmetric_zero'])
def test_dense_narrow_layer_on_a_long_batch(ops, oracle, shape, mode):
    """Narrow layers with one shift on 4096 rows or more go to the kernel that walks a chain of layers (a chain of one):
    signed and unsigned rows and results, with and without ReLU and bias, rows of 20 bytes (cut out of the dwords that
    cover them); 300 outputs, per-channel shifts and 16-bit results are outside it and take the GEMM kernels, with the
    same integers."""
    M, K, N = shape
    run_dense(ops, oracle, M, K, N, mode, per_channel=False, seed=M + K + N)
    run_dense(ops, oracle, M, K, N, mode, a_dtype=np.uint8, relu=False, per_channel=False, out='uint8', seed=M + K + N + 1)
    run_dense(ops, oracle, M, K, N, mode, relu=False, per_channel=False, bias=False, seed=M + K + N + 2)
    run_dense(ops, oracle, M, K, N, mode, per_channel=True, seed=M + K + N + 3)
    run_dense(ops, oracle, M, K, N, mode, per_channel=False, out='int16', seed=M + K + N + 4)


@pytest.mark.parametrize('shape', [(5000, 192, 576), (700, 80, 384), (130, 16, 1024), (64, 656, 768), (333, 208, 512),
                                   (1, 48, 16), (129, 752, 272)])
@pytest.mark.parametrize('mode', ['conv_even', 'symmetric_inf'])
def test_dense_reduction_that_ends_inside_a_tile(ops, oracle, shape, mode):
    """K a multiple of 16 but not of 128 (192 inputs of a small vision transformer): the weights-in-registers kernel
    takes it, fetching nothing for the part of the last 128-byte tile past K (unsigned activations are biased in
    registers: the chunks past K are left out of that, up to K = 640; 752 keeps the tiled kernel). Per-channel and single
    shifts, every output kind it has."""
    M, K, N = shape
    run_dense(ops, oracle, M, K, N, mode, seed=M + K + N)
    run_dense(ops, oracle, M, K, N, mode, per_channel=False, relu=False, out='uint8', seed=M + K + N + 1)
    run_dense(ops, oracle, M, K, N, mode, a_dtype=np.uint8, seed=M + K + N + 2)
    run_dense(ops, oracle, M, K, N, mode, bias=False, out='int16', seed=M + K + N + 3)


@pytest.mark.parametrize('shape', [(5, 3, 2), (64, 17, 33), (9, 100, 12), (128, 250, 64)])
def test_dense_ragged_k_generic_path(ops, oracle, shape):
    M, K, N = shape
    run_dense(ops, oracle, M, K, N, 'symmetric_inf', seed=M * K + N)
    run_dense(ops, oracle, M, K, N, 'conv_even', a_dtype=np.uint8, seed=M * K + N + 1)


@pytest.mark.parametrize('mode', MODES)
def test_dense_rounding_modes(ops, oracle, mode):
    run_dense(ops, oracle, 96, 64, 96, mode, relu=False, seed=11)
    run_dense(ops, oracle, 96, 64, 96, mode, relu=True, per_channel=False, seed=12)


@pytest.mark.parametrize('out', ['int8', 'uint8', 'int16'])
@pytest.mark.parametrize('a_dtype', [np.int8, np.uint8])
def test_dense_kinds(ops, oracle, out, a_dtype):
    run_dense(ops, oracle, 200, 128, 136, 'conv_even', a_dtype=a_dtype, relu=False, out=out, seed=21)
    run_dense(ops, oracle, 200, 128, 136, 'floor', a_dtype=a_dtype, relu=True, out=out, bias=False, seed=22)


def test_dense_ties_saturation_identity(ops, oracle):
    K = 64
    A = rng(5).integers(-128, 128, (32, K)).astype(np.int8)
    eye = np.eye(K, dtype=np.int8)
    p = ops.pack_dense(dev(eye), None, 0)
    assert np.array_equal(host(ops.dense(dev(A), p, 'floor')), A)
    # W = 0 -> out = srs(bias): exact ties +-2^(s-1), saturation at the int32 extremes
    bias = np.array([64, -64, 63, -65, 192, -192, 2**31 - 1, -2**31] * 8, dtype=np.int32)
    p = ops.pack_dense(dev(np.zeros((K, K), np.int8)), dev(bias), 7)
    for mode in MODES:
        got = host(ops.dense(dev(A), p, mode))
        assert np.array_equal(got, oracle.dense(A, np.zeros((K, K), np.int8), bias, 7, mode)), mode


def test_dense_accumulator_wraps(ops, oracle):
    K, N = 4096, 64
    A = np.full((40, K), 127, np.int8)
    W = np.full((K, N), 127, np.int8)
    bias = np.full(N, 2**31 - 1, np.int32)
    p = ops.pack_dense(dev(W), dev(bias), 12)
    got = host(ops.dense(dev(A), p, 'conv_even'))
    assert np.array_equal(got, oracle.dense(A, W, bias, 12, 'conv_even'))


@pytest.mark.parametrize('mode', MODES)
@pytest.mark.parametrize('shift_set', ['1..15', 'with zero', 'beyond 15'])
def test_dense_requantisation_paths_with_extreme_accumulators(ops, oracle, mode, shift_set):
    # the tiled kernels choose their requantisation form from the shifts of a tile: all within 1..15, some
    # zero, some above 15; the bias puts accumulators next to both int32 extremes and on exact ties
    r = rng(31)
    M, K, N = 160, 128, 192
    A = gauss8(r, 40, (M, K))
    W = gauss8(r, 30, (K, N))
    W[:, ::3] = 0  # those columns give srs(bias) exactly
    lo, hi = {'1..15': (1, 16), 'with zero': (0, 16), 'beyond 15': (0, 25)}[shift_set]
    shifts = r.integers(lo, hi, N).astype(np.int32)
    shifts[:hi - lo] = np.arange(lo, hi)
    bias = r.integers(-2**20, 2**20, N).astype(np.int64)
    bias[0::12] = 2**31 - 1 - r.integers(0, 70000, len(bias[0::12]))
    bias[3::12] = -2**31 + r.integers(0, 70000, len(bias[3::12]))
    bias[6::12] = (1 << shifts[6::12].astype(np.int64)) // 2 * r.choice([-3, -1, 1, 3], len(bias[6::12]))
    bias = bias.astype(np.int32)
    p = ops.pack_dense(dev(W), dev(bias), shifts)
    for out, relu in (('int8', False), ('uint8', False), ('int16', True)):
        got = host(ops.dense(dev(A), p, mode, relu=relu, out_kind=out))
        exp = oracle.dense(A, W, bias, shifts, mode, relu=relu, out=out)
        assert np.array_equal(got, exp), (out, np.argwhere(got != exp)[:5])


def test_dense_width_multiple_of_192(ops, oracle):
    # 56 x 4 = 224 tiles of 128 x 192: the tile shape picked for widths such as 768 on 256 CUs
    run_dense(ops, oracle, 7168, 128, 768, 'conv_even', seed=41)
    run_dense(ops, oracle, 7100, 256, 768, 'symmetric_inf', a_dtype=np.uint8, out='int16', seed=42)


# Reductions of one to six 128-byte tiles with one-byte outputs take the kernel that keeps the weights in registers:
# every reduction length, runs of rows that end in a 64-row step or mid-tile, widths that are not whole column blocks,
# both activation types, and the encoder's projection shapes at full size.
@pytest.mark.parametrize('case', [
    (4096, 128, 4096, 'conv_even', np.int8), (4096, 256, 4096, 'symmetric_inf', np.int8), (4096, 384, 4096, 'symmetric_inf', np.uint8),
    (4096, 512, 4096, 'conv_odd', np.int8), (4096, 640, 4096, 'floor', np.uint8), (4173, 256, 4112, 'conv_even', np.int8),
    (4173, 384, 4112, 'conv_odd', np.uint8), (8192, 768, 2304, 'conv_even', np.int8), (8192, 768, 3072, 'conv_even', np.uint8),
    (8192, 768, 768, 'symmetric_zero', np.int8), (1, 256, 128, 'conv_even', np.int8), (63, 768, 16, 'conv_even', np.int8),
    (65, 640, 144, 'positive_inf', np.uint8), (193, 768, 272, 'negative_inf', np.int8), (2048, 768, 768, 'ceil', np.int8),
    (320, 512, 3088, 'conv_even', np.uint8)], ids=lambda c: 'x'.join(str(v) for v in c[:3]))
def test_dense_short_reduction_weights_in_registers(ops, oracle, case):
    M, K, N, mode, a_dtype = case
    run_dense(ops, oracle, M, K, N, mode, a_dtype=a_dtype, relu=(M % 2 == 0), out='int8' if a_dtype == np.int8 else 'uint8',
              seed=M + K + N)


@pytest.mark.parametrize('mode', MODES)
@pytest.mark.parametrize('shift_set', ['1..15', 'with zero', 'beyond 15', 'large bias'])
def test_dense_short_reduction_requantisation_forms(ops, oracle, mode, shift_set):
    # the quick form (shifts 1..15, start values below 2^30) and the general one, with accumulators on exact ties and, for
    # 'large bias', next to both int32 extremes
    r = rng(57)
    M, K, N = 200, 384, 272
    A = gauss8(r, 40, (M, K))
    W = gauss8(r, 30, (K, N))
    W[:, ::3] = 0  # those columns give srs(bias) exactly
    lo, hi = {'1..15': (1, 16), 'with zero': (0, 16), 'beyond 15': (0, 25), 'large bias': (1, 16)}[shift_set]
    shifts = r.integers(lo, hi, N).astype(np.int32)
    shifts[:hi - lo] = np.arange(lo, hi)
    bias = r.integers(-2**20, 2**20, N).astype(np.int64)
    bias[6::12] = (1 << shifts[6::12].astype(np.int64)) // 2 * r.choice([-3, -1, 1, 3], len(bias[6::12]))
    if shift_set == 'large bias':
        bias[0::12] = 2**31 - 1 - r.integers(0, 70000, len(bias[0::12]))
        bias[3::12] = -2**31 + r.integers(0, 70000, len(bias[3::12]))
        bias[9::12] = r.choice([2**30 - 1, 2**30, 2**30 + 1, -2**30, -2**30 - 1], len(bias[9::12]))
    bias = bias.astype(np.int32)
    p = ops.pack_dense(dev(W), dev(bias), shifts)
    for out, relu in (('int8', False), ('uint8', False), ('int8', True)):
        got = host(ops.dense(dev(A), p, mode, relu=relu, out_kind=out))
        exp = oracle.dense(A, W, bias, shifts, mode, relu=relu, out=out)
        assert np.array_equal(got, exp), (out, np.argwhere(got != exp)[:5])


def test_dense_short_reduction_with_and_without_fragment_order_weights(ops, oracle):
    """a4g_dense_i8_wf with the fragment-order copy (64-row pieces, weights fetched with whole-line loads) and with NULL
    in its place (the kernel that takes them from the row-major weights) give the oracle's integers. Of the four
    256-column blocks only the third needs the general requantisation (a zero shift, a shift of 20 and biases next to
    the int32 limits), so the runs of pieces go from the quick form into the general one and back; 2000 rows end inside a
    piece, 1000 columns inside a column block."""
    import dataclasses
    r = rng(61)
    for (M, K, N, a_dtype, mode) in [(2000, 768, 1000 // 16 * 16, np.int8, 'conv_even'), (4100, 320, 1024, np.uint8, 'symmetric_inf'),
                                     (8192, 768, 2304, np.int8, 'positive_inf'), (70, 128, 1024, np.int8, 'conv_even')]:
        A = r.integers(0, 256, (M, K)).astype(np.uint8) if a_dtype == np.uint8 else gauss8(r, 40, (M, K))
        W = gauss8(r, 30, (K, N))
        shifts = r.integers(1, 16, N).astype(np.int32)
        bias = r.integers(-2**20, 2**20, N).astype(np.int64)
        if N > 600:
            shifts[520] = 0
            shifts[530] = 20
            bias[540], bias[541] = 2**31 - 5, -2**31 + 7
        bias = bias.astype(np.int32)
        p = ops.pack_dense(dev(W), dev(bias), shifts)
        # a layer with a shift outside 1..15 is packed without the fragment-order copy (the other kernel does its general
        # requantisation faster); the copy is made here and forced on the call, which is what a C caller may do
        assert p.wf is None and not p.quick_shifts
        from aie4ml_amd.ops import _rowpack
        _rowpack(p)
        forced = dataclasses.replace(p, quick_shifts=True)
        exp = oracle.dense(A, W, bias, shifts, mode, relu=False, out='int8')
        got = host(ops.dense(dev(A), forced, mode, relu=False, out_kind='int8'))
        assert np.array_equal(got, exp), (M, K, N, np.argwhere(got != exp)[:5])
        got = host(ops.dense(dev(A), p, mode, relu=False, out_kind='int8'))
        assert np.array_equal(got, exp), ('row-major weights', M, K, N, np.argwhere(got != exp)[:5])
    # shifts within 1..15: the copy is made at pack time and used
    shifts = r.integers(1, 16, 1024).astype(np.int32)
    W, A = gauss8(r, 30, (256, 1024)), gauss8(r, 40, (300, 256))
    p = ops.pack_dense(dev(W), None, shifts)
    assert p.wf is not None and p.quick_shifts
    assert np.array_equal(host(ops.dense(dev(A), p, 'conv_even', out_kind='int8')), oracle.dense(A, W, None, shifts, 'conv_even', out='int8'))


# Longer reductions on at most 256 tiles of 128 x 192 take the kernel that splits the reduction inside the workgroup.
@pytest.mark.parametrize('case', [
    (8192, 3072, 768, 'conv_even', np.int8), (8192, 3072, 768, 'conv_even', np.uint8), (8192, 1024, 768, 'symmetric_inf', np.int8),
    (4096, 2048, 1536, 'conv_odd', np.uint8), (1000, 1152, 400, 'symmetric_zero', np.uint8), (129, 1024, 208, 'floor', np.int8),
    (1, 1024, 16, 'conv_even', np.int8), (512, 4096, 1024, 'positive_inf', np.int8), (1024, 8192, 384, 'negative_inf', np.uint8),
    (8192, 896, 768, 'ceil', np.int8)], ids=lambda c: 'x'.join(str(v) for v in c[:3]))
def test_dense_long_reduction_split_in_workgroup(ops, oracle, case):
    M, K, N, mode, a_dtype = case
    run_dense(ops, oracle, M, K, N, mode, a_dtype=a_dtype, relu=(M % 2 == 0), out='int8' if a_dtype == np.int8 else 'uint8',
              seed=M + K + N)


@pytest.mark.parametrize('mode', MODES)
@pytest.mark.parametrize('shift_set', ['1..15', 'beyond 15', 'large bias'])
def test_dense_long_reduction_requantisation_forms(ops, oracle, mode, shift_set):
    r = rng(59)
    M, K, N = 200, 1280, 272
    A = gauss8(r, 40, (M, K))
    W = gauss8(r, 30, (K, N))
    W[:, ::3] = 0  # those columns give srs(bias) exactly
    lo, hi = {'1..15': (1, 16), 'beyond 15': (0, 25), 'large bias': (1, 16)}[shift_set]
    shifts = r.integers(lo, hi, N).astype(np.int32)
    shifts[:hi - lo] = np.arange(lo, hi)
    bias = r.integers(-2**20, 2**20, N).astype(np.int64)
    bias[6::12] = (1 << shifts[6::12].astype(np.int64)) // 2 * r.choice([-3, -1, 1, 3], len(bias[6::12]))
    if shift_set == 'large bias':
        bias[0::12] = 2**31 - 1 - r.integers(0, 70000, len(bias[0::12]))
        bias[3::12] = -2**31 + r.integers(0, 70000, len(bias[3::12]))
        bias[9::12] = r.choice([2**30 - 1, 2**30, 2**30 + 1, -2**30, -2**30 - 1], len(bias[9::12]))
    bias = bias.astype(np.int32)
    p = ops.pack_dense(dev(W), dev(bias), shifts)
    for out, relu in (('int8', False), ('uint8', True)):
        got = host(ops.dense(dev(A), p, mode, relu=relu, out_kind=out))
        exp = oracle.dense(A, W, bias, shifts, mode, relu=relu, out=out)
        assert np.array_equal(got, exp), (out, np.argwhere(got != exp)[:5])


def test_dense_short_reduction_pitched_views(ops, oracle):
    # activations and outputs that are column slices of wider tensors: row pitches larger than the rows
    r = rng(58)
    M, K, N = 700, 256, 400
    A_full = gauss8(r, 40, (M, 3 * K))
    W = gauss8(r, 30, (K, N))
    b = r.integers(-2**14, 2**14, N).astype(np.int32)
    p = ops.pack_dense(dev(W), dev(b), 7)
    y_full = torch.zeros((M, 2 * N), dtype=torch.int8, device='cuda')
    ops.dense(dev(A_full)[:, K:2 * K], p, 'conv_even', relu=True, out=y_full[:, N:])
    exp = oracle.dense(np.ascontiguousarray(A_full[:, K:2 * K]), W, b, 7, 'conv_even', relu=True)
    got = host(y_full)
    assert np.array_equal(got[:, N:], exp)
    assert not got[:, :N].any()


def test_dense_nd_input_and_empty(ops, oracle):
    r = rng(6)
    A = gauss8(r, 30, (3, 5, 32))
    W = gauss8(r, 30, (32, 48))
    p = ops.pack_dense(dev(W), None, 6)
    got = host(ops.dense(dev(A), p, 'conv_even'))
    assert got.shape == (3, 5, 48)
    assert np.array_equal(got.reshape(15, 48), oracle.dense(A.reshape(15, 32), W, None, 6, 'conv_even'))
    empty = ops.dense(torch.empty((0, 32), dtype=torch.int8, device='cuda'), p, 'conv_even')
    assert tuple(empty.shape) == (0, 48)


# ---- MatMul ---------------------------------------------------------------------------------------------

@pytest.mark.parametrize('trans_b', [True, False])
@pytest.mark.parametrize('shape', [((2, 3), 64, 64, 64), ((4,), 128, 96, 32), ((), 130, 70, 48), ((2,), 50, 17, 24),
                                   ((3,), 33, 64, 19)])
def test_matmul_batched(ops, oracle, shape, trans_b):
    lead, M, N, K = shape
    r = rng(M + N + K)
    A = gauss8(r, 24, lead + (M, K))
    B = gauss8(r, 24, lead + ((N, K) if trans_b else (K, N)))
    for mode in ('conv_even', 'symmetric_inf'):
        got = host(ops.matmul(dev(A), dev(B), 6, mode, trans_b=trans_b))
        assert np.array_equal(got, oracle.matmul(A, B, 6, mode, trans_b=trans_b))


@pytest.mark.parametrize('a_dtype', [np.int8, np.uint8])
@pytest.mark.parametrize('trans_b', [True, False])
@pytest.mark.parametrize('shape', [(300, 272, 256), (1000, 128, 768), (129, 400, 1024), (2048, 768, 2048), (65, 16, 128)])
def test_matmul_single_problem_on_the_dense_kernels(ops, oracle, shape, trans_b, a_dtype):
    # one problem with K a multiple of 128: the Dense kernels that requantise from registers (weights in registers up to
    # K = 768, reduction split in the workgroup beyond), here without bias and with a scalar shift
    M, N, K = shape
    r = rng(M + N + K + 5)
    A = r.integers(0, 256, (M, K)).astype(np.uint8) if a_dtype == np.uint8 else gauss8(r, 24, (M, K))
    B = gauss8(r, 24, (N, K) if trans_b else (K, N))
    for mode, shift, kind in (('conv_even', 9, 'int8'), ('symmetric_inf', 0, 'int8'), ('floor', 17, 'uint8')):
        got = host(ops.matmul(dev(A), dev(B), shift, mode, trans_b=trans_b, out_kind=kind))
        assert np.array_equal(got, oracle.matmul(A, B, shift, mode, trans_b=trans_b, out=kind)), (mode, shift, kind)


@pytest.mark.parametrize('a_unsigned', [False, True])
@pytest.mark.parametrize('trans_b', [True, False])
@pytest.mark.parametrize('shape', [((2, 3), 64, 64, 64), ((4,), 128, 96, 32), ((), 130, 70, 48), ((2,), 50, 17, 24),
                                   ((3,), 33, 64, 19), ((), 517, 260, 203), ((2,), 256, 128, 320)])
def test_matmul_transposed_lhs_in_kernel(ops, oracle, shape, trans_b, a_unsigned):
    """The left operand stored as [..., K, M] (matmul.cpp:60-66, TRANSPOSE_A): the kernel transposes its tiles; the
    oracle gets the materialised transpose. Row counts off the dword grid take the byte loads."""
    lead, M, N, K = shape
    r = rng(M + 2 * N + 3 * K)
    At = r.integers(0, 256, lead + (K, M)).astype(np.uint8) if a_unsigned else gauss8(r, 40, lead + (K, M))
    B = gauss8(r, 24, lead + ((N, K) if trans_b else (K, N)))
    A = np.ascontiguousarray(np.swapaxes(At, -1, -2))
    for mode, out in (('conv_even', 'int8'), ('floor', 'int16')):
        got = host(ops.matmul(dev(At), dev(B), 7, mode, trans_b=trans_b, out_kind=out, trans_a=True))
        assert np.array_equal(got, oracle.matmul(A, B, 7, mode, trans_b=trans_b, out=out))


@pytest.mark.parametrize('shape', [((), 64, 64, 64), ((3,), 130, 70, 48), ((2, 2), 33, 19, 100), ((), 1000, 200, 512)])
def test_dense_transposed_lhs_in_kernel(ops, oracle, shape):
    """Dense whose input arrives through a last-two-axes transpose view (dense_bias_relu.cpp:95-101), with bias,
    per-channel shifts and ReLU, signed and unsigned activations."""
    lead, M, N, K = shape
    r = rng(7 * M + N + K)
    W = gauss8(r, 16, (K, N))
    bias = r.integers(-20000, 20000, N).astype(np.int32)
    shifts = r.integers(5, 11, N).astype(np.int32)
    p = ops.pack_dense(dev(W), dev(bias), shifts)
    for unsigned in (False, True):
        Xt = r.integers(0, 256, lead + (K, M)).astype(np.uint8) if unsigned else gauss8(r, 32, lead + (K, M))
        X = np.ascontiguousarray(np.swapaxes(Xt, -1, -2))
        got = host(ops.dense(dev(Xt), p, 'conv_even', relu=True, trans_a=True))
        want = oracle.dense(X.reshape(-1, K), W, bias, shifts, 'conv_even', relu=True).reshape(lead + (M, N))
        assert np.array_equal(got, want)


@pytest.mark.parametrize('wide', [False, True])
@pytest.mark.parametrize('shape', [((), 64, 64, 64), ((3,), 130, 70, 48), ((2,), 33, 19, 100), ((), 1000, 200, 512), ((), 517, 260, 203)])
def test_transposed_lhs_in_kernel_16_bit(ops, oracle, shape, wide):
    """The 16-bit Dense and MatMul entry points read a left operand stored as [..., K, M] themselves (TRANSPOSE_A,
    matmul.cpp:60-66, dense_bias_relu.cpp:95-101): (16, 8) and (16, 16), every leading index, reductions off the tile grid,
    checked against the oracle on the materialised transpose."""
    lead, M, N, K = shape
    r = rng(11 * M + N + K + wide)
    At = r.integers(-32768, 32768, lead + (K, M)).astype(np.int16)
    A = np.ascontiguousarray(np.swapaxes(At, -1, -2))
    W = r.integers(-32768, 32768, (K, N)).astype(np.int16) if wide else gauss8(r, 16, (K, N))
    bias = r.integers(-20000, 20000, N).astype(np.int32)
    shifts = r.integers(17, 23, N).astype(np.int32) if wide else r.integers(9, 15, N).astype(np.int32)
    p = ops.pack_dense(dev(W), dev(bias), shifts)
    for mode, kind, relu in (('conv_even', 'int16', False), ('symmetric_inf', 'int8', True)):
        got = host(ops.dense(dev(At), p, mode, relu=relu, out_kind=kind, trans_a=True))
        want = oracle.dense(A.reshape(-1, K), W, bias, shifts, mode, relu=relu, out=kind).reshape(lead + (M, N))
        assert np.array_equal(got, want), ('dense', mode, kind)
    for trans_b in (True, False):
        B = (r.integers(-32768, 32768, lead + ((N, K) if trans_b else (K, N))).astype(np.int16) if wide
             else gauss8(r, 24, lead + ((N, K) if trans_b else (K, N))))
        sh = 22 if wide else 14
        got = host(ops.matmul(dev(At), dev(B), sh, 'conv_even', trans_b=trans_b, out_kind='int16', trans_a=True))
        assert np.array_equal(got, oracle.matmul(A, B, sh, 'conv_even', trans_b=trans_b, out='int16')), ('matmul', trans_b)


@pytest.mark.parametrize('trans_b', [True, False])
def test_matmul_unsigned_lhs(ops, oracle, trans_b):
    r = rng(9)
    P = r.integers(0, 256, (2, 4, 96, 128)).astype(np.uint8)
    V = gauss8(r, 24, (2, 4) + ((64, 128) if trans_b else (128, 64)))
    for out in ('int8', 'int16'):
        got = host(ops.matmul(dev(P), dev(V), 8, 'conv_even', trans_b=trans_b, out_kind=out))
        assert np.array_equal(got, oracle.matmul(P, V, 8, 'conv_even', trans_b=trans_b, out=out))


@pytest.mark.parametrize('shape', [(300, 200, 256), (128, 128, 64), (33, 17, 48), (70, 130, 1000), (5, 9, 23), (1024, 512, 512)])
def test_dense_int16_activations(ops, oracle, shape):
    """(16, 8) Dense: int16 activations split into byte planes on the matrix cores, acc32 semantics; aligned shapes take
    the tiled kernel, the others the generic one; int16 / int8 / uint8 outputs, ReLU, per-channel shifts, a wrapping bias."""
    M, N, K = shape
    r = rng(M + N + K)
    A = r.integers(-32768, 32768, (M, K)).astype(np.int16)
    A[0, :] = 32767
    A[-1, :] = -32768
    W = gauss8(r, 40, (K, N))
    bias = r.integers(-2**24, 2**24, N).astype(np.int32)
    shifts = r.integers(10, 16, N).astype(np.int32)
    p = ops.pack_dense(dev(W), dev(bias), shifts)
    for mode, relu, kind in (('conv_even', False, 'int16'), ('symmetric_inf', True, 'int8'), ('floor', False, 'uint8')):
        got = host(ops.dense(dev(A), p, mode, relu=relu, out_kind=kind))
        assert np.array_equal(got, oracle.dense(A, W, bias, shifts, mode, relu=relu, out=kind)), (mode, kind)
    big = np.full(N, 2**31 - 77, dtype=np.int32)      # the 32-bit accumulator wraps, as acc32 does
    got = host(ops.dense(dev(np.abs(A)), ops.pack_dense(dev(np.abs(W)), dev(big), 16), 'conv_even', out_kind='int16'))
    assert np.array_equal(got, oracle.dense(np.abs(A), np.abs(W), big, 16, 'conv_even', out='int16'))


@pytest.mark.parametrize('shape', [(2085, 3000, 1024), (4096, 1536, 1152), (2085, 3000, 256)])
def test_dense_int16_activations_large(ops, oracle, shape):
    """Problems with K >= 1024 in whole 128-element tiles and at least 192 tiles of 128 x 256 take the software-pipelined
    kernel that splits the activations into byte planes while staging them, the last shape the tiled one: ragged M and
    N, every rounding mode, the three output kinds, rows at the int16 extremes, a bias that makes the 32-bit
    accumulator wrap."""
    M, N, K = shape
    r = rng(M + N + K)
    A = r.integers(-32768, 32768, (M, K)).astype(np.int16)
    A[0, :], A[1, :], A[-1, :] = 32767, -32768, -32768
    A[2, ::2], A[2, 1::2] = 255, -256          # planes at their own extremes: low byte 0xff / 0x00
    W = gauss8(r, 40, (K, N))
    W[:, 0], W[:, 1] = 127, -128
    bias = r.integers(-2**24, 2**24, N).astype(np.int32)
    shifts = r.integers(10, 16, N).astype(np.int32)
    p = ops.pack_dense(dev(W), dev(bias), shifts)
    dA = dev(A)
    for mode in MODES:
        got = host(ops.dense(dA, p, mode, out_kind='int16'))
        assert np.array_equal(got, oracle.dense(A, W, bias, shifts, mode, out='int16')), mode
    for mode, relu, kind in (('symmetric_inf', True, 'int8'), ('floor', False, 'uint8')):
        got = host(ops.dense(dA, p, mode, relu=relu, out_kind=kind))
        assert np.array_equal(got, oracle.dense(A, W, bias, shifts, mode, relu=relu, out=kind)), (mode, kind)
    big = np.full(N, 2**31 - 77, dtype=np.int32)
    got = host(ops.dense(dev(np.abs(A)), ops.pack_dense(dev(np.abs(W)), dev(big), 16), 'conv_even', out_kind='int16'))
    assert np.array_equal(got, oracle.dense(np.abs(A), np.abs(W), big, 16, 'conv_even', out='int16'))


MODES8 = ('floor', 'ceil', 'positive_inf', 'negative_inf', 'symmetric_inf', 'symmetric_zero', 'conv_even', 'conv_odd')


@pytest.mark.parametrize('shape', [(300, 200, 256), (64, 128, 64), (33, 17, 48), (70, 130, 1000), (5, 9, 23), (512, 384, 512),
                                   (65, 129, 4096)])
def test_dense_int16_activations_int16_weights(ops, oracle, shape):
    # the (16, 16) width combination: 64-bit accumulator, byte-plane matrix-core kernel or the generic one
    M, N, K = shape
    r = rng(M + N + K)
    A = r.integers(-32768, 32768, (M, K)).astype(np.int16)
    W = r.integers(-32768, 32768, (K, N)).astype(np.int16)
    A[0, :], W[:, 0] = -32768, -32768
    if M > 1 and N > 1:
        A[1, :], W[:, 1] = 32767, -32768
    bias = r.integers(-2**31, 2**31, N).astype(np.int32)
    shifts = r.integers(14, 32, N).astype(np.int32)
    p = ops.pack_dense(dev(W), dev(bias), shifts)
    for mode in MODES:
        got = host(ops.dense(dev(A), p, mode, out_kind='int16'))
        assert np.array_equal(got, oracle.dense(A, W, bias, shifts, mode, out='int16')), mode
    p2 = ops.pack_dense(dev(W), None, 40)
    assert np.array_equal(host(ops.dense(dev(A), p2, 'conv_even', relu=True, out_kind='int8')),
                          oracle.dense(A, W, None, 40, 'conv_even', relu=True, out='int8'))
    with pytest.raises(RuntimeError, match='int8 x int16'):
        ops.dense(dev(A.astype(np.int8)), p, 'floor')


@pytest.mark.parametrize('shape', [(2085, 3000, 1024), (1024, 3072, 1152), (1024, 3072, 640)])
def test_dense_int16x16_large(ops, oracle, shape):
    """int16 x int16 problems with K >= 1024 in whole 128-element tiles and at least 192 output tiles of 128 x 128 take
    the software-pipelined kernel (both operands as byte planes in one tile, row sums gathered while the activations
    are split), the last shape the tiled one: ragged edges, every rounding mode, extreme rows and columns, all three
    output kinds."""
    M, N, K = shape
    r = rng(M + N + K)
    A = r.integers(-32768, 32768, (M, K)).astype(np.int16)
    W = r.integers(-32768, 32768, (K, N)).astype(np.int16)
    A[0, :], A[1, :], A[-1, :] = -32768, 32767, -32768
    A[2, ::2], A[2, 1::2] = 255, -256
    W[:, 0], W[:, 1], W[:, -1] = -32768, 32767, -32768
    W[::2, 2], W[1::2, 2] = 255, -256
    bias = r.integers(-2**31, 2**31, N).astype(np.int32)
    shifts = r.integers(14, 32, N).astype(np.int32)
    p = ops.pack_dense(dev(W), dev(bias), shifts)
    dA = dev(A)
    for mode in MODES:
        got = host(ops.dense(dA, p, mode, out_kind='int16'))
        assert np.array_equal(got, oracle.dense(A, W, bias, shifts, mode, out='int16')), mode
    for mode, relu, kind in (('symmetric_inf', True, 'int8'), ('floor', False, 'uint8')):
        got = host(ops.dense(dA, p, mode, relu=relu, out_kind=kind))
        assert np.array_equal(got, oracle.dense(A, W, bias, shifts, mode, relu=relu, out=kind)), (mode, kind)
    p2 = ops.pack_dense(dev(W), None, 40)
    assert np.array_equal(host(ops.dense(dA, p2, 'conv_even', relu=True, out_kind='int8')),
                          oracle.dense(A, W, None, 40, 'conv_even', relu=True, out='int8'))


@pytest.mark.parametrize('b_dtype', [np.int8, np.int16])
@pytest.mark.parametrize('trans_b', [True, False])
@pytest.mark.parametrize('shape', [((2, 3), 64, 64, 64), ((4,), 130, 96, 48), ((), 70, 17, 24), ((2,), 128, 256, 512),
                                   ((3,), 1100, 2000, 256), ((3,), 1100, 2000, 1024), ((1,), 300, 200, 4096)])
def test_matmul_int16_left_operand(ops, oracle, shape, trans_b, b_dtype):
    # the 16-bit width combinations of the dynamic MatMul: int16 x int8 (acc32) and int16 x int16 (acc64)
    lead, M, N, K = shape
    r = rng(M + N + K + int(trans_b))
    A = r.integers(-32768, 32768, lead + (M, K)).astype(np.int16)
    lo, hi = (-128, 128) if b_dtype == np.int8 else (-32768, 32768)
    B = r.integers(lo, hi, lead + ((N, K) if trans_b else (K, N))).astype(b_dtype)
    shift = 14 if b_dtype == np.int8 else 22
    for mode, out in (('conv_even', 'int16'), ('symmetric_inf', 'int8'), ('floor', 'int16')):
        got = host(ops.matmul(dev(A), dev(B), shift, mode, trans_b=trans_b, out_kind=out))
        assert np.array_equal(got, oracle.matmul(A, B, shift, mode, trans_b=trans_b, out=out)), (mode, out)


RAGGED = [(300, 200, 100, 0, 0), (257, 130, 1000, 0, 0), (129, 70, 37, 3, 1), (64, 33, 7, 5, 3), (500, 256, 1030, 2, 2),
          (1, 1, 1, 0, 0), (140, 128, 200, 56, 8),
          # from two K tiles on, rows 4- or 8-byte aligned: descriptor loads by dwords / by 8 bytes, the bytes past K cleared
          (300, 144, 1004, 0, 0), (200, 256, 300, 4, 4), (130, 200, 1001, 7, 0), (260, 130, 2042, 6, 8)]


@pytest.mark.parametrize('case', RAGGED)
@pytest.mark.parametrize('kind', ['int8', 'uint8', 'int16x8', 'int16x16'])
def test_dense_ragged_reduction_and_unaligned_rows(ops, oracle, kind, case):
    """K that is not a multiple of 16 and activation rows that start at any byte (a column window of a wider matrix)
    run on the tiled kernels with loads that stop at the row ends: bytes past K must count as zero whatever lies
    behind them (here: the rest of the wider matrix, filled with extreme values)."""
    M, N, K, extra, off = case
    r = rng(M + N + K + len(kind))
    adt = {'int8': np.int8, 'uint8': np.uint8}.get(kind, np.int16)
    info = np.iinfo(adt)
    wide = np.full((M, off + K + extra), info.max, dtype=adt)
    wide[:, off + K:] = info.min
    A = r.integers(info.min, info.max + 1, (M, K)).astype(adt)
    wide[:, off:off + K] = A
    W = (r.integers(-32768, 32768, (K, N)).astype(np.int16) if kind == 'int16x16' else gauss8(r, 40, (K, N)))
    bias = r.integers(-2**15, 2**15, N).astype(np.int32)
    top = 28 if kind == 'int16x16' else (18 if kind == 'int16x8' else 12)
    shifts = r.integers(top - 5, top + 1, N).astype(np.int32)
    p = ops.pack_dense(dev(W), dev(bias), shifts)
    x = dev(wide)[:, off:off + K]
    out = 'int16' if kind.startswith('int16') else 'int8'
    for mode, relu in (('conv_even', False), ('symmetric_inf', True), ('floor', False)):
        got = host(ops.dense(x, p, mode, relu=relu, out_kind=out))
        assert np.array_equal(got, oracle.dense(A, W, bias, shifts, mode, relu=relu, out=out)), (mode, relu)


@pytest.mark.parametrize('case', [(300, 200, 784, 16), (1, 128, 784, 0), (1000, 130, 800, 240), (700, 520, 272, 112),
                                  (4096, 4096, 1040, 0), (4100, 4096, 528, 16)])
@pytest.mark.parametrize('a_dtype', [np.int8, np.uint8])
def test_dense_reduction_in_whole_chunks_but_not_whole_tiles(ops, oracle, case, a_dtype):
    """Aligned rows, K a multiple of 16 but not of 128, from two K tiles on (a 784-input classifier): the pipelined
    kernel fetches the last tile's missing chunks from outside the operands' descriptors. What lies behind K in a row
    (the rest of a wider matrix, extreme values) and behind the last row must count as zero; 128 x 128 and 256 x 256 tiles."""
    M, N, K, extra = case
    r = rng(M + N + K)
    info = np.iinfo(a_dtype)
    wide = np.full((M, K + extra), info.max, dtype=a_dtype)
    A = r.integers(info.min, info.max + 1, (M, K)).astype(a_dtype)
    wide[:, :K] = A
    W = gauss8(r, 40, (K, N))
    bias = r.integers(-2**15, 2**15, N).astype(np.int32)
    shifts = r.integers(7, 13, N).astype(np.int32)
    p = ops.pack_dense(dev(W), dev(bias), shifts)
    x = dev(wide)[:, :K]
    for mode, relu in (('conv_even', True), ('symmetric_inf', False)):
        got = host(ops.dense(x, p, mode, relu=relu, out_kind='int8'))
        assert np.array_equal(got, oracle.dense(A, W, bias, shifts, mode, relu=relu, out='int8')), (mode, relu)


@pytest.mark.parametrize('trans_b', [True, False])
@pytest.mark.parametrize('a_dtype,b_dtype', [(np.int8, np.int8), (np.uint8, np.int8), (np.int16, np.int8), (np.int16, np.int16)])
@pytest.mark.parametrize('shape', [((2,), 130, 70, 100), ((3,), 64, 129, 37), ((), 257, 200, 1001), ((2, 2), 33, 17, 7)])
def test_matmul_ragged_reduction(ops, oracle, shape, a_dtype, b_dtype, trans_b):
    """The dynamic MatMul with K off the 16-element grid (rows of either operand then start at odd addresses)."""
    lead, M, N, K = shape
    r = rng(M + N + K + int(trans_b))
    ia, ib = np.iinfo(a_dtype), np.iinfo(b_dtype)
    A = r.integers(ia.min, ia.max + 1, lead + (M, K)).astype(a_dtype)
    B = r.integers(ib.min, ib.max + 1, lead + ((N, K) if trans_b else (K, N))).astype(b_dtype)
    shift = {1: 9, 2: 16}[np.dtype(a_dtype).itemsize] + (8 if b_dtype == np.int16 else 0)
    out = 'int16' if a_dtype == np.int16 else 'int8'
    for mode in ('conv_even', 'symmetric_zero', 'ceil'):
        got = host(ops.matmul(dev(A), dev(B), shift, mode, trans_b=trans_b, out_kind=out))
        assert np.array_equal(got, oracle.matmul(A, B, shift, mode, trans_b=trans_b, out=out)), mode


@pytest.mark.parametrize('shape', [((2, 3), 200, 96, 32), ((5,), 129, 544, 64), ((2,), 31, 1056, 96), ((), 512, 512, 128),
                                   ((3,), 1, 32, 64)])
def test_matmul_short_reduction_transposed_rhs(ops, oracle, shape):
    """Q.K^T shapes (K <= 128, right operand transposed): the register-resident kernel, all rounding modes,
    ragged row counts, more than one 512-column chunk, uint8 output."""
    lead, M, N, K = shape
    r = rng(M + N + K)
    A = gauss8(r, 30, lead + (M, K))
    B = gauss8(r, 30, lead + (N, K))
    for i, mode in enumerate(MODES8):
        shift = (0, 3, 6, 9)[i % 4]
        got = host(ops.matmul(dev(A), dev(B), shift, mode, trans_b=True))
        assert np.array_equal(got, oracle.matmul(A, B, shift, mode, trans_b=True)), (mode, shift)
    got = host(ops.matmul(dev(A), dev(B), 5, 'conv_even', trans_b=True, out_kind='uint8'))
    assert np.array_equal(got, oracle.matmul(A, B, 5, 'conv_even', trans_b=True, out='uint8'))


@pytest.mark.parametrize('unsigned', [True, False])
@pytest.mark.parametrize('shape', [((2, 2), 200, 64, 512), ((3,), 129, 32, 128), ((), 300, 128, 256), ((2,), 7, 64, 384)])
def test_matmul_narrow_result(ops, oracle, shape, unsigned):
    """P.V shapes (N in 32/64/128, K a multiple of 128, right operand [K][N]): the kernel that transposes
    V into LDS itself, with int8 and uint8 left operands."""
    lead, M, N, K = shape
    r = rng(M + N + K + unsigned)
    A = r.integers(0, 256, lead + (M, K)).astype(np.uint8) if unsigned else gauss8(r, 30, lead + (M, K))
    B = gauss8(r, 30, lead + (K, N))
    for i, mode in enumerate(MODES8):
        shift = (8, 11, 0, 14)[i % 4]
        got = host(ops.matmul(dev(A), dev(B), shift, mode))
        assert np.array_equal(got, oracle.matmul(A, B, shift, mode)), (mode, shift)


def test_matmul_rejects_bad_arguments(ops):
    a = torch.zeros((2, 16, 16), dtype=torch.int8, device='cuda')
    with pytest.raises(ValueError):
        ops.matmul(a, a.to(torch.uint8), 0)  # RHS must be signed
    with pytest.raises(ValueError):
        ops.matmul(a, a, 40)  # shift out of range


# ---- LayerNorm ------------------------------------------------------------------------------------------

def ln_params(r, cols):
    gamma = r.integers(32, 128, cols).astype(np.int16)
    beta = (r.integers(-16, 17, cols).astype(np.int32) << 10).astype(np.int16)
    return gamma, beta


@pytest.mark.parametrize('cols', [16, 32, 64, 128, 192, 256, 384, 512, 768, 1024, 2048, 4096, 48, 100, 8192])
def test_layernorm_columns(ops, oracle, cols):
    r = rng(cols)
    rows = 37
    x = gauss8(r, 20, (rows, cols)) + np.int8(3)
    gamma, beta = ln_params(r, cols)
    for mode in ('conv_even', 'symmetric_inf'):
        got = host(ops.layernorm(dev(x), dev(gamma), dev(beta), 5, mode))
        assert np.array_equal(got, oracle.layernorm(x, gamma, beta, 5, mode)), (cols, mode)


@pytest.mark.parametrize('mode', MODES)
def test_layernorm_modes_and_shifts(ops, oracle, mode):
    r = rng(31)
    x = gauss8(r, 35, (64, 256))
    gamma = r.integers(-256, 256, 256).astype(np.int16)
    beta = r.integers(-32768, 32768, 256).astype(np.int16)
    for out_shift in (0, 4, 7, 15):
        got = host(ops.layernorm(dev(x), dev(gamma), dev(beta), out_shift, mode, eps_q0=3))
        assert np.array_equal(got, oracle.layernorm(x, gamma, beta, out_shift, mode, eps_q0=3)), (mode, out_shift)


def test_layernorm_degenerate_rows(ops, oracle):
    cols = 1024
    r = rng(32)
    gamma = np.full(cols, 32767, np.int16)  # forces the int16 saturation of inv_std * gamma
    beta = r.integers(-32768, 32768, cols).astype(np.int16)
    x = np.zeros((6, cols), np.int8)
    x[0] = 17                      # constant row: variance 0
    x[1, :cols // 2] = 1           # mean rounds half up
    x[2, :cols // 2] = -1
    x[3] = 127
    x[4] = -128
    x[5, ::2], x[5, 1::2] = 127, -128   # maximum variance
    got = host(ops.layernorm(dev(x), dev(gamma), dev(beta), 5, 'conv_even'))
    assert np.array_equal(got, oracle.layernorm(x, gamma, beta, 5, 'conv_even'))


@pytest.mark.parametrize('mode', MODES)
@pytest.mark.parametrize('gmax', [511, 512])
def test_layernorm_gamma_at_the_float_limit(ops, oracle, mode, gmax):
    """The row kernel normalises in float arithmetic while every |gamma| <= 511 and in integers otherwise; both must
    be the reference's integers. Rows of tiny variance make inv_std16 as large as it gets (products next to 2^24),
    beta spans int16, the shifts span their ranges."""
    cols = 512
    r = rng(gmax)
    gamma = r.integers(-gmax, gmax + 1, cols).astype(np.int16)
    gamma[:4] = (gmax, -gmax, gmax - 1, 1 - gmax)
    beta = r.integers(-32768, 32768, cols).astype(np.int16)
    beta[:4] = (32767, -32768, 32767, -32768)
    x = gauss8(r, 40, (48, cols))
    x[:8] = 0
    x[0, 0] = 1                 # variance rounds to 0: inv_std16 = 32767 at eps 1
    x[1, :3] = (127, -128, 127)
    x[2] = 5
    x[3, ::2], x[3, 1::2] = 127, -128
    x[4, :4] = (-128, -128, 127, 127)
    for gamma_shift, out_shift, eps in ((7, 5, 1), (0, 15, 1), (15, 0, 2), (3, 8, 1), (7, 0, 1)):
        got = host(ops.layernorm(dev(x), dev(gamma), dev(beta), out_shift, mode, eps_q0=eps, gamma_shift=gamma_shift))
        exp = oracle.layernorm(x, gamma, beta, out_shift, mode, eps_q0=eps, gamma_shift=gamma_shift)
        assert np.array_equal(got, exp), (mode, gmax, gamma_shift, out_shift)
    a, b = gauss8(r, 70, (48, cols)), gauss8(r, 70, (48, cols))
    got = host(ops.add_layernorm(dev(a), dev(b), dev(gamma), dev(beta), 6, mode))
    assert np.array_equal(got, oracle.add_layernorm(a, b, gamma, beta, 6, mode)), (mode, gmax)


def test_layernorm_tensor_beyond_two_gib(ops, oracle):
    """The row kernel addresses its tensors with 32-bit offsets; the host splits a larger tensor over several launches.
    Rows on both sides of the split and at the very end are checked."""
    import torch

    cols = 4096
    per_launch = (2**31 - 1) // cols
    rows = per_launch + 5
    r = rng(99)
    gamma, beta = ln_params(r, cols)
    x = torch.randint(-128, 128, (rows, cols), dtype=torch.int8, device='cuda')
    y = ops.layernorm(x, dev(gamma), dev(beta), 5, 'conv_even')
    pick = torch.tensor([0, 1, per_launch - 1, per_launch, per_launch + 1, rows - 1], device='cuda')
    exp = oracle.layernorm(host(x[pick]), gamma, beta, 5, 'conv_even')
    assert np.array_equal(host(y[pick]), exp)
    del x, y
    torch.cuda.empty_cache()


@pytest.mark.parametrize('cols', [4112, 5120, 6144, 7168, 8192, 8208, 12288, 16384, 16400])
@pytest.mark.parametrize('mode', ['conv_even', 'floor', 'symmetric_zero', 'conv_odd'])
def test_layernorm_long_rows(ops, oracle, cols, mode):
    """Rows of thousands of columns (the hidden sizes of large transformers): five to sixteen 16-byte chunks per lane,
    the staged parameters up to 128 KiB of LDS; 16400 is past the row kernel and takes the general one. Both forms of
    the normalisation (float where the mode has one), more rows than one round of waves, a ragged last round."""
    r = rng(cols + 3)
    rows = 301
    x = gauss8(r, 25, (rows, cols)) + np.int8(-5)
    gamma, beta = ln_params(r, cols)
    got = host(ops.layernorm(dev(x), dev(gamma), dev(beta), 6, mode, eps_q0=2))
    assert np.array_equal(got, oracle.layernorm(x, gamma, beta, 6, mode, eps_q0=2)), (cols, mode)


@pytest.mark.parametrize('cols', [4112, 5120, 6144, 7168, 8192, 8208])
@pytest.mark.parametrize('mode', ['conv_even', 'ceil', 'symmetric_inf'])
def test_add_layernorm_long_rows(ops, oracle, cols, mode):
    r = rng(cols + 11)
    a = gauss8(r, 60, (150, cols))
    b = gauss8(r, 60, (150, cols))
    gamma, beta = ln_params(r, cols)
    s, out = ops.add_layernorm(dev(a), dev(b), dev(gamma), dev(beta), 5, mode, return_sum=True)
    es, eo = oracle.add_layernorm(a, b, gamma, beta, 5, mode, return_sum=True)
    assert np.array_equal(host(s), es) and np.array_equal(host(out), eo), (cols, mode)
    assert np.array_equal(host(ops.add_layernorm(dev(a), dev(b), dev(gamma), dev(beta), 5, mode)), eo)


@pytest.mark.parametrize('cols', [64, 128, 192, 384, 768, 1024, 100])
def test_add_layernorm_fused(ops, oracle, cols):
    r = rng(cols + 7)
    a = gauss8(r, 60, (41, cols))
    b = gauss8(r, 60, (41, cols))
    gamma, beta = ln_params(r, cols)
    s, out = ops.add_layernorm(dev(a), dev(b), dev(gamma), dev(beta), 5, 'conv_even', return_sum=True)
    es, eo = oracle.add_layernorm(a, b, gamma, beta, 5, 'conv_even', return_sum=True)
    assert np.array_equal(host(s), es)
    assert np.array_equal(host(out), eo)
    out2 = ops.add_layernorm(dev(a), dev(b), dev(gamma), dev(beta), 5, 'conv_even')
    assert np.array_equal(host(out2), eo)


# ---- Dense + Add + LayerNorm in one launch ---------------------------------------------------------------------

def run_dense_add_layernorm(ops, oracle, M, K, N, seed, dmode='conv_even', lmode='conv_even', shift=9, a_dtype=np.int8,
                            relu=False, residual=True, bias=True, gmax=None, out_shift=5, eps=1, gamma_shift=7, sigma=40):
    """The row-complete kernel against the oracle's dense -> add -> layernorm, operator by operator."""
    r = rng(seed)
    A = r.integers(0, 256, (M, K)).astype(np.uint8) if a_dtype == np.uint8 else gauss8(r, sigma, (M, K))
    W = gauss8(r, 30, (K, N))
    b = r.integers(-2**14, 2**14, N).astype(np.int32) if bias else None
    res = gauss8(r, 50, (M, N)) if residual else None
    if gmax is None:
        gamma, beta = ln_params(r, N)
    else:
        gamma = r.integers(-gmax, gmax + 1, N).astype(np.int16)
        beta = r.integers(-32768, 32768, N).astype(np.int16)
    p = ops.pack_dense(dev(W), dev(b) if bias else None, np.array([shift], np.int32))
    got = host(ops.dense_add_layernorm(dev(A), p, dev(res) if residual else None, dev(gamma), dev(beta), out_shift, dmode,
                                       relu, lmode, eps_q0=eps, gamma_shift=gamma_shift))
    y = oracle.dense(A, W, b, shift, dmode, relu=relu, out='int8')
    if residual:
        exp = oracle.add_layernorm(y, res, gamma, beta, out_shift, lmode, eps_q0=eps, gamma_shift=gamma_shift)
    else:
        exp = oracle.layernorm(y, gamma, beta, out_shift, lmode, eps_q0=eps, gamma_shift=gamma_shift)
    assert np.array_equal(got, exp), f'mismatch at {np.argwhere(got != exp)[:5]}'


@pytest.mark.parametrize('case', [(1, 128, 32), (31, 128, 768), (33, 256, 256), (100, 768, 768), (64, 384, 512),
                                  (257, 512, 384), (96, 640, 160), (40, 3072, 768), (700, 1024, 64), (65, 4096, 96),
                                  # more than 256 workgroups of 32 rows: workgroups of 64 rows, the last one ragged
                                  (8200, 256, 128), (16390, 128, 64), (9216, 768, 768)])
def test_dense_add_layernorm_shapes(ops, oracle, case):
    M, K, N = case
    run_dense_add_layernorm(ops, oracle, M, K, N, seed=sum(case))
    run_dense_add_layernorm(ops, oracle, M, K, N, seed=sum(case) + 1, a_dtype=np.uint8, relu=True, residual=False)


@pytest.mark.parametrize('lmode', MODES)
@pytest.mark.parametrize('dmode', MODES)
def test_dense_add_layernorm_rounding_modes(ops, oracle, dmode, lmode):
    """Every pair of rounding modes: the Dense requantisation takes its rounding bit at run time, the LayerNorm has a
    float form for five of the modes and the integer form for the rest."""
    run_dense_add_layernorm(ops, oracle, 70, 256, 96, seed=MODES.index(dmode) * 8 + MODES.index(lmode), dmode=dmode, lmode=lmode,
                            shift=8, sigma=60)


@pytest.mark.parametrize('shift', [0, 1, 15, 22, 23, 31])
def test_dense_add_layernorm_shifts(ops, oracle, shift):
    """Shifts on both sides of the quick requantisation's limit (22), and none at all."""
    for dmode in ('conv_even', 'symmetric_inf', 'ceil'):
        run_dense_add_layernorm(ops, oracle, 45, 128, 64, seed=shift, dmode=dmode, shift=shift, sigma=90 if shift > 15 else 8)


def test_dense_add_layernorm_large_start_values(ops, oracle):
    """A bias next to the int32 limits sends a wave to the general requantisation (the accumulator wraps like the sum)."""
    r = rng(77)
    M, K, N = 40, 128, 64
    A, W = gauss8(r, 40, (M, K)), gauss8(r, 30, (K, N))
    b = r.integers(-2**14, 2**14, N).astype(np.int32)
    b[3], b[40] = 2**31 - 5, -2**31 + 9
    res = gauss8(r, 50, (M, N))
    gamma, beta = ln_params(r, N)
    p = ops.pack_dense(dev(W), dev(b), np.array([12], np.int32))
    got = host(ops.dense_add_layernorm(dev(A), p, dev(res), dev(gamma), dev(beta), 5, 'conv_even', False, 'conv_even'))
    exp = oracle.add_layernorm(oracle.dense(A, W, b, 12, 'conv_even', out='int8'), res, gamma, beta, 5, 'conv_even')
    assert np.array_equal(got, exp)


@pytest.mark.parametrize('gmax', [511, 512, 32767])
def test_dense_add_layernorm_gamma_at_the_float_limit(ops, oracle, gmax):
    for lmode, gs, osft in (('conv_even', 7, 5), ('floor', 0, 15), ('negative_inf', 15, 0), ('symmetric_zero', 3, 8)):
        run_dense_add_layernorm(ops, oracle, 50, 128, 128, seed=gmax % 97, lmode=lmode, gmax=gmax, gamma_shift=gs, out_shift=osft)


def test_dense_add_layernorm_degenerate_rows(ops, oracle):
    """Constant and extreme rows after the add: zero variance, the int8 limits, maximum variance."""
    M, K, N = 6, 128, 256
    A = np.zeros((M, K), np.int8)          # the Dense output is the requantised bias
    W = np.ones((K, N), np.int8)
    b = np.zeros(N, np.int32)
    res = np.zeros((M, N), np.int8)
    res[0] = 17
    res[1, :N // 2] = 1
    res[2] = 127
    res[3] = -128
    res[4, ::2], res[4, 1::2] = 127, -128
    res[5, 0] = 1
    r = rng(5)
    gamma = np.full(N, 32767, np.int16)
    beta = r.integers(-32768, 32768, N).astype(np.int16)
    p = ops.pack_dense(dev(W), dev(b), np.array([3], np.int32))
    for lmode in ('conv_even', 'symmetric_inf'):
        got = host(ops.dense_add_layernorm(dev(A), p, dev(res), dev(gamma), dev(beta), 5, 'floor', False, lmode))
        exp = oracle.add_layernorm(oracle.dense(A, W, b, 3, 'floor', out='int8'), res, gamma, beta, 5, lmode)
        assert np.array_equal(got, exp), lmode


def test_dense_add_layernorm_pitched_through_the_c_abi(ops, oracle):
    """Activations, residual and result as column windows of wider buffers (row pitches larger than the rows), 64 rows
    per workgroup not taken; what lies outside the result window must stay untouched."""
    import ctypes
    from aie4ml_amd import _lib
    L = _lib.load()
    r = rng(123)
    M, K, N = 77, 256, 96
    lda, ldr, ldo = 320, 128, 160
    abuf = gauss8(r, 40, (M, lda))
    rbuf = gauss8(r, 50, (M, ldr))
    W = gauss8(r, 30, (K, N))
    b = r.integers(-2**14, 2**14, N).astype(np.int32)
    gamma, beta = ln_params(r, N)
    p = ops.pack_dense(dev(W), dev(b), np.array([8], np.int32))
    wf = torch.empty(N * K, dtype=torch.int8, device='cuda')
    vp = lambda t: ctypes.c_void_p(t.data_ptr())  # noqa: E731
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    assert L.a4g_rowpack_weights_i8(vp(p.wt), p.ldwt, N, K, vp(wf), stream) == 0
    da, dr, dg, dbt = dev(abuf), dev(rbuf), dev(gamma), dev(beta)
    out = torch.full((M, ldo), 99, dtype=torch.int8, device='cuda')
    a_win, r_win, o_win = da[:, 64:], dr[:, 32:], out[:, 16:]   # 16-byte aligned windows
    rc = L.a4g_dense_add_layernorm_i8(vp(a_win), 0, lda, vp(wf), None, vp(p.bias), 8, 6, 0, vp(r_win), ldr, vp(dg), vp(dbt),
                                      vp(o_win), ldo, M, N, K, 1, 7, 5, 6, stream)
    assert rc == 0, L.a4g_last_error()
    got = host(out)
    y = oracle.dense(abuf[:, 64:64 + K], W, b, 8, 'conv_even', out='int8')
    exp = oracle.add_layernorm(y, rbuf[:, 32:32 + N], gamma, beta, 5, 'conv_even')
    assert np.array_equal(got[:, 16:16 + N], exp)
    assert (got[:, :16] == 99).all() and (got[:, 16 + N:] == 99).all()


@pytest.mark.parametrize('with_residual', [True, False])
def test_mlp_add_layernorm_pitched_through_the_c_abi(ops, oracle, with_residual):
    """a4g_mlp_add_layernorm_i8 with a residual and a result that are column windows of wider buffers (ld_res > N,
    ldy > N), and with no residual at all: the same bytes as a4g_mlp_i8 -> a4g_add -> a4g_layernorm_i8 through their own
    entry points, and as the oracle; nothing outside the result window is written."""
    import ctypes
    from aie4ml_amd import _lib
    L = _lib.load()
    r = rng(63 + with_residual)
    M, widths = 5000, [48, 128, 64]
    x = gauss8(r, 40, (M, widths[0]))
    specs, layers_np = [], []
    for i in range(len(widths) - 1):
        W = gauss8(r, 30, (widths[i], widths[i + 1]))
        b = r.integers(-2**12, 2**12, widths[i + 1]).astype(np.int32)
        last = i == len(widths) - 2
        specs.append(ops.MlpLayerSpec(ops.pack_dense(dev(W), dev(b), 7), 7, not last, 'int8'))
        layers_np.append((W, b, 7, not last, 'int8'))
    N = widths[-1]
    ldr, ldy = N + 48, N + 32
    rbuf = gauss8(r, 40, (M, ldr))
    gamma = r.integers(32, 128, N).astype(np.int16)
    beta = (r.integers(-16, 17, N).astype(np.int32) << 10).astype(np.int16)
    vp = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None  # noqa: E731
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    arr = ops._mlp_layer_array(specs)
    dx, dr, dg, dbt = dev(x), dev(rbuf), dev(gamma), dev(beta)
    r_win = dr[:, 32:] if with_residual else None
    out = torch.full((M, ldy), 99, dtype=torch.int8, device='cuda')
    rc = L.a4g_mlp_add_layernorm_i8(arr, len(specs), vp(dx), 0, widths[0], vp(r_win), ldr, vp(dg), vp(dbt), vp(out[:, 16:]), ldy, M,
                                    6, 1, 7, 5, 6, stream)
    assert rc == 0, L.a4g_last_error()
    got = host(out)
    # the three entry points it replaces
    y = torch.empty((M, N), dtype=torch.int8, device='cuda')
    assert L.a4g_mlp_i8(arr, len(specs), vp(dx), 0, widths[0], vp(y), N, M, 6, stream) == 0
    ref = torch.empty((M, N), dtype=torch.int8, device='cuda')
    if with_residual:
        res = dr[:, 32:32 + N].contiguous()
        ssum = torch.empty((M, N), dtype=torch.int8, device='cuda')
        assert L.a4g_add(vp(y), vp(res), vp(ssum), M * N, 0, 0, 6, stream) == 0
        y = ssum
    assert L.a4g_layernorm_i8(vp(y), vp(dg), vp(dbt), vp(ref), M, N, 1, 7, 5, 6, stream) == 0
    assert np.array_equal(got[:, 16:16 + N], host(ref))
    yo = oracle.mlp(x, layers_np, 'conv_even')
    want = (oracle.add_layernorm(yo, rbuf[:, 32:32 + N], gamma, beta, 5, 'conv_even') if with_residual
            else oracle.layernorm(yo, gamma, beta, 5, 'conv_even'))
    assert np.array_equal(got[:, 16:16 + N], want)
    assert (got[:, :16] == 99).all() and (got[:, 16 + N:] == 99).all()
    # and through the wrapper, which hands the windows over as they lie
    out2 = torch.full((M, ldy), 77, dtype=torch.int8, device='cuda')
    ops.mlp_add_layernorm(dx, specs, r_win[:, :N] if with_residual else None, dg, dbt, 5, 'conv_even', 'conv_even', out=out2[:, 16:16 + N])
    got2 = host(out2)
    assert np.array_equal(got2[:, 16:16 + N], want) and (got2[:, :16] == 77).all() and (got2[:, 16 + N:] == 77).all()


def test_dense_add_layernorm_refuses_what_it_cannot_take(ops):
    r = rng(9)
    W = gauss8(r, 30, (100, 64))  # K not a multiple of 128
    p = ops.pack_dense(dev(W), None, np.array([7], np.int32))
    assert not ops.dense_add_layernorm_applicable(dev(gauss8(r, 40, (8, 100))), p)
    with pytest.raises(NotImplementedError):
        ops.dense_add_layernorm(dev(gauss8(r, 40, (8, 100))), p, None, dev(np.ones(64, np.int16)), dev(np.zeros(64, np.int16)), 5)


# ---- Softmax --------------------------------------------------------------------------------------------

@pytest.mark.parametrize('cols', [16, 32, 64, 128, 512, 1024, 2048, 4096, 48, 96, 100, 8192])
def test_softmax_exp_columns(ops, oracle, cols):
    r = rng(cols + 100)
    x = gauss8(r, 24, (53, cols))
    for kq in (23, 1, 128):
        got = host(ops.softmax_exp(dev(x), kq))
        assert np.array_equal(got, oracle.softmax_exp(x, kq)), (cols, kq)
    got16 = host(ops.softmax_exp(dev(x), 23, out_kind='int16'))
    assert np.array_equal(got16, oracle.softmax_exp(x, 23, out='int16'))


@pytest.mark.parametrize('cols', [4112, 5120, 8192, 8208, 12288, 16384, 16400])
def test_softmax_long_rows(ops, oracle, cols):
    """Rows beyond 4096 columns: eight or sixteen chunks per lane, scores looked up once for the sum and once more for
    the products; 16400 is past the row kernel. Both score forms, both output types, a clamping and a plain shift."""
    r = rng(cols + 19)
    x = gauss8(r, 30, (131, cols))
    x[5] = -128
    x[6, ::7] = 127
    for kq, inv_shift in ((23, 15), (128, 15), (1, 12)):
        got = host(ops.softmax_exp(dev(x), kq, inv_shift))
        assert np.array_equal(got, oracle.softmax_exp(x, kq, inv_shift)), (cols, kq, inv_shift)
    got16 = host(ops.softmax_exp(dev(x), 23, out_kind='int16'))
    assert np.array_equal(got16, oracle.softmax_exp(x, 23, out='int16'))
    B = 32767 // cols
    if B >= 2:
        got = host(ops.softmax_hccs(dev(x), B, 1, B - 1))
        assert np.array_equal(got, oracle.softmax_hccs(x, B, 1, B - 1)), cols


def test_softmax_exp_every_gap_and_kq(ops, oracle):
    # a row containing every gap 0..255, for every legal KQ: the whole exp table is exercised
    base = np.arange(-128, 128, dtype=np.int8)
    x = np.stack([np.roll(base, i) for i in range(8)])
    for kq in range(1, 129):
        got = host(ops.softmax_exp(dev(x), kq))
        assert np.array_equal(got, oracle.softmax_exp(x, kq)), kq


def test_softmax_exp_special_rows(ops, oracle):
    x = np.zeros((4, 512), np.int8)
    x[1] = -128
    x[2, 7] = 127
    x[2, :7] = -128
    x[3] = 127
    got = host(ops.softmax_exp(dev(x), 23))
    assert np.array_equal(got, oracle.softmax_exp(x, 23))
    assert not got[0].any()  # uniform row of 512: floor(510/512) = 0 -> all zero


@pytest.mark.parametrize('offset', [0, 1, 4, 16])
@pytest.mark.parametrize('cols', [1, 7, 33, 100, 197, 1000, 1001, 1030, 4090, 4095])
def test_softmax_ragged_rows(ops, oracle, cols, offset):
    """Row lengths off the 16-element grid and rows that start at any byte (a window into a larger buffer whose
    surroundings hold the extreme values): the chunked kernel with row-end-aware loads and stores. Both variants,
    both output types; the bytes around the output window must stay untouched."""
    rows = 37
    r = rng(cols * 7 + offset)
    x = gauss8(r, 24, (rows, cols))
    x[0, :] = -128
    x[1, :] = 127
    x[2, -1] = 127
    flat = np.full(offset + rows * cols + 19, 127, dtype=np.int8)
    flat[offset:offset + rows * cols] = x.ravel()
    xin = dev(flat)[offset:offset + rows * cols].reshape(rows, cols)
    for out_kind, tdt in (('uint8', torch.uint8), ('int16', torch.int16)):
        buf = torch.full((offset + rows * cols + 19,), 77, dtype=tdt, device='cuda')
        out = buf[offset:offset + rows * cols].reshape(rows, cols)
        ops.softmax_exp(xin, 23, out_kind=out_kind, out=out)
        got = host(buf)
        assert np.array_equal(got[offset:offset + rows * cols].reshape(rows, cols), oracle.softmax_exp(x, 23, out=out_kind))
        assert (got[:offset] == 77).all() and (got[offset + rows * cols:] == 77).all()
    B = max(1, min(300, 32767 // cols))
    S, Dmax = (1, B - 1) if cols * 1 >= 256 else (0, 0)
    if cols * (B - S * Dmax) >= 256:
        got = host(ops.softmax_hccs(xin, B, S, Dmax))
        assert np.array_equal(got, oracle.softmax_hccs(x, B, S, Dmax))


@pytest.mark.parametrize('cols,params', [(512, (60, 1, 59)), (512, (63, 2, 31)), (128, (255, 2, 126)),
                                         (64, (400, 3, 100)), (96, (33, 1, 30)), (100, (300, 2, 127))])
def test_softmax_hccs(ops, oracle, cols, params):
    B, S, Dmax = params
    r = rng(cols + B)
    x = gauss8(r, 24, (77, cols))
    for out in ('uint8', 'int16'):
        for clb in (False, True):
            got = host(ops.softmax_hccs(dev(x), B, S, Dmax, use_clb=clb, out_kind=out))
            assert np.array_equal(got, oracle.softmax_hccs(x, B, S, Dmax, use_clb=clb, out=out)), (out, clb)
    for inv_shift in (8, 12, 20):
        got = host(ops.softmax_hccs(dev(x), B, S, Dmax, inv_shift=inv_shift))
        assert np.array_equal(got, oracle.softmax_hccs(x, B, S, Dmax, inv_shift=inv_shift)), inv_shift


@pytest.mark.parametrize('cols', [512, 256, 1024, 2048])
def test_softmax_large_inputs(ops, oracle, cols):
    # 2^24 elements: every workgroup makes many passes over its rows
    rows = (1 << 24) // cols + 37
    x = gauss8(rng(cols), 30, (rows, cols))
    x[5, :] = 7                       # uniform row
    x[6, :], x[6, 3] = -128, 127      # widest gap
    assert np.array_equal(host(ops.softmax_exp(dev(x), 23)), oracle.softmax_exp(x, 23))
    if cols == 512:
        assert np.array_equal(host(ops.softmax_hccs(dev(x), 60, 1, 59)), oracle.softmax_hccs(x, 60, 1, 59))


def test_softmax_validation_errors(ops):
    x = torch.zeros((4, 512), dtype=torch.int8, device='cuda')
    with pytest.raises(ValueError, match='cols \\* B <= 32767'):
        ops.softmax_hccs(x, 100, 1, 59)
    with pytest.raises(ValueError, match='B - S\\*Dmax >= 0'):
        ops.softmax_hccs(x, 10, 1, 59)
    with pytest.raises(ValueError, match='EXP_KQ'):
        ops.softmax_exp(x, 200)
    with pytest.raises(ValueError, match='uint8 or int16'):
        ops.softmax_exp(x, 23, out_kind='int8')


# ---- fused MLP ------------------------------------------------------------------------------------------

def make_mlp(ops, r, widths, relu_kind='int8'):
    layers_np, specs = [], []
    for i, (k, n) in enumerate(zip(widths[:-1], widths[1:])):
        W = r.integers(-64, 64, (k, n)).astype(np.int8)
        b = r.integers(-4096, 4097, n).astype(np.int32)
        last = i == len(widths) - 2
        relu = not last
        out = relu_kind if relu else 'int8'
        layers_np.append((W, b, 7, relu, out))
        specs.append(ops.MlpLayerSpec(ops.pack_dense(dev(W), dev(b), 7), 7, relu, out))
    return layers_np, specs


@pytest.mark.parametrize('mode', ['positive_inf', 'symmetric_inf', 'conv_even', 'floor'])
@pytest.mark.parametrize('batch', [1, 63, 1024, 5000])
def test_mlp_fused_matches_layerwise_oracle(ops, oracle, mode, batch):
    r = rng(17)
    x = r.integers(-128, 128, (batch, 16)).astype(np.int8)
    layers_np, specs = make_mlp(ops, r, [16, 64, 32, 32, 5])
    got = host(ops.mlp(dev(x), specs, mode))
    assert np.array_equal(got, oracle.mlp(x, layers_np, mode))


def test_mlp_unsigned_hidden_activations_and_odd_widths(ops, oracle):
    r = rng(18)
    x = r.integers(-128, 128, (300, 23)).astype(np.int8)
    layers_np, specs = make_mlp(ops, r, [23, 50, 7, 256, 3], relu_kind='uint8')
    got = host(ops.mlp(dev(x), specs, 'conv_even'))
    assert np.array_equal(got, oracle.mlp(x, layers_np, 'conv_even'))


def make_mlp_general(ops, r, widths, shifts, relus, outs, bias_span=4096, wmax=64):
    layers_np, specs = [], []
    for (k, n), sh, relu, out in zip(zip(widths[:-1], widths[1:]), shifts, relus, outs):
        W = r.integers(-wmax, wmax, (k, n)).astype(np.int8)
        b = r.integers(-bias_span, bias_span + 1, n).astype(np.int32)
        layers_np.append((W, b, sh, relu, out))
        specs.append(ops.MlpLayerSpec(ops.pack_dense(dev(W), dev(b), sh), sh, relu, out))
    return layers_np, specs


@pytest.mark.parametrize('mode', MODES)
def test_mlp_large_batch_every_rounding_mode(ops, oracle, mode):
    """Batches from 4096 samples run the chain on the matrix units (activations stay in registers from layer to layer):
    the C1 widths, a batch that is not a multiple of 32, every rounding mode."""
    r = rng(31)
    x = r.integers(-128, 128, (4096 + 77, 16)).astype(np.int8)
    layers_np, specs = make_mlp(ops, r, [16, 64, 32, 32, 5])
    assert np.array_equal(host(ops.mlp(dev(x), specs, mode)), oracle.mlp(x, layers_np, mode)), mode


@pytest.mark.parametrize('case', [
    dict(widths=[16, 64, 32, 32, 5], shifts=[7, 0, 15, 3], relus=[1, 1, 0, 0], outs=['int8', 'uint8', 'int8', 'int8']),
    dict(widths=[32, 256, 256, 16], shifts=[9, 10, 8], relus=[1, 1, 0], outs=['uint8', 'uint8', 'int8']),
    dict(widths=[48, 50, 7, 200, 3], shifts=[6, 5, 4, 7], relus=[1, 0, 1, 0], outs=['uint8', 'int8', 'uint8', 'int8']),
    dict(widths=[64, 33, 5], shifts=[8, 20], relus=[0, 0], outs=['int8', 'int16']),
    dict(widths=[16, 32], shifts=[24], relus=[1], outs=['uint8']),
    dict(widths=[128, 96, 64], shifts=[12, 31], relus=[1, 0], outs=['int8', 'int8']),
])
@pytest.mark.parametrize('x_kind', ['int8', 'uint8'])
def test_mlp_large_batch_shapes(ops, oracle, case, x_kind):
    """Widths off the 32-grid (zero-padded fragments), uint8 inputs and hidden activations (biased to int8, corrected by
    the column sums), a 16-bit last layer, shifts from 0 to 31 (the quick requantisation up to 22, the general one
    above), outputs stored as 16-byte pieces (16 columns) and byte by byte (5, 3)."""
    r = rng(len(case['widths']) * 100 + case['widths'][0])
    k0 = case['widths'][0]
    x = (r.integers(0, 256, (5000, k0)).astype(np.uint8) if x_kind == 'uint8' else r.integers(-128, 128, (5000, k0)).astype(np.int8))
    layers_np, specs = make_mlp_general(ops, r, case['widths'], case['shifts'], case['relus'], case['outs'])
    for mode in ('conv_even', 'symmetric_zero'):
        assert np.array_equal(host(ops.mlp(dev(x), specs, mode)), oracle.mlp(x, layers_np, mode)), (case, mode)


def test_mlp_large_batch_large_bias(ops, oracle):
    """Biases next to the int32 limits: the quick requantisation (which adds its rounding constant to the accumulator)
    would overflow, so the kernel notices them while staging and takes the general form."""
    r = rng(41)
    x = r.integers(-128, 128, (4500, 32)).astype(np.int8)
    layers_np, specs = make_mlp_general(ops, r, [32, 64, 16], [9, 9], [1, 0], ['int8', 'int8'], bias_span=2**31 - 2**22)
    assert np.array_equal(host(ops.mlp(dev(x), specs, 'conv_even')), oracle.mlp(x, layers_np, 'conv_even'))


def test_mlp_large_batch_pitched_rows(ops, oracle):
    """Rows of a wider matrix as input (pitch 64, 16 used) and a column window as output."""
    r = rng(43)
    wide = r.integers(-128, 128, (6000, 64)).astype(np.int8)
    layers_np, specs = make_mlp(ops, r, [16, 64, 32, 32, 5])
    dx = dev(wide)[:, :16]
    got = ops.mlp(dx, specs, 'positive_inf')
    assert np.array_equal(host(got), oracle.mlp(np.ascontiguousarray(wide[:, :16]), layers_np, 'positive_inf'))


@pytest.mark.parametrize('widths', [[57, 200, 200, 200, 3], [23, 50, 7, 256, 3], [17, 33, 5], [1, 8, 1], [5, 16]])
def test_mlp_large_batch_rows_at_any_address(ops, oracle, widths):
    """Input rows whose pitch is not a multiple of 16 bytes (57 features), at byte offsets 0, 1 and 3 from an aligned
    address: the kernel cuts each 16-byte piece out of the dwords that cover it; the last row ends inside the last dword
    the kernel may read."""
    r = rng(sum(widths))
    batch = 4096 + widths[0]
    layers_np, specs = make_mlp(ops, r, widths)
    x = r.integers(-128, 128, (batch, widths[0])).astype(np.int8)
    want = oracle.mlp(x, layers_np, 'conv_even')
    for off in (0, 1, 3):
        buf = torch.zeros(batch * widths[0] + 16, dtype=torch.int8, device='cuda')
        xv = buf[off:off + batch * widths[0]].view(batch, widths[0])
        xv.copy_(torch.from_numpy(x))
        assert np.array_equal(host(ops.mlp(xv, specs, 'conv_even')), want), (widths, off)
    # rows of a wider matrix whose pitch is a multiple of 16 while the row length is not a multiple of 4
    wide = torch.zeros((batch, 64), dtype=torch.int8, device='cuda')
    wide[:, :widths[0]] = torch.from_numpy(x)
    assert np.array_equal(host(ops.mlp(wide[:, :widths[0]], specs, 'conv_even')), want), widths


@pytest.mark.parametrize('case', [
    dict(widths=[64, 128, 64], batch=3000, residual=True),
    dict(widths=[64, 64], batch=100, residual=True),
    dict(widths=[128, 256, 128], batch=5000, residual=True),
    dict(widths=[32, 64, 16], batch=33, residual=False),
    dict(widths=[57, 200, 96, 48], batch=700, residual=True),
    dict(widths=[256, 256], batch=1, residual=True),
])
@pytest.mark.parametrize('modes', [('conv_even', 'conv_even'), ('positive_inf', 'floor'), ('symmetric_inf', 'symmetric_zero'),
                                   ('floor', 'conv_odd')])
def test_mlp_add_layernorm(ops, oracle, case, modes):
    """A chain of layers, the residual Add and the LayerNorm in one launch against the oracle's three operators: the two
    halves of a small transformer block (one projection, or the feed-forward pair), widths on and off the 32-grid, uint8
    hidden activations, batches from one sample to thousands, with and without a residual, gamma beyond 511."""
    widths, batch = case['widths'], case['batch']
    r = rng(sum(widths) + batch)
    n_l = len(widths) - 1
    outs = ['uint8' if i % 2 == 0 else 'int8' for i in range(n_l - 1)] + ['int8']
    layers_np, specs = make_mlp_general(ops, r, widths, [int(r.integers(5, 10)) for _ in range(n_l)],
                                        [i < n_l - 1 for i in range(n_l)], outs)
    x = gauss8(r, 40, (batch, widths[0]))
    N = widths[-1]
    res = gauss8(r, 50, (batch, N)) if case['residual'] else None
    gamma = r.integers(-700, 700, N).astype(np.int16)
    beta = r.integers(-30000, 30000, N).astype(np.int16)
    mode, lmode = modes
    got = host(ops.mlp_add_layernorm(dev(x), specs, dev(res) if res is not None else None, dev(gamma), dev(beta), 6, mode,
                                     lmode, eps_q0=3, gamma_shift=8))
    y = oracle.mlp(x, layers_np, mode)
    if res is not None:
        want = oracle.add_layernorm(y, res, gamma, beta, 6, lmode, eps_q0=3, gamma_shift=8)
    else:
        want = oracle.layernorm(y, gamma, beta, 6, lmode, eps_q0=3, gamma_shift=8)
    assert np.array_equal(got, want), (case, modes)


def test_mlp_add_layernorm_refuses_what_it_cannot_take(ops):
    r = rng(77)
    _, specs = make_mlp_general(ops, r, [64, 40], [7], [False], ['int8'])       # 40 columns: not in 16-column pieces
    x = torch.zeros((8, 64), dtype=torch.int8, device='cuda')
    g = torch.ones(40, dtype=torch.int16, device='cuda')
    with pytest.raises(NotImplementedError):
        ops.mlp_add_layernorm(x, specs, None, g, g, 5)
    _, specs = make_mlp_general(ops, r, [64, 32], [7], [False], ['uint8'])      # the sum is defined on int8
    g = torch.ones(32, dtype=torch.int16, device='cuda')
    with pytest.raises(NotImplementedError):
        ops.mlp_add_layernorm(x, specs, None, g, g, 5)


def test_mlp_limits(ops):
    r = rng(19)
    _, specs = make_mlp(ops, r, [16, 300, 4])
    with pytest.raises(NotImplementedError):
        ops.mlp(torch.zeros((4, 16), dtype=torch.int8, device='cuda'), specs, 'floor')


@pytest.mark.parametrize('axis', [-1, 1, 0])
@pytest.mark.parametrize('dtype', [torch.int8, torch.int16])
def test_concat_places_parts_with_the_device_copy(ops, axis, dtype):
    """Concat of producer outputs: every part lands in its slice of one new tensor (last, middle and first axis; parts of
    different extents along it, a non-contiguous part, an empty part)."""
    r = np.random.default_rng(77)
    shapes = {-1: [(3, 5, 7), (3, 5, 1), (3, 5, 0), (3, 5, 16)], 1: [(3, 2, 7), (3, 9, 7)], 0: [(1, 5, 7), (4, 5, 7)]}[axis]
    info = np.iinfo(np.int8 if dtype == torch.int8 else np.int16)
    parts = [r.integers(info.min, info.max + 1, s).astype(info.dtype) for s in shapes]
    dev_parts = [torch.from_numpy(p).cuda() for p in parts]
    dev_parts[0] = torch.from_numpy(np.ascontiguousarray(parts[0].swapaxes(0, 1))).cuda().transpose(0, 1)  # same values, strided
    got = ops.concat(dev_parts, axis)
    np.testing.assert_array_equal(got.cpu().numpy(), np.concatenate(parts, axis=axis))
    with pytest.raises(ValueError, match='share dtype'):
        ops.concat([dev_parts[0], dev_parts[0][:, :1, :1]], axis)
