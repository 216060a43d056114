"""a4g_matmul_i8_static, the MatMul entry point that allocates nothing: its repacked right operand and column sums
live in a fixed device array inside the library instead of a caller's workspace. Checked through the C ABI against
a4g_matmul_i8 (same kernels, caller workspace) and the oracle, bit for bit, on two calls in a row — the second with a
smaller input, so stale contents of the shared array from the first call would show."""

import numpy as np
import pytest

torch = pytest.importorskip('torch')
pytestmark = pytest.mark.gpu

STATIC_MAX = 16 << 20


def _call(lib_fn, a, b, out, shift, mode, trans_b, out_kind, extra):
    from aie4ml_amd import _lib

    batch, M, K = a.shape
    N = b.shape[1] if trans_b else b.shape[2]
    akind = _lib.KIND['uint8' if a.dtype == torch.uint8 else 'int8']
    st = lib_fn(a.data_ptr(), akind, 0, K, M * K, b.data_ptr(), b.shape[2], b.shape[1] * b.shape[2], int(trans_b), out.data_ptr(), N,
                M * N, batch, M, N, K, shift, _lib.ROUNDING[mode], _lib.KIND[out_kind], *extra,
                torch.cuda.current_stream().cuda_stream)
    _lib.check(st)


def _case(seed, batch, M, N, K, a_unsigned, trans_b, shift, mode, out_kind):
    r = np.random.default_rng(seed)
    a = r.integers(0, 256, (batch, M, K)).astype(np.uint8) if a_unsigned else r.integers(-128, 128, (batch, M, K)).astype(np.int8)
    b = r.integers(-128, 128, (batch, N, K) if trans_b else (batch, K, N)).astype(np.int8)
    return a, b, dict(shift=shift, mode=mode, trans_b=trans_b, out_kind=out_kind)


def _run_both(a, b, prm):
    from aie4ml_amd import _lib
    from oracle import oracle

    L = _lib.load()
    da, db = torch.from_numpy(a).cuda(), torch.from_numpy(b).cuda()
    batch, M, K = a.shape
    N = b.shape[1] if prm['trans_b'] else b.shape[2]
    tdt = {'int8': torch.int8, 'uint8': torch.uint8, 'int16': torch.int16}[prm['out_kind']]
    need = int(L.a4g_matmul_i8_workspace_bytes(batch, M, N, K, int(prm['trans_b']), 1 if a.dtype == np.uint8 else 0))
    ws = torch.empty((max(need, 16),), dtype=torch.uint8, device='cuda')
    ref = torch.full((batch, M, N), 77, dtype=tdt, device='cuda')
    got = torch.full((batch, M, N), 55, dtype=tdt, device='cuda')
    _call(L.a4g_matmul_i8, da, db, ref, prm['shift'], prm['mode'], prm['trans_b'], prm['out_kind'], (ws.data_ptr(), ws.numel()))
    _call(L.a4g_matmul_i8_static, da, db, got, prm['shift'], prm['mode'], prm['trans_b'], prm['out_kind'], ())
    torch.cuda.synchronize()
    exp = oracle.matmul(a, b, prm['shift'], prm['mode'], trans_b=prm['trans_b'], out=prm['out_kind'])
    assert np.array_equal(ref.cpu().numpy(), exp), 'a4g_matmul_i8 differs from the oracle'
    assert torch.equal(got, ref), 'a4g_matmul_i8_static differs from a4g_matmul_i8'
    return need


def test_static_matmul_two_calls_second_smaller():
    # uint8 x int8 with a [K][N] right operand: both halves of the scratch (transposed operand, column sums) in use
    big = _case(1, 5, 300, 200, 272, True, False, 9, 'conv_even', 'int8')
    small = _case(2, 2, 70, 40, 48, True, False, 7, 'symmetric_inf', 'int8')
    assert _run_both(*big) > 0
    assert _run_both(*small) > 0
    # and once more the other way round, signed left operand, ragged reduction, int16 output
    assert _run_both(*_case(3, 3, 130, 96, 100, False, False, 5, 'floor', 'int16')) > 0
    assert _run_both(*big) > 0


def test_static_matmul_shapes_without_scratch():
    # transposed right operand, signed left operand: no repack, the array is not touched
    assert _run_both(*_case(4, 4, 128, 128, 64, False, True, 6, 'conv_even', 'int8')) == 0
    # uint8 left operand with a transposed right operand: column sums only
    assert _run_both(*_case(5, 2, 96, 80, 64, True, True, 8, 'positive_inf', 'uint8')) > 0


def test_static_matmul_rejects_operands_beyond_the_array():
    from aie4ml_amd import _lib

    L = _lib.load()
    batch, M, N, K = 3, 16, 2048, 4096  # 3 * 2048 * 4096 = 24 MiB of repacked operand
    assert int(L.a4g_matmul_i8_workspace_bytes(batch, M, N, K, 0, 0)) > STATIC_MAX
    a = torch.zeros((batch, M, K), dtype=torch.int8, device='cuda')
    b = torch.zeros((batch, K, N), dtype=torch.int8, device='cuda')
    out = torch.zeros((batch, M, N), dtype=torch.int8, device='cuda')
    st = L.a4g_matmul_i8_static(a.data_ptr(), 0, 0, K, M * K, b.data_ptr(), N, K * N, 0, out.data_ptr(), N, M * N, batch, M, N, K, 8, 6,
                                0, torch.cuda.current_stream().cuda_stream)
    assert st == _lib.A4G_ERR_WORKSPACE
    assert b'static scratch array holds' in L.a4g_last_error()
    # the largest operand that fits runs
    assert _run_both(*_case(6, 1, 64, 2048, 4096, False, False, 10, 'conv_even', 'int8')) <= STATIC_MAX
