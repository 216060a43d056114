"""GPU parity of the fused attention core against the oracle's three separate operators
(MatMul with transposed K -> integer Softmax -> MatMul with a uint8 left operand)."""

import numpy as np
import pytest
import torch

from aie4ml_amd import ops

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def reference(oracle, q, k, v, lshift, lmode, sm, oshift, omode):
    logits = oracle.matmul(q, k, lshift, lmode, trans_b=True)
    if sm['kind'] == 'exp':
        p = oracle.softmax_exp(logits, sm['exp_kq'], sm.get('inv_shift', 15))
    else:
        p = oracle.softmax_hccs(logits, sm['B'], sm['S'], sm['Dmax'], sm.get('inv_shift', 15), sm.get('use_clb', False))
    return oracle.matmul(p, v, oshift, omode)


def qkv(seed, shape_q, shape_k, sigma=24.0):
    r = np.random.default_rng(seed)
    g = lambda s: np.clip(np.rint(r.normal(0, sigma, s)), -128, 127).astype(np.int8)  # noqa: E731
    return g(shape_q), g(shape_k), g(shape_k)


HCCS = {32: (255, 4, 60), 64: (255, 3, 80), 96: (255, 3, 80), 128: (255, 2, 126), 160: (200, 2, 90), 192: (170, 1, 126),
        256: (127, 1, 126), 384: (85, 1, 80), 512: (60, 1, 59)}


@pytest.mark.parametrize('sk', [32, 64, 96, 128, 160, 192, 256, 384, 512])
@pytest.mark.parametrize('kind', ['exp', 'hccs'])
def test_attention_matches_three_operators(oracle, sk, kind):
    q, k, v = qkv(sk, (2, 3, sk, 64), (2, 3, sk, 64))
    if kind == 'exp':
        sm = {'kind': 'exp', 'exp_kq': 23}
    else:
        B, S, D = HCCS[sk]
        sm = {'kind': 'hccs', 'B': B, 'S': S, 'Dmax': D}
    got = ops.attention(dev(q), dev(k), dev(v), 6, 'conv_even', sm, 7, 'conv_even').cpu().numpy()
    want = reference(oracle, q, k, v, 6, 'conv_even', sm, 7, 'conv_even')
    np.testing.assert_array_equal(got, want)
    assert len(np.unique(got)) > 16


@pytest.mark.parametrize('mode', ['floor', 'ceil', 'positive_inf', 'negative_inf', 'symmetric_inf', 'symmetric_zero',
                                  'conv_even', 'conv_odd'])
def test_attention_rounding_modes(oracle, mode):
    q, k, v = qkv(7, (4, 128, 64), (4, 128, 64), sigma=40.0)
    sm = {'kind': 'exp', 'exp_kq': 40}
    got = ops.attention(dev(q), dev(k), dev(v), 5, mode, sm, 6, mode).cpu().numpy()
    np.testing.assert_array_equal(got, reference(oracle, q, k, v, 5, mode, sm, 6, mode))


@pytest.mark.parametrize('sq', [1, 31, 100, 129, 300])
def test_attention_ragged_query_count(oracle, sq):
    q, k, v = qkv(sq, (2, 2, sq, 64), (2, 2, 128, 64))
    sm = {'kind': 'hccs', 'B': 255, 'S': 2, 'Dmax': 126, 'use_clb': True}
    got = ops.attention(dev(q), dev(k), dev(v), 6, 'symmetric_inf', sm, 8, 'floor').cpu().numpy()
    np.testing.assert_array_equal(got, reference(oracle, q, k, v, 6, 'symmetric_inf', sm, 8, 'floor'))


@pytest.mark.parametrize('sk', [1, 5, 31, 33, 90, 96, 100, 150, 180, 197, 250, 300, 370, 511])
@pytest.mark.parametrize('kind', ['exp', 'hccs'])
def test_attention_key_count_off_the_tile_grid(oracle, sk, kind):
    """Any number of keys up to 512: the kernel of the next tile count that has one runs with the missing keys masked (they
    must neither raise a row's maximum, nor add to its sum, nor to the output). Self-attention shapes (sq == sk, as
    a 197-token ViT block has them), plus a query count of its own; both forms of the logit requantisation."""
    for sq in (sk, 70):
        q, k, v = qkv(1000 + sk + sq, (2, 3, sq, 64), (2, 3, sk, 64), sigma=30.0)
        if kind == 'exp':
            sm = {'kind': 'exp', 'exp_kq': 23}
        else:
            if sk == 1:
                return  # the parameter rules of HCCS (cols * (B - S * Dmax) >= 256, B <= 255) leave nothing for one key
            B = min(255, 32767 // sk)
            sm = {'kind': 'hccs', 'B': B, 'S': 1, 'Dmax': min(126, B - (256 + sk - 1) // sk)}
        lmode = 'conv_even' if sk % 2 else 'symmetric_inf'
        got = ops.attention(dev(q), dev(k), dev(v), 6, lmode, sm, 7, 'conv_even').cpu().numpy()
        np.testing.assert_array_equal(got, reference(oracle, q, k, v, 6, lmode, sm, 7, 'conv_even'))


@pytest.mark.parametrize('d,sk', [(32, 32), (32, 128), (32, 512), (32, 197), (128, 64), (128, 256), (128, 100), (16, 32),
                                  (16, 128), (16, 512), (16, 77)])
@pytest.mark.parametrize('kind', ['exp', 'hccs'])
def test_attention_head_dimensions_16_32_and_128(oracle, d, sk, kind):
    """One and four MFMA K steps per key tile instead of two (16: one, its upper half masked); sequence lengths on and off the tile grid; a query count
    of its own; both logit requantisations."""
    for sq in (sk, 45):
        q, k, v = qkv(7000 + d + sk + sq, (2, 3, sq, d), (2, 3, sk, d), sigma=24.0 if d <= 64 else 16.0)
        if kind == 'exp':
            sm = {'kind': 'exp', 'exp_kq': 23}
        else:
            B = min(255, 32767 // sk)
            sm = {'kind': 'hccs', 'B': B, 'S': 1, 'Dmax': min(126, B - (256 + sk - 1) // sk)}
        lmode = 'conv_even' if sq == sk else 'floor'
        lshift = 6 if d <= 64 else 7
        got = ops.attention(dev(q), dev(k), dev(v), lshift, lmode, sm, 7, 'conv_even').cpu().numpy()
        np.testing.assert_array_equal(got, reference(oracle, q, k, v, lshift, lmode, sm, 7, 'conv_even'))


@pytest.mark.parametrize('d,sk', [(16, 64), (16, 100), (48, 128), (80, 96), (96, 256), (112, 33)])
def test_attention_head_dimensions_between_the_kernels(oracle, d, sk):
    """Head dimensions 16, 48, 80, 96, 112 run on the next wider kernel with the missing pieces of a row masked; also into
    a strided output (the heads of a concatenated result) and from head slices of packed projections, where the bytes
    behind a head's row are the next head's."""
    q, k, v = qkv(9000 + d + sk, (2, 3, sk, d), (2, 3, sk, d), sigma=24.0)
    sm = {'kind': 'exp', 'exp_kq': 23}
    want = reference(oracle, q, k, v, 6, 'conv_even', sm, 7, 'symmetric_inf')
    got = ops.attention(dev(q), dev(k), dev(v), 6, 'conv_even', sm, 7, 'symmetric_inf').cpu().numpy()
    np.testing.assert_array_equal(got, want)
    out = torch.zeros((2, sk, 3 * d), dtype=torch.int8, device='cuda')
    ops.attention(dev(q), dev(k), dev(v), 6, 'conv_even', sm, 7, 'symmetric_inf', out=out.unflatten(-1, (3, d)).permute(0, 2, 1, 3))
    np.testing.assert_array_equal(out.cpu().numpy().reshape(2, sk, 3, d).transpose(0, 2, 1, 3), want)
    packed = [dev(np.ascontiguousarray(t.transpose(0, 2, 1, 3))).permute(0, 2, 1, 3) for t in (q, k, v)]  # [2, sk, 3, d] in memory
    got = ops.attention(packed[0], packed[1], packed[2], 6, 'conv_even', sm, 7, 'symmetric_inf').cpu().numpy()
    np.testing.assert_array_equal(got, want)


def test_attention_masked_keys_do_not_leak(oracle):
    """The rows behind the last key are other tensors' memory: whatever they hold, the result is that of the keys that
    exist (K rows past the end read as zero inside the kernel and their logits are forced to the minimum, V rows past the
    end are not read)."""
    sk = 100
    r = np.random.default_rng(5)
    big_k = np.full((2, 128, 64), 127, np.int8)
    big_v = np.full((2, 128, 64), -128, np.int8)
    big_k[:, :sk] = np.clip(np.rint(r.normal(0, 30, (2, sk, 64))), -128, 127)
    big_v[:, :sk] = np.clip(np.rint(r.normal(0, 30, (2, sk, 64))), -128, 127)
    q = np.clip(np.rint(r.normal(0, 30, (2, sk, 64))), -128, 127).astype(np.int8)
    sm = {'kind': 'exp', 'exp_kq': 23}
    got = ops.attention(dev(q), dev(big_k)[:, :sk], dev(big_v)[:, :sk], 6, 'conv_even', sm, 7, 'floor').cpu().numpy()
    want = reference(oracle, q, big_k[:, :sk].copy(), big_v[:, :sk].copy(), 6, 'conv_even', sm, 7, 'floor')
    np.testing.assert_array_equal(got, want)


@pytest.mark.parametrize('sq,sk', [(512, 512), (300, 256), (256, 512), (512, 384), (300, 384), (384, 384), (320, 512), (576, 256)])
@pytest.mark.parametrize('mode', ['conv_even', 'symmetric_inf', 'floor'])
def test_attention_with_256_row_workgroups(oracle, sq, sk, mode):
    # at least 256 workgroups of 256 query rows and 256 or more keys: the eight-wave form with the score table
    # stored once per LDS bank (six waves, blocks of 192 rows, where those leave fewer rows empty: 300, 320, 384, 576
    # queries); a clamped (non fast-path) probability shift as well
    nb = 256 // ((sq + 255) // 256) // 16
    q, k, v = qkv(sq + sk, (nb, 16, sq, 64), (nb, 16, sk, 64), sigma=30.0)
    B, S, D = HCCS[sk]
    for sm in ({'kind': 'exp', 'exp_kq': 23}, {'kind': 'hccs', 'B': B, 'S': S, 'Dmax': D},
               {'kind': 'exp', 'exp_kq': 23, 'inv_shift': 17}):
        got = ops.attention(dev(q), dev(k), dev(v), 6, mode, sm, 7, mode).cpu().numpy()
        np.testing.assert_array_equal(got, reference(oracle, q, k, v, 6, mode, sm, 7, mode))


@pytest.mark.parametrize('sk', [96, 160, 192, 384])
@pytest.mark.parametrize('mode', ['floor', 'symmetric_inf', 'symmetric_zero', 'conv_even', 'conv_odd'])
def test_attention_tile_counts_between_the_powers_of_two(oracle, sk, mode):
    """3, 5, 6 and 12 key tiles have kernels of their own for 64-wide heads: every form of the logit requantisation, both
    forms of the probability (the shift of 17 needs the clamp), a ragged query count."""
    q, k, v = qkv(4000 + sk, (2, 3, sk - 7, 64), (2, 3, sk, 64), sigma=36.0)
    for sm in ({'kind': 'exp', 'exp_kq': 31}, {'kind': 'exp', 'exp_kq': 23, 'inv_shift': 17}):
        got = ops.attention(dev(q), dev(k), dev(v), 5, mode, sm, 7, mode).cpu().numpy()
        np.testing.assert_array_equal(got, reference(oracle, q, k, v, 5, mode, sm, 7, mode))


def test_attention_zero_shift_and_saturation(oracle):
    # shift 0 on the logits saturates most of them; shift 0 on the output saturates everything
    q, k, v = qkv(3, (2, 64, 64), (2, 64, 64), sigma=60.0)
    sm = {'kind': 'exp', 'exp_kq': 128}
    got = ops.attention(dev(q), dev(k), dev(v), 0, 'conv_even', sm, 0, 'conv_even').cpu().numpy()
    np.testing.assert_array_equal(got, reference(oracle, q, k, v, 0, 'conv_even', sm, 0, 'conv_even'))
    got = ops.attention(dev(q), dev(k), dev(v), 10, 'conv_even', sm, 3, 'conv_even').cpu().numpy()
    np.testing.assert_array_equal(got, reference(oracle, q, k, v, 10, 'conv_even', sm, 3, 'conv_even'))


@pytest.mark.parametrize('sq,sk', [(96, 64), (256, 256)])
def test_attention_nearest_even_logits_at_every_shift(oracle, sq, sk):
    """Nearest-even logits are requantised in float arithmetic inside the kernel: every shift it covers, operands
    at the int8 extremes (accumulators of +-64 * 2^14, saturating both ways) and rows built to land on exact ties."""
    r = np.random.default_rng(sq + sk)
    q, k, v = qkv(11, (2, 2, sq, 64), (2, 2, sk, 64), sigma=50.0)
    q[0, 0, :8] = -128
    q[0, 0, 8:16] = 127
    k[0, 0, :8] = -128
    k[0, 0, 8:16] = 127
    # ties: q row = one-hot * 1, k rows with odd small values -> acc = odd multiples of 2^(s-1) for several s
    q[1, 1, :32] = 0
    q[1, 1, np.arange(32), np.arange(32)] = 1 << (np.arange(32) % 7)
    k[1, 1] = r.integers(-5, 6, (sk, 64)).astype(np.int8)
    sm = {'kind': 'exp', 'exp_kq': 23}
    for shift in range(0, 16):
        got = ops.attention(dev(q), dev(k), dev(v), shift, 'conv_even', sm, 7, 'conv_even').cpu().numpy()
        np.testing.assert_array_equal(got, reference(oracle, q, k, v, shift, 'conv_even', sm, 7, 'conv_even'), str(shift))
    for shift in (16, 20, 24):  # beyond the float form's range: the integer form
        got = ops.attention(dev(q), dev(k), dev(v), shift, 'conv_even', sm, 7, 'conv_even').cpu().numpy()
        np.testing.assert_array_equal(got, reference(oracle, q, k, v, shift, 'conv_even', sm, 7, 'conv_even'), str(shift))


def test_attention_on_head_slices_of_a_packed_projection(oracle):
    """Q, K, V as strided views of one [batch, seq, 3*hidden] tensor, output written into the head's
    columns of a [batch, seq, hidden] tensor: the layout of an encoder block, no copies."""
    batch, seq, heads, hd = 3, 128, 4, 64
    hidden = heads * hd
    r = np.random.default_rng(12)
    qkv_np = np.clip(np.rint(r.normal(0, 30, (batch, seq, 3 * hidden))), -128, 127).astype(np.int8)
    t = dev(qkv_np)
    out = torch.zeros((batch, seq, hidden), dtype=torch.int8, device='cuda')
    sm = {'kind': 'hccs', 'B': 255, 'S': 4, 'Dmax': 62}
    for h in range(heads):
        qs = t[:, :, h * hd:(h + 1) * hd]
        ks = t[:, :, hidden + h * hd:hidden + (h + 1) * hd]
        vs = t[:, :, 2 * hidden + h * hd:2 * hidden + (h + 1) * hd]
        ops.attention(qs, ks, vs, 7, 'conv_even', sm, 7, 'conv_even', out=out[:, :, h * hd:(h + 1) * hd])
    got = out.cpu().numpy()
    for h in range(heads):
        sl = lambda o: np.ascontiguousarray(qkv_np[:, :, o + h * hd:o + (h + 1) * hd])  # noqa: E731
        want = reference(oracle, sl(0), sl(hidden), sl(2 * hidden), 7, 'conv_even', sm, 7, 'conv_even')
        np.testing.assert_array_equal(got[:, :, h * hd:(h + 1) * hd], want, err_msg=f'head {h}')
    # all heads in one launch: [batch, heads, seq, hd] views with head stride hd
    q4 = t[:, :, :hidden].view(batch, seq, heads, hd).permute(0, 2, 1, 3)
    k4 = t[:, :, hidden:2 * hidden].view(batch, seq, heads, hd).permute(0, 2, 1, 3)
    v4 = t[:, :, 2 * hidden:].view(batch, seq, heads, hd).permute(0, 2, 1, 3)
    out2 = torch.zeros((batch, seq, hidden), dtype=torch.int8, device='cuda')
    ops.attention(q4, k4, v4, 7, 'conv_even', sm, 7, 'conv_even', out=out2.view(batch, seq, heads, hd).permute(0, 2, 1, 3))
    np.testing.assert_array_equal(out2.cpu().numpy(), got)


def test_attention_uncovered_shapes_and_bad_parameters():
    q = torch.zeros((2, 64, 40), dtype=torch.int8, device='cuda')
    with pytest.raises(NotImplementedError, match='fused path covers head dimensions that are multiples of 16'):
        ops.attention(q, q, q, 6, 'floor', {'kind': 'exp', 'exp_kq': 23}, 7, 'floor')
    q = torch.zeros((2, 544, 64), dtype=torch.int8, device='cuda')
    with pytest.raises(NotImplementedError, match='fused path covers'):
        ops.attention(q, q, q, 6, 'floor', {'kind': 'exp', 'exp_kq': 23}, 7, 'floor')
    q = torch.zeros((2, 64, 64), dtype=torch.int8, device='cuda')
    with pytest.raises(ValueError, match='1 <= EXP_KQ <= 128'):
        ops.attention(q, q, q, 6, 'floor', {'kind': 'exp', 'exp_kq': 0}, 7, 'floor')
    with pytest.raises(ValueError, match=r'cols \* B <= 32767'):
        ops.attention(q, q, q, 6, 'floor', {'kind': 'hccs', 'B': 600, 'S': 1, 'Dmax': 5}, 7, 'floor')
    with pytest.raises(ValueError, match='incompatible shapes'):
        ops.attention(q, q[:, :32], q, 6, 'floor', {'kind': 'exp', 'exp_kq': 23}, 7, 'floor')
