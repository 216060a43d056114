"""Inputs beyond 2^31 bytes / elements: every kernel's addressing must be 64-bit where it has to be.
Data is generated on the GPU; the oracle checks slices from the start, the middle and the very end."""

import numpy as np
import pytest

torch = pytest.importorskip('torch')

pytestmark = pytest.mark.gpu


@pytest.fixture(scope='module')
def ops():
    if not torch.cuda.is_available():
        pytest.skip('no GPU')
    from aie4ml_amd import ops as _ops

    return _ops


def slices(n, width=257):
    return [slice(0, width), slice(n // 2 - 3, n // 2 - 3 + width), slice(n - width, n)]


def host(t):
    return t.cpu().numpy()


def test_dense_more_than_2gib_of_activations(ops, oracle):
    M, K, N = (1 << 21) + 5, 1024, 64
    g = torch.Generator(device='cuda').manual_seed(1)
    A = torch.randint(-128, 128, (M, K), dtype=torch.int8, device='cuda', generator=g)
    W = torch.randint(-128, 128, (K, N), dtype=torch.int8, device='cuda', generator=g)
    bias = torch.randint(-2 ** 14, 2 ** 14, (N,), dtype=torch.int32, device='cuda', generator=g)
    y = ops.dense(A, ops.pack_dense(W, bias, 11), 'conv_even', relu=True)
    torch.cuda.synchronize()
    for s in slices(M):
        assert np.array_equal(host(y[s]), oracle.dense(host(A[s]), host(W), host(bias), 11, 'conv_even', relu=True))


def test_add_more_than_2_31_elements(ops, oracle):
    n = (1 << 31) + 1000
    g = torch.Generator(device='cuda').manual_seed(2)
    a = torch.randint(-128, 128, (n,), dtype=torch.int8, device='cuda', generator=g)
    b = torch.randint(-128, 128, (n,), dtype=torch.int8, device='cuda', generator=g)
    y = ops.add(a, b)
    torch.cuda.synchronize()
    for s in slices(n, 4099):
        assert np.array_equal(host(y[s]), oracle.add(host(a[s]), host(b[s])))


def test_row_kernels_more_than_2_31_elements(ops, oracle):
    rows, cols = (1 << 21) + 3, 1024
    g = torch.Generator(device='cuda').manual_seed(3)
    x = (torch.randn((rows, cols), device='cuda', generator=g) * 24).round().clamp(-128, 127).to(torch.int8)
    gamma = torch.randint(32, 128, (cols,), dtype=torch.int16, device='cuda', generator=g)
    beta = (torch.randint(-16, 17, (cols,), dtype=torch.int32, device='cuda', generator=g) << 10).to(torch.int16)
    ln = ops.layernorm(x, gamma, beta, 5, 'conv_even')
    sm = ops.softmax_exp(x, 23)
    torch.cuda.synchronize()
    for s in slices(rows, 33):
        assert np.array_equal(host(ln[s]), oracle.layernorm(host(x[s]), host(gamma), host(beta), 5, 'conv_even'))
        assert np.array_equal(host(sm[s]), oracle.softmax_exp(host(x[s]), 23))


def test_matmul_batch_beyond_2gib_output(ops, oracle):
    # 4200 heads of 512 x 512 logits: 1.1 G output elements through the short-reduction kernel
    heads = 4200
    g = torch.Generator(device='cuda').manual_seed(4)
    q = (torch.randn((heads, 512, 64), device='cuda', generator=g) * 24).round().clamp(-128, 127).to(torch.int8)
    k = (torch.randn((heads, 512, 64), device='cuda', generator=g) * 24).round().clamp(-128, 127).to(torch.int8)
    y = ops.matmul(q, k, 6, 'conv_even', trans_b=True)
    torch.cuda.synchronize()
    for h in (0, heads // 2, heads - 1):
        assert np.array_equal(host(y[h]), oracle.matmul(host(q[h]), host(k[h]), 6, 'conv_even', trans_b=True))
