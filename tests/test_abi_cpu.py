"""CPU-only checks of the C-ABI boundary: the library builds in-tree, loads, exports every symbol the
public header declares, and the Python binding table names exactly those symbols. No kernels run."""

import ctypes
import re
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / 'include' / 'aie4ml_gfx950.h'


def declared_symbols():
    text = HEADER.read_text()
    return sorted(set(re.findall(r'^A4G_API [\w\s\*]*?\b(a4g_\w+)\(', text, flags=re.M)))


@pytest.fixture(scope='module')
def libpath():
    from aie4ml_amd import _lib

    if not _lib.LIB_PATH.exists():
        from aie4ml_amd import build

        build.build()
    return _lib.LIB_PATH


def test_header_declares_expected_entry_points():
    syms = declared_symbols()
    for name in ('a4g_version', 'a4g_last_error', 'a4g_add', 'a4g_pack_weights_i8', 'a4g_dense_i8', 'a4g_matmul_i8',
                 'a4g_matmul_i8_workspace_bytes', 'a4g_layernorm_i8', 'a4g_add_layernorm_i8', 'a4g_softmax_exp_i8',
                 'a4g_softmax_hccs_i8', 'a4g_mlp_i8', 'a4g_packed_ld'):
        assert name in syms


def test_library_exports_every_declared_symbol(libpath):
    lib = ctypes.CDLL(str(libpath))
    for name in declared_symbols():
        assert hasattr(lib, name), f'{name} declared in the header but not exported'


def test_binding_table_matches_header(libpath):
    from aie4ml_amd import _lib

    assert sorted(_lib.SIGNATURES) == declared_symbols()
    lib = _lib.load()
    assert lib.a4g_version() == _lib.EXPECTED_VERSION == 300
    assert lib.a4g_packed_ld(1) == 16 and lib.a4g_packed_ld(16) == 16 and lib.a4g_packed_ld(17) == 32
    # pure host-side query, no GPU needed: K x N operand transposed into the workspace + colsum
    assert lib.a4g_matmul_i8_workspace_bytes(2, 8, 64, 512, 1, 0) == 0
    assert lib.a4g_matmul_i8_workspace_bytes(2, 8, 64, 512, 0, 0) == 2 * 64 * 512
    assert lib.a4g_matmul_i8_workspace_bytes(2, 8, 64, 512, 0, 1) == 2 * 64 * 512 + 512


def test_mlp_layer_struct_layout():
    from aie4ml_amd._lib import MlpLayer

    # wt(8) ldwt(8) colsum(8) bias(8) + five int32 -> 52, padded to 56
    assert ctypes.sizeof(MlpLayer) == 56
    assert MlpLayer.K.offset == 32 and MlpLayer.out_kind.offset == 48


def test_argument_validation_happens_before_any_launch(libpath):
    """Error paths return a status and a message without touching the GPU (null stream, no device)."""
    from aie4ml_amd import _lib

    lib = _lib.load()
    st = lib.a4g_add(None, None, None, 16, 9, 0, 0, None)  # null pointers
    assert st == _lib.A4G_ERR_INVALID_ARGUMENT
    st = lib.a4g_softmax_hccs_i8(None, None, 4, 512, 100, 1, 59, 15, 0, 1, None)  # cols*B > 32767
    assert st == _lib.A4G_ERR_INVALID_ARGUMENT
    assert b'cols * B <= 32767' in lib.a4g_last_error()
    with pytest.raises(ValueError):
        _lib.check(st)
    st = lib.a4g_transpose(None, 3, 8, 64, None, 8, 64, 1, 8, 8, None)  # 3-byte elements
    assert st == _lib.A4G_ERR_UNSUPPORTED and b'a4g_transpose' in lib.a4g_last_error()
    assert lib.a4g_transpose(None, 2, 4, 64, None, 8, 64, 1, 8, 8, None) == _lib.A4G_ERR_INVALID_ARGUMENT  # pitch < row
    assert lib.a4g_transpose(None, 2, 8, 64, None, 8, 64, 0, 8, 8, None) == 0  # empty batch
    # the row-complete Dense + Add + LayerNorm: shapes outside its limits are refused before anything else happens
    st = lib.a4g_dense_add_layernorm_i8(None, 0, 800, None, None, None, 9, 0, 0, None, 800, None, None, None, 800, 64, 800, 768,
                                        1, 7, 5, 0, None)  # 800 columns
    assert st == _lib.A4G_ERR_UNSUPPORTED and b'a4g_dense_add_layernorm_i8' in lib.a4g_last_error()
    assert lib.a4g_dense_add_layernorm_i8(None, 0, 768, None, None, None, 9, 0, 0, None, 768, None, None, None, 768, 64, 768, 700,
                                          1, 7, 5, 0, None) == _lib.A4G_ERR_UNSUPPORTED  # K not a multiple of 128
    assert lib.a4g_dense_add_layernorm_i8(None, 0, 768, None, None, None, 40, 0, 0, None, 768, None, None, None, 768, 64, 768, 768,
                                          1, 7, 5, 0, None) == _lib.A4G_ERR_INVALID_ARGUMENT  # shift 40
    assert lib.a4g_dense_add_layernorm_i8(None, 0, 768, None, None, None, 9, 0, 0, None, 768, None, None, None, 768, 0, 768, 768,
                                          1, 7, 5, 0, None) == 0  # no rows
    assert lib.a4g_rowpack_weights_i8(None, 768, 100, 760, None, None) == _lib.A4G_ERR_UNSUPPORTED  # K off the 16-byte grid
    assert lib.a4g_rowpack_weights_i8(None, 768, 100, 768, None, None) == _lib.A4G_ERR_INVALID_ARGUMENT  # null pointers
    assert lib.a4g_rowpacked_bytes(100, 200) == 128 * 256 and lib.a4g_rowpacked_bytes(0, 64) == 0
    # the chain that ends in Add + LayerNorm checks the normalisation's constants before it looks at the chain
    st = lib.a4g_mlp_add_layernorm_i8(None, 1, None, 0, 64, None, 64, None, None, None, 64, 32, 0, 0, 7, 5, 0, None)  # eps_q0 < 1
    assert st == _lib.A4G_ERR_INVALID_ARGUMENT and b'a4g_mlp_add_layernorm_i8: eps_q0' in lib.a4g_last_error()
    assert lib.a4g_mlp_add_layernorm_i8(None, 1, None, 0, 64, None, 64, None, None, None, 64, 32, 0, 1, 7, 16, 0,
                                        None) == _lib.A4G_ERR_INVALID_ARGUMENT  # out_shift 16
    assert lib.a4g_mlp_add_layernorm_i8(None, 1, None, 0, 64, None, 64, None, None, None, 64, 32, 0, 1, 16, 5, 0,
                                        None) == _lib.A4G_ERR_INVALID_ARGUMENT  # gamma_shift 16
    assert lib.a4g_mlp_add_layernorm_i8(None, 1, None, 0, 64, None, 64, None, None, None, 64, 32, 0, 1, 7, 5, 9,
                                        None) == _lib.A4G_ERR_INVALID_ARGUMENT  # rounding mode 9
    st = lib.a4g_softmax_exp_i8(None, None, 4, 512, 0, 15, 1, None)  # exp_kq out of range
    assert st == _lib.A4G_ERR_INVALID_ARGUMENT and b'EXP_KQ' in lib.a4g_last_error()
    st = lib.a4g_layernorm_i8(None, None, None, None, 4, 64, 0, 7, 5, 6, None)  # eps_q0 < 1
    assert st == _lib.A4G_ERR_INVALID_ARGUMENT and b'eps_q0' in lib.a4g_last_error()
    st = lib.a4g_layernorm_i8(None, None, None, None, 4, 64, 1, 7, 16, 6, None)  # out_shift > 15
    assert st == _lib.A4G_ERR_INVALID_ARGUMENT and b'out_shift' in lib.a4g_last_error()
    st = lib.a4g_dense_i8(None, 2, 0, 16, None, 16, None, None, None, 1, 0, 0, 0, None, 16, 4, 16, 16, None)  # int16 lhs
    assert st == _lib.A4G_ERR_UNSUPPORTED
    with pytest.raises(NotImplementedError):
        _lib.check(st)
    # the entry point without a workspace validates like a4g_matmul_i8, before it looks at the device
    st = lib.a4g_matmul_i8_static(None, 0, 0, 16, 0, None, 16, 0, 0, None, 16, 0, 1, 4, 16, 16, 40, 0, 0, None)  # shift 40
    assert st == _lib.A4G_ERR_INVALID_ARGUMENT and b'a4g_matmul_i8_static' in lib.a4g_last_error()
    assert lib.a4g_matmul_i8_static(None, 0, 0, 16, 0, None, 16, 0, 0, None, 16, 0, 0, 4, 16, 16, 3, 0, 0, None) == 0  # batch 0
    # empty problems are fine and do nothing
    assert lib.a4g_add(None, None, None, 0, 0, 0, 0, None) == 0
    assert lib.a4g_layernorm_i8(None, None, None, None, 0, 64, 1, 7, 5, 6, None) == 0
