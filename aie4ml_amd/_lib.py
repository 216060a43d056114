"""ctypes loader for libaie4ml_gfx950.so — the only way the Python host reaches the HIP kernels.

There is no CPU fallback: if the library is missing or a symbol cannot be bound, importing an operator
raises, loudly.
"""

from __future__ import annotations

import ctypes
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / 'libaie4ml_gfx950.so'

A4G_OK = 0
A4G_ERR_INVALID_ARGUMENT = -1
A4G_ERR_UNSUPPORTED = -2
A4G_ERR_WORKSPACE = -3
A4G_ERR_HIP = -4

ROUNDING = {
    'floor': 0,
    'ceil': 1,
    'positive_inf': 2,
    'negative_inf': 3,
    'symmetric_inf': 4,
    'symmetric_zero': 5,
    'conv_even': 6,
    'conv_odd': 7,
}
KIND = {'int8': 0, 'uint8': 1, 'int16': 2, 'uint16': 3, 'int32': 4}
FLOAT_FORMAT = {'bfloat16': 16, 'float32': 17, 'fp8_e4m3': 18}

_i64, _i32, _vp, _sz = ctypes.c_int64, ctypes.c_int, ctypes.c_void_p, ctypes.c_size_t


class MlpLayer(ctypes.Structure):
    """Mirror of ``a4g_mlp_layer`` (include/aie4ml_gfx950.h)."""

    _fields_ = [
        ('wt', _vp),
        ('ldwt', _i64),
        ('colsum', _vp),
        ('bias', _vp),
        ('K', ctypes.c_int32),
        ('N', ctypes.c_int32),
        ('shift', ctypes.c_int32),
        ('relu', ctypes.c_int32),
        ('out_kind', ctypes.c_int32),
    ]


# The interface revision (A4G_VERSION of include/aie4ml_gfx950.h) the signatures below were written for. load() refuses
# a library of any other revision: a stale build would misread every argument behind a changed one without an error.
EXPECTED_VERSION = 300

# name -> (restype, argtypes); must list every symbol the public header declares
SIGNATURES = {
    'a4g_version': (_i32, []),
    'a4g_last_error': (ctypes.c_char_p, []),
    'a4g_add': (_i32, [_vp, _vp, _vp, _i64, _i32, _i32, _i32, _vp]),
    'a4g_packed_ld': (_i64, [_i64]),
    'a4g_pack_weights_i8': (_i32, [_vp, _i64, _i64, _i64, _vp, _vp, _vp]),
    'a4g_dense_i8': (_i32, [_vp, _i32, _i32, _i64, _vp, _i64, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp, _i64, _i64, _i64,
                            _i64, _vp]),
    'a4g_dense_i8_wf': (_i32, [_vp, _i32, _i32, _i64, _vp, _i64, _vp, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp, _i64, _i64, _i64,
                               _i64, _vp]),
    'a4g_matmul_i8_workspace_bytes': (_sz, [_i64, _i64, _i64, _i64, _i32, _i32]),
    'a4g_matmul_i8': (_i32, [_vp, _i32, _i32, _i64, _i64, _vp, _i64, _i64, _i32, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
                             _i32, _i32, _i32, _vp, _sz, _vp]),
    'a4g_matmul_i8_static': (_i32, [_vp, _i32, _i32, _i64, _i64, _vp, _i64, _i64, _i32, _vp, _i64, _i64, _i64, _i64, _i64, _i64,
                                    _i32, _i32, _i32, _vp]),
    'a4g_layernorm_i8': (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, ctypes.c_int32, _i32, _i32, _i32, _vp]),
    'a4g_add_layernorm_i8': (_i32, [_vp, _vp, _i32, _i32, _vp, _vp, _vp, _vp, _i64, _i64, ctypes.c_int32, _i32, _i32,
                                    _i32, _vp]),
    'a4g_rowpacked_bytes': (_i64, [_i64, _i64]),
    'a4g_rowpack_weights_i8': (_i32, [_vp, _i64, _i64, _i64, _vp, _vp]),
    'a4g_dense_add_layernorm_i8': (_i32, [_vp, _i32, _i64, _vp, _vp, _vp, _i32, _i32, _i32, _vp, _i64, _vp, _vp, _vp, _i64,
                                          _i64, _i64, _i64, ctypes.c_int32, _i32, _i32, _i32, _vp]),
    'a4g_softmax_exp_i8': (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, _i32, _vp]),
    'a4g_softmax_hccs_i8': (_i32, [_vp, _vp, _i64, _i64, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    'a4g_mlp_i8': (_i32, [ctypes.POINTER(MlpLayer), _i32, _vp, _i32, _i64, _vp, _i64, _i64, _i32, _vp]),
    'a4g_mlp_add_layernorm_i8': (_i32, [ctypes.POINTER(MlpLayer), _i32, _vp, _i32, _i64, _vp, _i64, _vp, _vp, _vp, _i64, _i64, _i32,
                                        _i32, _i32, _i32, _i32, _vp]),
    'a4g_dense_i16': (_i32, [_vp, _i32, _i64, _vp, _i64, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp, _i64, _i64, _i64, _i64, _vp]),
    'a4g_pack_weights_i16': (_i32, [_vp, _i64, _i64, _i64, _vp, _vp, _vp, _vp]),
    'a4g_dense_i16x16': (_i32, [_vp, _i32, _i64, _vp, _vp, _i64, _vp, _vp, _vp, _i32, _i32, _i32, _i32, _vp, _i64, _i64, _i64, _i64,
                                _vp]),
    'a4g_matmul_i16_workspace_bytes': (_sz, [_i64, _i64, _i64, _i32]),
    'a4g_matmul_i16': (_i32, [_vp, _i32, _i64, _i64, _vp, _i32, _i64, _i64, _i32, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32,
                              _i32, _vp, _sz, _vp]),
    'a4g_attention_i8': (_i32, [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, ctypes.POINTER(ctypes.c_int64), _i32, _i32,
                                _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _i32, _vp]),
    'a4g_packed_ld_f': (_i64, [_i64, _i32]),
    'a4g_pack_weights_f': (_i32, [_vp, _i32, _i64, _i64, _i64, _vp, _vp]),
    'a4g_dense_f': (_i32, [_vp, _i32, _i32, _i64, _vp, _i64, _vp, _i32, _vp, _i64, _i64, _i64, _i64, _vp]),
    'a4g_matmul_f_workspace_bytes': (_sz, [_i64, _i64, _i64, _i32, _i32]),
    'a4g_matmul_f': (_i32, [_vp, _i32, _i32, _i64, _i64, _vp, _i64, _i64, _i32, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _vp, _sz,
                            _vp]),
    'a4g_add_f': (_i32, [_vp, _vp, _vp, _i64, _i32, _vp]),
    'a4g_transpose': (_i32, [_vp, _i32, _i64, _i64, _vp, _i64, _i64, _i64, _i64, _i64, _vp]),
    'a4g_copy_2d': (_i32, [_vp, _i64, _vp, _i64, _i64, _i64, _vp]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library and bind every entry point. Raises if anything is missing."""
    global _lib
    if _lib is not None:
        return _lib
    # PyTorch's bundled HIP runtime must be the one this process initialises: load it first so that the
    # library below binds to the same libamdhip64 that owns torch's device memory and streams.
    import torch  # noqa: F401

    if not LIB_PATH.exists():
        raise RuntimeError(
            f'{LIB_PATH} is missing: build it with `python -m aie4ml_amd.build` (hipcc, gfx950). '
            'aie4ml_amd has no CPU fallback.'
        )
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is not exported
        fn.restype = restype
        fn.argtypes = argtypes
    have = int(lib.a4g_version())
    if have != EXPECTED_VERSION:
        raise RuntimeError(f'{LIB_PATH} is interface revision {have}, these bindings are written for {EXPECTED_VERSION}: '
                           'rebuild it with `python -m aie4ml_amd.build --force`')
    _lib = lib
    return lib


_EXC = {
    A4G_ERR_INVALID_ARGUMENT: ValueError,
    A4G_ERR_UNSUPPORTED: NotImplementedError,
    A4G_ERR_WORKSPACE: RuntimeError,
    A4G_ERR_HIP: RuntimeError,
}


def check(status: int) -> None:
    """Translate a C status into the exception class the reference raises for the same condition."""
    if status == A4G_OK:
        return
    msg = load().a4g_last_error().decode('utf-8', 'replace')
    raise _EXC.get(status, RuntimeError)(msg)
