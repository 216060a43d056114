"""Builds libaie4ml_gfx950.so (the HIP kernels + C ABI) in-tree with hipcc for gfx950.

Usage:  python -m aie4ml_amd.build [--force]
"""

from __future__ import annotations

import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

CSRC = Path(__file__).resolve().parent / 'csrc'
LIB_PATH = Path(__file__).resolve().parent / 'libaie4ml_gfx950.so'
# measurement aids of bench.py (the matrix-core calibration loop), kept out of the library an integrator ships
BENCH_LIB_PATH = Path(__file__).resolve().parent / 'libaie4ml_bench_gfx950.so'
BENCH_SOURCES = ('calib.hip',)
SOURCES = ('abi.hip', 'rowops.hip', 'gemm.hip', 'mlp.hip', 'attention.hip', 'matmul_lean.hip', 'gemm_i16.hip', 'gemm_float.hip', 'gemm_wreg.hip', 'gemm_wrow.hip', 'gemm_wrow_plain.hip', 'gemm_wrow_sym_inf.hip', 'gemm_wrow_conv_even.hip', 'gemm_sk.hip', 'gemm_rowln.hip')

HIPCC_FLAGS = [
    '--offload-arch=gfx950',
    '-O3',
    '-std=c++17',
    '-fPIC',
    '-fvisibility=hidden',
    '-fvisibility-inlines-hidden',
    '-Wall',
    '-Wno-unused-function',
    # packed-FP32 instruction selection is switched off for every kernel in this library
    '-Xclang', '-target-feature', '-Xclang', '-packed-fp32-ops',
]


def _hipcc() -> str:
    rocm = os.environ.get('ROCM_PATH', '/opt/rocm')
    cand = Path(rocm) / 'bin' / 'hipcc'
    return str(cand) if cand.exists() else 'hipcc'


def _stale() -> bool:
    if not LIB_PATH.exists() or not BENCH_LIB_PATH.exists():
        return True
    t = LIB_PATH.stat().st_mtime
    # every source and header under csrc/ plus the public header: an edited epilogue header must trigger a rebuild
    deps = [*CSRC.glob('*.hip'), *CSRC.glob('*.hpp'), *(CSRC.parent.parent / 'include').glob('*.h')]
    return any(d.stat().st_mtime > t for d in deps)


def build(force: bool = False, verbose: bool = False) -> Path:
    """Compile every HIP source for gfx950 and link the shared library. Returns its path."""
    if not force and not _stale():
        return LIB_PATH
    objdir = CSRC / 'build'
    objdir.mkdir(exist_ok=True)
    hipcc = _hipcc()

    headers = [*CSRC.glob('*.hpp'), *(CSRC.parent.parent / 'include').glob('*.h')]
    newest_header = max(h.stat().st_mtime for h in headers)

    def compile_one(src: str) -> Path:
        obj = objdir / (Path(src).stem + '.o')
        # an object newer than its source and every header is kept (never with force: the build check compiles everything)
        if not force and obj.exists() and obj.stat().st_mtime > max((CSRC / src).stat().st_mtime, newest_header):
            return obj
        cmd = [hipcc, *HIPCC_FLAGS, '-c', str(CSRC / src), '-o', str(obj)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        errs = '\n'.join(line for line in res.stderr.splitlines()
                         if "is not a recognized feature" not in line)
        if res.returncode != 0:
            raise RuntimeError(f'hipcc failed on {src}:\n{errs}')
        if verbose and errs.strip():
            print(errs, file=sys.stderr)
        return obj

    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as pool:
        objs = list(pool.map(compile_one, SOURCES + BENCH_SOURCES))
    for path, group in ((LIB_PATH, objs[:len(SOURCES)]), (BENCH_LIB_PATH, objs[len(SOURCES):])):
        cmd = [hipcc, '--offload-arch=gfx950', '-shared', '-fPIC', '-o', str(path), *map(str, group)]
        res = subprocess.run(cmd, capture_output=True, text=True)
        if res.returncode != 0:
            raise RuntimeError(f'link failed:\n{res.stderr}')
    return LIB_PATH


if __name__ == '__main__':
    print(build(force='--force' in sys.argv, verbose=True))
