"""Operator-level host API: torch device tensors in, torch device tensors out, HIP kernels underneath.

Each function is a thin shim over one C-ABI entry point of ``libaie4ml_gfx950.so``; PyTorch only
supplies device memory and the current stream. Argument meaning follows the reference's kernel
configuration structs (templates/firmware/variants/*/parameters.h.jinja).
"""

from __future__ import annotations

import ctypes
from dataclasses import dataclass
from typing import Tuple, List, Optional, Sequence

import torch

from . import _lib
from ._lib import KIND, ROUNDING, MlpLayer, check

_TORCH_KIND = {torch.int8: 0, torch.uint8: 1, torch.int16: 2, torch.int32: 4}
_KIND_TORCH = {0: torch.int8, 1: torch.uint8, 2: torch.int16, 4: torch.int32}


def _mode(mode) -> int:
    if isinstance(mode, str):
        try:
            return ROUNDING[mode]
        except KeyError:
            raise ValueError(f'Unsupported rounding mode {mode!r} for the GPU kernels.') from None
    return int(mode)


def _kind(kind) -> int:
    return KIND[kind] if isinstance(kind, str) else int(kind)


def _dev(t: torch.Tensor, name: str) -> torch.Tensor:
    if not t.is_cuda:
        raise ValueError(f'{name}: expected a tensor in GPU memory, got device {t.device}.')
    return t


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else None


def _pitched_rows(t: torch.Tensor, name: str) -> torch.Tensor:
    """t as a 2-D [rows, cols] view whose rows the kernels can read in place: a contiguous last axis, a row pitch that is
    a multiple of 16 bytes and a 16-byte aligned start (a column window of a wider tensor qualifies); anything else is
    copied to a dense buffer."""
    t2 = _rows2d(t, name)
    if t2.dim() == 2 and t2.stride(1) == 1 and (t2.shape[0] <= 1 or (t2.stride(0) * t2.element_size()) % 16 == 0) \
            and t2.data_ptr() % 16 == 0 and (t2.shape[0] <= 1 or t2.stride(0) >= t2.shape[1]):
        return t2
    return t2.contiguous()


def _pitch(t2: torch.Tensor) -> int:
    return int(t2.stride(0)) if t2.shape[0] > 1 else int(t2.shape[1])


def _stream() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _rows2d(t: torch.Tensor, name: str) -> torch.Tensor:
    """View a tensor as [rows, cols] with a contiguous last axis."""
    _dev(t, name)
    if t.dim() < 1:
        raise ValueError(f'{name}: need at least one axis.')
    t2 = t.reshape(-1, t.shape[-1])
    if t2.stride(-1) != 1 and t2.shape[-1] > 1:
        t2 = t2.contiguous()
    return t2


def transpose_last2(t: torch.Tensor) -> torch.Tensor:
    """[..., R, C] -> a new contiguous [..., C, R] through the library's transpose kernel (elements of 1, 2 or 4 bytes):
    how the 16-bit and floating-point operators take a left operand that the graph hands over transposed."""
    _dev(t, 't')
    if t.dim() < 2:
        raise ValueError('transpose needs rank >= 2')
    t = t.contiguous()
    R, C = int(t.shape[-2]), int(t.shape[-1])
    batch = t.numel() // max(R * C, 1)
    out = torch.empty(tuple(t.shape[:-2]) + (C, R), dtype=t.dtype, device=t.device)
    if t.numel():
        src, dst = t.reshape(-1, R, C), out.reshape(-1, C, R)
        for b0 in range(0, batch, 65535):  # the batch rides on gridDim.z
            nb = min(65535, batch - b0)
            check(_lib.load().a4g_transpose(_ptr(src[b0:]), t.element_size(), C, R * C, _ptr(dst[b0:]), R, R * C, nb, R, C, _stream()))
    return out


def concat(parts: Sequence[torch.Tensor], axis: int) -> torch.Tensor:
    """The parts side by side along `axis` in one new tensor, each placed with the library's 2-D device copy (the
    reference's Concat is a view: its producers write their slices of one buffer, docs/support.md:13-15)."""
    if not parts:
        raise ValueError('concat needs at least one tensor')
    first = parts[0]
    axis = axis % first.dim()
    for t in parts:
        _dev(t, 'part')
        if t.dtype != first.dtype or t.dim() != first.dim() or any(
                t.shape[i] != first.shape[i] for i in range(first.dim()) if i != axis):
            raise ValueError('concat: parts must share dtype and every extent but the one along the axis')
    shape = list(first.shape)
    shape[axis] = sum(int(t.shape[axis]) for t in parts)
    out = torch.empty(shape, dtype=first.dtype, device=first.device)
    rows = 1
    for e in shape[:axis]:
        rows *= int(e)
    inner = first.element_size()
    for e in shape[axis + 1:]:
        inner *= int(e)
    ld_dst, at = shape[axis] * inner, 0
    for t in parts:
        t = t.contiguous()
        row_bytes = int(t.shape[axis]) * inner
        if rows and row_bytes:
            check(_lib.load().a4g_copy_2d(_ptr(t), row_bytes, out.data_ptr() + at, ld_dst, rows, row_bytes, _stream()))
        at += row_bytes
    return out


def add(a: torch.Tensor, b: torch.Tensor, shift: int = 0, rounding='floor', out: Optional[torch.Tensor] = None):
    """Saturating elementwise add of two tensors that share shape and storage type."""
    _dev(a, 'a'), _dev(b, 'b')
    if a.shape != b.shape:
        raise ValueError(f'elementwise Add requires exact-shape inputs, got {tuple(a.shape)} and {tuple(b.shape)}.')
    if a.dtype != b.dtype or a.dtype not in _TORCH_KIND:
        raise ValueError('elementwise Add requires lhs/rhs/output to use the same storage type.')
    a, b = a.contiguous(), b.contiguous()
    if out is None:
        out = torch.empty_like(a)
    check(_lib.load().a4g_add(_ptr(a), _ptr(b), _ptr(out), a.numel(), _TORCH_KIND[a.dtype], int(shift), _mode(rounding),
                              _stream()))
    return out


@dataclass
class PackedDense:
    """Device-resident Dense parameters in the layout the GEMM kernel consumes."""

    wt: torch.Tensor       # [N, ldwt] int8, reduction axis contiguous, zero padded (int16 weights: their high bytes)
    colsum: torch.Tensor   # [N] int32
    bias: Optional[torch.Tensor]  # [N] int32 or None
    shifts: torch.Tensor   # [1] or [N] int32
    K: int
    N: int
    wt_lo: Optional[torch.Tensor] = None  # int16 weights only: the low-byte plane (bytes ^ 0x80)
    shift0: Optional[int] = None          # the shift as a host integer when there is one for every column
    wf: Optional[torch.Tensor] = None     # int8 weights in fragment order (short reductions: at pack time; else on
                                          # first use by dense_add_layernorm)
    quick_shifts: bool = True             # every shift lies in 1..15: the requantisation that the kernel fed by `wf`
                                          # overlaps with its matrix work covers exactly those

    @property
    def ldwt(self) -> int:
        return int(self.wt.shape[1])


def pack_dense(weight: torch.Tensor, bias: Optional[torch.Tensor], shifts) -> PackedDense:
    """weight: logical [K, N] int8 on the device; bias: [N] int32 or None; shifts: int or [N] ints."""
    _dev(weight, 'weight')
    if weight.dtype not in (torch.int8, torch.int16) or weight.dim() != 2:
        raise ValueError('weight matrix must be a rank-2 int8 (or int16) tensor')
    weight = weight.contiguous()
    K, N = int(weight.shape[0]), int(weight.shape[1])
    L = _lib.load()
    ldwt = int(L.a4g_packed_ld(K))
    wt = torch.empty((N, ldwt), dtype=torch.int8, device=weight.device)
    colsum = torch.empty((N,), dtype=torch.int32, device=weight.device)
    wt_lo = None
    if weight.dtype == torch.int16:
        wt_lo = torch.empty((N, ldwt), dtype=torch.int8, device=weight.device)
        check(L.a4g_pack_weights_i16(_ptr(weight), N, K, N, _ptr(wt), _ptr(wt_lo), _ptr(colsum), _stream()))
    else:
        check(L.a4g_pack_weights_i8(_ptr(weight), N, K, N, _ptr(wt), _ptr(colsum), _stream()))
    if bias is not None:
        bias = _dev(bias, 'bias').to(torch.int32).contiguous()
        if bias.numel() != N:
            raise ValueError(f'dense bias requires exactly {N} elements, got {bias.numel()}.')
    sh = torch.as_tensor(shifts, dtype=torch.int32).reshape(-1)
    if sh.numel() not in (1, N):
        raise ValueError(f'shifts must hold 1 or {N} entries, got {sh.numel()}')
    top = 62 if wt_lo is not None else 31
    if int(sh.min()) < 0 or int(sh.max()) > top:
        raise ValueError(f'dense accumulator output shift must be in [0, {top}], got [{int(sh.min())}, {int(sh.max())}].')
    p = PackedDense(wt=wt, colsum=colsum, bias=bias, shifts=sh.to(weight.device), K=K, N=N, wt_lo=wt_lo,
                    shift0=int(sh[0]) if sh.numel() == 1 else None, quick_shifts=bool(int(sh.min()) >= 1 and int(sh.max()) <= 15))
    if wt_lo is None and K <= 768 and K % 16 == 0 and p.quick_shifts:
        _rowpack(p)  # the Dense kernel for short reductions fetches its weights in this order
    return p


def _rowpack(p: PackedDense) -> torch.Tensor:
    """The fragment-order copy of p's int8 weights (made once, kept in p.wf)."""
    if p.wf is None:
        L = _lib.load()
        wf = torch.empty((int(L.a4g_rowpacked_bytes(p.N, p.K)),), dtype=torch.int8, device=p.wt.device)
        check(L.a4g_rowpack_weights_i8(_ptr(p.wt), p.ldwt, p.N, p.K, _ptr(wf), _stream()))
        p.wf = wf
    return p.wf


def dense(x: torch.Tensor, p: PackedDense, rounding='floor', relu: bool = False, out_kind='int8',
          out: Optional[torch.Tensor] = None, trans_a: bool = False):
    """y = saturate(round((x @ W + bias) >> shift)), optionally ReLU. x: [..., K] int8 / uint8 / int16.
    ``trans_a``: x is [..., K, M], the operand is consumed through a last-two-axes transpose view and transposed inside
    the kernel, one launch per leading index."""
    if trans_a:
        _dev(x, 'x')
        if x.dim() < 2 or int(x.shape[-2]) != p.K:
            raise ValueError(f'dense input (transposed) has {tuple(x.shape)}, weights expect {p.K} on the second-to-last axis')
        if x.dtype not in (torch.int8, torch.uint8, torch.int16):
            raise NotImplementedError(f'dense activations must be int8, uint8 or int16, got {x.dtype}')
        if p.wt_lo is not None and x.dtype != torch.int16:
            raise RuntimeError('unsupported int8 x int16 precision mix for AIE implementations; no implementation variant '
                               'available.')
        xs = x.contiguous().reshape(-1, p.K, int(x.shape[-1]))
        Mt = int(xs.shape[-1])
        ok = _kind(out_kind)
        if out is None:
            out = torch.empty(tuple(x.shape[:-2]) + (Mt, p.N), dtype=_KIND_TORCH[ok], device=x.device)
        ys = out.reshape(-1, Mt, p.N)
        L = _lib.load()
        tail = (_ptr(p.colsum), _ptr(p.bias), _ptr(p.shifts), int(p.shifts.numel()), _mode(rounding), int(bool(relu)), ok)
        for i in range(int(xs.shape[0])):  # the operand is transposed inside the kernel, one launch per leading index
            if p.wt_lo is not None:
                check(L.a4g_dense_i16x16(_ptr(xs[i]), 1, Mt, _ptr(p.wt), _ptr(p.wt_lo), p.ldwt, *tail, _ptr(ys[i]), p.N, Mt, p.N, p.K,
                                         _stream()))
            elif xs.dtype == torch.int16:
                check(L.a4g_dense_i16(_ptr(xs[i]), 1, Mt, _ptr(p.wt), p.ldwt, *tail, _ptr(ys[i]), p.N, Mt, p.N, p.K, _stream()))
            else:
                check(L.a4g_dense_i8(_ptr(xs[i]), _TORCH_KIND[xs.dtype], 1, Mt, _ptr(p.wt), p.ldwt, *tail, _ptr(ys[i]), p.N, Mt, p.N,
                                     p.K, _stream()))
        return out
    x2 = _rows2d(x, 'x')
    if x2.dtype not in (torch.int8, torch.uint8, torch.int16):
        raise NotImplementedError(f'dense activations must be int8, uint8 or int16, got {x2.dtype}')
    if x2.shape[1] != p.K:
        raise ValueError(f'dense input has {x2.shape[1]} features, weights expect {p.K}')
    M = int(x2.shape[0])
    ok = _kind(out_kind)
    if out is None:
        out = torch.empty(tuple(x.shape[:-1]) + (p.N,), dtype=_KIND_TORCH[ok], device=x.device)
    y2 = out.reshape(-1, p.N)
    if p.wt_lo is not None:
        if x2.dtype != torch.int16:
            raise RuntimeError('unsupported int8 x int16 precision mix for AIE implementations; no implementation variant '
                               'available.')
        check(_lib.load().a4g_dense_i16x16(_ptr(x2), 0, x2.stride(0) if M > 0 else p.K, _ptr(p.wt), _ptr(p.wt_lo), p.ldwt,
                                           _ptr(p.colsum), _ptr(p.bias), _ptr(p.shifts), int(p.shifts.numel()), _mode(rounding),
                                           int(bool(relu)), ok, _ptr(y2), y2.stride(0) if M > 0 else p.N, M, p.N, p.K,
                                           _stream()))
        return out
    if x2.dtype == torch.int16:
        check(_lib.load().a4g_dense_i16(_ptr(x2), 0, x2.stride(0) if M > 0 else p.K, _ptr(p.wt), p.ldwt, _ptr(p.colsum),
                                        _ptr(p.bias), _ptr(p.shifts), int(p.shifts.numel()), _mode(rounding),
                                        int(bool(relu)), ok, _ptr(y2), y2.stride(0) if M > 0 else p.N, M, p.N, p.K, _stream()))
        return out
    if _narrow_dense_as_chain(x2, p, ok, M):
        # a narrow layer on a long batch is bound by its rows' traffic, not by arithmetic: the kernel that walks a chain
        # of layers over 32 samples per wave does a chain of one at 3-5 TB/s (1 Mi x 16 -> 64: 23 us against 151 us)
        mlp(x2, [MlpLayerSpec(p, int(p.shift0), bool(relu), 'uint8' if ok == 1 else 'int8')], rounding, out=y2)
        return out
    # A shift of 0 or above 15 sends a column block of the kernel that takes `wf` through its general requantisation, which
    # keeps no weights in registers (8192 x 768 -> 3072: 50 us against 26 us); the kernel without `wf` does such layers in 33 us.
    check(_lib.load().a4g_dense_i8_wf(_ptr(x2), _TORCH_KIND[x2.dtype], 0, x2.stride(0) if M > 0 else p.K, _ptr(p.wt), p.ldwt,
                                      _ptr(p.wf if p.quick_shifts else None), _ptr(p.colsum), _ptr(p.bias), _ptr(p.shifts), int(p.shifts.numel()),
                                      _mode(rounding), int(bool(relu)), ok, _ptr(y2), y2.stride(0) if M > 0 else p.N, M, p.N,
                                      p.K, _stream()))
    return out


def _narrow_dense_as_chain(x2: torch.Tensor, p: PackedDense, out_kind: int, rows: int) -> bool:
    """Dense layers that a4g_mlp_i8 with one layer runs faster than a4g_dense_i8: up to 256 wide both ways, one shift,
    8-bit result, a batch on which a4g_mlp_i8 uses the matrix units, and either a shape the weights-in-registers GEMM
    does not take (that one wants K and N in multiples of 16 and 16-byte aligned rows: a classifier's 10 outputs are not),
    or at most 64 outputs behind a reduction that ends inside a 128-byte tile. Measured, chain / GEMM in us:
    1 Mi x 16 -> 64 23.8 / 38.1 (151 on the tiled kernel), 1 Mi x 64 -> 32 19.4 / 36.2, 1 Mi x 16 -> 16 15.4 / 35.3,
    65 536 x 64 -> 64 5.3 / 6.6, 65 536 x 128 -> 10 6.3 / 10.6, 262 144 x 128 -> 8 11.3 / 31.4; but 50 432 x 192 -> 192
    14.0 / 10.7, 262 144 x 48 -> 256 32.9 / 24.6, 32 768 x 240 -> 240 13.8 / 8.3, and level at 128 or 256 inputs with 16 to
    64 outputs."""
    if not (p.shift0 is not None and p.wt_lo is None and p.K <= 256 and p.N <= 256 and out_kind in (0, 1)
            and x2.dtype in (torch.int8, torch.uint8) and x2.stride(1) == 1
            and mlp_runs_on_matrix_units(rows, int(x2.stride(0)), [(p.K, p.N)])):
        return False
    gemm_takes_it = (p.K % 16 == 0 and p.N % 16 == 0 and int(x2.stride(0)) % 16 == 0 and x2.data_ptr() % 16 == 0
                     and (p.K % 128 == 0 or x2.dtype == torch.int8 or p.K <= 640))
    return not gemm_takes_it or (p.N <= 64 and p.K % 128 != 0)


def matmul(a: torch.Tensor, b: torch.Tensor, shift: int, rounding='floor', trans_b: bool = False, out_kind='int8',
           out: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None, trans_a: bool = False):
    """Batched dynamic MatMul. a: [..., M, K] int8/uint8/int16; b: [..., K, N] int8 (int16 with an int16 a), or [..., N, K] when
    ``trans_b`` (the operand is consumed through a last-two-axes transpose view). ``trans_a``: a is [..., K, M] and is
    transposed inside the kernel."""
    _dev(a, 'a'), _dev(b, 'b')
    if b.dtype not in (torch.int8, torch.int16):
        raise ValueError('matmul RHS must use a signed integer precision.')
    if a.dtype not in (torch.int8, torch.uint8, torch.int16):
        raise NotImplementedError(f'matmul LHS must be int8, uint8 or int16, got {a.dtype}')
    if b.dtype == torch.int16 and a.dtype != torch.int16:
        raise RuntimeError('unsupported int8 x int16 precision mix for AIE implementations; no implementation variant available.')
    if a.dim() < 2 or b.dim() < 2:
        raise ValueError('matmul operands need rank >= 2')
    a, b = a.contiguous(), b.contiguous()
    M, K = (int(a.shape[-1]), int(a.shape[-2])) if trans_a else (int(a.shape[-2]), int(a.shape[-1]))
    N = int(b.shape[-2] if trans_b else b.shape[-1])
    Kb = int(b.shape[-1] if trans_b else b.shape[-2])
    if K != Kb:
        raise ValueError(f'matmul reduction extents differ: {K} vs {Kb}')
    lead = tuple(a.shape[:-2])
    if tuple(b.shape[:-2]) != lead:
        raise ValueError(f'matmul leading axes differ: {lead} vs {tuple(b.shape[:-2])}')
    batch = 1
    for d in lead:
        batch *= int(d)
    ok = _kind(out_kind)
    if out is None:
        out = torch.empty(lead + (M, N), dtype=_KIND_TORCH[ok], device=a.device)
    L = _lib.load()
    if a.dtype == torch.int16:  # 16-bit left operand: (16, 8) in acc32, (16, 16) in acc64
        bkind = _TORCH_KIND[b.dtype]
        need = int(L.a4g_matmul_i16_workspace_bytes(batch, N, K, bkind))
        if workspace is None or workspace.numel() * workspace.element_size() < need:
            workspace = torch.empty((need,), dtype=torch.uint8, device=a.device)
        check(L.a4g_matmul_i16(_ptr(a), int(bool(trans_a)), M if trans_a else K, M * K, _ptr(b), bkind, int(b.shape[-1]), K * N, int(bool(trans_b)), _ptr(out), N, M * N,
                               batch, M, N, K, int(shift), _mode(rounding), ok, _ptr(workspace),
                               workspace.numel() * workspace.element_size(), _stream()))
        return out
    akind = _TORCH_KIND[a.dtype]
    need = int(L.a4g_matmul_i8_workspace_bytes(batch, M, N, K, int(trans_b), akind))
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty((need,), dtype=torch.uint8, device=a.device)
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    check(L.a4g_matmul_i8(_ptr(a), akind, int(bool(trans_a)), M if trans_a else K, M * K, _ptr(b), int(b.shape[-1]), K * N,
                          int(bool(trans_b)), _ptr(out), N,
                          M * N, batch, M, N, K, int(shift), _mode(rounding), ok, _ptr(workspace), ws_bytes, _stream()))
    return out


def layernorm(x: torch.Tensor, gamma_q7: torch.Tensor, beta_q15: torch.Tensor, out_shift: int, rounding='floor',
              eps_q0: int = 1, gamma_shift: int = 7, out: Optional[torch.Tensor] = None):
    """Integer LayerNorm over the last axis, int8 -> int8. gamma int16 Q7, beta int16 Q15."""
    x2 = _rows2d(x, 'x').contiguous()
    if x2.dtype != torch.int8:
        raise NotImplementedError('integer LayerNorm needs signed 8-bit input and output')
    cols = int(x2.shape[1])
    g = _dev(gamma_q7, 'gamma').to(torch.int16).contiguous()
    b = _dev(beta_q15, 'beta').to(torch.int16).contiguous()
    if g.numel() != cols or b.numel() != cols:
        raise ValueError(f'LayerNorm parameter length does not match full_inner={cols}.')
    if out is None:
        out = torch.empty_like(x2).reshape(x.shape)
    check(_lib.load().a4g_layernorm_i8(_ptr(x2), _ptr(g), _ptr(b), _ptr(out), int(x2.shape[0]), cols, int(eps_q0),
                                       int(gamma_shift), int(out_shift), _mode(rounding), _stream()))
    return out


def add_layernorm(a: torch.Tensor, b: torch.Tensor, gamma_q7: torch.Tensor, beta_q15: torch.Tensor, out_shift: int,
                  rounding='floor', eps_q0: int = 1, gamma_shift: int = 7, add_shift: int = 0, add_rounding='floor',
                  return_sum: bool = False, out: Optional[torch.Tensor] = None, sum_out: Optional[torch.Tensor] = None):
    """Residual add fused in front of the LayerNorm (same result as add() then layernorm())."""
    if a.shape != b.shape or a.dtype != torch.int8 or b.dtype != torch.int8:
        raise ValueError('add_layernorm requires two int8 tensors of one shape')
    a2 = _rows2d(a, 'a').contiguous()
    b2 = _rows2d(b, 'b').contiguous()
    cols = int(a2.shape[1])
    g = _dev(gamma_q7, 'gamma').to(torch.int16).contiguous()
    bt = _dev(beta_q15, 'beta').to(torch.int16).contiguous()
    if g.numel() != cols or bt.numel() != cols:
        raise ValueError(f'LayerNorm parameter length does not match full_inner={cols}.')
    if out is None:
        out = torch.empty_like(a2).reshape(a.shape)
    elif out.shape != a.shape or out.dtype != torch.int8 or not out.is_contiguous():
        raise ValueError('add_layernorm: out must be a contiguous int8 tensor of the input shape')
    s = None
    if return_sum:
        s = sum_out if sum_out is not None else torch.empty_like(a2).reshape(a.shape)
        if s.shape != a.shape or s.dtype != torch.int8 or not s.is_contiguous():
            raise ValueError('add_layernorm: sum_out must be a contiguous int8 tensor of the input shape')
    check(_lib.load().a4g_add_layernorm_i8(_ptr(a2), _ptr(b2), int(add_shift), _mode(add_rounding), _ptr(g), _ptr(bt),
                                           _ptr(s), _ptr(out), int(a2.shape[0]), cols, int(eps_q0), int(gamma_shift),
                                           int(out_shift), _mode(rounding), _stream()))
    return (s, out) if return_sum else out


def dense_add_layernorm_applicable(x: torch.Tensor, p: PackedDense) -> bool:
    """Whether dense_add_layernorm() takes this Dense (the limits of a4g_dense_add_layernorm_i8)."""
    return (p.wt_lo is None and p.shift0 is not None and p.N % 32 == 0 and p.N <= 768 and p.K % 128 == 0 and p.K <= 4096
            and x.dtype in (torch.int8, torch.uint8) and x.dim() >= 1 and int(x.shape[-1]) == p.K)


def dense_add_layernorm_pays(rows: int, p: PackedDense) -> bool:
    """Whether the one-launch form is the faster one. Every workgroup of that kernel streams the whole weight matrix,
    one per 32 rows, and a single round of workgroups has nothing to hide its first loads and its normalisation behind;
    measured against dense() + add_layernorm() at 768 outputs: 768 inputs 12.2 / 14.1 / 23.1 us against 14.2 / 19.6 /
    28.7 us at 4096 / 8192 / 16384 rows, but 11.6 against 11.3 us at 2048 rows and 45.4 against 46.3 us at 32768;
    1024 inputs 16.1 against 22.1 us, 1536 inputs 20.2 against 25.2 us, 2048 inputs 26.1 against 27.9 us, 3072 inputs
    35.2 against 34.2 us (8192 rows); 512 -> 512: 11.0 against 13.7 us; 256 outputs (one 32-column block per wave) 8.8
    against 10.0 us at 8192 rows, 26.5 against 17.7 us at 32768. The LayerNorm's rounding mode does not matter: 13.3-14.9 us for
    every pair of modes at 8192 x 768 -> 768 against 17.7-19.0 us for the two launches."""
    return 4096 <= rows <= 16384 and p.K <= 1536 and p.N >= 384


def dense_add_layernorm(x: torch.Tensor, p: PackedDense, residual: Optional[torch.Tensor], gamma_q7: torch.Tensor,
                        beta_q15: torch.Tensor, out_shift: int, dense_rounding='floor', relu: bool = False,
                        rounding='floor', eps_q0: int = 1, gamma_shift: int = 7, out: Optional[torch.Tensor] = None):
    """layernorm(saturate_i8(dense(x) + residual)) in one launch: the same result as dense() (int8 output), add() with
    shift 0 and layernorm(). ``residual`` may be None. Raises NotImplementedError outside the limits of the fused kernel
    (dense_add_layernorm_applicable)."""
    if not dense_add_layernorm_applicable(x, p):
        raise NotImplementedError('dense_add_layernorm: needs int8 / uint8 rows, one shift, N % 32 == 0, N <= 768, '
                                  'K % 128 == 0, K <= 4096')
    x2 = _rows2d(x, 'x')
    if x2.stride(1) != 1 or x2.stride(0) % 16:
        x2 = x2.contiguous()
    M = int(x2.shape[0])
    r2 = None
    if residual is not None:
        if residual.dtype != torch.int8 or tuple(residual.shape) != tuple(x.shape[:-1]) + (p.N,):
            raise ValueError('dense_add_layernorm: the residual must be an int8 tensor of the output shape')
        r2 = _pitched_rows(residual, 'residual')  # a window of a wider tensor is read where it lies
    g = _dev(gamma_q7, 'gamma').to(torch.int16).contiguous()
    bt = _dev(beta_q15, 'beta').to(torch.int16).contiguous()
    if g.numel() != p.N or bt.numel() != p.N:
        raise ValueError(f'LayerNorm parameter length does not match full_inner={p.N}.')
    L = _lib.load()
    _rowpack(p)
    if out is None:
        out = torch.empty(tuple(x.shape[:-1]) + (p.N,), dtype=torch.int8, device=x.device)
    elif tuple(out.shape) != tuple(x.shape[:-1]) + (p.N,) or out.dtype != torch.int8:
        raise ValueError('dense_add_layernorm: out must be an int8 tensor of the output shape')
    o2 = _pitched_rows(out, 'out')
    if o2.data_ptr() != out.data_ptr():
        raise ValueError('dense_add_layernorm: out needs a contiguous last axis, a row pitch in whole 16 bytes and a 16-byte aligned start')
    check(L.a4g_dense_add_layernorm_i8(_ptr(x2), _TORCH_KIND[x2.dtype], x2.stride(0) if M > 0 else p.K, _ptr(p.wf),
                                       _ptr(p.colsum), _ptr(p.bias), int(p.shift0), _mode(dense_rounding), int(bool(relu)),
                                       _ptr(r2), _pitch(r2) if r2 is not None else p.N, _ptr(g), _ptr(bt), _ptr(o2),
                                       _pitch(o2) if M > 0 else p.N, M, p.N, p.K, int(eps_q0),
                                       int(gamma_shift), int(out_shift), _mode(rounding), _stream()))
    return out


def softmax_exp(x: torch.Tensor, exp_kq: int, inv_shift: int = 15, out_kind='uint8', out: Optional[torch.Tensor] = None):
    """Accurate integer-exp Softmax over the last axis: int8 -> uint8 (scale 1/256) or int16."""
    x2 = _rows2d(x, 'x').contiguous()
    if x2.dtype != torch.int8:
        raise NotImplementedError('integer Softmax needs int8 input')
    ok = _kind(out_kind)
    if out is None:
        out = torch.empty(x.shape, dtype=_KIND_TORCH.get(ok, torch.uint8), device=x.device)
    check(_lib.load().a4g_softmax_exp_i8(_ptr(x2), _ptr(out), int(x2.shape[0]), int(x2.shape[1]), int(exp_kq),
                                         int(inv_shift), ok, _stream()))
    return out


def softmax_hccs(x: torch.Tensor, B: int, S: int, Dmax: int, inv_shift: int = 15, use_clb: bool = False,
                 out_kind='uint8', out: Optional[torch.Tensor] = None):
    """HCCS clipped-linear surrogate Softmax over the last axis."""
    x2 = _rows2d(x, 'x').contiguous()
    if x2.dtype != torch.int8:
        raise NotImplementedError('integer Softmax needs int8 input')
    ok = _kind(out_kind)
    if out is None:
        out = torch.empty(x.shape, dtype=_KIND_TORCH.get(ok, torch.uint8), device=x.device)
    check(_lib.load().a4g_softmax_hccs_i8(_ptr(x2), _ptr(out), int(x2.shape[0]), int(x2.shape[1]), int(B), int(S),
                                          int(Dmax), int(inv_shift), int(bool(use_clb)), ok, _stream()))
    return out


@dataclass
class MlpLayerSpec:
    params: PackedDense
    shift: int
    relu: bool
    out_kind: str = 'int8'


def mlp_runs_on_matrix_units(rows: int, x_pitch: int, layers: Sequence[Tuple[int, int]], last_out_kind='int8',
                             y_pitch: Optional[int] = None) -> bool:
    """Whether a4g_mlp_i8 takes its large-batch form for this chain (``layers``: (K, N) per layer; ``x_pitch``: bytes
    between input rows, 0 if unknown; ``y_pitch``: elements between result rows, the last width if not given): from 512
    rows, an 8-bit last layer, weight fragments of 1 KiB per 32 x 32 block plus 128 bytes of start values per 32
    neurons within 128 KiB of LDS, and both ends addressable with 32-bit offsets (the conditions of csrc/mlp.hip)."""
    blocks = sum(((k + 31) // 32) * ((n + 31) // 32) for k, n in layers) + 1
    start = sum((n + 31) // 32 * 32 for _k, n in layers)
    ldy = int(y_pitch) if y_pitch else layers[-1][1]
    limit = (1 << 31) - 64
    return (rows >= 512 and x_pitch >= 1 and _kind(last_out_kind) in (0, 1) and blocks * 1024 + start * 4 + 32 <= 128 * 1024
            and (rows - 1) * x_pitch + layers[0][0] < limit and ((rows - 1) * ldy + layers[-1][1]) * 2 < limit)


def mlp(x: torch.Tensor, layers: Sequence[MlpLayerSpec], rounding='floor', out: Optional[torch.Tensor] = None):
    """Whole MLP in one launch (weights resident in LDS). x: [batch, K0] int8/uint8; rows of a wider matrix are taken
    where they lie."""
    x2 = _rows2d(x, 'x')
    if x2.stride(1) != 1 or (x2.shape[0] > 1 and x2.stride(0) < x2.shape[1]):
        x2 = x2.contiguous()
    n = len(layers)
    arr = (MlpLayer * max(n, 1))()
    keep: List[torch.Tensor] = []
    for i, spec in enumerate(layers):
        p = spec.params
        arr[i].wt = p.wt.data_ptr()
        arr[i].ldwt = p.ldwt
        arr[i].colsum = p.colsum.data_ptr()
        arr[i].bias = p.bias.data_ptr() if p.bias is not None else None
        arr[i].K, arr[i].N = p.K, p.N
        arr[i].shift = int(spec.shift)
        arr[i].relu = int(bool(spec.relu))
        arr[i].out_kind = _kind(spec.out_kind)
        keep.append(p.wt)
    last = layers[-1]
    ok = _kind(last.out_kind)
    if out is None:
        out = torch.empty((x2.shape[0], last.params.N), dtype=_KIND_TORCH[ok], device=x.device)
    check(_lib.load().a4g_mlp_i8(arr, n, _ptr(x2), _TORCH_KIND[x2.dtype], x2.stride(0) if x2.shape[0] else x2.shape[1],
                                 _ptr(out), out.stride(0) if out.shape[0] else last.params.N, int(x2.shape[0]),
                                 _mode(rounding), _stream()))
    return out


def _mlp_layer_array(layers: Sequence[MlpLayerSpec]):
    arr = (MlpLayer * max(len(layers), 1))()
    for i, spec in enumerate(layers):
        p = spec.params
        arr[i].wt = p.wt.data_ptr()
        arr[i].ldwt = p.ldwt
        arr[i].colsum = p.colsum.data_ptr()
        arr[i].bias = p.bias.data_ptr() if p.bias is not None else None
        arr[i].K, arr[i].N = p.K, p.N
        arr[i].shift = int(spec.shift)
        arr[i].relu = int(bool(spec.relu))
        arr[i].out_kind = _kind(spec.out_kind)
    return arr


def mlp_add_layernorm_applicable(x: torch.Tensor, layers: Sequence[MlpLayerSpec]) -> bool:
    """Whether mlp_add_layernorm() takes this chain (the limits of a4g_mlp_add_layernorm_i8)."""
    if not layers or len(layers) > 8 or x.dtype not in (torch.int8, torch.uint8) or x.dim() < 1:
        return False
    shapes = [(s.params.K, s.params.N) for s in layers]
    last = layers[-1]
    blocks = sum(((k + 31) // 32) * ((n + 31) // 32) for k, n in shapes) + 1
    start = sum((n + 31) // 32 * 32 for _k, n in shapes)
    return (all(s.params.wt_lo is None and s.params.K <= 256 and s.params.N <= 256 for s in layers)
            and all(a[1] == b[0] for a, b in zip(shapes[:-1], shapes[1:])) and int(x.shape[-1]) == shapes[0][0]
            and all(_kind(s.out_kind) in (0, 1) for s in layers) and _kind(last.out_kind) == 0 and last.params.N % 16 == 0
            and sum(s.params.N * s.params.ldwt for s in layers) <= 96 * 1024
            and blocks * 1024 + start * 4 + 32 + 8 * last.params.N + 16 <= 128 * 1024)


def mlp_add_layernorm_pays(rows: int, shapes: Sequence[Tuple[int, int]]) -> bool:
    """Whether the one-launch form is the faster one (``shapes``: (K, N) per layer). Its normalisation is serial work of
    the two lanes that hold a row, where the row kernel spreads a row over as many lanes as it has 16-byte pieces: the
    launch it saves pays up to 128 columns. Measured against mlp() + add_layernorm() at 2048 / 32768 / 131072 rows:
    64 -> 64: 9.6 / 10.3 / 14.9 us against 11.6 / 12.3 / 17.2; 64 -> 128 -> 64: 13.2 / 13.9 / 21.5 against 14.5 / 15.6 /
    22.6; 128 -> 128: 13.1 / 13.9 / 25.9 against 13.8 / 16.0 / 29.2; but 64 -> 256 -> 64: 17.8 / 19.2 / 32.8 against
    17.5 / 19.0 / 31.0 and 256 -> 256: 25.2 / 28.0 / 44.7 against 20.3 / 25.1 / 48.3."""
    return rows >= 1 and all(k <= 128 and n <= 128 for k, n in shapes)


def mlp_add_layernorm(x: torch.Tensor, layers: Sequence[MlpLayerSpec], residual: Optional[torch.Tensor], gamma_q7: torch.Tensor,
                      beta_q15: torch.Tensor, out_shift: int, rounding='floor', ln_rounding='floor', eps_q0: int = 1,
                      gamma_shift: int = 7, out: Optional[torch.Tensor] = None):
    """layernorm(saturate_i8(mlp(x) + residual)) in one launch: the same result as mlp() (int8 last layer), add() with
    shift 0 and layernorm(). ``residual`` may be None. Raises NotImplementedError outside the limits of the fused kernel
    (mlp_add_layernorm_applicable)."""
    if not mlp_add_layernorm_applicable(x, layers):
        raise NotImplementedError('mlp_add_layernorm: needs int8 / uint8 rows, up to 8 layers up to 256 wide whose fragments fit '
                                  '128 KiB of LDS, and an int8 last layer of N % 16 == 0 columns')
    x2 = _rows2d(x, 'x')
    if x2.stride(1) != 1 or (x2.shape[0] > 1 and x2.stride(0) < x2.shape[1]):
        x2 = x2.contiguous()
    M, N = int(x2.shape[0]), layers[-1].params.N
    r2 = None
    if residual is not None:
        if residual.dtype != torch.int8 or tuple(residual.shape) != tuple(x.shape[:-1]) + (N,):
            raise ValueError('mlp_add_layernorm: the residual must be an int8 tensor of the output shape')
        r2 = _pitched_rows(residual, 'residual')  # a window of a wider tensor is read where it lies
    g = _dev(gamma_q7, 'gamma').to(torch.int16).contiguous()
    bt = _dev(beta_q15, 'beta').to(torch.int16).contiguous()
    if g.numel() != N or bt.numel() != N:
        raise ValueError(f'LayerNorm parameter length does not match full_inner={N}.')
    if out is None:
        out = torch.empty(tuple(x.shape[:-1]) + (N,), dtype=torch.int8, device=x.device)
    elif tuple(out.shape) != tuple(x.shape[:-1]) + (N,) or out.dtype != torch.int8:
        raise ValueError('mlp_add_layernorm: out must be an int8 tensor of the output shape')
    o2 = _pitched_rows(out, 'out')
    if o2.data_ptr() != out.data_ptr():
        raise ValueError('mlp_add_layernorm: out needs a contiguous last axis, a row pitch in whole 16 bytes and a 16-byte aligned start')
    arr = _mlp_layer_array(layers)
    check(_lib.load().a4g_mlp_add_layernorm_i8(
        arr, len(layers), _ptr(x2), _TORCH_KIND[x2.dtype], x2.stride(0) if M > 0 else layers[0].params.K, _ptr(r2),
        _pitch(r2) if r2 is not None else N, _ptr(g), _ptr(bt), _ptr(o2), _pitch(o2) if M > 0 else N, M, _mode(rounding), int(eps_q0), int(gamma_shift), int(out_shift), _mode(ln_rounding), _stream()))
    return out


def attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, logit_shift: int, logit_rounding, softmax: dict,
              out_shift: int, out_rounding, out: Optional[torch.Tensor] = None):
    """Fused attention core: srs(softmax(srs(q k^T)) v) per (batch, head), one launch.

    q: [..., sq, d], k and v: [..., sk, d] int8 with up to two leading axes (batch, head); any strides with a
    contiguous last axis (head slices of a packed projection are fine). `softmax` is
    {'kind': 'exp', 'exp_kq': .., 'inv_shift': 15} or {'kind': 'hccs', 'B': .., 'S': .., 'Dmax': .., 'inv_shift': 15,
    'use_clb': False}. Bit-identical to matmul(trans_b) -> softmax_* -> matmul. Raises NotImplementedError for
    shapes the fused kernel does not cover (head_dim not a multiple of 16 or above 128, more than 512 keys - 256 from
    head_dim 80 on -, unaligned views). Head dimensions 16, 48, 80, 96 and 112 run on the next wider kernel (32, 64, 128) with the pieces of a
    row that do not exist masked inside it.
    """
    for name, t in (('q', q), ('k', k), ('v', v)):
        _dev(t, name)
        if t.dtype != torch.int8 or t.dim() < 2 or t.dim() > 4 or t.stride(-1) != 1:
            raise ValueError(f'attention: {name} must be int8 with 2..4 axes and a contiguous last axis')
    if k.shape != v.shape or q.shape[:-2] != k.shape[:-2] or q.shape[-1] != k.shape[-1]:
        raise ValueError(f'attention: incompatible shapes {tuple(q.shape)}, {tuple(k.shape)}, {tuple(v.shape)}')
    lead = tuple(q.shape[:-2])
    sq, d, sk = int(q.shape[-2]), int(q.shape[-1]), int(k.shape[-2])
    if out is None:
        out = torch.empty(lead + (sq, d), dtype=torch.int8, device=q.device)
    elif out.shape != lead + (sq, d) or out.dtype != torch.int8 or out.stride(-1) != 1:
        raise ValueError('attention: out must be int8 of shape [..., sq, d] with a contiguous last axis')

    def strides3(t):  # (batch, head, row) byte strides with missing leading axes as 0
        st = [0] * (4 - t.dim()) + [int(x) for x in t.stride()]
        return st[0], st[1], st[2]

    batch = int(lead[0]) if len(lead) >= 1 else 1
    heads = int(lead[1]) if len(lead) == 2 else 1
    if len(lead) == 1:  # [batch, s, d]: one head
        flat = [(int(t.stride(0)), 0, int(t.stride(1))) for t in (q, k, v, out)]
    else:
        flat = [strides3(t) for t in (q, k, v, out)]
    arr = (ctypes.c_int64 * 12)(*[x for trip in flat for x in trip])
    kind = softmax.get('kind', 'exp')
    if kind not in ('exp', 'hccs'):
        raise ValueError(f"attention: unknown softmax kind {kind!r}")
    check(_lib.load().a4g_attention_i8(_ptr(q), _ptr(k), _ptr(v), _ptr(out), batch, heads, sq, sk, d, arr, int(logit_shift),
                                       _mode(logit_rounding), 0 if kind == 'exp' else 1, int(softmax.get('exp_kq', 1)),
                                       int(softmax.get('B', 0)), int(softmax.get('S', 0)), int(softmax.get('Dmax', 0)),
                                       int(softmax.get('inv_shift', 15)), int(bool(softmax.get('use_clb', False))),
                                       int(out_shift), _mode(out_rounding), _stream()))
    return out


# ---- floating-point compute path (bfloat16 / float32 operands, float32 accumulation) ---------------------------

_TORCH_FLOAT = {torch.bfloat16: 16, torch.float32: 17, torch.float8_e4m3fn: 18}


def _float_format(t: torch.Tensor, name: str) -> int:
    try:
        return _TORCH_FLOAT[t.dtype]
    except KeyError:
        raise NotImplementedError(f'{name}: the float path takes bfloat16, float32 or float8_e4m3fn tensors, got {t.dtype}') from None


@dataclass
class PackedDenseFloat:
    """Device-resident float Dense parameters: weights [N, ldwt] with the reduction axis contiguous."""

    wt: torch.Tensor
    bias: Optional[torch.Tensor]  # [N] float32 or None
    K: int
    N: int

    @property
    def ldwt(self) -> int:
        return int(self.wt.shape[1])


def pack_dense_float(weight: torch.Tensor, bias: Optional[torch.Tensor]) -> PackedDenseFloat:
    """weight: logical [K, N] bfloat16 / float32 on the device; bias: [N] (kept in float32) or None."""
    _dev(weight, 'weight')
    fmt = _float_format(weight, 'weight')
    if weight.dim() != 2:
        raise ValueError('weight matrix must be a rank-2 tensor')
    weight = weight.contiguous()
    K, N = int(weight.shape[0]), int(weight.shape[1])
    L = _lib.load()
    wt = torch.empty((N, int(L.a4g_packed_ld_f(K, fmt))), dtype=weight.dtype, device=weight.device)
    check(L.a4g_pack_weights_f(_ptr(weight), fmt, N, K, N, _ptr(wt), _stream()))
    if bias is not None:
        bias = _dev(bias, 'bias').to(torch.float32).contiguous()
        if bias.numel() != N:
            raise ValueError(f'dense bias requires exactly {N} elements, got {bias.numel()}.')
    return PackedDenseFloat(wt=wt, bias=bias, K=K, N=N)


def dense_float(x: torch.Tensor, p: PackedDenseFloat, relu: bool = False, out: Optional[torch.Tensor] = None,
                trans_a: bool = False):
    """y = fmt(relu?(bias + x @ W)) with float32 accumulation; x: [..., K] in the weights' format. ``trans_a``: x is
    [..., K, M] and is transposed inside the kernel, one launch per leading index."""
    if trans_a:
        _dev(x, 'x')
        fmt = _float_format(x, 'x')
        if x.dtype != p.wt.dtype:
            raise ValueError(f'float dense requires lhs/rhs/output to share float precision, got {x.dtype} and {p.wt.dtype}.')
        if x.dim() < 2 or int(x.shape[-2]) != p.K:
            raise ValueError(f'dense input (transposed) has {tuple(x.shape)}, weights expect {p.K} on the second-to-last axis')
        xs = x.contiguous().reshape(-1, p.K, int(x.shape[-1]))
        Mt = int(xs.shape[-1])
        if out is None:
            out = torch.empty(tuple(x.shape[:-2]) + (Mt, p.N), dtype=x.dtype, device=x.device)
        ys = out.reshape(-1, Mt, p.N)
        for i in range(int(xs.shape[0])):
            check(_lib.load().a4g_dense_f(_ptr(xs[i]), fmt, 1, Mt, _ptr(p.wt), p.ldwt, _ptr(p.bias), int(bool(relu)), _ptr(ys[i]), p.N,
                                          Mt, p.N, p.K, _stream()))
        return out
    x2 = _rows2d(x, 'x')
    fmt = _float_format(x2, 'x')
    if x2.dtype != p.wt.dtype:
        raise ValueError(f'float dense requires lhs/rhs/output to share float precision, got {x2.dtype} and {p.wt.dtype}.')
    if x2.shape[1] != p.K:
        raise ValueError(f'dense input has {x2.shape[1]} features, weights expect {p.K}')
    M = int(x2.shape[0])
    if out is None:
        out = torch.empty(tuple(x.shape[:-1]) + (p.N,), dtype=x.dtype, device=x.device)
    y2 = out.reshape(-1, p.N)
    check(_lib.load().a4g_dense_f(_ptr(x2), fmt, 0, x2.stride(0) if M > 0 else p.K, _ptr(p.wt), p.ldwt, _ptr(p.bias),
                                  int(bool(relu)), _ptr(y2), y2.stride(0) if M > 0 else p.N, M, p.N, p.K, _stream()))
    return out


def matmul_float(a: torch.Tensor, b: torch.Tensor, trans_b: bool = False, out: Optional[torch.Tensor] = None,
                 workspace: Optional[torch.Tensor] = None, trans_a: bool = False):
    """Batched float MatMul. a: [..., M, K] (``trans_a``: [..., K, M], transposed inside the kernel); b: [..., K, N], or
    [..., N, K] when ``trans_b``."""
    _dev(a, 'a'), _dev(b, 'b')
    fmt = _float_format(a, 'a')
    if a.dtype != b.dtype:
        raise ValueError(f'float matmul requires lhs/rhs/output to share float precision, got {a.dtype} and {b.dtype}.')
    if a.dim() < 2 or b.dim() < 2:
        raise ValueError('matmul operands need rank >= 2')
    a, b = a.contiguous(), b.contiguous()
    M, K = (int(a.shape[-1]), int(a.shape[-2])) if trans_a else (int(a.shape[-2]), int(a.shape[-1]))
    N = int(b.shape[-2] if trans_b else b.shape[-1])
    Kb = int(b.shape[-1] if trans_b else b.shape[-2])
    if K != Kb:
        raise ValueError(f'matmul reduction extents differ: {K} vs {Kb}')
    lead = tuple(a.shape[:-2])
    if tuple(b.shape[:-2]) != lead:
        raise ValueError(f'matmul leading axes differ: {lead} vs {tuple(b.shape[:-2])}')
    batch = 1
    for d in lead:
        batch *= int(d)
    if out is None:
        out = torch.empty(lead + (M, N), dtype=a.dtype, device=a.device)
    L = _lib.load()
    need = int(L.a4g_matmul_f_workspace_bytes(batch, N, K, int(trans_b), fmt))
    if need and (workspace is None or workspace.numel() * workspace.element_size() < need):
        workspace = torch.empty((need,), dtype=torch.uint8, device=a.device)
    ws_bytes = workspace.numel() * workspace.element_size() if workspace is not None else 0
    check(L.a4g_matmul_f(_ptr(a), fmt, int(bool(trans_a)), M if trans_a else K, M * K, _ptr(b), int(b.shape[-1]), K * N, int(bool(trans_b)), _ptr(out), N, M * N,
                         batch, M, N, K, _ptr(workspace), ws_bytes, _stream()))
    return out


def add_float(a: torch.Tensor, b: torch.Tensor, out: Optional[torch.Tensor] = None):
    """Elementwise a + b in float32, rounded to the operands' format."""
    _dev(a, 'a'), _dev(b, 'b')
    if a.shape != b.shape:
        raise ValueError(f'elementwise Add requires exact-shape inputs, got {tuple(a.shape)} and {tuple(b.shape)}.')
    if a.dtype != b.dtype:
        raise ValueError('elementwise Add requires lhs/rhs/output to use the same storage type.')
    fmt = _float_format(a, 'a')
    a, b = a.contiguous(), b.contiguous()
    if out is None:
        out = torch.empty_like(a)
    check(_lib.load().a4g_add_f(_ptr(a), _ptr(b), _ptr(out), a.numel(), fmt, _stream()))
    return out
