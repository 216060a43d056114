// Shared device helpers: shift-round-saturate, storage kinds, wave-level reductions, error plumbing.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/aie4ml_gfx950.h"

namespace a4g {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef short v2s __attribute__((ext_vector_type(2)));
typedef unsigned short v2us __attribute__((ext_vector_type(2)));

// ---- host-side error plumbing -------------------------------------------------------------------
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);
int check_hip(hipError_t e, const char* what);

#define A4G_REQUIRE(cond, code, ...)                    \
    do {                                                \
        if (!(cond)) return ::a4g::fail(code, __VA_ARGS__); \
    } while (0)

static inline bool valid_round(int m) { return m >= 0 && m <= 7; }
static inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static inline int kind_bytes(int kind) { return (kind == A4G_I8 || kind == A4G_U8) ? 1 : (kind == A4G_I32 ? 4 : 2); }

// ---- rounding ---------------------------------------------------------------------------------------
// round(acc / 2^s) for the eight aie::rounding_mode values; s in [0,31]. 32-bit only: the quotient
// plus a 0/1 increment never overflows for s >= 1.
template <int MODE>
__device__ __forceinline__ int round_shift(int acc, int s) {
    if (s == 0) return acc;
    const int q = acc >> s;
    if (MODE == A4G_RND_FLOOR) return q;
    const unsigned mask = (1u << s) - 1u;
    const unsigned r = static_cast<unsigned>(acc) & mask;
    const unsigned h = 1u << (s - 1);
    if (MODE == A4G_RND_CEIL) return q + (r != 0u);
    if (MODE == A4G_RND_POSITIVE_INF) return q + (r >= h);
    if (MODE == A4G_RND_NEGATIVE_INF) return q + (r > h);
    if (MODE == A4G_RND_SYMMETRIC_INF) return q + ((r > h) | ((r == h) & (acc >= 0)));
    if (MODE == A4G_RND_SYMMETRIC_ZERO) return q + ((r > h) | ((r == h) & (acc < 0)));
    if (MODE == A4G_RND_CONV_EVEN) return q + ((r > h) | ((r == h) & (q & 1)));
    /* conv_odd */ return q + ((r > h) | ((r == h) & ((q & 1) == 0)));
}

__device__ __forceinline__ int round_shift_rt(int acc, int s, int mode) {
    switch (mode) {
    case A4G_RND_FLOOR: return round_shift<A4G_RND_FLOOR>(acc, s);
    case A4G_RND_CEIL: return round_shift<A4G_RND_CEIL>(acc, s);
    case A4G_RND_POSITIVE_INF: return round_shift<A4G_RND_POSITIVE_INF>(acc, s);
    case A4G_RND_NEGATIVE_INF: return round_shift<A4G_RND_NEGATIVE_INF>(acc, s);
    case A4G_RND_SYMMETRIC_INF: return round_shift<A4G_RND_SYMMETRIC_INF>(acc, s);
    case A4G_RND_SYMMETRIC_ZERO: return round_shift<A4G_RND_SYMMETRIC_ZERO>(acc, s);
    case A4G_RND_CONV_EVEN: return round_shift<A4G_RND_CONV_EVEN>(acc, s);
    default: return round_shift<A4G_RND_CONV_ODD>(acc, s);
    }
}

// The same eight modes without a per-element switch: every mode is floor((acc + off) / 2^s) with
// off = c0 + cx * bit, where bit is either the sign of acc or the parity of the floor quotient.
// The offset is added to the remainder, not to acc, so nothing can overflow.
struct RoundCfg {
    int s;          // shift, 0..31
    unsigned mask;  // 2^s - 1
    int c0, cx;     // offset constants
    int bs;         // which bit of acc feeds `bit`: 31 (sign) or s (quotient parity)
};

__host__ __device__ __forceinline__ RoundCfg make_round(int mode, int s) {
    RoundCfg rc;
    rc.s = s;
    rc.mask = s > 0 ? ((1u << s) - 1u) : 0u;
    rc.c0 = 0;
    rc.cx = 0;
    rc.bs = 31;
    if (s <= 0) return rc;
    const int h = 1 << (s - 1);
    switch (mode) {
    case A4G_RND_FLOOR: break;
    case A4G_RND_CEIL: rc.c0 = static_cast<int>(rc.mask); break;
    case A4G_RND_POSITIVE_INF: rc.c0 = h; break;
    case A4G_RND_NEGATIVE_INF: rc.c0 = h - 1; break;
    case A4G_RND_SYMMETRIC_INF: rc.c0 = h; rc.cx = -1; break;
    case A4G_RND_SYMMETRIC_ZERO: rc.c0 = h - 1; rc.cx = 1; break;
    case A4G_RND_CONV_EVEN: rc.c0 = h - 1; rc.cx = 1; rc.bs = s; break;
    default: rc.c0 = h; rc.cx = -1; rc.bs = s; break;  // conv_odd
    }
    return rc;
}

__device__ __forceinline__ int apply_round(int acc, const RoundCfg& rc) {
    const int q = acc >> rc.s;
    const unsigned r = static_cast<unsigned>(acc) & rc.mask;
    const int bit = (acc >> rc.bs) & 1;
    const unsigned t = r + static_cast<unsigned>(rc.c0 + rc.cx * bit);
    return q + static_cast<int>(t >> rc.s);
}

// Cheaper form for accumulators of bounded magnitude: three VALU instructions per value.
struct FastRound {  // (acc + c0 + cx * bit) >> s, bit = one bit of acc at `pos` (width w = 0 disables it)
    int s, c0, pos, w, cx;
};

static inline FastRound make_fast_round(int mode, int s) {
    FastRound r{s, 0, 31, 0, 0};
    if (s <= 0) return r;
    const int h = 1 << (s - 1);
    switch (mode) {
    case A4G_RND_FLOOR: break;
    case A4G_RND_CEIL: r.c0 = (1 << s) - 1; break;
    case A4G_RND_POSITIVE_INF: r.c0 = h; break;
    case A4G_RND_NEGATIVE_INF: r.c0 = h - 1; break;
    case A4G_RND_SYMMETRIC_INF: r.c0 = h; r.cx = -1; r.w = 1; break;
    case A4G_RND_SYMMETRIC_ZERO: r.c0 = h - 1; r.cx = 1; r.w = 1; break;
    case A4G_RND_CONV_EVEN: r.c0 = h - 1; r.cx = 1; r.w = 1; r.pos = s; break;
    default: r.c0 = h; r.cx = -1; r.w = 1; r.pos = s; break;  // conv_odd
    }
    return r;
}

// Callers guarantee |acc| + 2^s < 2^31 (short reductions of 8-bit products, s <= 24), so nothing overflows.
__device__ __forceinline__ int fast_round(int acc, const FastRound& r) {
    const int bit = static_cast<int>(__builtin_amdgcn_ubfe(static_cast<unsigned>(acc), r.pos, r.w));
    return (acc + r.c0 + __mul24(bit, r.cx)) >> r.s;
}

// The same with the bit's sign fixed at compile time: BIT 0 no bit, 1 add it, 2 subtract it (kind from
// fast_round_kind). Two or three VALU instructions per value.
static inline int fast_round_kind(const FastRound& r) { return r.w == 0 || r.cx == 0 ? 0 : (r.cx > 0 ? 1 : 2); }
template <int BIT>
__device__ __forceinline__ int fast_round_k(int acc, const FastRound& r) {
    int bit = 0;
    if (BIT == 1) bit = static_cast<int>(__builtin_amdgcn_ubfe(static_cast<unsigned>(acc), r.pos, 1));
    if (BIT == 2) bit = __builtin_amdgcn_sbfe(acc, r.pos, 1);
    return (acc + r.c0 + bit) >> r.s;
}

__device__ __forceinline__ int clamp_i(int v, int lo, int hi) { return min(max(v, lo), hi); }

// clamp_i as one instruction for bounds that are only known at run time (callers guarantee lo <= hi,
// which the compiler would have to prove before it forms the median by itself).
// Not to be the first reader of an MFMA result: the compiler's hazard recogniser does not look into inline asm, so it
// inserts no wait states between the MFMA and this instruction. Every caller either applies it to a sum formed by an
// ordinary instruction, or reads the accumulator through one first (mlp_mfma_kernel).
__device__ __forceinline__ int clamp_med3(int v, int lo, int hi) {
    int y;
    asm("v_med3_i32 %0, %1, %2, %3" : "=v"(y) : "v"(v), "v"(lo), "v"(hi));
    return y;
}

// Low bytes of four ints -> one dword, through v_perm_b32. Shift-and-or packing of clamped shifts is
// avoided on purpose: the compiler folds that shape into gfx950's v_ashr_pk_u8_i32 / _i8_i32 and then
// treats the upper half of its result as zero, which the hardware does not guarantee.
__device__ __forceinline__ unsigned pack4_bytes(int y0, int y1, int y2, int y3) {
    const unsigned lo = __builtin_amdgcn_perm(static_cast<unsigned>(y1), static_cast<unsigned>(y0), 0x0c0c0400u);
    const unsigned hi = __builtin_amdgcn_perm(static_cast<unsigned>(y3), static_cast<unsigned>(y2), 0x04000c0cu);
    return lo | hi;
}
// Low halves of two ints -> one dword.
__device__ __forceinline__ unsigned pack2_halves(int y0, int y1) {
    return __builtin_amdgcn_perm(static_cast<unsigned>(y1), static_cast<unsigned>(y0), 0x05040100u);
}

// Requantise four accumulators straight into the four bytes of one dword: the clamp is applied before the shift
// (to [lo << s, (hi << s) + 2^s - 1], which selects exactly the sums whose shifted value lies in [lo, hi]) and the
// shift then writes its low byte into byte n of the result (SDWA destination select, other bytes preserved), so
// no separate packing instructions are needed. Valid for hi << s within int32 (s <= 22 for 8-bit outputs).
struct ByteRequant {
    FastRound fr;
    int lo_s, hi_s;
};
static inline ByteRequant make_byte_requant(const FastRound& fr, int lo, int hi) {
    ByteRequant b;
    b.fr = fr;
    b.lo_s = static_cast<int>(static_cast<unsigned>(lo) << fr.s);
    b.hi_s = static_cast<int>((static_cast<unsigned>(hi) << fr.s) | ((1u << fr.s) - 1u));
    return b;
}
static inline bool byte_requant_ok(const FastRound& fr) { return fr.s >= 0 && fr.s <= 22; }

template <int N>
__device__ __forceinline__ void shift_into_byte(unsigned& packed, int v, int s) {
    if (N == 0) asm("v_ashrrev_i32_sdwa %0, %1, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(packed) : "v"(s), "v"(v));
    if (N == 1) asm("v_ashrrev_i32_sdwa %0, %1, %2 dst_sel:BYTE_1 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(packed) : "v"(s), "v"(v));
    if (N == 2) asm("v_ashrrev_i32_sdwa %0, %1, %2 dst_sel:BYTE_2 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(packed) : "v"(s), "v"(v));
    if (N == 3) asm("v_ashrrev_i32_sdwa %0, %1, %2 dst_sel:BYTE_3 dst_unused:UNUSED_PRESERVE src0_sel:DWORD src1_sel:DWORD" : "+v"(packed) : "v"(s), "v"(v));
}

// acc[0..3] -> one dword of four requantised bytes (rounding kind BIT as in fast_round_k).
template <int BIT>
__device__ __forceinline__ unsigned requant4_bytes(int a0, int a1, int a2, int a3, const ByteRequant& b) {
    auto pre = [&](int acc) {
        int bit = 0;
        if (BIT == 1) bit = static_cast<int>(__builtin_amdgcn_ubfe(static_cast<unsigned>(acc), b.fr.pos, 1));
        if (BIT == 2) bit = __builtin_amdgcn_sbfe(acc, b.fr.pos, 1);
        return clamp_med3(acc + b.fr.c0 + bit, b.lo_s, b.hi_s);
    };
    unsigned packed;  // byte 0 is written with the other bytes zeroed, bytes 1..3 are then merged in
    {
        const int v0 = pre(a0);
        asm("v_ashrrev_i32_sdwa %0, %1, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:DWORD"
            : "=v"(packed)
            : "v"(b.fr.s), "v"(v0));
    }
    shift_into_byte<1>(packed, pre(a1), b.fr.s);
    shift_into_byte<2>(packed, pre(a2), b.fr.s);
    shift_into_byte<3>(packed, pre(a3), b.fr.s);
    return packed;
}

// The same with the rounding bit's position, width and sign given at run time (|acc| + 2^s < 2^31, s <= 22).
__device__ __forceinline__ unsigned requant4_bytes_rt(int a0, int a1, int a2, int a3, const ByteRequant& b) {
    auto pre = [&](int acc) {
        const int bit = static_cast<int>(__builtin_amdgcn_ubfe(static_cast<unsigned>(acc), b.fr.pos, b.fr.w));
        return clamp_med3(acc + b.fr.c0 + __mul24(bit, b.fr.cx), b.lo_s, b.hi_s);
    };
    unsigned packed = 0;
    shift_into_byte<0>(packed, pre(a0), b.fr.s);
    shift_into_byte<1>(packed, pre(a1), b.fr.s);
    shift_into_byte<2>(packed, pre(a2), b.fr.s);
    shift_into_byte<3>(packed, pre(a3), b.fr.s);
    return packed;
}

// Actual column (within a block of 32) whose weights the lanes j and j + 32 supply as row j of the MFMA's first operand:
// accumulator register 4g + i of lane (m, half) is output column 8g + 4half + i of the block, and we want that to be
// actual column 16half + 4g + i, so that a lane's 16 registers are 16 neighbouring bytes of its output row.
__device__ __forceinline__ int direct_col_of_operand_row(int j) { return ((j >> 2) & 1) * 16 + (j >> 3) * 4 + (j & 3); }

__device__ __forceinline__ int kind_lo(int kind) {
    return kind == A4G_I8 ? -128 : (kind == A4G_I16 ? -32768 : (kind == A4G_I32 ? INT32_MIN : 0));
}
__device__ __forceinline__ int kind_hi(int kind) {
    return kind == A4G_I8 ? 127 : (kind == A4G_U8 ? 255 : (kind == A4G_I16 ? 32767 : (kind == A4G_U16 ? 65535 : INT32_MAX)));
}

__device__ __forceinline__ int load_kind(const void* p, int64_t i, int kind) {
    switch (kind) {
    case A4G_I8: return static_cast<const int8_t*>(p)[i];
    case A4G_U8: return static_cast<const uint8_t*>(p)[i];
    case A4G_I16: return static_cast<const int16_t*>(p)[i];
    case A4G_U16: return static_cast<const uint16_t*>(p)[i];
    default: return static_cast<const int32_t*>(p)[i];
    }
}
__device__ __forceinline__ void store_kind(void* p, int64_t i, int kind, int v) {
    switch (kind) {
    case A4G_I8: static_cast<int8_t*>(p)[i] = static_cast<int8_t>(v); break;
    case A4G_U8: static_cast<uint8_t*>(p)[i] = static_cast<uint8_t>(v); break;
    case A4G_I16: static_cast<int16_t*>(p)[i] = static_cast<int16_t>(v); break;
    case A4G_U16: static_cast<uint16_t*>(p)[i] = static_cast<uint16_t>(v); break;
    default: static_cast<int32_t*>(p)[i] = v; break;
    }
}

// ---- cross-lane helpers (64-wide wavefront) -------------------------------------------------------------
// xor-butterfly partner exchange. Masks 1,2 use DPP quad permutes, 4 and 8 the row mirrors (valid
// as reduction steps once the lower levels are already combined), 16 ds_swizzle, 32 ds_bpermute.
template <int MASK>
__device__ __forceinline__ int lane_xor(int v) {
    if (MASK == 1) return __builtin_amdgcn_mov_dpp(v, 0xB1, 0xF, 0xF, true);  // quad_perm [1,0,3,2]
    if (MASK == 2) return __builtin_amdgcn_mov_dpp(v, 0x4E, 0xF, 0xF, true);  // quad_perm [2,3,0,1]
    if (MASK == 4) return __builtin_amdgcn_mov_dpp(v, 0x141, 0xF, 0xF, true); // row_half_mirror
    if (MASK == 8) return __builtin_amdgcn_mov_dpp(v, 0x140, 0xF, 0xF, true); // row_mirror
    if (MASK == 16) return __builtin_amdgcn_ds_swizzle(v, (0x10 << 10) | 0x1F);
    return __builtin_amdgcn_ds_bpermute(((__lane_id() ^ 32) << 2), v);
}

struct OpAdd {
    __device__ __forceinline__ int operator()(int a, int b) const { return a + b; }
};
struct OpMax {
    __device__ __forceinline__ int operator()(int a, int b) const { return max(a, b); }
};

// All-reduce over aligned groups of L consecutive lanes (L a power of two, 1..64).
template <int L, typename Op>
__device__ __forceinline__ int group_allreduce(int v, Op op) {
    if (L >= 2) v = op(v, lane_xor<1>(v));
    if (L >= 4) v = op(v, lane_xor<2>(v));
    if (L >= 8) v = op(v, lane_xor<4>(v));
    if (L >= 16) v = op(v, lane_xor<8>(v));
    if (L >= 32) v = op(v, lane_xor<16>(v));
    if (L >= 64) v = op(v, lane_xor<32>(v));
    return v;
}

__device__ __forceinline__ int64_t floordiv64(int64_t a, int64_t b) {
    int64_t q = a / b, r = a % b;
    return (r != 0 && ((r < 0) != (b < 0))) ? q - 1 : q;
}

// One 16-byte chunk of an operand row for shapes the aligned kernels cannot take (K not a multiple of 16, rows that
// are not 16-byte aligned): `rem` of its bytes belong to the row's K values, the rest read as zero, and no byte
// past the end of the row's pitch is touched. mode 0: the chunk is aligned and lies inside the pitch; mode 1: rows
// are 4-byte aligned with a pitch that is a multiple of 4; mode 2: neither.
__device__ __forceinline__ v4i load_chunk_ragged(const int8_t* p, int rem, int mode) {
    v4i r = {0, 0, 0, 0};
    if (rem <= 0) return r;
    if (mode == 0) {
        r = *reinterpret_cast<const v4i*>(p);
    } else if (mode == 1) {
#pragma unroll
        for (int j = 0; j < 4; ++j)
            if (4 * j < rem) r[j] = *reinterpret_cast<const int*>(p + 4 * j);
    } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            unsigned w = 0;
#pragma unroll
            for (int b = 0; b < 4; ++b)
                if (4 * j + b < rem) w |= static_cast<unsigned>(static_cast<uint8_t>(p[4 * j + b])) << (8 * b);
            r[j] = static_cast<int>(w);
        }
    }
    if (rem < 16) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int v = rem - 4 * j;  // valid bytes of this dword
            if (v <= 0) r[j] = 0;
            else if (v < 4) r[j] &= static_cast<int>((1u << (8 * v)) - 1u);
        }
    }
    return r;
}

// One 16-byte chunk of a row of A when A is stored transposed ([K][ld], TRANSPOSE_A of matmul.cpp:60-66 and
// dense_bias_relu.cpp:95-101): element e of the chunk is the `es`-byte element (1, 2 or 4 bytes) at
// col + (k0 + e) * ld_bytes, `col` pointing at the row's element of k = 0; elements at or past K read as zero.
__device__ __forceinline__ v4i load_chunk_transposed(const int8_t* col, int64_t ld_bytes, int k0, int K, int es) {
    v4i r = {0, 0, 0, 0};
    const int8_t* p = col + static_cast<int64_t>(k0) * ld_bytes;
    if (es == 4) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
            if (k0 + e < K) r[e] = *reinterpret_cast<const int*>(p + e * ld_bytes);
    } else if (es == 2) {
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (k0 + e < K) r[e >> 1] |= static_cast<int>(static_cast<unsigned>(*reinterpret_cast<const uint16_t*>(p + e * ld_bytes)) << (16 * (e & 1)));
    } else {
#pragma unroll
        for (int e = 0; e < 16; ++e)
            if (k0 + e < K) r[e >> 2] |= static_cast<int>(static_cast<unsigned>(static_cast<uint8_t>(p[e * ld_bytes])) << (8 * (e & 3)));
    }
    return r;
}

// The store that goes with it: the first `rem` bytes of a 16-byte chunk, in pieces the row's alignment allows.
__device__ __forceinline__ void store_chunk_ragged(int8_t* p, const v4i& v, int rem, int mode) {
    if (rem <= 0) return;
    if (mode == 0 && rem >= 16) {
        *reinterpret_cast<v4i*>(p) = v;
        return;
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int n = rem - 4 * j;  // bytes of this dword to write
        if (n <= 0) break;
        if (mode <= 1 && n >= 4) {
            *reinterpret_cast<int*>(p + 4 * j) = v[j];
        } else {
#pragma unroll
            for (int b = 0; b < 4; ++b)
                if (b < n) p[4 * j + b] = static_cast<int8_t>(static_cast<unsigned>(v[j]) >> (8 * b));
        }
    }
}

}  // namespace a4g
