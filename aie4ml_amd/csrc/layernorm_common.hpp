// Integer LayerNorm arithmetic shared by the row kernels (rowops.hip) and the Dense kernel that normalises its own
// output rows (gemm_rowln.hip): row statistics, the exact Q15 reciprocal square root, the two requantisations in
// their integer and float forms, and the packed saturating int8 add of the residual in front.
// (reference: layer_norm.cpp:14-121, elementwise_add.cpp:12-37)
#pragma once
#include "common.hpp"

namespace a4g {

// Saturating add of four packed int8 lanes. Even and odd bytes are moved to the high byte of each 16-bit half (one
// v_perm each for the even ones, one mask for the odd ones) so that the packed 16-bit saturating add clamps exactly
// where the int8 add would; a last v_perm gathers the four high bytes.
__device__ __forceinline__ unsigned sat_add_i8x4(unsigned a, unsigned b) {
    const v2s ae = __builtin_bit_cast(v2s, __builtin_amdgcn_perm(a, 0u, 0x060c040cu));  // [0, a0, 0, a2]
    const v2s be = __builtin_bit_cast(v2s, __builtin_amdgcn_perm(b, 0u, 0x060c040cu));
    const v2s ao = __builtin_bit_cast(v2s, a & 0xFF00FF00u);                            // [0, a1, 0, a3]
    const v2s bo = __builtin_bit_cast(v2s, b & 0xFF00FF00u);
    const unsigned se = __builtin_bit_cast(unsigned, __builtin_elementwise_add_sat(ae, be));
    const unsigned so = __builtin_bit_cast(unsigned, __builtin_elementwise_add_sat(ao, bo));
    return __builtin_amdgcn_perm(so, se, 0x07030501u);  // bytes: se.1, so.1, se.3, so.3
}

// Nearest Q15 of 1/sqrt(v), v >= 1, clamped to 32767: the answer is the largest q with
// (2q-1)^2 * v <= 2^32. A float seed is within one of it (relative error of v_rsq_f32 and of the
// int->float conversion are ~2^-22, q < 2^15), so testing the seed and its successor decides.
__device__ __forceinline__ bool rsqrt_q15_fits(unsigned q, unsigned v) {
    const unsigned a = (2u * q - 1u) * (2u * q - 1u);  // q <= 23172 here: no overflow
    const unsigned lo = a * v, hi = __umulhi(a, v);
    return hi == 0u || (hi == 1u && lo == 0u);
}
__device__ __forceinline__ int rsqrt_q15(int vi) {
    const unsigned v = vi < 1 ? 1u : static_cast<unsigned>(vi);
    if (v < 2u) return 32767;  // exact value 32768 saturates
    unsigned q = static_cast<unsigned>(32768.0f * __frsqrt_rn(static_cast<float>(v)) + 0.5f);
    if (q < 1u) q = 1u;
    const bool t0 = rsqrt_q15_fits(q, v), t1 = rsqrt_q15_fits(q + 1u, v);
    q = t0 ? (t1 ? q + 1u : q) : q - 1u;
    if (q < 1u) q = 1u;
    return static_cast<int>(q);
}

// floor(n / d) for any int32 n and 1 <= d <= 65536: float quotient (within one of the answer,
// |n|/d * 2^-23 < 1), then exact remainder fix-up.
__device__ __forceinline__ int floordiv_small(int n, int d) {
    int q = static_cast<int>(floorf(static_cast<float>(n) / static_cast<float>(d)));
    int r = n - q * d;  // |r| < 3d: no overflow
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        if (r < 0) { r += d; --q; }
        if (r >= d) { r -= d; ++q; }
    }
    return q;
}

struct RowStats {
    int mu;
    int inv;
};

// layer_norm.cpp:22-34. log2c >= 0 when cols is a power of two (the reference's shift form); the
// floor divisions are the same numbers otherwise.
__device__ __forceinline__ RowStats row_stats(int sx, int sq, int cols, int log2c, int eps_q0) {
    RowStats st;
    int mu, var;
    if (log2c >= 0) {
        mu = (sx + (cols >> 1)) >> log2c;
        const int csq = static_cast<int>(static_cast<unsigned>(sq) - 2u * static_cast<unsigned>(mu) * static_cast<unsigned>(sx) +
                                         static_cast<unsigned>(cols) * static_cast<unsigned>(mu) * static_cast<unsigned>(mu));
        var = csq >> log2c;
    } else {
        mu = floordiv_small(sx + (cols >> 1), cols);
        const int csq = static_cast<int>(static_cast<unsigned>(sq) - 2u * static_cast<unsigned>(mu) * static_cast<unsigned>(sx) +
                                         static_cast<unsigned>(cols) * static_cast<unsigned>(mu) * static_cast<unsigned>(mu));
        var = floordiv_small(csq, cols);
    }
    if (var < 0) var = 0;
    st.mu = static_cast<int16_t>(mu);
    st.inv = rsqrt_q15(static_cast<int>(static_cast<unsigned>(var) + static_cast<unsigned>(eps_q0)));
    return st;
}

__device__ __forceinline__ int sext8(unsigned w, int j) { return static_cast<int>(w << (24 - 8 * j)) >> 24; }

// Rounding of the two requantisations in the row kernel. Every mode is (acc + c0 + bit) >> s with bit
// taken from acc itself; BIT selects where: 0 none, 1 minus the sign bit (symmetric_inf), 2 plus the
// sign bit (symmetric_zero), 3 plus the parity of acc >> s (conv_even), 4 minus it (conv_odd).
// w is the extracted field's width: 1, or 0 when s == 0 (then c0 == 0 too and acc passes unchanged).
// |acc| < 2^30 here, so the additions cannot overflow.
struct LnRound {
    int s, c0, w;
};
static LnRound make_ln_round(int mode, int s, int* bit_kind) {
    LnRound r{s, 0, s > 0 ? 1 : 0};
    const int h = s > 0 ? (1 << (s - 1)) : 0;
    int kind = 0;
    switch (mode) {
    case A4G_RND_FLOOR: break;
    case A4G_RND_CEIL: r.c0 = s > 0 ? (1 << s) - 1 : 0; break;
    case A4G_RND_POSITIVE_INF: r.c0 = h; break;
    case A4G_RND_NEGATIVE_INF: r.c0 = s > 0 ? h - 1 : 0; break;
    case A4G_RND_SYMMETRIC_INF: r.c0 = h; kind = 1; break;
    case A4G_RND_SYMMETRIC_ZERO: r.c0 = s > 0 ? h - 1 : 0; kind = 2; break;
    case A4G_RND_CONV_EVEN: r.c0 = s > 0 ? h - 1 : 0; kind = 3; break;
    default: r.c0 = h; kind = 4; break;
    }
    *bit_kind = kind;
    return r;
}
template <int BIT>
__device__ __forceinline__ int ln_round(int acc, const LnRound& r) {
    int bit = 0;
    if (BIT == 1) bit = __builtin_amdgcn_sbfe(acc, 31, r.w);
    if (BIT == 2) bit = static_cast<int>(__builtin_amdgcn_ubfe(static_cast<unsigned>(acc), 31, r.w));
    if (BIT == 3) bit = static_cast<int>(__builtin_amdgcn_ubfe(static_cast<unsigned>(acc), r.s, r.w));
    if (BIT == 4) bit = __builtin_amdgcn_sbfe(acc, r.s, r.w);
    return (acc + r.c0 + bit) >> r.s;
}

// The normalisation in float arithmetic, exact for the modes whose rounding the float unit has
// (FR 0: nearest-even, 1: floor of x + h, 2: ceil of x + h) as long as every gamma is within +-511:
// inv <= 32767 makes |inv * gamma| < 2^24 - 2^14, |x - mu| <= 255 and |fscale| <= 32768 make
// |vd * fscale + beta + 2^(7+s)| < 2^24 for s <= 15, so each product and sum below is an integer times a
// power of two that a float holds exactly, and v_rndne / v_floor / v_ceil round the same rational the
// integer path rounds. The output is produced biased by 128: v_cvt_pk_u8_f32 rounds to nearest even,
// saturates to 0..255 and inserts the byte, which is the int8 saturation once the bias is removed.
struct LnFloat {
    float s1, h1;  // 2^-gamma_shift and the rounding offset of fscale
    float c, h2;   // 2^-final_shift and 128 + the rounding offset of the output
};
static LnFloat make_ln_float(int mode, int gamma_shift, int final_shift, int* fr) {
    float half = 0.f;
    int kind = -1;
    switch (mode) {
    case A4G_RND_CONV_EVEN: kind = 0; break;
    case A4G_RND_FLOOR: kind = 1; break;
    case A4G_RND_POSITIVE_INF: kind = 1; half = 0.5f; break;
    case A4G_RND_CEIL: kind = 2; break;
    case A4G_RND_NEGATIVE_INF: kind = 2; half = -0.5f; break;
    default: break;
    }
    *fr = kind;
    return LnFloat{ldexpf(1.f, -gamma_shift), gamma_shift > 0 ? half : 0.f, ldexpf(1.f, -final_shift),
                   128.f + (final_shift > 0 ? half : 0.f)};
}
constexpr int LN_FLOAT_MAX_GAMMA = 511;

}  // namespace a4g
