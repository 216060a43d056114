// Pieces of the integer Softmax shared by the row kernel and the fused attention kernel
// (reference: templates/nnet_utils/softmax/softmax.cpp:19-127, 252-384).
#pragma once

#include "common.hpp"

namespace a4g {

__device__ __forceinline__ int sat16(int v) { return clamp_i(v, -32768, 32767); }

// softmax.cpp:252-273 under rounding_mode::floor.
__device__ __forceinline__ int exp_score16(int d, int kq) {
    const int z = sat16(d * kq);
    const int zint = z >> 8;
    const int zfrac = z & 255;
    const int t = sat16((zfrac * 2811) >> 8);
    const int inner = sat16(t - 11004);
    const int t2 = sat16((inner * zfrac) >> 8);
    int e = static_cast<int16_t>(t2 + 16384);
    e = e >> (zint & 15);
    return zint >= 16 ? 0 : e;
}

struct SoftmaxParams {
    int is_hccs;
    int exp_kq;
    int B, S, Dmax;
    int numer;      // 255 << inv_shift, or 32767
    int inv_shift;  // for the use_clb branch
    int use_clb;
    int out_shift;
    int out_i16;
};

__device__ __forceinline__ int table_entry(const SoftmaxParams& p, int d) {
    if (p.is_hccs) return sat16(p.B - p.S * min(d, p.Dmax));
    return exp_score16(d, p.exp_kq);
}

// softmax.cpp:62-79 (HCCS) / :108-127 (exact floor(NUMER/sum)); the int16 narrowing is the
// broadcast<int16>(inv_q0) of softmax.cpp:79 and the (int16_t) cast of :375.
__device__ __forceinline__ int row_inverse(const SoftmaxParams& p, int sum) {
    const int s = sum > 0 ? sum : 1;
    int inv;
    if (p.use_clb) {
        const int k = 31 - __builtin_clz(static_cast<unsigned>(s));
        inv = p.out_i16 ? (32767 >> k) : (k <= p.inv_shift ? (255 << (p.inv_shift - k)) : 0);
    } else {
        inv = static_cast<int>(static_cast<unsigned>(p.numer) / static_cast<unsigned>(s));
    }
    return static_cast<int16_t>(inv);
}


// (byte n of w) * 4 in one instruction: the LDS byte offset of a table entry.
template <int N>
__device__ __forceinline__ unsigned byte_x4(unsigned w, unsigned two) {
    unsigned r;
    if (N == 0) asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_0" : "=v"(r) : "v"(two), "v"(w));
    if (N == 1) asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_1" : "=v"(r) : "v"(two), "v"(w));
    if (N == 2) asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_2" : "=v"(r) : "v"(two), "v"(w));
    if (N == 3) asm("v_lshlrev_b32_sdwa %0, %1, %2 dst_sel:DWORD dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:BYTE_3" : "=v"(r) : "v"(two), "v"(w));
    return r;
}

// Parameter checks of the two Softmax forms (softmax.py:339-349, softmax/common.py:59-89); both fill
// `p` and say whether the final clamp to [0,255] can be skipped.
static inline int make_exp_params(const char* who, int exp_kq, int inv_shift, int out_kind, SoftmaxParams* p,
                                  bool* noclamp) {
    A4G_REQUIRE(out_kind == A4G_U8 || out_kind == A4G_I16, A4G_ERR_INVALID_ARGUMENT,
                "%s: requires uint8 or int16 output, got kind %d", who, out_kind);
    A4G_REQUIRE(exp_kq >= 1 && exp_kq <= 128, A4G_ERR_INVALID_ARGUMENT, "%s: exp Softmax needs 1 <= EXP_KQ <= 128, got %d",
                who, exp_kq);
    A4G_REQUIRE(inv_shift >= 1 && inv_shift <= 21, A4G_ERR_INVALID_ARGUMENT, "%s: inv_shift %d outside [1,21]", who,
                inv_shift);
    *p = SoftmaxParams{};
    p->is_hccs = 0;
    p->exp_kq = exp_kq;
    p->out_i16 = out_kind == A4G_I16;
    p->numer = p->out_i16 ? 32767 : (255 << inv_shift);
    p->inv_shift = inv_shift;
    p->use_clb = 0;
    p->out_shift = p->out_i16 ? 0 : inv_shift;
    // every score <= sum and inv = floor(numer/sum) fits int16, so score*inv >> shift <= 255
    *noclamp = true;
    return A4G_OK;
}

static inline int make_hccs_params(const char* who, int64_t cols, int B, int S, int Dmax, int inv_shift, int use_clb,
                                   int out_kind, SoftmaxParams* p, bool* noclamp) {
    A4G_REQUIRE(out_kind == A4G_U8 || out_kind == A4G_I16, A4G_ERR_INVALID_ARGUMENT,
                "%s: requires uint8 or int16 output, got kind %d", who, out_kind);
    A4G_REQUIRE(B >= 0 && B <= 32767, A4G_ERR_INVALID_ARGUMENT, "%s: HCCS Softmax parameter 'B' must be in [0, 32767]", who);
    A4G_REQUIRE(S >= 0 && S <= 127, A4G_ERR_INVALID_ARGUMENT, "%s: HCCS Softmax parameter 'S' must be in [0, 127]", who);
    A4G_REQUIRE(Dmax >= 0 && Dmax <= 127, A4G_ERR_INVALID_ARGUMENT, "%s: HCCS Softmax parameter 'Dmax' must be in [0, 127]",
                who);
    A4G_REQUIRE(B - S * Dmax >= 0, A4G_ERR_INVALID_ARGUMENT, "%s: HCCS Softmax requires B - S*Dmax >= 0, got %d", who,
                B - S * Dmax);
    A4G_REQUIRE(static_cast<int64_t>(B - S * Dmax) * cols >= 256, A4G_ERR_INVALID_ARGUMENT,
                "%s: HCCS Softmax requires cols * (B - S*Dmax) >= 256 for reciprocal range, got %lld", who,
                (long long)(static_cast<int64_t>(B - S * Dmax) * cols));
    A4G_REQUIRE(static_cast<int64_t>(B) * cols <= 32767, A4G_ERR_INVALID_ARGUMENT,
                "%s: HCCS Softmax requires cols * B <= 32767 so score sum fits int16 range", who);
    A4G_REQUIRE(inv_shift >= 1 && inv_shift <= 23, A4G_ERR_INVALID_ARGUMENT, "%s: inv_shift %d outside [1,23]", who,
                inv_shift);
    *p = SoftmaxParams{};
    p->is_hccs = 1;
    p->B = B;
    p->S = S;
    p->Dmax = Dmax;
    p->out_i16 = out_kind == A4G_I16;
    p->numer = p->out_i16 ? 32767 : (255 << inv_shift);
    p->inv_shift = inv_shift;
    p->use_clb = use_clb != 0;
    p->out_shift = p->out_i16 ? 0 : inv_shift;
    *noclamp = !p->use_clb && inv_shift <= 15;
    return A4G_OK;
}

}  // namespace a4g
