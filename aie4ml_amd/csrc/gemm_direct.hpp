// Pieces shared by the Dense kernels that requantise straight from the accumulator registers (gemm_wreg.hip,
// gemm_sk.hip): the per-column parameters in LDS, the quick requantisation of four neighbouring columns into one dword,
// and the order in which weight rows are handed to the MFMA so that a lane ends up with 16 neighbouring output bytes.
// (dense_bias_relu.cpp:153-163: to_vector<result_t>(acc, SHIFT), then the optional ReLU.)
#pragma once
#include "common.hpp"
#include "gemm_epilogue.hpp"
#include "gemm_rs.hpp"

namespace a4g {

// Per-column requantisation parameters in LDS: the accumulator's start value (bias + 128 * colsum), the constants of
// RoundCfg, and the output range moved in front of the shift ([lo << s, (hi << s) + 2^s - 1]).
template <int BN>
struct DirectParams {
    int *add, *s, *c0, *cx, *bs, *lo_s, *hi_s;
    __device__ __forceinline__ explicit DirectParams(int8_t* base)
        : add(reinterpret_cast<int*>(base)), s(add + BN), c0(s + BN), cx(c0 + BN), bs(cx + BN), lo_s(bs + BN), hi_s(lo_s + BN) {}
    static constexpr int BYTES = 7 * 4 * BN;
};

// Parks the parameters; returns (workgroup-uniform) whether some column needs the general requantisation: a shift
// outside 1..15 or a start value so large that start + dot product + rounding offset could leave int32 (the dot product
// of K <= 32768 pairs of 8-bit values stays below 2^29). Barrier inside.
template <int BN>
__device__ __forceinline__ bool direct_park(const GemmArgs& g, const DirectParams<BN>& wp, int tid, int col_add, int col_shift, int lo,
                                            int hi) {
    int general = g.K > 32768;
    if (tid < BN) {
        const RoundCfg rc = make_round(g.mode, col_shift);
        wp.add[tid] = col_add;
        wp.s[tid] = rc.s;
        wp.c0[tid] = rc.c0;
        wp.cx[tid] = rc.cx;
        wp.bs[tid] = rc.bs;
        const int sc = min(max(rc.s, 0), 15);
        wp.lo_s[tid] = static_cast<int>(static_cast<unsigned>(lo) << sc);
        wp.hi_s[tid] = static_cast<int>((static_cast<unsigned>(hi) << sc) | ((1u << sc) - 1u));
        general |= rc.s < 1 || rc.s > 15 || col_add > (1 << 30) || col_add < -(1 << 30);
    }
    return __syncthreads_or(general) != 0;
}

// Four accumulators of four neighbouring columns -> four requantised bytes, for shifts within 1..15 and sums that stay
// inside int32: rounding offset (BIT 0 none, 1 plus, 2 minus the tie bit, taken at bit s when CONV, else the sign), the
// clamp in front of the shift, and a shift that writes its low byte straight into byte n of the result.
template <int BIT, bool CONV>
__device__ __forceinline__ unsigned direct_requant4(int a0, int a1, int a2, int a3, const v4i& s4, const v4i& c04, const v4i& lo4,
                                                  const v4i& hi4) {
    auto pre = [&](int a, int t) {
        int bit = 0;
        if (BIT == 1) bit = static_cast<int>(__builtin_amdgcn_ubfe(static_cast<unsigned>(a), CONV ? s4[t] : 31, 1));
        if (BIT == 2) bit = __builtin_amdgcn_sbfe(a, CONV ? s4[t] : 31, 1);
        return clamp_med3(a + c04[t] + bit, lo4[t], hi4[t]);
    };
    unsigned packed;
    {
        const int v0 = pre(a0, 0);
        asm("v_ashrrev_i32_sdwa %0, %1, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:DWORD"
            : "=v"(packed)
            : "v"(s4[0]), "v"(v0));
    }
    shift_into_byte<1>(packed, pre(a1, 1), s4[1]);
    shift_into_byte<2>(packed, pre(a2, 2), s4[2]);
    shift_into_byte<3>(packed, pre(a3, 3), s4[3]);
    return packed;
}

// The general requantisation of the same four values: any shift, any start value (`add4` is added here, the accumulators
// started from zero).
__device__ __forceinline__ unsigned direct_requant4_general(int a0, int a1, int a2, int a3, const v4i& add4, const v4i& s4, const v4i& c04,
                                                            const v4i& cx4, const v4i& bs4, int lo, int hi) {
    const int a[4] = {a0, a1, a2, a3};
    int y[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        RoundCfg rc;
        rc.s = s4[t];
        rc.mask = (1u << s4[t]) - 1u;
        rc.c0 = c04[t];
        rc.cx = cx4[t];
        rc.bs = bs4[t];
        y[t] = clamp_i(apply_round(static_cast<int>(static_cast<unsigned>(a[t]) + static_cast<unsigned>(add4[t])), rc), lo, hi);
    }
    return pack4_bytes(y[0], y[1], y[2], y[3]);
}

}  // namespace a4g
