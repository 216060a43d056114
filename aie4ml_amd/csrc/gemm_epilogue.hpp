// The requantising epilogue shared by the int8 GEMM kernels and the byte-plane int16 kernels: per-column
// parameters parked in LDS, accumulators requantised into an LDS image of the output tile, whole rows stored.
// (dense_bias_relu.cpp:153-163 and matmul.cpp:112-115: to_vector<result_t>(acc, SHIFT), then the optional ReLU.)
#pragma once
#include <type_traits>

#include "common.hpp"
#include "gemm_rs.hpp"

namespace a4g {

__device__ __forceinline__ int column_shift(const GemmArgs& g, int n) {
    const int s = g.shifts ? g.shifts[static_cast<int64_t>(n) * g.shift_stride] : g.shift;
    return min(max(s, 0), 31);
}

// Per-column epilogue parameters, 5 ints per tile column in LDS: add (bias + 128*colsum), shift, and
// the rounding constants c0, cx, bs of RoundCfg.
template <int BN>
struct ColParams {
    int* add;
    int* s;
    int* c0;
    int* cx;
    int* bs;
    __device__ __forceinline__ explicit ColParams(int8_t* base)
        : add(reinterpret_cast<int*>(base)), s(add + BN), c0(s + BN), cx(c0 + BN), bs(cx + BN) {}
    static constexpr int BYTES = 5 * 4 * BN;
};

// Issues the global loads of this thread's column parameters (threads tid < BN own one column each).
template <int BN, bool A_UNSIGNED>
__device__ __forceinline__ void fetch_col_params(const GemmArgs& g, const TileCoord& tc, int tid, int& col_add, int& col_shift) {
    col_add = 0;
    col_shift = 0;
    if (tid < BN) {
        const int nn = min(tc.n0 + tid, g.N - 1);
        col_add = g.bias ? g.bias[nn] : 0;
        if (A_UNSIGNED && g.colsum) col_add += 128 * g.colsum[tc.batch * g.stride_colsum + nn];
        col_shift = column_shift(g, nn);
    }
}

// Parks them in LDS; returns (workgroup-uniform) which requantisation path the tile takes: 0 = every
// shift is within 1..15 (or the mode needs no tie bit), 1 = some shift is 0, 2 = some shift exceeds 15.
// Contains barriers.
template <int BN>
__device__ __forceinline__ int park_col_params(const GemmArgs& g, const ColParams<BN>& cp, int tid, int col_add, int col_shift) {
    int big_shift = 0, zero_shift = 0;
    if (tid < BN) {
        const RoundCfg rc = make_round(g.mode, col_shift);
        cp.add[tid] = col_add;
        cp.s[tid] = rc.s;
        cp.c0[tid] = rc.c0;
        cp.cx[tid] = rc.cx;
        cp.bs[tid] = rc.bs;
        big_shift = rc.s > 15;
        zero_shift = rc.s <= 0;
    }
    if (__syncthreads_or(big_shift) != 0) return 2;
    return __syncthreads_or(zero_shift) != 0 ? 1 : 0;
}

// Epilogue shared by the pipelined kernels: requantise the accumulators into an LDS image of the
// output tile (row pitch BN*obytes + 16), then store whole rows with coalesced 16-byte writes.
// Rounding: floor((acc + off) / 2^s), off = c0 + cx*bit (see RoundCfg). With every shift <= 15 the
// offset is added with a saturating add: a sum that would overflow lies far above any output range
// either way, so the clamp gives the same value. Larger shifts take the overflow-free form.
// The caller has made sure that no tile load is in flight and that all waves are past the main loop.
// PERM: the weight rows were taken in the order of direct_col_of_operand_row, so accumulator 4 q + t of a lane is column
// 16 * (lane / 32) + 4 q + t of its block (not 8 q + 4 * (lane / 32) + t); ADDED: the accumulators started from `add`.
template <int BM, int BN, int WTM, int WTN, int NT, bool PERM = false, bool ADDED = false>
__device__ __forceinline__ void epilogue_store(const GemmArgs& g, const TileCoord& tc, v16i (&acc)[WTM / 32][WTN / 32],
                                               int8_t* smem, const ColParams<BN>& cp, int round_path, int wm, int wn, int lane,
                                               int tid) {
    constexpr int TM = WTM / 32, TN = WTN / 32;
    const int lo = g.relu ? max(kind_lo(g.out_kind), 0) : kind_lo(g.out_kind), hi = kind_hi(g.out_kind);
    const int obytes = (g.out_kind == A4G_I16 || g.out_kind == A4G_U16) ? 2 : 1;
    const int cpitch = BN * obytes + 16;
    auto store_quad = [&](int ml, int nl, const int (&y)[4]) {
        if (obytes == 1) {
            *reinterpret_cast<unsigned*>(smem + ml * cpitch + nl) = pack4_bytes(y[0], y[1], y[2], y[3]);
        } else {
            v2i o = {static_cast<int>(pack2_halves(y[0], y[1])), static_cast<int>(pack2_halves(y[2], y[3]))};
            *reinterpret_cast<v2i*>(smem + ml * cpitch + nl * 2) = o;
        }
    };
    // General forms: PATH 1 multiplies the tie bit by its per-column sign, PATH 2 is the overflow-free one.
    auto requantise = [&](auto slow_tag) {
        constexpr bool SLOW = decltype(slow_tag)::value;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int nl = wn * WTN + j * 32 + (PERM ? 16 * (lane >> 5) + 4 * q : 8 * q + 4 * (lane >> 5));  // column inside the tile
                const v4i add4 = ADDED ? v4i{0, 0, 0, 0} : *reinterpret_cast<const v4i*>(cp.add + nl);
                const v4i s4 = *reinterpret_cast<const v4i*>(cp.s + nl);
                const v4i c04 = *reinterpret_cast<const v4i*>(cp.c0 + nl);
                const v4i cx4 = *reinterpret_cast<const v4i*>(cp.cx + nl);
                const v4i bs4 = *reinterpret_cast<const v4i*>(cp.bs + nl);
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    const int ml = wm * WTM + i * 32 + (lane & 31);
                    int y[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int a = static_cast<int>(static_cast<unsigned>(acc[i][j][q * 4 + t]) + static_cast<unsigned>(add4[t]));
                        if (!SLOW) {
                            const int bit = (a >> bs4[t]) & 1;
                            const int sum = __builtin_elementwise_add_sat(a, c04[t] + cx4[t] * bit);
                            y[t] = clamp_i(sum >> s4[t], lo, hi);
                        } else {
                            RoundCfg rc;
                            rc.s = s4[t];
                            rc.mask = (1u << s4[t]) - 1u;
                            rc.c0 = c04[t];
                            rc.cx = cx4[t];
                            rc.bs = bs4[t];
                            y[t] = clamp_i(apply_round(a, rc), lo, hi);
                        }
                    }
                    store_quad(ml, nl, y);
                }
            }
        }
    };
    // Shifts within 1..15: the sign of the tie bit (BIT 0 none, 1 added, 2 subtracted) and where it sits
    // (CONV: bit s of the sum, else its sign) are compile-time facts of the rounding mode, which leaves
    // add, bit extract, add, saturating add, shift and one median per value.
    auto requantise_fast = [&](auto bit_tag, auto conv_tag) {
        constexpr int BIT = decltype(bit_tag)::value;
        constexpr bool CONV = decltype(conv_tag)::value;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int nl = wn * WTN + j * 32 + (PERM ? 16 * (lane >> 5) + 4 * q : 8 * q + 4 * (lane >> 5));
                const v4i add4 = ADDED ? v4i{0, 0, 0, 0} : *reinterpret_cast<const v4i*>(cp.add + nl);
                const v4i s4 = *reinterpret_cast<const v4i*>(cp.s + nl);
                const v4i c04 = *reinterpret_cast<const v4i*>(cp.c0 + nl);
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    const int ml = wm * WTM + i * 32 + (lane & 31);
                    int y[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int a = static_cast<int>(static_cast<unsigned>(acc[i][j][q * 4 + t]) + static_cast<unsigned>(add4[t]));
                        int off = c04[t];
                        if (BIT == 1) off += static_cast<int>(__builtin_amdgcn_ubfe(static_cast<unsigned>(a), CONV ? s4[t] : 31, 1));
                        if (BIT == 2) off += __builtin_amdgcn_sbfe(a, CONV ? s4[t] : 31, 1);
                        y[t] = clamp_med3(__builtin_elementwise_add_sat(a, off) >> s4[t], lo, hi);
                    }
                    store_quad(ml, nl, y);
                }
            }
        }
    };
    using B0 = std::integral_constant<int, 0>;
    using B1 = std::integral_constant<int, 1>;
    using B2 = std::integral_constant<int, 2>;
    if (round_path == 2) requantise(std::true_type{});
    else if (g.mode <= A4G_RND_NEGATIVE_INF) requantise_fast(B0{}, std::false_type{});
    else if (round_path == 1) requantise(std::false_type{});
    else if (g.mode == A4G_RND_SYMMETRIC_INF) requantise_fast(B2{}, std::false_type{});
    else if (g.mode == A4G_RND_SYMMETRIC_ZERO) requantise_fast(B1{}, std::false_type{});
    else if (g.mode == A4G_RND_CONV_EVEN) requantise_fast(B1{}, std::true_type{});
    else requantise_fast(B2{}, std::true_type{});
    __syncthreads();
    A4G_STAMP(4);
    store_tile_image<BM, BN, NT>(g, tc, smem, obytes, tid);
}

}  // namespace a4g
