// int8 x int8 -> int32 GEMM on the gfx950 matrix cores (v_mfma_i32_32x32x32_i8) with the fused
// requantisation epilogue of the reference's Dense and MatMul kernels
// (dense_bias_relu.cpp:112-163, matmul.cpp:80-115): bias, shift / round / saturate, ReLU.
//
// Operand layout ("NT"): A is [M][lda] and the right-hand side is [N][ldb], both with the
// reduction axis contiguous, so every MFMA operand is one 16-byte read. Dense weights are packed to
// that layout once (a4g_pack_weights_i8); a K x N activation operand is transposed by a pre-pass.
// uint8 left operands are biased to int8 with x ^ 0x80 when fragments are read; the epilogue adds
// back 128 * colsum[n] (exact in wrapping int32).
#include <algorithm>
#include <cstdlib>
#include <mutex>
#include <type_traits>

#include "common.hpp"
#include "gemm_direct.hpp"
#include "gemm_epilogue.hpp"
#include "gemm_rs.hpp"
#include "matmul_lean.hpp"


namespace a4g {

// lo already includes the ReLU floor (max(lo, 0)) when the layer has one
__device__ __forceinline__ int requant(int acc, const RoundCfg& rc, int lo, int hi) {
    return clamp_i(apply_round(acc, rc), lo, hi);
}

// -----------------------------------------------------------------------------------------------------
// Tiled MFMA kernel. Block tile BM x BN, K step BK, WAVES_M x WAVES_N waves; each wave owns a
// (BM/WAVES_M) x (BN/WAVES_N) sub-tile as TM x TN blocks of 32x32 int32 accumulators.
// Requirements checked by the host: K % 16 == 0, lda % 16 == 0, ldb % 16 == 0, 16-byte aligned bases.
// -----------------------------------------------------------------------------------------------------
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N>
struct GemmCfg {
    static constexpr int NT = WAVES_M * WAVES_N * 64;
    static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    static constexpr int TM = WTM / 32, TN = WTN / 32;
    static constexpr int CPR = BK / 16;          // 16-byte chunks per tile row
    static constexpr int PITCH = BK + 16;        // LDS row pitch: breaks the power-of-two bank stride
    static constexpr int A_CHUNKS = BM * CPR, B_CHUNKS = BN * CPR;
    static constexpr int A_PER_T = A_CHUNKS / NT, B_PER_T = B_CHUNKS / NT;
    static constexpr int LDS_BYTES = 2 * (BM + BN) * PITCH;
    static_assert(A_CHUNKS % NT == 0 && B_CHUNKS % NT == 0, "tile loads must divide evenly over the threads");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0 && BK % 32 == 0, "wave tile must be whole 32x32x32 MFMA blocks");
};

// TRANS_A: the left operand is stored transposed, [K][lda] with the rows of the product contiguous (TRANSPOSE_A of the
// reference kernels, matmul.cpp:60-66 / dense_bias_relu.cpp:95-101). Its tile is then fetched as 4 (k) x 4 (m) byte
// blocks, four dword loads along m, transposed in registers (v_perm) and written to LDS as four dwords along k, so the
// MFMA side sees the usual [m][k] tile. Rows (m >= M) and reduction positions (k >= K) outside the operand read as zero.
template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool RAGGED = false, bool TRANS_A = false>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gemm_i8_nt_kernel(GemmArgs g) {
    using Cfg = GemmCfg<BM, BN, BK, WAVES_M, WAVES_N>;
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];
    constexpr int BUF = (BM + BN) * Cfg::PITCH;  // one stage: A tile then B tile
    constexpr int B_OFF = BM * Cfg::PITCH;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    // Workgroup -> tile mapping. Hardware deals consecutive workgroup ids round-robin over the 8
    // XCDs, each with a private L2, so id % 8 names the XCD: give every XCD one contiguous range of
    // tiles, and order that range in bands of GROUP_M tile rows (row index fastest inside a band) so
    // that the tiles resident on an XCD at one time share both activation and weight panels.
    const int tiles_m = (g.M + BM - 1) / BM;
    const int tiles_n = (g.N + BN - 1) / BN;
    const int tiles = tiles_m * tiles_n;
    const int per_xcd = (tiles + 7) / 8;
    const int tile = tiles < 8 ? static_cast<int>(blockIdx.x) : (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;  // grid_for_tiles
    if (tile >= tiles) return;
    constexpr int GROUP_M = 8;
    const int band = tile / (GROUP_M * tiles_n);
    const int band_rows = min(GROUP_M, tiles_m - band * GROUP_M);
    const int in_band = tile % (GROUP_M * tiles_n);
    const int m0 = (band * GROUP_M + in_band % band_rows) * BM;
    const int n0 = (in_band / band_rows) * BN;
    const int batch = blockIdx.y;

    const int8_t* __restrict__ Ab = g.A + batch * g.stride_a;
    const int8_t* __restrict__ Bb = g.Bt + batch * g.stride_b;

    // global -> register staging of the next K tile
    v4i ra[Cfg::A_PER_T], rb[Cfg::B_PER_T];
    const int8_t* pa[Cfg::A_PER_T];
    const int8_t* pb[Cfg::B_PER_T];
    int ka[Cfg::A_PER_T], kb[Cfg::B_PER_T];
    int offa[Cfg::A_PER_T], offb[Cfg::B_PER_T];
#pragma unroll
    for (int i = 0; i < Cfg::A_PER_T; ++i) {
        const int c = tid + i * Cfg::NT;
        const int row = c / Cfg::CPR, kc = c % Cfg::CPR;
        const int gm = min(m0 + row, g.M - 1);
        pa[i] = Ab + static_cast<int64_t>(gm) * g.lda + kc * 16;
        ka[i] = kc * 16;
        offa[i] = row * Cfg::PITCH + kc * 16;
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_PER_T; ++i) {
        const int c = tid + i * Cfg::NT;
        const int row = c / Cfg::CPR, kc = c % Cfg::CPR;
        const int gn = min(n0 + row, g.N - 1);
        pb[i] = Bb + static_cast<int64_t>(gn) * g.ldb + kc * 16;
        kb[i] = kc * 16;
        offb[i] = row * Cfg::PITCH + kc * 16;
    }

    // TRANS_A: 4 x 4 blocks of the [k][m] tile; block b of a thread covers k = 4 * (b / (BM/4)) .., m = 4 * (b % (BM/4)) ..
    constexpr int TA_BLOCKS = TRANS_A ? (BM / 4) * (BK / 4) / Cfg::NT : 1;
    static_assert(!TRANS_A || ((BM / 4) * (BK / 4)) % Cfg::NT == 0, "transposed tile blocks must divide over the threads");
    unsigned ta[TA_BLOCKS][4];
    auto load_a_transposed = [&](int k0) {
#pragma unroll
        for (int b = 0; b < TA_BLOCKS; ++b) {
            const int blk = tid + b * Cfg::NT;
            const int mq = (blk % (BM / 4)) * 4, kq = (blk / (BM / 4)) * 4;
            const int m = m0 + mq;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int k = k0 + kq + i;
                unsigned w = 0;
                if (k < g.K && m < g.M) {
                    const int8_t* src = Ab + static_cast<int64_t>(k) * g.lda + m;
                    if (g.ragged_a == 0 && m + 4 <= g.M) {
                        w = *reinterpret_cast<const unsigned*>(src);
                    } else {
#pragma unroll
                        for (int j = 0; j < 4; ++j)
                            if (m + j < g.M) w |= static_cast<unsigned>(static_cast<uint8_t>(src[j])) << (8 * j);
                    }
                }
                ta[b][i] = w;
            }
        }
    };
    auto store_a_transposed = [&](int buf) {
#pragma unroll
        for (int b = 0; b < TA_BLOCKS; ++b) {
            const int blk = tid + b * Cfg::NT;
            const int mq = (blk % (BM / 4)) * 4, kq = (blk / (BM / 4)) * 4;
            // in: ta[b][i] byte j = A^T[k + i][m + j]; out: c[j] byte i = the same element, k-contiguous for row m + j
            const unsigned lo01 = __builtin_amdgcn_perm(ta[b][1], ta[b][0], 0x05010400u);
            const unsigned hi01 = __builtin_amdgcn_perm(ta[b][1], ta[b][0], 0x07030602u);
            const unsigned lo23 = __builtin_amdgcn_perm(ta[b][3], ta[b][2], 0x05010400u);
            const unsigned hi23 = __builtin_amdgcn_perm(ta[b][3], ta[b][2], 0x07030602u);
            const unsigned c[4] = {__builtin_amdgcn_perm(lo23, lo01, 0x05040100u), __builtin_amdgcn_perm(lo23, lo01, 0x07060302u),
                                   __builtin_amdgcn_perm(hi23, hi01, 0x05040100u), __builtin_amdgcn_perm(hi23, hi01, 0x07060302u)};
#pragma unroll
            for (int j = 0; j < 4; ++j) *reinterpret_cast<unsigned*>(smem + buf * BUF + (mq + j) * Cfg::PITCH + kq) = c[j];
        }
    };

    auto load_tile = [&](int k0) {
        if constexpr (TRANS_A) {
            static_assert(!TRANS_A || RAGGED, "the transposed-A form takes B through the ragged loads");
            load_a_transposed(k0);
#pragma unroll
            for (int i = 0; i < Cfg::B_PER_T; ++i) rb[i] = load_chunk_ragged(pb[i] + k0, g.K - (k0 + kb[i]), g.ragged_b);
        } else if constexpr (RAGGED) {
#pragma unroll
            for (int i = 0; i < Cfg::A_PER_T; ++i) ra[i] = load_chunk_ragged(pa[i] + k0, g.K - (k0 + ka[i]), g.ragged_a);
#pragma unroll
            for (int i = 0; i < Cfg::B_PER_T; ++i) rb[i] = load_chunk_ragged(pb[i] + k0, g.K - (k0 + kb[i]), g.ragged_b);
        } else {
#pragma unroll
            for (int i = 0; i < Cfg::A_PER_T; ++i)
                ra[i] = (k0 + ka[i] < g.K) ? *reinterpret_cast<const v4i*>(pa[i] + k0) : v4i{0, 0, 0, 0};
#pragma unroll
            for (int i = 0; i < Cfg::B_PER_T; ++i)
                rb[i] = (k0 + kb[i] < g.K) ? *reinterpret_cast<const v4i*>(pb[i] + k0) : v4i{0, 0, 0, 0};
        }
    };
    auto store_tile = [&](int buf) {
        if constexpr (TRANS_A) store_a_transposed(buf);
#pragma unroll
        for (int i = 0; i < (TRANS_A ? 0 : Cfg::A_PER_T); ++i) *reinterpret_cast<v4i*>(smem + buf * BUF + offa[i]) = ra[i];
#pragma unroll
        for (int i = 0; i < Cfg::B_PER_T; ++i) *reinterpret_cast<v4i*>(smem + buf * BUF + B_OFF + offb[i]) = rb[i];
    };

    v16i acc[Cfg::TM][Cfg::TN];
#pragma unroll
    for (int i = 0; i < Cfg::TM; ++i)
#pragma unroll
        for (int j = 0; j < Cfg::TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    // fragment addressing: lane%32 picks the row of the operand block, lane/32 the 16-byte half of
    // the 32-wide K step
    const int frag_row = lane & 31;
    const int frag_k = (lane >> 5) * 16;
    const int a_frag_off = (wm * Cfg::WTM + frag_row) * Cfg::PITCH + frag_k;
    const int b_frag_off = (wn * Cfg::WTN + frag_row) * Cfg::PITCH + frag_k;
    const int xor_mask = g.a_unsigned ? static_cast<int>(0x80808080u) : 0;

    const int ktiles = (g.K + BK - 1) / BK;
    load_tile(0);
    store_tile(0);
    __syncthreads();

    for (int kt = 0; kt < ktiles; ++kt) {
        const int buf = kt & 1;
        if (kt + 1 < ktiles) load_tile((kt + 1) * BK);
#pragma unroll
        for (int kk = 0; kk < BK / 32; ++kk) {
            v4i af[Cfg::TM], bf[Cfg::TN];
#pragma unroll
            for (int i = 0; i < Cfg::TM; ++i) {
                af[i] = *reinterpret_cast<const v4i*>(smem + buf * BUF + a_frag_off + i * 32 * Cfg::PITCH + kk * 32);
                af[i] ^= xor_mask;
            }
#pragma unroll
            for (int j = 0; j < Cfg::TN; ++j)
                bf[j] = *reinterpret_cast<const v4i*>(smem + buf * BUF + B_OFF + b_frag_off + j * 32 * Cfg::PITCH + kk * 32);
#pragma unroll
            for (int i = 0; i < Cfg::TM; ++i)
#pragma unroll
                for (int j = 0; j < Cfg::TN; ++j)
                    // operands swapped: the block's first index (registers) runs over n, lanes over m
                    acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[j], af[i], acc[i][j], 0, 0, 0);
        }
        if (kt + 1 < ktiles) store_tile(buf ^ 1);
        __syncthreads();
    }

    // ---- epilogue: lane owns row m = lane%32 of each block and, per register quad q, the four
    // consecutive columns 8q + 4*(lane/32) .. +3.
    const int lo = g.relu ? max(kind_lo(g.out_kind), 0) : kind_lo(g.out_kind), hi = kind_hi(g.out_kind);
    const int obytes = (g.out_kind == A4G_I16 || g.out_kind == A4G_U16) ? 2 : 1;
    int8_t* Cb = static_cast<int8_t*>(g.C) + batch * g.stride_c * obytes;
    const int32_t* cs = (g.a_unsigned && g.colsum) ? g.colsum + batch * g.stride_colsum : nullptr;
    const bool vec_ok = (g.ldc % 4 == 0) && ((reinterpret_cast<uintptr_t>(Cb) & 7) == 0);
#pragma unroll
    for (int j = 0; j < Cfg::TN; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int n = n0 + wn * Cfg::WTN + j * 32 + 8 * q + 4 * (lane >> 5);
            int add[4];
            RoundCfg rc[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int nn = min(n + t, g.N - 1);
                int a = g.bias ? g.bias[nn] : 0;
                if (cs) a += 128 * cs[nn];
                add[t] = a;
                rc[t] = make_round(g.mode, column_shift(g, nn));
            }
#pragma unroll
            for (int i = 0; i < Cfg::TM; ++i) {
                const int m = m0 + wm * Cfg::WTM + i * 32 + (lane & 31);
                int y[4];
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    y[t] = requant(static_cast<int>(static_cast<unsigned>(acc[i][j][q * 4 + t]) + static_cast<unsigned>(add[t])),
                                   rc[t], lo, hi);
                int8_t* dst = Cb + (static_cast<int64_t>(m) * g.ldc + n) * obytes;
                if (m >= g.M || n >= g.N) {
                    // outside the matrix: nothing to store
                } else if (n + 3 < g.N && vec_ok) {
                    if (obytes == 1) {
                        *reinterpret_cast<unsigned*>(dst) = pack4_bytes(y[0], y[1], y[2], y[3]);
                    } else {
                        v2i o = {static_cast<int>(pack2_halves(y[0], y[1])), static_cast<int>(pack2_halves(y[2], y[3]))};
                        *reinterpret_cast<v2i*>(dst) = o;
                    }
                } else {
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        if (n + t < g.N) {
                            if (obytes == 1) dst[t] = static_cast<int8_t>(y[t]);
                            else reinterpret_cast<int16_t*>(dst)[t] = static_cast<int16_t>(y[t]);
                        }
                    }
                }
            }
        }
    }
}

// -----------------------------------------------------------------------------------------------------
// Pipelined MFMA kernel (K % BK == 0). Tiles go global -> LDS directly (global_load_lds, 16 bytes per
// lane, no register staging) into a ring of STAGES buffers; fragments are read with ds_read_b128 one
// K step (32) ahead of the MFMAs that consume them, one read issued behind each MFMA, so LDS latency
// and the per-wave LDS issue rate hide behind the matrix pipe. One workgroup barrier per K tile,
// placed before the tile's last K step.
//
// LDS layout of one operand tile: rows of BK bytes = CPR 16-byte chunks, unpadded (a wave-wide direct
// load writes 64 consecutive chunks). Chunk c of row r lives at slot r*CPR + (c ^ swz(r)) with
// swz(r) = (r>>2)&3 for BK = 64 and (r>>1)&7 for BK = 128: the 16 lanes that read one chunk column of
// 16 consecutive rows then touch 16 distinct 16-byte bank groups. The swizzle is applied on the
// global side: lane l of wave-load j fetches the chunk that belongs in slot j*64 + l. With BK = 128
// every row segment is one whole 128-byte cache line.
// -----------------------------------------------------------------------------------------------------
typedef __attribute__((address_space(1))) const void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

// What the shared pipelined kernel needs to know about int8 operands with an integer epilogue.
template <bool A_UNSIGNED>
struct I8Policy {
    using acc_t = v16i;
    static constexpr int MMAS = 1, KSTEP_BYTES = 32;
    static constexpr bool FIX_A = A_UNSIGNED;
    static constexpr bool SPLIT_A = false, SPLIT_B = false;
    static constexpr bool PERM_B = false;
    struct Extra {};
    static constexpr int MAX_OUT_BYTES = 2;
    template <int BN>
    static constexpr int param_bytes() { return ColParams<BN>::BYTES; }
    struct ColRegs {
        int add, shift;
    };
    __device__ static __forceinline__ void fix_a(v4i& a) { a ^= static_cast<int>(0x80808080u); }
    __device__ static __forceinline__ v16i mma(const v4i (&b)[1], const v4i (&a)[1], const v16i& c) {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(b[0], a[0], c, 0, 0, 0);
    }
    template <int BN>
    __device__ static __forceinline__ void fetch_params(const GemmArgs& g, const TileCoord& tc, int tid, ColRegs& r) {
        fetch_col_params<BN, A_UNSIGNED>(g, tc, tid, r.add, r.shift);
    }
    template <int BN>
    __device__ static __forceinline__ int park_params(const GemmArgs& g, int8_t* lds, int tid, const ColRegs& r) {
        return park_col_params<BN>(g, ColParams<BN>(lds), tid, r.add, r.shift);
    }
    template <int BM, int BN, int WTM, int WTN, int NT>
    __device__ static __forceinline__ void epilogue(const GemmArgs& g, const TileCoord& tc, v16i (&acc)[WTM / 32][WTN / 32],
                                                    int8_t* smem, int8_t* lds_params, int path, int wm, int wn, int lane,
                                                    int tid, Extra&) {
        epilogue_store<BM, BN, WTM, WTN, NT>(g, tc, acc, smem, ColParams<BN>(lds_params), path, wm, wn, lane, tid);
    }
};

// The int8 policy with the epilogue of the register-requantising kernels (gemm_direct.hpp): weight rows in the order that
// makes a lane's 16 accumulators of a block 16 neighbouring columns, accumulators started from bias + 128 * colsum, four
// vector instructions per value in the quick form (shifts within 1..15, sums inside int32), 16-byte stores straight from
// registers: no LDS image of the output tile. For one-byte outputs in whole 16-column pieces on 16-byte aligned rows;
// column blocks that need the general requantisation leave through the LDS image as before (same bits either way:
// int32 addition wraps, so where the bias joins the sum does not matter).
template <bool A_UNSIGNED>
struct I8DirectPolicy : I8Policy<A_UNSIGNED> {
    static constexpr bool PERM_B = true;
    using Extra = typename I8Policy<A_UNSIGNED>::Extra;
    using ColRegs = typename I8Policy<A_UNSIGNED>::ColRegs;
    template <int BN>
    static constexpr int param_bytes() { return DirectParams<BN>::BYTES; }
    template <int BN>
    __device__ static __forceinline__ int park_params(const GemmArgs& g, int8_t* lds, int tid, const ColRegs& r) {
        const int lo = g.relu ? max(kind_lo(g.out_kind), 0) : kind_lo(g.out_kind), hi = kind_hi(g.out_kind);
        return direct_park<BN>(g, DirectParams<BN>(lds), tid, r.add, r.shift, lo, hi) ? 2 : 0;
    }
    template <int BN, int WTN, int TM, int TN>
    __device__ static __forceinline__ void start_acc(v16i (&acc)[TM][TN], int8_t* lds_params, int wn, int lane) {
        const DirectParams<BN> wp(lds_params);
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4i add4 = *reinterpret_cast<const v4i*>(wp.add + wn * WTN + j * 32 + 16 * (lane >> 5) + 4 * q);
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int t = 0; t < 4; ++t) acc[i][j][q * 4 + t] = add4[t];
            }
    }
    template <int BM, int BN, int WTM, int WTN, int NT>
    __device__ static __forceinline__ void epilogue(const GemmArgs& g, const TileCoord& tc, v16i (&acc)[WTM / 32][WTN / 32],
                                                    int8_t* smem, int8_t* lds_params, int path, int wm, int wn, int lane,
                                                    int tid, Extra&) {
        if (path != 0) {  // some column of the tile needs the general form
            epilogue_store<BM, BN, WTM, WTN, NT, true, true>(g, tc, acc, smem, ColParams<BN>(lds_params), 2, wm, wn, lane, tid);
            return;
        }
        constexpr int TM = WTM / 32, TN = WTN / 32;
        const DirectParams<BN> wp(lds_params);
        const int half = lane >> 5, frow = lane & 31;
        auto quick = [&](auto bit_tag, auto conv_tag) {
            constexpr int BIT = decltype(bit_tag)::value;
            constexpr bool CONV = decltype(conv_tag)::value;
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nl = wn * WTN + j * 32 + 16 * half + 4 * q;
                    const v4i s4 = *reinterpret_cast<const v4i*>(wp.s + nl);
                    const v4i c04 = *reinterpret_cast<const v4i*>(wp.c0 + nl);
                    const v4i lo4 = *reinterpret_cast<const v4i*>(wp.lo_s + nl);
                    const v4i hi4 = *reinterpret_cast<const v4i*>(wp.hi_s + nl);
#pragma unroll
                    for (int i = 0; i < TM; ++i)
                        acc[i][j][q] = static_cast<int>(direct_requant4<BIT, CONV>(acc[i][j][q * 4], acc[i][j][q * 4 + 1], acc[i][j][q * 4 + 2],
                                                                                     acc[i][j][q * 4 + 3], s4, c04, lo4, hi4));
                }
        };
        using B0 = std::integral_constant<int, 0>;
        using B1 = std::integral_constant<int, 1>;
        using B2 = std::integral_constant<int, 2>;
        if (g.mode <= A4G_RND_NEGATIVE_INF) quick(B0{}, std::false_type{});
        else if (g.mode == A4G_RND_SYMMETRIC_INF) quick(B2{}, std::false_type{});
        else if (g.mode == A4G_RND_SYMMETRIC_ZERO) quick(B1{}, std::false_type{});
        else if (g.mode == A4G_RND_CONV_EVEN) quick(B1{}, std::true_type{});
        else quick(B2{}, std::true_type{});
        int8_t* Cb = static_cast<int8_t*>(g.C) + tc.batch * g.stride_c;
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int m = tc.m0 + wm * WTM + i * 32 + frow;
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const int n = tc.n0 + wn * WTN + j * 32 + 16 * half;
                if (m < g.M && n + 16 <= g.N) {
                    const v4i o = {acc[i][j][0], acc[i][j][1], acc[i][j][2], acc[i][j][3]};
                    *reinterpret_cast<v4i*>(Cb + static_cast<int64_t>(m) * g.ldc + n) = o;
                }
            }
        }
    }
};

// int16 activations: A is split into its signed high bytes and its low bytes (biased by 128 to be signed too)
// while it is staged, the two planes being alternate runs of rows of the tile, so the unchanged main loop
// leaves a wave with the two partial products of every output in the same lane and register of two of its
// accumulator blocks: acc = 256 * sum(hi * w) + sum((lo - 128) * w) + 128 * sum(w), the last term joining the
// bias as it does for an unsigned operand. Wrapping 32-bit arithmetic throughout, as acc32 does.
struct I16Policy : I8Policy<false> {
    static constexpr bool SPLIT_A = true;
    __device__ static __forceinline__ void split_a(v4i& x, v4i& y, Extra&, int, bool) {
        v4i hi, lo;
        hi[0] = static_cast<int>(__builtin_amdgcn_perm(x[1], x[0], 0x07050301u));
        hi[1] = static_cast<int>(__builtin_amdgcn_perm(x[3], x[2], 0x07050301u));
        hi[2] = static_cast<int>(__builtin_amdgcn_perm(y[1], y[0], 0x07050301u));
        hi[3] = static_cast<int>(__builtin_amdgcn_perm(y[3], y[2], 0x07050301u));
        lo[0] = static_cast<int>(__builtin_amdgcn_perm(x[1], x[0], 0x06040200u) ^ 0x80808080u);
        lo[1] = static_cast<int>(__builtin_amdgcn_perm(x[3], x[2], 0x06040200u) ^ 0x80808080u);
        lo[2] = static_cast<int>(__builtin_amdgcn_perm(y[1], y[0], 0x06040200u) ^ 0x80808080u);
        lo[3] = static_cast<int>(__builtin_amdgcn_perm(y[3], y[2], 0x06040200u) ^ 0x80808080u);
        x = hi;
        y = lo;
    }
    template <int BN>
    __device__ static __forceinline__ void fetch_params(const GemmArgs& g, const TileCoord& tc, int tid, ColRegs& r) {
        fetch_col_params<BN, true>(g, tc, tid, r.add, r.shift);  // + 128 * column sum
    }
    template <int BM, int BN, int WTM, int WTN, int NT>
    __device__ static __forceinline__ void epilogue(const GemmArgs& g, const TileCoord& tc, v16i (&acc)[WTM / 32][WTN / 32],
                                                    int8_t* smem, int8_t* lds_params, int path, int wm, int wn, int lane,
                                                    int tid, Extra&) {
        constexpr int PB = NT / 256;  // 32-row blocks per run of one plane (rows covered by one load per thread / 32)
        v16i sum[WTM / 64][WTN / 32];
#pragma unroll
        for (int i = 0; i < WTM / 64; ++i) {
            const int hi_blk = (i / PB) * 2 * PB + i % PB, lo_blk = hi_blk + PB;
#pragma unroll
            for (int j = 0; j < WTN / 32; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    sum[i][j][r] = static_cast<int>((static_cast<unsigned>(acc[hi_blk][j][r]) << 8) +
                                                    static_cast<unsigned>(acc[lo_blk][j][r]));
        }
        epilogue_store<BM / 2, BN, WTM / 2, WTN, NT>(g, tc, sum, smem, ColParams<BN>(lds_params), path, wm, wn, lane, tid);
    }
};

template <int BM, int BN, int BK_, int WAVES_M, int WAVES_N, int STAGES>
struct DtlCfg {
    static constexpr int BK = BK_;
    static constexpr int CPR = BK / 16;    // chunks per row
    static constexpr int KSTEPS = BK / 32; // MFMA K steps per tile
    static constexpr int NW = WAVES_M * WAVES_N;
    static constexpr int NT = NW * 64;
    static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    static constexpr int TM = WTM / 32, TN = WTN / 32;
    static constexpr int A_WL = BM * CPR / 64, B_WL = BN * CPR / 64;  // wave-wide loads per tile (64 chunks each)
    static constexpr int A_PER_W = A_WL / NW, B_PER_W = B_WL / NW;
    static constexpr int LOADS = A_PER_W + B_PER_W;  // per thread per K tile
    static constexpr int STAGE_BYTES = (BM + BN) * BK;
    static constexpr int C_PITCH1 = BN + 16, C_PITCH2 = 2 * BN + 16;
    static constexpr int EPI_BYTES = BM * C_PITCH2;
    // per-column epilogue parameters (5 ints per column) live behind the stages / output image
    static constexpr int PARAM_OFF = STAGES * STAGE_BYTES > EPI_BYTES ? STAGES * STAGE_BYTES : EPI_BYTES;
    static constexpr int LDS_BYTES = PARAM_OFF + ColParams<BN>::BYTES;
    static_assert(BK == 64 || BK == 128, "BK is 64 or 128");
    static_assert(A_WL % NW == 0 && B_WL % NW == 0, "every wave must issue the same number of tile loads");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be whole 32x32 MFMA blocks");
    static_assert(TM >= TN, "fragment read order assumes TM >= TN");
    static_assert(TM * TN >= TM + TN, "one fragment read is issued behind each MFMA");
    static_assert(STAGES >= 2 && STAGES <= 4, "2..4 stages");
    static_assert(LOADS * (STAGES - 1) < 64, "vmcnt is a 6-bit counter");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
    __host__ __device__ static constexpr int swz(int r) { return BK == 64 ? ((r >> 2) & 3) : ((r >> 1) & 7); }
};

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
    // s_waitcnt vmcnt(N) only (lgkmcnt / expcnt left at their maxima); gfx9 encoding:
    // vmcnt[3:0] = simm16[3:0], vmcnt[5:4] = simm16[15:14], expcnt = [6:4], lgkmcnt = [11:8]
    __builtin_amdgcn_s_waitcnt(((N & 0xF) | ((N >> 4) << 14)) | (0x7 << 4) | (0xF << 8));
}

template <int BM, int BN, int BK_, int WAVES_M, int WAVES_N, int STAGES, bool A_UNSIGNED>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gemm_i8_dtl_kernel(GemmArgs g) {
    using Cfg = DtlCfg<BM, BN, BK_, WAVES_M, WAVES_N, STAGES>;
    constexpr int BK = Cfg::BK, CPR = Cfg::CPR, KSTEPS = Cfg::KSTEPS;
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    const TileCoord tc = tile_coord<BM, BN>(g);
    if (!tc.valid) return;
    const int m0 = tc.m0, n0 = tc.n0, batch = tc.batch;

    const int8_t* __restrict__ Ab = g.A + batch * g.stride_a;
    const int8_t* __restrict__ Bb = g.Bt + batch * g.stride_b;

    // per-column epilogue parameters: fetched first, parked in LDS once the tile loads are in flight
    const ColParams<BN> cp(smem + Cfg::PARAM_OFF);
    int col_add, col_shift;
    fetch_col_params<BN, A_UNSIGNED>(g, tc, tid, col_add, col_shift);

    // ---- global -> LDS assignment: wave-load j covers chunk slots [j*64, j*64+64) of the tile
    const int8_t* pa[Cfg::A_PER_W];
    const int8_t* pb[Cfg::B_PER_W];
#pragma unroll
    for (int i = 0; i < Cfg::A_PER_W; ++i) {
        const int slot = (wave + i * Cfg::NW) * 64 + lane;
        const int r = slot / CPR, c = (slot % CPR) ^ Cfg::swz(r);
        pa[i] = Ab + static_cast<int64_t>(min(m0 + r, g.M - 1)) * g.lda + c * 16;
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_PER_W; ++i) {
        const int slot = (wave + i * Cfg::NW) * 64 + lane;
        const int r = slot / CPR, c = (slot % CPR) ^ Cfg::swz(r);
        pb[i] = Bb + static_cast<int64_t>(min(n0 + r, g.N - 1)) * g.ldb + c * 16;
    }
    auto issue_tile = [&](int kt, int stage) {
        int8_t* base = smem + stage * Cfg::STAGE_BYTES + wave * 1024;
#pragma unroll
        for (int i = 0; i < Cfg::A_PER_W; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(pa[i] + static_cast<int64_t>(kt) * BK),
                                             (lptr_t)(base + i * Cfg::NW * 1024), 16, 0, 0);
#pragma unroll
        for (int i = 0; i < Cfg::B_PER_W; ++i)
            __builtin_amdgcn_global_load_lds((gptr_t)(pb[i] + static_cast<int64_t>(kt) * BK),
                                             (lptr_t)(base + BM * BK + i * Cfg::NW * 1024), 16, 0, 0);
    };

    const int ktiles = g.K / BK;
    // prologue: fill every stage. Tiles past the end are still issued (the last tile again, into a
    // stage nobody reads any more) so that the outstanding-load count stays a compile-time constant.
#pragma unroll
    for (int st = 0; st < STAGES; ++st) issue_tile(min(st, ktiles - 1), st);

    const int round_path = park_col_params<BN>(g, cp, tid, col_add, col_shift);

    // ---- fragment addressing: row = lane%32 of the block, 16-byte half of the 32-wide K step = lane/32
    const int frow = lane & 31;
    int koff[KSTEPS];
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk) koff[kk] = ((kk * 2 + (lane >> 5)) ^ Cfg::swz(frow)) * 16;
    const int a_off = (wm * Cfg::WTM + frow) * BK;
    const int b_off = BM * BK + (wn * Cfg::WTN + frow) * BK;

    v16i acc[Cfg::TM][Cfg::TN];
#pragma unroll
    for (int i = 0; i < Cfg::TM; ++i)
#pragma unroll
        for (int j = 0; j < Cfg::TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    v4i af[2][Cfg::TM], bf[2][Cfg::TN];
    constexpr int NR = Cfg::TM + Cfg::TN, NM = Cfg::TM * Cfg::TN;
    auto read_one = [&](int set, const int8_t* base, int kk, int idx) {
        // order B0, A0, B1, A1, ... so that the first MFMA of the next step can start early
        constexpr int TMIN = Cfg::TM < Cfg::TN ? Cfg::TM : Cfg::TN;
        if (idx < 2 * TMIN) {
            if (idx & 1) af[set][idx >> 1] = *reinterpret_cast<const v4i*>(base + a_off + (idx >> 1) * 32 * BK + koff[kk]);
            else bf[set][idx >> 1] = *reinterpret_cast<const v4i*>(base + b_off + (idx >> 1) * 32 * BK + koff[kk]);
        } else if (Cfg::TM > Cfg::TN) {
            const int i = idx - TMIN;
            af[set][i] = *reinterpret_cast<const v4i*>(base + a_off + i * 32 * BK + koff[kk]);
        } else {
            const int j = idx - TMIN;
            bf[set][j] = *reinterpret_cast<const v4i*>(base + b_off + j * 32 * BK + koff[kk]);
        }
    };
    // MFMAs of the fragment set `cur`, with the reads of set `nxt` threaded between them
    auto step = [&](int cur, int nxt, const int8_t* next_base, int next_kk) {
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            const int i = m / Cfg::TN, j = m % Cfg::TN;
            if (A_UNSIGNED && j == 0) af[cur][i] ^= static_cast<int>(0x80808080u);
            // operands swapped: the block's first index (registers) runs over n, lanes over m
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[cur][j], af[cur][i], acc[i][j], 0, 0, 0);
            if (m < NR) read_one(nxt, next_base, next_kk, m);
        }
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            if (A_UNSIGNED && m % Cfg::TN == 0) __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // operand fix-up
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                                      // one MFMA
            if (m < NR) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                          // one LDS read
        }
    };

    wait_vmcnt<Cfg::LOADS*(STAGES - 1)>();
    __syncthreads();  // tile 0 visible to every wave
#pragma unroll
    for (int r = 0; r < NR; ++r) read_one(0, smem, 0, r);

    for (int kt = 0; kt < ktiles; ++kt) {
        const int8_t* cur_base = smem + (kt % STAGES) * Cfg::STAGE_BYTES;
        const int8_t* nxt_base = smem + ((kt + 1) % STAGES) * Cfg::STAGE_BYTES;
#pragma unroll
        for (int kk = 0; kk < KSTEPS - 1; ++kk) {
            step(kk & 1, (kk + 1) & 1, cur_base, kk + 1);
            __builtin_amdgcn_sched_barrier(0);
        }
        // every read of tile kt has been issued; once they have returned its stage can be refilled
        wait_vmcnt<Cfg::LOADS*(STAGES - 2)>();  // this wave's share of tile kt+1 has landed
        wait_lgkmcnt0();
        __builtin_amdgcn_s_barrier();            // ... and everyone's; nobody reads stage kt%S any more
        __builtin_amdgcn_sched_barrier(0);
        issue_tile(min(kt + STAGES, ktiles - 1), kt % STAGES);
        step((KSTEPS - 1) & 1, KSTEPS & 1, nxt_base, 0);  // after the last tile this reads a stale stage: unused
        __builtin_amdgcn_sched_barrier(0);
    }

    // drain the direct loads still in flight before the stages are reused as the output tile
    wait_vmcnt<0>();
    __syncthreads();

    epilogue_store<BM, BN, Cfg::WTM, Cfg::WTN, Cfg::NT>(g, tc, acc, smem, cp, round_path, wm, wn, lane, tid);
}


// -----------------------------------------------------------------------------------------------------
// Right-hand-side preparation: [K][ldb] -> [N][ldt] (zero padded to ldt) and column sums.
// -----------------------------------------------------------------------------------------------------
__global__ __launch_bounds__(256) void transpose_kn_kernel(const int8_t* __restrict__ B, int64_t ldb, int64_t stride_b,
                                                            int8_t* __restrict__ Bt, int64_t ldt, int64_t stride_t, int K,
                                                            int N) {
    __shared__ int8_t tile[64][65];
    const int batch = blockIdx.z;
    const int k0 = blockIdx.x * 64, n0 = blockIdx.y * 64;
    const int8_t* src = B + batch * stride_b;
    int8_t* dst = Bt + batch * stride_t;
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int kk = i >> 6, nn = i & 63;
        const int k = k0 + kk, n = n0 + nn;
        tile[kk][nn] = (k < K && n < N) ? src[static_cast<int64_t>(k) * ldb + n] : static_cast<int8_t>(0);
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int nn = i >> 6, kk = i & 63;
        const int k = k0 + kk, n = n0 + nn;
        if (n < N && k < ldt) dst[static_cast<int64_t>(n) * ldt + k] = tile[kk][nn];
    }
}

// The same for operands whose rows are 4-byte aligned (ldb, stride_b and the base multiples of 4): a thread takes a
// 4 x 4 block of bytes as four dwords from four rows of k, transposes it in registers (v_perm) and parks its four
// dwords in an LDS tile [64 n][64 k + 4]; the tile then leaves in 16-byte pieces, four lanes per row of 64 k. The
// byte-at-a-time kernel above moved 16.8 MB in 17 us.
__global__ __launch_bounds__(256) void transpose_kn4_kernel(const int8_t* __restrict__ B, int64_t ldb, int64_t stride_b,
                                                             int8_t* __restrict__ Bt, int64_t ldt, int64_t stride_t, int K,
                                                             int N) {
    constexpr int PITCH = 64 + 4;  // dwords of a tile row land in different banks for the sixteen n of a k block
    __shared__ __attribute__((aligned(16))) int8_t tile[64 * PITCH];
    const int batch = blockIdx.z;
    const int k0 = blockIdx.x * 64, n0 = blockIdx.y * 64;
    const int8_t* src = B + batch * stride_b;
    int8_t* dst = Bt + batch * stride_t;
    const int kb = threadIdx.x >> 4, nb = threadIdx.x & 15;
    unsigned in[4], out[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int k = k0 + 4 * kb + i, n = n0 + 4 * nb;
        unsigned w = 0;
        if (k < K) {
            if (n + 4 <= N) {
                w = *reinterpret_cast<const unsigned*>(src + static_cast<int64_t>(k) * ldb + n);
            } else {  // the matrix ends inside the block
                for (int j = 0; j < 4; ++j)
                    if (n + j < N) w |= static_cast<unsigned>(static_cast<uint8_t>(src[static_cast<int64_t>(k) * ldb + n + j])) << (8 * j);
            }
        }
        in[i] = w;
    }
    // in[i] byte j = element (k 4 kb + i, n 4 nb + j)  ->  out[j] byte i
    {
        const unsigned lo01 = __builtin_amdgcn_perm(in[1], in[0], 0x05010400u);
        const unsigned hi01 = __builtin_amdgcn_perm(in[1], in[0], 0x07030602u);
        const unsigned lo23 = __builtin_amdgcn_perm(in[3], in[2], 0x05010400u);
        const unsigned hi23 = __builtin_amdgcn_perm(in[3], in[2], 0x07030602u);
        out[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
        out[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
        out[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
        out[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) *reinterpret_cast<unsigned*>(tile + (4 * nb + j) * PITCH + 4 * kb) = out[j];
    __syncthreads();
    const int n = threadIdx.x >> 2, kq = threadIdx.x & 3;
    if (n0 + n < N && k0 + 16 * kq < ldt) {  // ldt is a multiple of 128 and Bt 16-byte aligned: whole pieces
        const unsigned* t = reinterpret_cast<const unsigned*>(tile + n * PITCH + 16 * kq);
        *reinterpret_cast<v4i*>(dst + static_cast<int64_t>(n0 + n) * ldt + k0 + 16 * kq) =
            v4i{static_cast<int>(t[0]), static_cast<int>(t[1]), static_cast<int>(t[2]), static_cast<int>(t[3])};
    }
}

// [K][ldb] -> [N][ldt] for `batch` operands, by the faster kernel where the operand's alignment allows it
static void launch_transpose_kn(const int8_t* B, int64_t ldb, int64_t stride_b, int8_t* Bt, int64_t ldt, int64_t stride_t, int64_t K,
                                int64_t N, int64_t batch, hipStream_t stream) {
    dim3 grid(static_cast<unsigned>((ldt + 63) / 64), static_cast<unsigned>((N + 63) / 64), static_cast<unsigned>(batch));
    const bool by_dwords = ldb % 4 == 0 && stride_b % 4 == 0 && (reinterpret_cast<uintptr_t>(B) & 3) == 0 && ldt % 16 == 0 &&
                           stride_t % 16 == 0 && aligned16(Bt);
    if (by_dwords) transpose_kn4_kernel<<<grid, 256, 0, stream>>>(B, ldb, stride_b, Bt, ldt, stride_t, static_cast<int>(K), static_cast<int>(N));
    else transpose_kn_kernel<<<grid, 256, 0, stream>>>(B, ldb, stride_b, Bt, ldt, stride_t, static_cast<int>(K), static_cast<int>(N));
}

// colsum[b][n] = sum_k rhs[k][n]; trans: rhs stored [N][ld] (sum along the contiguous axis).
// A workgroup owns 64 columns; its four waves take every fourth k (rows of 64 contiguous bytes when the operand
// is [K][N]; when it is [N][ld] a thread walks its own row in steps of four) and add up through LDS.
// k_chunk < K splits the reduction over gridDim.z: every workgroup then adds its partial sums into colsum with
// integer atomics, and the caller clears colsum first (clear_i32_kernel, not a memset, so that a caller may capture
// the sequence into a graph).
__global__ __launch_bounds__(256) void colsum_kernel(const int8_t* __restrict__ B, int64_t ld, int64_t stride_b, int trans,
                                                      int32_t* __restrict__ colsum, int64_t stride_c, int K, int N,
                                                      int k_chunk) {
    __shared__ int part[4][64];
    const int batch = blockIdx.y;
    const int8_t* src = B + batch * stride_b;
    const int c = threadIdx.x & 63, ks = threadIdx.x >> 6;
    const int n = blockIdx.x * 64 + c;
    const int k0 = blockIdx.z * k_chunk, k1 = min(K, k0 + k_chunk);
    int s = 0;
    if (n < N) {
        if (trans) {
            const int8_t* r = src + static_cast<int64_t>(n) * ld;
            for (int k = k0 + ks; k < k1; k += 4) s += r[k];
        } else {
            for (int k = k0 + ks; k < k1; k += 4) s += src[static_cast<int64_t>(k) * ld + n];
        }
    }
    part[ks][c] = s;
    __syncthreads();
    if (ks == 0 && n < N) {
        const int total = part[0][c] + part[1][c] + part[2][c] + part[3][c];
        if (k_chunk < K) atomicAdd(colsum + batch * stride_c + n, total);
        else colsum[batch * stride_c + n] = total;
    }
}

__global__ __launch_bounds__(256) void clear_i32_kernel(int32_t* __restrict__ p, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

static inline int64_t round_up(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, bool RAGGED = false, bool TRANS_A = false>
static hipError_t launch_tiled(const GemmArgs& g, int batch, hipStream_t stream) {
    using Cfg = GemmCfg<BM, BN, BK, WAVES_M, WAVES_N>;
    auto kern = gemm_i8_nt_kernel<BM, BN, BK, WAVES_M, WAVES_N, RAGGED, TRANS_A>;
    static bool attr_set = false;  // benign race: the attribute is idempotent
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           Cfg::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int tiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
    const int grid_x = grid_for_tiles(tiles);
    hipLaunchKernelGGL(kern, dim3(grid_x, batch), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, g);
    return hipGetLastError();
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int STAGES, bool A_UNSIGNED>
static hipError_t launch_dtl_u(const GemmArgs& g, int batch, hipStream_t stream) {
    using Cfg = DtlCfg<BM, BN, BK, WAVES_M, WAVES_N, STAGES>;
    auto kern = gemm_i8_dtl_kernel<BM, BN, BK, WAVES_M, WAVES_N, STAGES, A_UNSIGNED>;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           Cfg::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int tiles = ((g.M + BM - 1) / BM) * ((g.N + BN - 1) / BN);
    const int grid_x = grid_for_tiles(tiles);
    hipLaunchKernelGGL(kern, dim3(grid_x, batch), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, g);
    return hipGetLastError();
}

// One-byte outputs in whole 16-column pieces on 16-byte aligned rows take the epilogue that requantises and stores from
// registers (I8DirectPolicy); everything else the LDS image.
static bool direct_epilogue_ok(const GemmArgs& g) {
    return (g.out_kind == A4G_I8 || g.out_kind == A4G_U8) && g.N % 16 == 0 && g.ldc % 16 == 0 && g.stride_c % 16 == 0 && aligned16(g.C);
}

template <int BM, int BN, int WAVES_M, int WAVES_N, bool A_UNSIGNED, bool EARLY = false>
static hipError_t launch_rs_u(const GemmArgs& g, int batch, hipStream_t stream) {
    if (direct_epilogue_ok(g)) return launch_rs_policy<I8DirectPolicy<A_UNSIGNED>, BM, BN, WAVES_M, WAVES_N, EARLY>(g, batch, stream);
    return launch_rs_policy<I8Policy<A_UNSIGNED>, BM, BN, WAVES_M, WAVES_N, EARLY>(g, batch, stream);
}

bool rs_i16i8_applicable(const GemmArgs& g, int batch) {
    // whole 128-element K tiles, 16-byte aligned rows, and enough 128 x 256 tiles to give every CU one; from K = 1024 on
    // (measured 3-7 % ahead of the tiled kernel there, level or behind for shorter reductions and for narrow outputs)
    return g.K % 128 == 0 && g.K >= 1024 && g.N >= 192 && g.lda % 16 == 0 && g.stride_a % 16 == 0 && g.ldb % 16 == 0 &&
           g.stride_b % 16 == 0 && aligned16(g.A) && aligned16(g.Bt) && g.colsum != nullptr &&
           static_cast<int64_t>((g.M + 127) / 128) * ((g.N + 255) / 256) * batch >= 192;
}

hipError_t launch_rs_i16i8(const GemmArgs& g, int batch, hipStream_t stream) {
    return launch_rs_policy<I16Policy, 256, 256, 2, 4, true>(g, batch, stream);
}

template <int BM, int BN, int WAVES_M, int WAVES_N>
static hipError_t launch_rs(const GemmArgs& g, int batch, hipStream_t stream) {
    return g.a_unsigned ? launch_rs_u<BM, BN, WAVES_M, WAVES_N, true>(g, batch, stream)
                        : launch_rs_u<BM, BN, WAVES_M, WAVES_N, false>(g, batch, stream);
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N, int STAGES>
static hipError_t launch_dtl(const GemmArgs& g, int batch, hipStream_t stream) {
    return g.a_unsigned ? launch_dtl_u<BM, BN, BK, WAVES_M, WAVES_N, STAGES, true>(g, batch, stream)
                        : launch_dtl_u<BM, BN, BK, WAVES_M, WAVES_N, STAGES, false>(g, batch, stream);
}

// Picks a kernel and tile shape for the problem. variant: 0 = automatic; 1..4 force a tile shape (tuning only,
// through the A4G_GEMM_VARIANT environment variable; a forced shape whose kernel's K granularity does not
// divide K falls back to the next finer kernel).
static hipError_t launch_gemm_nt(const GemmArgs& g, int batch, hipStream_t stream, int variant) {
    if (variant == 0) {
        // 256 x 256 tiles halve the L2 traffic per MAC but cost a long fill / drain per workgroup:
        // they pay off only for deep reductions with enough tiles to keep 256 CUs busy. Everything
        // else (attention-sized batches, short K, narrow N) measured faster with 128 x 128.
        const int64_t tiles256 = static_cast<int64_t>((g.M + 255) / 256) * ((g.N + 255) / 256) * batch;
        const int64_t rounds256 = (tiles256 + 255) / 256;  // one workgroup per CU at a time
        // the last round must be 85 % full, or 75 % for deep reductions (8192 x 3072 x 3072, 384 tiles: 94 us against
        // 103 us with 128 x 128; the same output with K = 768 inside the encoder block: 128 x 128 ahead by 2 %)
        const bool fills = tiles256 * 100 >= rounds256 * 256 * (g.K >= 2048 ? 75 : 85);
        variant = (g.M >= 256 && g.N >= 256 && g.K >= 512 && fills) ? 1 : 2;
        // Widths that are multiples of 192 but not of 256 (768 = 3 * 256 columns on 256 CUs): 128 x 192
        // tiles that make exactly one round of workgroups measured 5-15 % faster than 128 x 128.
        const int64_t tiles192 = static_cast<int64_t>((g.M + 127) / 128) * ((g.N + 191) / 192) * batch;
        if (variant == 2 && g.N % 192 == 0 && g.K % 128 == 0 && tiles192 <= 256 && tiles192 >= 224) variant = 4;
    }
    const bool k128 = g.K % 128 == 0, k64 = g.K % 64 == 0;
    switch (variant) {
    case 1:  // 256 x 256
        if (k128) return g.a_unsigned ? launch_rs_u<256, 256, 2, 4, true, true>(g, batch, stream)
                                      : launch_rs_u<256, 256, 2, 4, false, true>(g, batch, stream);
        if (k64) return launch_dtl<256, 256, 64, 2, 4, 4>(g, batch, stream);
        // K in whole 16-byte chunks but not whole tiles: the pipelined kernel with the last tile's missing chunks
        // fetched from outside the operands' descriptors
        return g.a_unsigned ? launch_rs_policy<I8Policy<true>, 256, 256, 2, 4, true, false, true>(g, batch, stream)
                            : launch_rs_policy<I8Policy<false>, 256, 256, 2, 4, true, false, true>(g, batch, stream);
    case 2:  // 128 x 128
        if (k128) return launch_rs<128, 128, 2, 2>(g, batch, stream);
        if (k64) return launch_dtl<128, 128, 64, 2, 2, 4>(g, batch, stream);
        if (g.K >= 256) {  // K in whole 16-byte chunks but not whole tiles: as above
            return g.a_unsigned ? launch_rs_policy<I8Policy<true>, 128, 128, 2, 2, false, false, true>(g, batch, stream)
                                : launch_rs_policy<I8Policy<false>, 128, 128, 2, 2, false, false, true>(g, batch, stream);
        }
        return launch_tiled<128, 128, 64, 2, 2>(g, batch, stream);
    case 4:  // 128 x 192
        if (k128) return g.a_unsigned ? launch_rs_u<128, 192, 2, 2, true, true>(g, batch, stream)
                                      : launch_rs_u<128, 192, 2, 2, false, true>(g, batch, stream);
        return launch_gemm_nt(g, batch, stream, 2);
    case 3:  // 256 x 64
        if (k64) return launch_dtl<256, 64, 64, 4, 1, 4>(g, batch, stream);
        return launch_tiled<256, 64, 64, 4, 1>(g, batch, stream);
    default: return hipErrorInvalidValue;
    }
}

// Tuning builds (-DA4G_TUNING) can force a tile shape through the A4G_GEMM_VARIANT environment variable; the shipped
// library reads no environment and always dispatches automatically.
static int env_variant() {
#ifdef A4G_TUNING
    static int v = -1;
    if (v < 0) {
        const char* e = getenv("A4G_GEMM_VARIANT");
        v = e ? atoi(e) : 0;
        if (v < 0) v = 0;
    }
    return v;
#else
    return 0;
#endif
}

// Shapes outside the aligned kernels' requirements: same tiles, chunk loads that respect the row ends.
static hipError_t launch_ragged(GemmArgs g, int batch, hipStream_t stream) {
    g.ragged_a = ragged_mode(g.A, g.lda, g.stride_a, g.K);
    g.ragged_b = ragged_mode(g.Bt, g.ldb, g.stride_b, g.K);
    // from two K tiles on, the pipelined kernel is ahead (25 us against 31 us at 8192 x 1024 x 1008): with descriptor loads
    // and no branches where the activations' rows are 4-byte aligned and the other operand's 16-byte aligned rows hold
    // K rounded up to 16 (packed weights always do) ...
    if (g.K >= 256 && g.ragged_a <= 1 && g.ragged_b == 0 && !g.trans_a_es && static_cast<int64_t>(g.lda) >= (g.K + 3) / 4 * 4) {
        // (8-byte aligned rows, a pitch of 1000 bytes: two loads per chunk instead of four)
        const bool by8 = g.lda % 8 == 0 && g.stride_a % 8 == 0 && (reinterpret_cast<uintptr_t>(g.A) & 7) == 0 &&
                         static_cast<int64_t>(g.lda) >= (g.K + 7) / 8 * 8;
        if (by8)
            return g.a_unsigned ? launch_rs_policy<I8Policy<true>, 128, 128, 2, 2, false, false, 3>(g, batch, stream)
                                : launch_rs_policy<I8Policy<false>, 128, 128, 2, 2, false, false, 3>(g, batch, stream);
        return g.a_unsigned ? launch_rs_policy<I8Policy<true>, 128, 128, 2, 2, false, false, 2>(g, batch, stream)
                            : launch_rs_policy<I8Policy<false>, 128, 128, 2, 2, false, false, 2>(g, batch, stream);
    }
    // ... else with chunk loads that respect the row ends
    if (g.K >= 256)
        return g.a_unsigned ? launch_rs_policy<I8Policy<true>, 128, 128, 2, 2, false, true>(g, batch, stream)
                            : launch_rs_policy<I8Policy<false>, 128, 128, 2, 2, false, true>(g, batch, stream);
    return launch_tiled<128, 128, 64, 2, 2, true>(g, batch, stream);
}

// Left operand stored transposed ([K][lda]): the tiled kernel with the in-register tile transpose.
static hipError_t launch_trans_a(GemmArgs g, int batch, hipStream_t stream) {
    // ragged_a here: 0 = rows of A^T are 4-byte aligned (dword loads along m), else byte loads
    const uintptr_t a = reinterpret_cast<uintptr_t>(g.A);
    g.ragged_a = (g.lda % 4 == 0 && g.stride_a % 4 == 0 && a % 4 == 0) ? 0 : 2;
    g.ragged_b = ragged_mode(g.Bt, g.ldb, g.stride_b, g.K);
    return launch_tiled<128, 128, 64, 2, 2, true, true>(g, batch, stream);
}

static bool out_kind_ok(int k) { return k == A4G_I8 || k == A4G_U8 || k == A4G_I16; }

}  // namespace a4g

using namespace a4g;

extern "C" int64_t a4g_packed_ld(int64_t K) { return K <= 0 ? 16 : round_up(K, 16); }

extern "C" int a4g_pack_weights_i8(const int8_t* W, int64_t ldw, int64_t K, int64_t N, int8_t* Wt, int32_t* colsum,
                                   a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    A4G_REQUIRE(W && Wt, A4G_ERR_INVALID_ARGUMENT, "a4g_pack_weights_i8: null pointer");
    A4G_REQUIRE(K >= 1 && N >= 1 && K <= (1 << 24) && N <= (1 << 24) && ldw >= N, A4G_ERR_INVALID_ARGUMENT,
                "a4g_pack_weights_i8: bad shape K=%lld N=%lld ldw=%lld", (long long)K, (long long)N, (long long)ldw);
    const int64_t ldt = a4g_packed_ld(K);
    launch_transpose_kn(W, ldw, 0, Wt, ldt, 0, K, N, 1, stream);
    if (colsum) {
        // one workgroup per 64 columns over all of K is 64 workgroups for a 4096 x 4096 matrix: split K so that the
        // launch has about 2048 workgroups
        const int64_t col_groups = (N + 63) / 64;
        int64_t splits = std::min<int64_t>(std::max<int64_t>(1, 2048 / col_groups), (K + 255) / 256);
        const int k_chunk = static_cast<int>((K + splits - 1) / splits);
        splits = (K + k_chunk - 1) / k_chunk;
        if (splits > 1)
            clear_i32_kernel<<<static_cast<unsigned>((N + 255) / 256), 256, 0, stream>>>(colsum, N);
        colsum_kernel<<<dim3(static_cast<unsigned>(col_groups), 1, static_cast<unsigned>(splits)), 256, 0, stream>>>(
            W, ldw, 0, 0, colsum, 0, static_cast<int>(K), static_cast<int>(N), k_chunk);
    }
    return check_hip(hipGetLastError(), "a4g_pack_weights_i8");
}

static int dense_i8(const char* who, const void* A, int a_kind, int trans_a, int64_t lda, const int8_t* Wt, int64_t ldwt, const int8_t* Wf,
                    const int32_t* colsum, const int32_t* bias, const int32_t* shifts, int n_shift, int round_mode, int relu,
                    int out_kind, void* Y, int64_t ldy, int64_t M, int64_t N, int64_t K, a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    A4G_REQUIRE(M >= 0 && N >= 1 && K >= 1 && M <= INT32_MAX && N <= (1 << 24) && K <= (1 << 24), A4G_ERR_INVALID_ARGUMENT,
                "%s: bad shape M=%lld N=%lld K=%lld", who, (long long)M, (long long)N, (long long)K);
    A4G_REQUIRE(a_kind == A4G_I8 || a_kind == A4G_U8, A4G_ERR_UNSUPPORTED, "%s: activations must be int8 or uint8 (kind %d)",
                who, a_kind);
    A4G_REQUIRE(out_kind_ok(out_kind), A4G_ERR_UNSUPPORTED, "%s: output kind %d is not int8/uint8/int16", who, out_kind);
    A4G_REQUIRE(valid_round(round_mode), A4G_ERR_INVALID_ARGUMENT, "%s: unknown rounding mode %d", who, round_mode);
    A4G_REQUIRE(n_shift == 1 || n_shift == N, A4G_ERR_INVALID_ARGUMENT, "%s: n_shift must be 1 or N=%lld, got %d", who,
                (long long)N, n_shift);
    A4G_REQUIRE(lda >= (trans_a ? M : K) && ldy >= N && ldwt >= K, A4G_ERR_INVALID_ARGUMENT, "%s: pitch smaller than the row", who);
    if (M == 0) return A4G_OK;
    A4G_REQUIRE(A && Wt && Y && shifts, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    A4G_REQUIRE(a_kind != A4G_U8 || colsum, A4G_ERR_INVALID_ARGUMENT, "%s: uint8 activations need the packed colsum vector",
                who);

    GemmArgs g{};
    g.A = static_cast<const int8_t*>(A);
    g.Bt = Wt;
    g.C = Y;
    g.bias = bias;
    g.colsum = colsum;
    g.shifts = shifts;
    g.lda = lda;
    g.ldb = ldwt;
    g.ldc = ldy;
    g.M = static_cast<int>(M);
    g.N = static_cast<int>(N);
    g.K = static_cast<int>(K);
    g.shift_stride = n_shift == 1 ? 0 : 1;
    g.a_unsigned = a_kind == A4G_U8;
    g.relu = relu != 0;
    g.out_kind = out_kind;
    g.mode = round_mode;
    g.Wf = Wf;

    const bool tiled = K % 16 == 0 && lda % 16 == 0 && ldwt % 16 == 0 && aligned16(A) && aligned16(Wt);
    hipError_t e;
    if (trans_a) {
        e = launch_trans_a(g, 1, stream);
    } else if (tiled && wreg_applicable(g)) {
        e = launch_wreg(g, stream);
    } else if (tiled && sk_applicable(g) && sk_preferred(g)) {
        e = launch_sk(g, stream);
    } else if (tiled) {
        e = launch_gemm_nt(g, 1, stream, env_variant());
    } else {
        e = launch_ragged(g, 1, stream);
    }
    return check_hip(e, who);
}

extern "C" int a4g_dense_i8(const void* A, int a_kind, int trans_a, int64_t lda, const int8_t* Wt, int64_t ldwt, const int32_t* colsum,
                            const int32_t* bias, const int32_t* shifts, int n_shift, int round_mode, int relu, int out_kind,
                            void* Y, int64_t ldy, int64_t M, int64_t N, int64_t K, a4g_stream_t stream_) {
    return dense_i8("a4g_dense_i8", A, a_kind, trans_a, lda, Wt, ldwt, nullptr, colsum, bias, shifts, n_shift, round_mode, relu, out_kind, Y,
                    ldy, M, N, K, stream_);
}

extern "C" int a4g_dense_i8_wf(const void* A, int a_kind, int trans_a, int64_t lda, const int8_t* Wt, int64_t ldwt, const int8_t* Wf,
                               const int32_t* colsum, const int32_t* bias, const int32_t* shifts, int n_shift, int round_mode, int relu,
                               int out_kind, void* Y, int64_t ldy, int64_t M, int64_t N, int64_t K, a4g_stream_t stream_) {
    return dense_i8("a4g_dense_i8_wf", A, a_kind, trans_a, lda, Wt, ldwt, Wf, colsum, bias, shifts, n_shift, round_mode, relu, out_kind, Y,
                    ldy, M, N, K, stream_);
}

extern "C" size_t a4g_matmul_i8_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K, int trans_b, int a_kind) {
    (void)M;
    if (batch <= 0 || N <= 0 || K <= 0) return 0;
    size_t bytes = 0;
    if (!trans_b) bytes += static_cast<size_t>(round_up(batch * N * a4g_packed_ld(K), 256));
    if (a_kind == A4G_U8) bytes += static_cast<size_t>(round_up(batch * N * 4, 256));
    return bytes;
}

// ---- a4g_matmul_i8_static: the same MatMul for callers that cannot allocate ---------------------------------
// The repacked right operand and its column sums go to a fixed array in device memory instead of a caller's
// workspace. Every GPU the library runs on holds its own copy of the array at its own address; host code never uses
// the array's name as an address (it is only a handle for hipGetSymbolAddress), it uses the per-device pointer
// resolved on the first call on that device.
static __device__ __align__(256) unsigned char scratch[A4G_MATMUL_I8_STATIC_MAX_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex scratch_mutex;
void* scratch_ptr[kMaxDevices] = {};  // device address of `scratch` on each device, resolved once

int static_scratch(const char* who, hipStream_t stream, void** out) {
    int dev = -1;
    if (int st = check_hip(hipGetDevice(&dev), who)) return st;
    A4G_REQUIRE(dev >= 0 && dev < kMaxDevices, A4G_ERR_UNSUPPORTED, "%s: device ordinal %d beyond %d", who, dev, kMaxDevices);
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (!scratch_ptr[dev]) {
        // Resolving the symbol is not a call a stream capture survives: the first call on a device has to come before any
        // capture, and says so instead of breaking the capture with an error nobody can place.
        hipStreamCaptureStatus cap = hipStreamCaptureStatusNone;
        if (int st = check_hip(hipStreamIsCapturing(stream, &cap), who)) return st;
        A4G_REQUIRE(cap == hipStreamCaptureStatusNone, A4G_ERR_UNSUPPORTED,
                    "%s: the first call on a device must be made outside stream capture (it resolves the scratch array's address)", who);
        void* p = nullptr;
        if (int st = check_hip(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)), who)) return st;
        A4G_REQUIRE(p != nullptr && aligned16(p), A4G_ERR_HIP, "%s: the scratch array resolved to a bad address", who);
        scratch_ptr[dev] = p;
    }
    *out = scratch_ptr[dev];
    return A4G_OK;
}
}  // namespace

// Body of both MatMul entry points. `own_scratch`: the workspace is the library's static scratch array rather than
// a caller's buffer; it is resolved here, after validation and only when the problem needs it.
static int matmul_i8_impl(const char* who, bool own_scratch, const void* A, int a_kind, int trans_a, int64_t lda, int64_t stride_a,
                          const int8_t* B, int64_t ldb, int64_t stride_b, int trans_b, void* C, int64_t ldc, int64_t stride_c,
                          int64_t batch, int64_t M, int64_t N, int64_t K, int shift, int round_mode, int out_kind,
                          void* workspace, size_t workspace_bytes, hipStream_t stream) {
    A4G_REQUIRE(batch >= 0 && batch <= 65535 && M >= 0 && N >= 1 && K >= 1 && M <= INT32_MAX && N <= (1 << 24) &&
                    K <= (1 << 24),
                A4G_ERR_INVALID_ARGUMENT, "%s: bad shape batch=%lld M=%lld N=%lld K=%lld", who, (long long)batch,
                (long long)M, (long long)N, (long long)K);
    A4G_REQUIRE(a_kind == A4G_I8 || a_kind == A4G_U8, A4G_ERR_UNSUPPORTED, "%s: lhs must be int8 or uint8 (kind %d)", who,
                a_kind);
    A4G_REQUIRE(out_kind_ok(out_kind), A4G_ERR_UNSUPPORTED, "%s: output kind %d is not int8/uint8/int16", who, out_kind);
    A4G_REQUIRE(valid_round(round_mode), A4G_ERR_INVALID_ARGUMENT, "%s: unknown rounding mode %d", who, round_mode);
    A4G_REQUIRE(shift >= 0 && shift <= 31, A4G_ERR_INVALID_ARGUMENT,
                "%s: accumulator output shift must be in [0,31], got %d", who, shift);
    A4G_REQUIRE(lda >= (trans_a ? M : K) && ldc >= N && ldb >= (trans_b ? K : N), A4G_ERR_INVALID_ARGUMENT,
                "%s: pitch smaller than the row", who);
    if (batch == 0 || M == 0) return A4G_OK;
    A4G_REQUIRE(A && B && C, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);

    // the two attention shapes have kernels of their own that need neither workspace nor K-loop barriers
    LeanArgs la{};
    const bool lean_shape = out_kind != A4G_I16 && env_variant() == 0 && !trans_a;
    if (lean_shape) {
        la.A = static_cast<const int8_t*>(A);
        la.B = B;
        la.C = static_cast<int8_t*>(C);
        la.lda = lda; la.stride_a = stride_a; la.ldb = ldb; la.stride_b = stride_b; la.ldc = ldc; la.stride_c = stride_c;
        la.M = static_cast<int>(M); la.N = static_cast<int>(N); la.K = static_cast<int>(K); la.batch = static_cast<int>(batch);
        la.a_unsigned = a_kind == A4G_U8;
        la.lo = out_kind == A4G_I8 ? -128 : 0;
        la.hi = out_kind == A4G_I8 ? 127 : 255;
        la.fr = make_fast_round(round_mode, shift);
        la.br = make_byte_requant(la.fr, la.lo, la.hi);
        // nearest even over a short reduction: the transposed-B kernel requantises in float (|acc| <= 128 * 2^14)
        la.fscale = (round_mode == A4G_RND_CONV_EVEN && shift >= 1 && shift <= 15) ? ldexpf(1.f, -shift) : 0.f;
        if (trans_b && lean_nt_applicable(la)) return check_hip(launch_lean_nt(la, stream), who);
        if (!trans_b && lean_nn_applicable(la)) return check_hip(launch_lean_nn(la, stream), who);
    }

    const size_t need = a4g_matmul_i8_workspace_bytes(batch, M, N, K, trans_b, a_kind);
    if (own_scratch && need > 0) {
        workspace_bytes = static_cast<size_t>(A4G_MATMUL_I8_STATIC_MAX_BYTES);
        A4G_REQUIRE(need <= workspace_bytes, A4G_ERR_WORKSPACE,
                    "%s: the repacked right operand needs %zu bytes, the static scratch array holds %zu "
                    "(A4G_MATMUL_I8_STATIC_MAX_BYTES); use a4g_matmul_i8 with a workspace of that size",
                    who, need, workspace_bytes);
        if (int st = static_scratch(who, stream, &workspace)) return st;
    }
    A4G_REQUIRE(need == 0 || (workspace && workspace_bytes >= need), A4G_ERR_WORKSPACE,
                "%s: workspace of %zu bytes required, got %zu", who, need, workspace ? workspace_bytes : (size_t)0);
    A4G_REQUIRE(need == 0 || aligned16(workspace), A4G_ERR_WORKSPACE, "%s: workspace must be 16-byte aligned", who);

    GemmArgs g{};
    g.A = static_cast<const int8_t*>(A);
    g.C = C;
    g.lda = lda;
    g.stride_a = stride_a;
    g.ldc = ldc;
    g.stride_c = stride_c;
    g.M = static_cast<int>(M);
    g.N = static_cast<int>(N);
    g.K = static_cast<int>(K);
    g.shift = shift;
    g.shifts = nullptr;
    g.a_unsigned = a_kind == A4G_U8;
    g.out_kind = out_kind;
    g.mode = round_mode;

    int8_t* ws = static_cast<int8_t*>(workspace);
    const int64_t ldt = a4g_packed_ld(K);
    int32_t* colsum = nullptr;
    if (g.a_unsigned) {
        colsum = reinterpret_cast<int32_t*>(ws + (trans_b ? 0 : round_up(batch * N * ldt, 256)));
        colsum_kernel<<<dim3(static_cast<unsigned>((N + 63) / 64), static_cast<unsigned>(batch)), 256, 0, stream>>>(
            B, ldb, stride_b, trans_b, colsum, N, static_cast<int>(K), static_cast<int>(N), static_cast<int>(K));
        g.colsum = colsum;
        g.stride_colsum = N;
    }

    const bool a_ok = K % 16 == 0 && lda % 16 == 0 && stride_a % 16 == 0 && aligned16(A);
    // a single problem is a Dense without bias: the kernels that requantise from registers take it where they apply
    auto launch_aligned = [&]() {
        if (batch == 1 && wreg_applicable(g)) return launch_wreg(g, stream);
        if (batch == 1 && sk_applicable(g) && sk_preferred(g)) return launch_sk(g, stream);
        return launch_gemm_nt(g, static_cast<int>(batch), stream, env_variant());
    };
    hipError_t e;
    if (trans_b) {
        g.Bt = B;
        g.ldb = ldb;
        g.stride_b = stride_b;
        if (trans_a) {
            e = launch_trans_a(g, static_cast<int>(batch), stream);
        } else if (a_ok && ldb % 16 == 0 && stride_b % 16 == 0 && aligned16(B)) {
            e = launch_aligned();
        } else {
            e = launch_ragged(g, static_cast<int>(batch), stream);
        }
    } else {
        launch_transpose_kn(B, ldb, stride_b, ws, ldt, N * ldt, K, N, batch, stream);
        g.Bt = ws;
        g.ldb = ldt;
        g.stride_b = N * ldt;
        if (lean_shape) {  // a short reduction against a wide right operand given as [K][N]: its transpose takes the lean kernel
            la.B = ws;
            la.ldb = ldt;
            la.stride_b = N * ldt;
            if (lean_nt_applicable(la)) return check_hip(launch_lean_nt(la, stream), who);
        }
        e = trans_a ? launch_trans_a(g, static_cast<int>(batch), stream)
            : a_ok  ? launch_aligned()
                    : launch_ragged(g, static_cast<int>(batch), stream);
    }
    return check_hip(e, who);
}

extern "C" int a4g_matmul_i8(const void* A, int a_kind, int trans_a, int64_t lda, int64_t stride_a, const int8_t* B, int64_t ldb,
                             int64_t stride_b, int trans_b, void* C, int64_t ldc, int64_t stride_c, int64_t batch, int64_t M,
                             int64_t N, int64_t K, int shift, int round_mode, int out_kind, void* workspace,
                             size_t workspace_bytes, a4g_stream_t stream_) {
    return matmul_i8_impl("a4g_matmul_i8", false, A, a_kind, trans_a, lda, stride_a, B, ldb, stride_b, trans_b, C, ldc, stride_c, batch, M,
                          N, K, shift, round_mode, out_kind, workspace, workspace_bytes, static_cast<hipStream_t>(stream_));
}

extern "C" int a4g_matmul_i8_static(const void* A, int a_kind, int trans_a, int64_t lda, int64_t stride_a, const int8_t* B, int64_t ldb,
                                    int64_t stride_b, int trans_b, void* C, int64_t ldc, int64_t stride_c, int64_t batch,
                                    int64_t M, int64_t N, int64_t K, int shift, int round_mode, int out_kind,
                                    a4g_stream_t stream_) {
    // Nothing in the array has to start at zero: the repack writes every byte the GEMM reads (rows are zero padded
    // to the packed pitch) and the column-sum kernel stores, never accumulates.
    return matmul_i8_impl("a4g_matmul_i8_static", true, A, a_kind, trans_a, lda, stride_a, B, ldb, stride_b, trans_b, C, ldc, stride_c,
                          batch, M, N, K, shift, round_mode, out_kind, nullptr, 0, static_cast<hipStream_t>(stream_));
}
