// Dense for short reductions (K <= 768) on many rows: the weights stay in registers, the activations stream.
//
// The tiled kernel of gemm_rs.hpp pays a fixed price per output tile (first loads from a cold start, parameter
// parking, the requantising epilogue through an LDS image); with K = 768 a 128 x 128 tile has only six K tiles of
// work to set against it, and the encoder's projections (8192 x 2304 x 768, 8192 x 3072 x 768) ran with the matrix pipe
// 17 % busy. Here a workgroup of four waves owns a block of 128 output columns for a long run of rows:
//   * wave w keeps the weights of its 32 columns for the whole reduction in registers (K / 32 fragments of 16 bytes
//     per lane, 96 registers at K = 768), loaded once per run;
//   * weights first, then activations, travel through ONE ring of four LDS stages of 128 rows x 128 bytes, filled by
//     buffer loads that write LDS directly (no staging registers), three tiles ahead of the one being consumed, so only
//     the first tile of a run sees a cold start;
//   * after the last K tile of every 128 rows the accumulators are requantised and stored straight from registers:
//     the weight rows are taken in a permuted order that leaves a lane with 16 contiguous output bytes per 32 x 32
//     block (an integer dot product does not care which lane supplies which column), so no LDS image is needed.
// Same arithmetic as the other Dense kernels (dense_bias_relu.cpp:112-163): int32 accumulation, + bias, shift / round /
// saturate, ReLU.
#include <algorithm>
#include <type_traits>

#include "gemm_direct.hpp"

namespace a4g {

constexpr int WR_BM = 128, WR_BN = 128, WR_BK = 128, WR_NT = 256;
constexpr int WR_STAGE = WR_BM * WR_BK;  // 16 KiB
constexpr int WR_NST = 4;                // stages of the ring (power of two); three tiles are in flight
constexpr int WR_WGS = 512;               // two workgroups per CU
using WregParams = DirectParams<WR_BN>;
constexpr int WR_LDS = WR_NST * WR_STAGE + WregParams::BYTES;

// One workgroup: one block of 128 output columns and a run of rows in 64-row halves, [h0, h1) of the `halves_m` halves
// of the matrix; the `wgs_per_cb` workgroups of a column block share its rows as evenly as halves allow. Rows are
// processed 128 at a time; a run of an odd number of halves ends with a step of 64 rows.
// PARTIAL: the reduction ends inside its last 128-byte tile (K a multiple of 16 only).
template <int NKT, bool A_UNSIGNED, bool PARTIAL = false>
__global__ __launch_bounds__(WR_NT, 2) void gemm_wreg_kernel(GemmArgs g, int halves_m, int wgs_per_cb, int a_bytes, int w_bytes) {
    constexpr int NKS = NKT * 4;  // K steps of 32 bytes
    extern __shared__ __attribute__((aligned(16))) int8_t wr_smem[];
    int8_t* const stages = wr_smem;  // the ring, then the column parameters
    const WregParams wp(wr_smem + WR_NST * WR_STAGE);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int frow = lane & 31, half = lane >> 5;

    // Workgroups go to the eight XCDs round robin. Renumbered so that an XCD gets consecutive indices, and with the column
    // block varying fastest, an XCD works on one slice of the rows for all column blocks: its L2 fetches those
    // activation rows once instead of every XCD fetching all of them.
    const int nb = gridDim.x, xcd = blockIdx.x & 7, per_xcd = nb >> 3, extra = nb & 7;
    const int index = xcd * per_xcd + min(xcd, extra) + (blockIdx.x >> 3);
    const int cbs = nb / wgs_per_cb;
    const int part = index / cbs, cb = index - part * cbs;
    const int h0 = part * halves_m / wgs_per_cb, h1 = (part + 1) * halves_m / wgs_per_cb;
    const int n0 = cb * WR_BN;
    const int m0 = h0 * 64, m_end = min(g.M, h1 * 64);
    const int steps = (h1 - h0 + 1) >> 1;
    const bool short_last = (h1 - h0) & 1;  // the last step has 64 rows
    A4G_STAMP(0);

    // Tiles go from global memory straight into LDS (buffer loads with the LDS bit: the 64 lanes of one instruction fill
    // 1 KiB, lane l at byte 16 l, from per-lane global addresses). Instruction j of wave w fills rows 32 w + 8 j .. + 7
    // of a stage; the 16-byte slot s of row r holds K chunk s ^ ((r >> 1) & 7), the swizzle the fragment reads undo.
    // Rows past the end of a matrix lie outside its buffer descriptor and read as zero.
    const int lrow8 = lane >> 3, slot = lane & 7;
    const int lda = static_cast<int>(g.lda), ldb = static_cast<int>(g.ldb);
    // rows 32 w + 8 j + lrow8: the swizzle term is (lrow8 >> 1) for even j and that ^ 4 for odd j, so two per-lane
    // offsets (j = 0, 1) cover all four instructions; j = 2, 3 add 16 rows, a scalar
    const int row0 = wave * 32 + lrow8, sw0 = (slot ^ (lrow8 >> 1)) * 16;
    const int va0 = row0 * lda + sw0, va1 = (row0 + 8) * lda + (sw0 ^ 64);
    // A reduction that ends inside its last 128-byte tile (K a multiple of 16 only): the lanes whose chunk of that tile
    // lies past K fetch nothing (an offset of the buffer's size: zeros), and zero activations make whatever the weight
    // tile holds there (the next weight row's first bytes) count for nothing.
    const int k_last = g.K - (NKT - 1) * WR_BK;  // bytes of the last tile that exist, 16 .. 128
    const int va0_last = (!PARTIAL || sw0 < k_last) ? va0 : a_bytes, va1_last = (!PARTIAL || (sw0 ^ 64) < k_last) ? va1 : a_bytes;
    const auto rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(g.A), 0, a_bytes, 0x00020000);
    const auto rsrc_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(g.Bt), 0, w_bytes, 0x00020000);

    int koff[4];  // activation fragment of K step kk: row frow (+ 32 i), chunk 2 kk + half
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) koff[kk] = frow * WR_BK + (((kk * 2 + half) ^ ((frow >> 1) & 7)) * 16);
    const int wrow = wave * 32 + direct_col_of_operand_row(frow);  // weight fragment: this lane's column of the block

    const int lo = g.relu ? max(kind_lo(g.out_kind), 0) : kind_lo(g.out_kind), hi = kind_hi(g.out_kind);

    // one tile: `toff` is the byte offset of its first row and K chunk, or (nothing to fetch) the size of the buffer, which
    // puts every lane out of range
    auto issue = [&](__amdgpu_buffer_rsrc_t rsrc, int v0, int v1, int ld, int toff, int st) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            int8_t* dst = stages + st * WR_STAGE + (wave * 4 + j) * 1024;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (__attribute__((address_space(3))) void*)dst, 16,
                                                     ((j & 1) ? v1 : v0) + (toff + (j >> 1) * 16 * ld), 0, 0, 0);
        }
    };
    // activation tile (step, kt) of the run; nothing is fetched past its end (the lower 64 rows of a short last step)
    auto issue_a = [&](int step, int kt, int st) {
        const bool live = step < steps && !(short_last && step == steps - 1 && wave >= 2);
        const bool last_kt = PARTIAL && kt == NKT - 1;
        issue(rsrc_a, last_kt ? va0_last : va0, last_kt ? va1_last : va1, lda, live ? (m0 + step * WR_BM) * lda + kt * WR_BK : a_bytes, st);
    };
    // ring position r: the NKT weight tiles of the column block, then the activation tiles
    auto issue_ring = [&](int r) {
        if (r < NKT) issue(rsrc_w, row0 * ldb + sw0, (row0 + 8) * ldb + (sw0 ^ 64), ldb, n0 * ldb + r * WR_BK, r & (WR_NST - 1));
        else issue_a((r - NKT) / NKT, (r - NKT) % NKT, r & (WR_NST - 1));
    };
    auto tile_ready = [&]() {
        // own loads of the oldest tile in flight have landed (the eight younger loads may be outstanding), own reads of the
        // previous tile are complete; after the barrier that holds for every wave
        asm volatile("s_waitcnt vmcnt(8) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
    };

    TileCoord tc;
    tc.m0 = m0;
    tc.n0 = n0;
    tc.batch = 0;
    tc.valid = true;
    int col_add, col_shift;
    fetch_col_params<WR_BN, A_UNSIGNED>(g, tc, tid, col_add, col_shift);
#pragma unroll
    for (int r = 0; r < 3; ++r) issue_ring(r);
    const bool general = direct_park<WR_BN>(g, wp, tid, col_add, col_shift, lo, hi);

    // ---- weights of this wave's 32 columns: ring -> registers
    v4i bw[NKS];
#pragma unroll
    for (int r = 0; r < NKT; ++r) {
        tile_ready();
        issue_ring(r + 3);  // into the stage of tile r - 1
        const int8_t* st = stages + (r & (WR_NST - 1)) * WR_STAGE + wrow * WR_BK;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) bw[r * 4 + kk] = *reinterpret_cast<const v4i*>(st + (((kk * 2 + half) ^ ((wrow >> 1) & 7)) * 16));
    }

    constexpr int AFS = NKT <= 4 ? 2 : 1;  // fragment sets: two where the weights leave room (a few percent faster)
    v4i af[AFS][4];
    tile_ready();  // the first activation tile
#pragma unroll
    for (int i = 0; i < 4; ++i) af[0][i] = *reinterpret_cast<const v4i*>(stages + (NKT & (WR_NST - 1)) * WR_STAGE + koff[0] + i * 32 * WR_BK);

    A4G_STAMP(1);
    int tv = NKT;  // ring position of the tile being computed
    const int nl_fixed = wave * 32 + 16 * half;  // first of this lane's 16 columns inside the block
    const bool cols_ok = n0 + nl_fixed + 16 <= g.N;
    v16i acc[4];

    // the NKT tiles of one step; NRB row blocks of 32 take part (4, or 2 in a short last step)
    auto reduce_step = [&](int step, auto nrb_tag) {
        constexpr int NRB = decltype(nrb_tag)::value;
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt, ++tv) {
            const int cur = (tv & (WR_NST - 1)) * WR_STAGE, nxt = ((tv + 1) & (WR_NST - 1)) * WR_STAGE;
            issue_a(step + (kt + 3) / NKT, (kt + 3) % NKT, (tv + 3) & (WR_NST - 1));  // into the stage of tile tv - 1
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                if (kk == 3) {
                    __builtin_amdgcn_sched_barrier(0);
                    tile_ready();  // tile tv + 1
                    __builtin_amdgcn_sched_barrier(0);
                }
                const int rd = (kk < 3 ? cur : nxt) + koff[(kk + 1) & 3];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (i < NRB) {
                        v4i a_op = af[kk % AFS][i];
                        // uint8 -> int8; 128 * colsum is in the start value. The chunks of the last tile that lie past K were
                        // fetched as zeros and stay zeros (biased they would count as -128 against whatever the weight tile
                        // holds there).
                        // (Not in the six-tile form, which has no register left for the mask: there K is 768.)
                        if (A_UNSIGNED)
                            a_op ^= (!PARTIAL || NKT == 6 || kt < NKT - 1 || kk * 32 + half * 16 < k_last) ? static_cast<int>(0x80808080u) : 0;
                        acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bw[kt * 4 + kk], a_op, acc[i], 0, 0, 0);
                    }
                    // the fragment of the next K step follows the MFMA that read this one: steps 1..3 from this tile, step
                    // 0 from the next
                    af[(kk + 1) % AFS][i] = *reinterpret_cast<const v4i*>(stages + rd + i * 32 * WR_BK);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };

    for (int step = 0; step < steps; ++step) {
        // The parameters are read from LDS again in every step: laundering the index keeps the compiler from holding all 80
        // of them in registers across the main loop, which the weights need.
        int nl = nl_fixed;
        asm volatile("" : "+v"(nl));
        // accumulators start from bias + 128 * colsum when the quick requantisation applies, else from zero
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            v4i add4 = {0, 0, 0, 0};
            if (!general) add4 = *reinterpret_cast<const v4i*>(wp.add + nl + 4 * q);
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[i][q * 4 + t] = add4[t];
        }
        if (short_last && step == steps - 1) reduce_step(step, std::integral_constant<int, 2>{});
        else reduce_step(step, std::integral_constant<int, 4>{});
        if (step == 0) A4G_STAMP(2);
        asm volatile("" : "+v"(nl));

        // ---- epilogue of these rows, straight from registers: lane (m, half) holds, per row block i, the 16 output bytes
        // of columns 16 * half .. + 15 of its wave's 32; dword q of them replaces accumulator q
        auto quick = [&](auto bit_tag, auto conv_tag) {
            constexpr int BIT = decltype(bit_tag)::value;
            constexpr bool CONV = decltype(conv_tag)::value;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4i s4 = *reinterpret_cast<const v4i*>(wp.s + nl + 4 * q);
                const v4i c04 = *reinterpret_cast<const v4i*>(wp.c0 + nl + 4 * q);
                const v4i lo4 = *reinterpret_cast<const v4i*>(wp.lo_s + nl + 4 * q);
                const v4i hi4 = *reinterpret_cast<const v4i*>(wp.hi_s + nl + 4 * q);
#pragma unroll
                for (int i = 0; i < 4; ++i)
                    acc[i][q] = static_cast<int>(direct_requant4<BIT, CONV>(acc[i][q * 4], acc[i][q * 4 + 1], acc[i][q * 4 + 2], acc[i][q * 4 + 3], s4, c04, lo4, hi4));
                __builtin_amdgcn_sched_barrier(0);  // one column group at a time: the weights leave few registers free
            }
        };
        using B0 = std::integral_constant<int, 0>;
        using B1 = std::integral_constant<int, 1>;
        using B2 = std::integral_constant<int, 2>;
        if (general) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4i add4 = *reinterpret_cast<const v4i*>(wp.add + nl + 4 * q);
                const v4i s4 = *reinterpret_cast<const v4i*>(wp.s + nl + 4 * q);
                const v4i c04 = *reinterpret_cast<const v4i*>(wp.c0 + nl + 4 * q);
                const v4i cx4 = *reinterpret_cast<const v4i*>(wp.cx + nl + 4 * q);
                const v4i bs4 = *reinterpret_cast<const v4i*>(wp.bs + nl + 4 * q);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    acc[i][q] = static_cast<int>(direct_requant4_general(acc[i][q * 4], acc[i][q * 4 + 1], acc[i][q * 4 + 2], acc[i][q * 4 + 3], add4, s4, c04, cx4, bs4, lo, hi));
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        } else if (g.mode <= A4G_RND_NEGATIVE_INF) quick(B0{}, std::false_type{});
        else if (g.mode == A4G_RND_SYMMETRIC_INF) quick(B2{}, std::false_type{});
        else if (g.mode == A4G_RND_SYMMETRIC_ZERO) quick(B1{}, std::false_type{});
        else if (g.mode == A4G_RND_CONV_EVEN) quick(B1{}, std::true_type{});
        else quick(B2{}, std::true_type{});

        int8_t* Cb = static_cast<int8_t*>(g.C);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int m = m0 + step * WR_BM + i * 32 + frow;
            if (m < m_end && cols_ok) {
                const v4i o = {acc[i][0], acc[i][1], acc[i][2], acc[i][3]};
                *reinterpret_cast<v4i*>(Cb + static_cast<int64_t>(m) * g.ldc + n0 + nl_fixed) = o;
            }
        }
    }
    A4G_STAMP(3);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the loads issued past the run's end have retired
    A4G_STAMP(4);
    A4G_STAMP(5);
}

template <int NKT, bool A_UNSIGNED, bool PARTIAL>
hipError_t launch_wreg_kernel(const GemmArgs& g, int halves_m, int wgs_per_cb, int cbs, int a_bytes, int w_bytes, hipStream_t stream) {
    auto kern = gemm_wreg_kernel<NKT, A_UNSIGNED, PARTIAL>;
    static bool attr_set = false;  // benign race: the attribute is idempotent
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, WR_LDS);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    kern<<<wgs_per_cb * cbs, WR_NT, WR_LDS, stream>>>(g, halves_m, wgs_per_cb, a_bytes, w_bytes);
    return hipGetLastError();
}
template <int NKT>
hipError_t launch_wreg_nkt(const GemmArgs& g, int halves_m, int wgs_per_cb, int cbs, int a_bytes, int w_bytes, hipStream_t stream) {
    if (g.K % 128 == 0)
        return g.a_unsigned ? launch_wreg_kernel<NKT, true, false>(g, halves_m, wgs_per_cb, cbs, a_bytes, w_bytes, stream)
                            : launch_wreg_kernel<NKT, false, false>(g, halves_m, wgs_per_cb, cbs, a_bytes, w_bytes, stream);
    if constexpr (NKT < 6) {
        if (g.a_unsigned) return launch_wreg_kernel<NKT, true, true>(g, halves_m, wgs_per_cb, cbs, a_bytes, w_bytes, stream);
    }
    return launch_wreg_kernel<NKT, false, true>(g, halves_m, wgs_per_cb, cbs, a_bytes, w_bytes, stream);
}

// Reductions of one to six whole 128-byte tiles, one-byte outputs, 16-byte aligned rows on both sides, widths in whole
// 16-column pieces, and operands small enough for 32-bit buffer offsets. Measured faster than the tiled kernel at every
// size tried, from one row to 8192 x 3072.
bool wreg_applicable(const GemmArgs& g) {
    // K in whole 128-byte tiles, or ending inside the last one on a multiple of 16 (unsigned activations: up to 640)
    return g.M > 0 && g.K % 16 == 0 && g.K >= 16 && g.K <= 768 && (g.K % 128 == 0 || !g.a_unsigned || g.K <= 640) && g.N % 16 == 0 && g.N >= 16 &&
           (g.out_kind == A4G_I8 || g.out_kind == A4G_U8) && g.lda % 16 == 0 && g.ldb % 16 == 0 && g.ldc % 16 == 0 && aligned16(g.A) &&
           aligned16(g.Bt) && aligned16(g.C) && (static_cast<int64_t>(g.M) + 2 * WR_BM) * g.lda < (int64_t{1} << 31) &&
           (static_cast<int64_t>(g.N) + WR_BN) * g.ldb < (int64_t{1} << 31) && (g.N + WR_BN - 1) / WR_BN <= 65536;
}

hipError_t launch_wreg(const GemmArgs& g, hipStream_t stream) {
    if (wrow_applicable(g)) return launch_wrow(g, stream);
    const int halves_m = (g.M + 63) / 64, cbs = (g.N + WR_BN - 1) / WR_BN;
    // 512 workgroups fill the chip (two per CU) and the column blocks get an equal share of them each; of the counts
    // that give the longest run the same number of halves, the smallest loads the weights least often
    const int most = std::min(halves_m, std::max(1, WR_WGS / cbs));
    const int longest = (halves_m + most - 1) / most;
    const int wgs_per_cb = (halves_m + longest - 1) / longest;
    const int a_bytes = static_cast<int>(static_cast<int64_t>(g.M - 1) * g.lda + g.K);
    const int w_bytes = static_cast<int>(static_cast<int64_t>(g.N - 1) * g.ldb + g.K);
    switch ((g.K + 127) / 128) {
    case 1: return launch_wreg_nkt<1>(g, halves_m, wgs_per_cb, cbs, a_bytes, w_bytes, stream);
    case 2: return launch_wreg_nkt<2>(g, halves_m, wgs_per_cb, cbs, a_bytes, w_bytes, stream);
    case 3: return launch_wreg_nkt<3>(g, halves_m, wgs_per_cb, cbs, a_bytes, w_bytes, stream);
    case 4: return launch_wreg_nkt<4>(g, halves_m, wgs_per_cb, cbs, a_bytes, w_bytes, stream);
    case 5: return launch_wreg_nkt<5>(g, halves_m, wgs_per_cb, cbs, a_bytes, w_bytes, stream);
    case 6: return launch_wreg_nkt<6>(g, halves_m, wgs_per_cb, cbs, a_bytes, w_bytes, stream);
    default: return hipErrorInvalidValue;
    }
}

}  // namespace a4g
