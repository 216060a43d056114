// Dense for long reductions on outputs too narrow to fill the chip with big tiles: 128 x 192 output tiles, the reduction
// split between the two halves of an eight-wave workgroup.
//
// A 8192 x 768 output with K = 3072 (the encoder's second feed-forward projection) has only 256 tiles of 128 x 192:
// one per CU. With four waves per tile every SIMD holds a single wave, and nothing runs while that wave waits on LDS
// or at a barrier: the tiled kernel of gemm_rs.hpp reached 27 % of the matrix peak there. Here
//   * the workgroup has eight waves in two groups of four (2 x 2 waves of 64 x 96 each); group 0 reduces the even
//     64-byte K tiles, group 1 the odd ones, so every SIMD always has two waves with independent work;
//   * each group streams its tiles (128 x 64 bytes of activations, 192 x 64 of weights) through its own ring of three
//     LDS stages, filled by buffer loads that write LDS directly, two tiles ahead of the one being consumed;
//   * at the end the groups swap halves of their partial sums through LDS (each keeps 32 of its 64 rows per wave),
//     and both requantise and store straight from registers, as in gemm_wreg.hip.
// Same arithmetic as the other Dense kernels (dense_bias_relu.cpp:112-163): int32 accumulation (wrapping addition is
// associative, so the split changes nothing), + bias, shift / round / saturate, ReLU.
#include <algorithm>
#include <type_traits>

#include "gemm_direct.hpp"

namespace a4g {

constexpr int SK_BM = 128, SK_BN = 192, SK_BK = 64, SK_NT = 512;
constexpr int SK_A = SK_BM * SK_BK, SK_W = SK_BN * SK_BK;  // 8 KiB + 12 KiB per stage
constexpr int SK_STAGE = SK_A + SK_W;
constexpr int SK_NST = 3;
constexpr int SK_RING = SK_NST * SK_STAGE;  // per group
using SkParams = DirectParams<SK_BN>;
constexpr int SK_LDS = 2 * SK_RING + SkParams::BYTES;

template <bool A_UNSIGNED>
__global__ __launch_bounds__(SK_NT, 1) void gemm_sk_kernel(GemmArgs g, int tiles_n, int a_bytes, int w_bytes) {
    extern __shared__ __attribute__((aligned(16))) int8_t sk_smem[];
    const SkParams wp(sk_smem + 2 * SK_RING);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int grp = wave >> 2, wq = wave & 3, wm = wq >> 1, wn = wq & 1;
    const int frow = lane & 31, half = lane >> 5;
    int8_t* const ring = sk_smem + grp * SK_RING;

    // Workgroups go to the eight XCDs round robin; numbering the tiles so that an XCD gets consecutive ones keeps the
    // column tiles that share activation rows on one L2.
    const int nb = gridDim.x, b = blockIdx.x;
    const int id = (nb & 7) == 0 ? (b & 7) * (nb >> 3) + (b >> 3) : b;
    const int tm = id / tiles_n, tn = id - tm * tiles_n;
    const int m0 = tm * SK_BM, n0 = tn * SK_BN;

    A4G_STAMP(0);
    const int nkt = g.K / SK_BK;  // K tiles of 64 bytes, an even number; this group takes tile 2 j + grp as its j-th
    const int ntl = nkt >> 1;     // tiles per group

    // Tiles go from global memory straight into LDS: one buffer load fills 1 KiB (16 rows of 64 bytes), lane l at byte
    // 16 l. The 16-byte slot s of an activation row r holds K chunk s ^ ((r >> 2) & 3), the swizzle the fragment reads undo. Per tile
    // a wave issues two instructions for the activations (rows 32 wq + 16 ja ..) and three for the weights (rows 48 wq +
    // 16 jb ..). Rows past the end of a matrix lie outside its buffer descriptor and read as zero.
    const int lda = static_cast<int>(g.lda), ldb = static_cast<int>(g.ldb);
    // (weights: s ^ (bit 2 of r | bit 4 of r << 1) instead, because the MFMA takes weight rows in a permuted order in which
    // rows r and r + 16 sit in neighbouring lanes)
    const int lrow = lane >> 2, sw = ((lane & 3) ^ ((lane >> 4) & 3)) * 16;
    const int va = lrow * lda + sw;
    const int vw_even = lrow * ldb + ((lane & 3) ^ ((lane >> 4) & 1)) * 16;        // rows 16 b .. with b even: bit 4 clear
    const int vw_odd = lrow * ldb + ((lane & 3) ^ (((lane >> 4) & 1) | 2)) * 16;  // b odd
    const auto rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(g.A), 0, a_bytes, 0x00020000);
    const auto rsrc_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(g.Bt), 0, w_bytes, 0x00020000);
    auto issue_tile = [&](int j, int st) {
        const int t = 2 * j + grp;
        const bool live = t < nkt;
        int8_t* stage = ring + st * SK_STAGE;
#pragma unroll
        for (int ja = 0; ja < 2; ++ja) {
            const int r0 = wq * 32 + ja * 16;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(stage + r0 * SK_BK), 16,
                                                     live ? va + ((m0 + r0) * lda + t * SK_BK) : a_bytes, 0, 0, 0);
        }
#pragma unroll
        for (int jb = 0; jb < 3; ++jb) {
            const int r0 = wq * 48 + jb * 16;
            const int vw = ((wq * 3 + jb) & 1) ? vw_odd : vw_even;
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_w, (__attribute__((address_space(3))) void*)(stage + SK_A + r0 * SK_BK), 16,
                                                     live ? vw + ((n0 + r0) * ldb + t * SK_BK) : w_bytes, 0, 0, 0);
        }
    };
    auto tile_ready = [&](auto younger_tag) {
        // own loads of the oldest tile in flight have landed (those of `younger` tiles, five each, may be outstanding), own
        // fragment reads are complete; after the barrier both hold for every wave
        constexpr int YOUNGER = decltype(younger_tag)::value;
        if (YOUNGER == 2) asm volatile("s_waitcnt vmcnt(10) lgkmcnt(0)" ::: "memory");
        else asm volatile("s_waitcnt vmcnt(5) lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
    };

    // fragments: activations row wm 64 + 32 i + frow, weights row wn 96 + 32 j + (permuted frow), chunk 2 kk + half
    const int pcol = direct_col_of_operand_row(frow);
    int offa[2], offb[2];
#pragma unroll
    for (int kk = 0; kk < 2; ++kk) {
        offa[kk] = (wm * 64 + frow) * SK_BK + (((kk * 2 + half) ^ ((frow >> 2) & 3)) * 16);
        offb[kk] = SK_A + (wn * 96 + pcol) * SK_BK + (((kk * 2 + half) ^ (((pcol >> 2) & 1) | (((pcol >> 4) & 1) << 1))) * 16);
    }

    const int lo = g.relu ? max(kind_lo(g.out_kind), 0) : kind_lo(g.out_kind), hi = kind_hi(g.out_kind);

    TileCoord tc;
    tc.m0 = m0;
    tc.n0 = n0;
    tc.batch = 0;
    tc.valid = true;
    int col_add, col_shift;
    fetch_col_params<SK_BN, A_UNSIGNED>(g, tc, tid, col_add, col_shift);
#pragma unroll
    for (int j = 0; j < 3; ++j) issue_tile(j, j);
    const bool general = direct_park<SK_BN>(g, wp, tid, col_add, col_shift, lo, hi);

    // accumulators: group 0 starts from bias + 128 * colsum when the quick requantisation applies, everything else from 0
    v16i acc[2][3];
#pragma unroll
    for (int j = 0; j < 3; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            v4i add4 = {0, 0, 0, 0};
            if (!general && grp == 0) add4 = *reinterpret_cast<const v4i*>(wp.add + wn * 96 + j * 32 + 16 * half + 4 * q);
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int t = 0; t < 4; ++t) acc[i][j][q * 4 + t] = add4[t];
        }
    }

    v4i fa[2][2], fb[2][3];
    tile_ready(std::integral_constant<int, 2>{});  // tile 0
#pragma unroll
    for (int i = 0; i < 2; ++i) fa[0][i] = *reinterpret_cast<const v4i*>(ring + offa[0] + i * 32 * SK_BK);
#pragma unroll
    for (int j = 0; j < 3; ++j) fb[0][j] = *reinterpret_cast<const v4i*>(ring + offb[0] + j * 32 * SK_BK);

    auto mfmas = [&](int set) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            v4i a_op = fa[set][i];
            if (A_UNSIGNED) a_op ^= static_cast<int>(0x80808080u);  // uint8 -> int8; 128 * colsum is in the start value
#pragma unroll
            for (int j = 0; j < 3; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[set][j], a_op, acc[i][j], 0, 0, 0);
        }
    };

    A4G_STAMP(1);
    int cur = 0;  // byte offset of the stage of the tile being computed
    for (int j = 0; j < ntl; ++j) {
        const int nxt = cur + SK_STAGE == SK_RING ? 0 : cur + SK_STAGE;
        // K step 1 of this tile -> second fragment set, behind the MFMAs of step 0
#pragma unroll
        for (int i = 0; i < 2; ++i) fa[1][i] = *reinterpret_cast<const v4i*>(ring + cur + offa[1] + i * 32 * SK_BK);
#pragma unroll
        for (int jj = 0; jj < 3; ++jj) fb[1][jj] = *reinterpret_cast<const v4i*>(ring + cur + offb[1] + jj * 32 * SK_BK);
        mfmas(0);
        __builtin_amdgcn_sched_barrier(0);
        // tile j + 1 has landed; every fragment of tile j is in registers, so its stage takes tile j + 3
        tile_ready(std::integral_constant<int, 1>{});
        issue_tile(j + 3, cur / SK_STAGE);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int i = 0; i < 2; ++i) fa[0][i] = *reinterpret_cast<const v4i*>(ring + nxt + offa[0] + i * 32 * SK_BK);
#pragma unroll
        for (int jj = 0; jj < 3; ++jj) fb[0][jj] = *reinterpret_cast<const v4i*>(ring + nxt + offb[0] + jj * 32 * SK_BK);
        mfmas(1);
        __builtin_amdgcn_sched_barrier(0);
        cur = nxt;
    }

    A4G_STAMP(2);
    // ---- the groups swap halves: group 0 keeps row block 0 of each wave tile, group 1 row block 1
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");  // the loads issued past the end have retired
    __builtin_amdgcn_s_barrier();                                // nobody reads the rings any more
    auto finish = [&](auto keep_tag) {
        constexpr int KEEP = decltype(keep_tag)::value;  // == grp
        v16i(&kept)[3] = acc[KEEP];
        v16i(&given)[3] = acc[KEEP ^ 1];
        int8_t* out_buf = sk_smem + (KEEP * 4 + wq) * (12 * 1024);
        const int8_t* in_buf = sk_smem + ((KEEP ^ 1) * 4 + wq) * (12 * 1024);
#pragma unroll
        for (int j = 0; j < 3; ++j)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const v4i v = {given[j][r4 * 4], given[j][r4 * 4 + 1], given[j][r4 * 4 + 2], given[j][r4 * 4 + 3]};
                *reinterpret_cast<v4i*>(out_buf + ((j * 4 + r4) * 64 + lane) * 16) = v;
            }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 3; ++j)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                const v4i v = *reinterpret_cast<const v4i*>(in_buf + ((j * 4 + r4) * 64 + lane) * 16);
#pragma unroll
                for (int t = 0; t < 4; ++t)
                    kept[j][r4 * 4 + t] = static_cast<int>(static_cast<unsigned>(kept[j][r4 * 4 + t]) + static_cast<unsigned>(v[t]));  // wrapping
            }

        A4G_STAMP(3);
        // ---- epilogue of the kept 32 rows x 96 columns, straight from registers: lane (m, half) holds, per column block
        // j, the 16 output bytes of columns 16 * half .. + 15; dword q of them replaces accumulator q
        const int nl0 = wn * 96 + 16 * half;
        auto quick = [&](auto bit_tag, auto conv_tag) {
            constexpr int BIT = decltype(bit_tag)::value;
            constexpr bool CONV = decltype(conv_tag)::value;
#pragma unroll
            for (int j = 0; j < 3; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nl = nl0 + j * 32 + 4 * q;
                    const v4i s4 = *reinterpret_cast<const v4i*>(wp.s + nl);
                    const v4i c04 = *reinterpret_cast<const v4i*>(wp.c0 + nl);
                    const v4i lo4 = *reinterpret_cast<const v4i*>(wp.lo_s + nl);
                    const v4i hi4 = *reinterpret_cast<const v4i*>(wp.hi_s + nl);
                    kept[j][q] = static_cast<int>(direct_requant4<BIT, CONV>(kept[j][q * 4], kept[j][q * 4 + 1], kept[j][q * 4 + 2], kept[j][q * 4 + 3], s4, c04, lo4, hi4));
                }
        };
        using B0 = std::integral_constant<int, 0>;
        using B1 = std::integral_constant<int, 1>;
        using B2 = std::integral_constant<int, 2>;
        if (general) {
#pragma unroll
            for (int j = 0; j < 3; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nl = nl0 + j * 32 + 4 * q;
                    const v4i add4 = *reinterpret_cast<const v4i*>(wp.add + nl);
                    const v4i s4 = *reinterpret_cast<const v4i*>(wp.s + nl);
                    const v4i c04 = *reinterpret_cast<const v4i*>(wp.c0 + nl);
                    const v4i cx4 = *reinterpret_cast<const v4i*>(wp.cx + nl);
                    const v4i bs4 = *reinterpret_cast<const v4i*>(wp.bs + nl);
                    kept[j][q] = static_cast<int>(direct_requant4_general(kept[j][q * 4], kept[j][q * 4 + 1], kept[j][q * 4 + 2], kept[j][q * 4 + 3], add4, s4, c04, cx4, bs4, lo, hi));
                }
        } else if (g.mode <= A4G_RND_NEGATIVE_INF) quick(B0{}, std::false_type{});
        else if (g.mode == A4G_RND_SYMMETRIC_INF) quick(B2{}, std::false_type{});
        else if (g.mode == A4G_RND_SYMMETRIC_ZERO) quick(B1{}, std::false_type{});
        else if (g.mode == A4G_RND_CONV_EVEN) quick(B1{}, std::true_type{});
        else quick(B2{}, std::true_type{});

        A4G_STAMP(4);
        int8_t* Cb = static_cast<int8_t*>(g.C);
        const int m = m0 + wm * 64 + KEEP * 32 + frow;
#pragma unroll
        for (int j = 0; j < 3; ++j) {
            const int n = n0 + nl0 + j * 32;
            if (m < g.M && n + 16 <= g.N) {
                const v4i o = {kept[j][0], kept[j][1], kept[j][2], kept[j][3]};
                *reinterpret_cast<v4i*>(Cb + static_cast<int64_t>(m) * g.ldc + n) = o;
            }
        }
    };
    if (grp == 0) finish(std::integral_constant<int, 0>{});
    else finish(std::integral_constant<int, 1>{});
    A4G_STAMP(5);
}

template <bool A_UNSIGNED>
hipError_t launch_sk_kernel(const GemmArgs& g, int tiles_m, int tiles_n, int a_bytes, int w_bytes, hipStream_t stream) {
    auto kern = gemm_sk_kernel<A_UNSIGNED>;
    static bool attr_set = false;  // benign race: the attribute is idempotent
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, SK_LDS);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    kern<<<tiles_m * tiles_n, SK_NT, SK_LDS, stream>>>(g, tiles_n, a_bytes, w_bytes);
    return hipGetLastError();
}

// Reductions in whole pairs of 64-byte tiles (one for each group), one-byte outputs, 16-byte aligned rows
// on both sides, widths in whole 16-column pieces, operands small enough for 32-bit buffer offsets.
bool sk_applicable(const GemmArgs& g) {
    const int64_t tiles = static_cast<int64_t>((g.M + SK_BM - 1) / SK_BM) * ((g.N + SK_BN - 1) / SK_BN);
    return g.M > 0 && g.K % 128 == 0 && g.K >= 128 && g.N % 16 == 0 && g.N >= 16 && (g.out_kind == A4G_I8 || g.out_kind == A4G_U8) &&
           g.lda % 16 == 0 && g.ldb % 16 == 0 && g.ldc % 16 == 0 && aligned16(g.A) && aligned16(g.Bt) && aligned16(g.C) &&
           (static_cast<int64_t>(g.M) + SK_BM) * g.lda < (int64_t{1} << 31) && (static_cast<int64_t>(g.N) + SK_BN) * g.ldb < (int64_t{1} << 31) &&
           tiles < (int64_t{1} << 31);
}

// Where it beats the tiled kernels (by 5 to 10 %): reductions too long for gemm_wreg.hip whose 128 x 192 tiles number at
// most one per CU, so that the tiled kernel would leave one wave on every SIMD. With more tiles than CUs the tiled
// kernels' larger tiles win (8192 x 4096 x 4096: 135 us against 181 us here).
bool sk_preferred(const GemmArgs& g) {
    const int64_t tiles = static_cast<int64_t>((g.M + SK_BM - 1) / SK_BM) * ((g.N + SK_BN - 1) / SK_BN);
    return g.K > 768 && tiles <= 256;
}

hipError_t launch_sk(const GemmArgs& g, hipStream_t stream) {
    const int tiles_m = (g.M + SK_BM - 1) / SK_BM, tiles_n = (g.N + SK_BN - 1) / SK_BN;
    const int a_bytes = static_cast<int>(static_cast<int64_t>(g.M - 1) * g.lda + g.K);
    const int w_bytes = static_cast<int>(static_cast<int64_t>(g.N - 1) * g.ldb + g.K);
    return g.a_unsigned ? launch_sk_kernel<true>(g, tiles_m, tiles_n, a_bytes, w_bytes, stream)
                        : launch_sk_kernel<false>(g, tiles_m, tiles_n, a_bytes, w_bytes, stream);
}

}  // namespace a4g
