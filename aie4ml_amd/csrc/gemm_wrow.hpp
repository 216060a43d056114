// Dense for short reductions (K <= 768) on many rows: the weights stay in registers, the activations stream in
// 64-row pieces, and the requantisation of one row block runs between the MFMAs of the next.
//
// One workgroup of four waves per CU, one wave per SIMD with the whole register file, works through a run of
// (column block, 64-row piece) pairs:
//   * wave w keeps the weights of its 64 columns of the 256-column block for the whole reduction in registers (two
//     column groups of K / 32 fragments of 16 bytes per lane, 192 registers at K = 768), fetched whenever the run
//     enters a new column block from a copy of the weights in fragment order (a4g_rowpack_weights_i8: one load
//     instruction fetches 1 KiB of consecutive bytes; taken from the row-major weights the same fragment touches 32
//     cache lines, and the 192 loads of a workgroup took 6.7 us);
//   * the activations travel through a ring of LDS slots of one piece each (K / 128 tiles of 64 rows x 128 bytes), filled
//     by buffer loads that write LDS directly, two pieces (more for shorter reductions) ahead of the one being read; a
//     piece is waited for and handed over with one barrier (per 96 MFMAs of a wave at K = 768), and the ring runs on
//     across column blocks, so only the first piece of a workgroup sees a cold start. A tile fetched into LDS once
//     serves 256 output columns (at the rate of the matrix pipe that is half of what a CU can take in from L2;
//     128-column blocks need all of it), and a fragment read from LDS serves two MFMAs, one per column group;
//   * a wave takes the piece's two 32-row blocks one after the other; the MFMAs of its two column groups alternate
//     and do not wait for each other. Two accumulator sets alternate by row block: while one is filled (starting from
//     bias + 128 * colsum through the MFMA's addend), the other, complete, is requantised one value per MFMA in the
//     shadow of the matrix pipe, with the shifts and rounding constants of the lane's 32 columns in registers, packed
//     and stored straight from registers (the weight rows are taken in a permuted order that leaves a lane with 16
//     contiguous output bytes per 32 x 32 block). With everything in one wave there is no second wave to cover a
//     stall, so nothing in the loop waits on anything younger than eight MFMAs;
//   * the pieces are shared out statically: an XCD owns one slice of the rows for all column blocks (its L2 then fetches
//     those activation rows once), and the workgroups of an XCD split its pairs, column block major, into equal runs.
// Same arithmetic as the other Dense kernels (dense_bias_relu.cpp:112-163): int32 accumulation, + bias, shift / round /
// saturate, ReLU.
#include <algorithm>
#include <type_traits>

#pragma once
#include "gemm_direct.hpp"

namespace a4g {

#define WS_INLINE __attribute__((always_inline))

// f(integral_constant<int, I>) for I = B .. E - 1, in order: an unrolled loop whose index is a compile-time constant in
// the body (a `#pragma unroll` loop of this size is past the optimizer's limit and would stay a loop)
template <int B, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
    if constexpr (B < E) {
        f(std::integral_constant<int, B>{});
        static_for<B + 1, E>(f);
    }
}

// acc += w * a on the matrix pipe with the weight fragment in accumulation registers, which only MFMAs can address:
// that leaves the 256 ordinary registers of the wave to everything else. The compiler does not look into these
// instructions for hazards, so their callers keep a written register away from the MFMA that reads it: the fragment
// comes from LDS behind a wait (or through a vector instruction, then two idle states in front), the addend was
// written long before, and a result is read again two MFMAs later at the earliest.
template <bool NOPS>
__device__ __forceinline__ void mfma_aw(v16i& acc, const v4i& w, const v4i& a) {
    if (NOPS) asm volatile("s_nop 1\n\tv_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc) : "a"(w), "v"(a));
    else asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %0" : "+v"(acc) : "a"(w), "v"(a));
}
template <bool NOPS>
__device__ __forceinline__ void mfma_aw_from(v16i& acc, const v4i& w, const v4i& a, const v16i& start) {
    if (NOPS) asm volatile("s_nop 1\n\tv_mfma_i32_32x32x32_i8 %0, %1, %2, %3" : "=&v"(acc) : "a"(w), "v"(a), "v"(start));
    else asm volatile("v_mfma_i32_32x32x32_i8 %0, %1, %2, %3" : "=&v"(acc) : "a"(w), "v"(a), "v"(start));
}
// Every MFMA issued so far has written its result (the longest takes 16 passes of 4 cycles).
__device__ __forceinline__ void mfma_drain() { asm volatile("s_nop 15\n\ts_nop 15\n\ts_nop 15\n\ts_nop 15" ::: "memory"); }

constexpr int WS_ROWS = 64, WS_BN = 256, WS_BK = 128, WS_NT = 256;
constexpr int WS_STAGE = WS_ROWS * WS_BK;  // 8 KiB: one 128-byte K tile of a piece
constexpr int WS_WGS = 256;                // one workgroup per CU
using WsParams = DirectParams<WS_BN>;
// Pieces the ring holds: the one being read, and up to sixteen tiles' worth (at least two pieces) on their way.
constexpr int ws_slots(int nkt) { return nkt >= 5 ? 3 : 16 / nkt; }
constexpr int ws_lds_bytes(int nkt) { return ws_slots(nkt) * nkt * WS_STAGE + WsParams::BYTES; }
static_assert(ws_lds_bytes(6) <= 160 * 1024, "LDS budget");

// NKT: 128-byte tiles of the reduction (the fragment-order weights are zero padded to whole tiles, so whatever the
// activation rows hold behind a K that ends inside the last tile counts for nothing).
// KIND: the quick requantisation the rounding mode takes: 0 no tie bit, 1 minus / 2 plus the sign, 3 plus / 4 minus bit s.
// `sliced`: XCD x takes the 64-row pieces [x * pieces / 8, (x + 1) * pieces / 8) for every column block.
template <int NKT, bool A_UNSIGNED, int KIND>
__global__ __launch_bounds__(WS_NT, 1) void gemm_wrow_kernel(GemmArgs g, int pieces_m, int cbs, int sliced, int a_bytes, int wf_bytes) {
    constexpr int NKS = NKT * 4;         // K steps of 32 bytes
    constexpr int NM = 2 * NKS;          // MFMAs of a row block: two column groups per K step
    constexpr int AFS = 4;               // activation fragments are read four K steps (eight MFMAs) ahead
    constexpr int SLOTS = ws_slots(NKT);
    extern __shared__ __attribute__((aligned(16))) int8_t ws_smem[];
    int8_t* const stages = ws_smem;
    const WsParams wp(ws_smem + SLOTS * NKT * WS_STAGE);

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int frow = lane & 31, half = lane >> 5;

    // ---- this workgroup's run of (column block, piece) pairs. Workgroups go to the eight XCDs round robin.
    const int nb = gridDim.x, bid = blockIdx.x, xcd = bid & 7;
    int hs0, hs1, j, nw;
    if (sliced) {
        hs0 = xcd * pieces_m / 8;
        hs1 = (xcd + 1) * pieces_m / 8;
        j = bid >> 3;
        nw = (nb >> 3) + (xcd < (nb & 7) ? 1 : 0);
    } else {  // few rows: one list, renumbered so that an XCD gets neighbouring runs
        hs0 = 0;
        hs1 = pieces_m;
        j = xcd * (nb >> 3) + min(xcd, nb & 7) + (bid >> 3);
        nw = nb;
    }
    const int hx = hs1 - hs0;
    // Pairs are numbered column block major; a run that enters a second column block fetches weights again, which costs
    // about three quarters of a piece, so the runs are cut on a scale where a piece counts 4 and a block boundary 3.
    const int64_t vlen = 4 * static_cast<int64_t>(hx) + 3, vtotal = vlen * cbs;
    auto pair_at = [&](int64_t u) { return static_cast<int>(u / vlen * hx + min(static_cast<int64_t>(hx), (u % vlen + 2) / 4)); };
    const int it0 = pair_at(j * vtotal / nw), it1 = pair_at((j + 1) * vtotal / nw);
    if (it0 >= it1) return;
    A4G_STAMP(0);

    // ---- ring loads: the 64 lanes of one instruction fill 1 KiB (8 rows), lane l at byte 16 l, from per-lane global
    // addresses. Instruction j2 of wave w fills rows 16 w + 8 j2 .. + 7 of a stage; the 16-byte slot s of row r holds K
    // chunk s ^ ((r >> 1) & 7), the swizzle the fragment reads undo. Rows past the end of the matrix lie outside the
    // buffer descriptor and read as zero.
    const int lrow8 = lane >> 3, slot16 = lane & 7;
    const int lda = static_cast<int>(g.lda);
    const int sw0 = (slot16 ^ (lrow8 >> 1)) * 16;
    const int va0 = (wave * 16 + lrow8) * lda + sw0, va1 = (wave * 16 + 8 + lrow8) * lda + (sw0 ^ 64);
    const auto rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(g.A), 0, a_bytes, 0x00020000);
    const auto rsrc_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(g.Wf), 0, wf_bytes, 0x00020000);

    const int h_first = hs0 + it0 % hx;  // piece of the run's first pair
    int itl = it0, hl = h_first;         // the piece the next issue fetches ...
    int sl = 0;                          // ... and the ring slot it goes to
    // Tile kt of the piece the issue cursor points at: two instructions per wave. `advance` moves the cursor on.
    auto issue_tile = [&](int kt, int j2) WS_INLINE {
        const int base = itl < it1 ? hl * WS_ROWS * lda : a_bytes;  // past the run: every lane out of range
        int8_t* dst = stages + (sl * NKT + kt) * WS_STAGE + wave * 2048 + j2 * 1024;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)dst, 16, (j2 ? va1 : va0) + base + kt * WS_BK, 0, 0, 0);
    };
    auto advance_issue = [&]() WS_INLINE {
        if (++sl == SLOTS) sl = 0;
        ++itl;
        if (++hl == hs1) hl = hs0;
    };
    auto issue_piece = [&]() WS_INLINE {
#pragma unroll
        for (int kt = 0; kt < NKT; ++kt) {
            issue_tile(kt, 0);
            issue_tile(kt, 1);
        }
        advance_issue();
    };
    // The piece about to be read has landed (own loads: those of the SLOTS - 2 younger pieces may be outstanding), after the
    // barrier for every wave; by then every wave has also issued the last MFMA of the piece before, whose slot the loads
    // issued during this piece refill (spread over its MFMAs: issued in one burst they hold the wave, and with it the
    // matrix pipe, for 0.4 us).
    // FIRST: a column block's first piece, whose weights were requested after the ring's loads and may still be on their
    // way (each MFMA of that piece waits for its own fragment).
    auto piece_sync = [&](auto first_tag) WS_INLINE {
        constexpr int YOUNGER = (SLOTS - 2) * NKT * 2 + (decltype(first_tag)::value ? 2 * NKS : 0);
        asm volatile("s_waitcnt vmcnt(%0)" ::"n"(YOUNGER < 63 ? YOUNGER : 63) : "memory");
        __builtin_amdgcn_s_barrier();
    };

    int koff[4];  // activation fragment of K step kk: row frow (+ 32 i), chunk 2 kk + half
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) koff[kk] = frow * WS_BK + (((kk * 2 + half) ^ ((frow >> 1) & 7)) * 16);
    const int nl = wave * 64 + 16 * half;  // first of this lane's 16 columns of column group 0 (group 1: + 32)

    const int lo = g.relu ? max(kind_lo(g.out_kind), 0) : kind_lo(g.out_kind), hi = kind_hi(g.out_kind);
    int lo_v = lo, hi_v = hi;  // the clamp takes both bounds from vector registers: held there, not moved there per value
    asm volatile("" : "+v"(lo_v), "+v"(hi_v));

    v4i bw[2][NKS];  // the weights of this wave's two groups of 32 columns
    v16i acc[2][2];  // [set][column group]: sets alternate by row block
    v16i addv[2];    // bias + 128 * colsum of the lane's 2 x 16 columns: where an accumulator starts
    v16i sh[2], c0[2];  // their shifts and rounding constants
    v4i af[AFS];     // activation fragments on their way to the next MFMAs
    bool general = false, cols_ok[2] = {false, false};
    int n0 = 0, woff = 0;

    // ---- the weights and column parameters of column block cb
    int col_add = 0, col_shift = 0;
    auto fetch_column_block = [&](int cb) WS_INLINE {
        n0 = cb * WS_BN;
        woff = (cb * (WS_BN / 32) + wave * 2) * (NKS * 1024) + lane * 16;  // fragment (column group, K step) is 1 KiB
        TileCoord tc;
        tc.m0 = 0;
        tc.n0 = n0;
        tc.batch = 0;
        tc.valid = true;
        fetch_col_params<WS_BN, A_UNSIGNED>(g, tc, tid, col_add, col_shift);
    };
    auto fetch_weights = [&]() WS_INLINE {  // in the order the MFMAs take them
#pragma unroll
        for (int s = 0; s < NKS; ++s)
#pragma unroll
            for (int c = 0; c < 2; ++c) {
                const auto w = __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, woff + (c * NKS + s) * 1024, 0, 0);
                bw[c][s] = v4i{static_cast<int>(w[0]), static_cast<int>(w[1]), static_cast<int>(w[2]), static_cast<int>(w[3])};
            }
    };
    auto park_column_block = [&]() WS_INLINE {  // barriers inside
        __syncthreads();  // nobody reads the previous block's parameters any more
        general = direct_park<WS_BN>(g, wp, tid, col_add, col_shift, lo, hi);
#pragma unroll
        for (int c = 0; c < 2; ++c) cols_ok[c] = n0 + nl + 32 * c + 16 <= g.N;
    };
    auto load_column_registers = [&]() WS_INLINE {
#pragma unroll
        for (int c = 0; c < 2; ++c)
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4i add4 = *reinterpret_cast<const v4i*>(wp.add + nl + 32 * c + 4 * q);
                const v4i s4 = *reinterpret_cast<const v4i*>(wp.s + nl + 32 * c + 4 * q);
                const v4i c04 = *reinterpret_cast<const v4i*>(wp.c0 + nl + 32 * c + 4 * q);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    addv[c][q * 4 + t] = add4[t];
                    sh[c][q * 4 + t] = s4[t];
                    c0[c][q * 4 + t] = c04[t];
                }
            }
    };

    // ---- requantisation of a complete accumulator set; dword q of a column group replaces its register q, and the 16 bytes
    // of the lane's row are stored after the fourth
    int pend_m0[2] = {0, 0}, pend_mend[2] = {0, 0};  // the rows a set holds (none: nothing is stored)
    int8_t* const Cb = static_cast<int8_t*>(g.C);
    auto store_group = [&](int P, int c) WS_INLINE {
        const int m = pend_m0[P] + frow;
        if (m < pend_mend[P] && cols_ok[c]) {
            const v4i o = {acc[P][c][0], acc[P][c][1], acc[P][c][2], acc[P][c][3]};
            *reinterpret_cast<v4i*>(Cb + static_cast<int64_t>(m) * g.ldc + n0 + nl + 32 * c) = o;
        }
    };
    // The quick form (shifts within 1..15, sums that stay inside int32: direct_park), value v = 16 c + 4 q + t of set P:
    // rounding offset (BIT 0 none, 1 plus, 2 minus the tie bit, taken at bit s when CONV, else the sign), shift, clamp; after
    // the fourth value of a dword the four low bytes are packed into it.
    auto epi_value = [&](int P, auto v_tag) WS_INLINE {
        constexpr int v = decltype(v_tag)::value, c = v >> 4, r = v & 15, q = r >> 2;
        constexpr int BIT = KIND == 0 ? 0 : (KIND == 2 || KIND == 3) ? 1 : 2;
        constexpr bool CONV = KIND >= 3;
        const int a = acc[P][c][r];
        int bit = 0;
        if (BIT == 1) bit = static_cast<int>(__builtin_amdgcn_ubfe(static_cast<unsigned>(a), CONV ? sh[c][r] : 31, 1));
        if (BIT == 2) bit = __builtin_amdgcn_sbfe(a, CONV ? sh[c][r] : 31, 1);
        acc[P][c][r] = clamp_med3((a + c0[c][r] + bit) >> sh[c][r], lo_v, hi_v);
        if ((r & 3) == 3) {
            acc[P][c][q] = static_cast<int>(pack4_bytes(acc[P][c][4 * q], acc[P][c][4 * q + 1], acc[P][c][4 * q + 2], acc[P][c][4 * q + 3]));
            if (q == 3) store_group(P, c);
        }
    };
    // the general form (any shift, any start value; the accumulators started from zero), not overlapped with anything
    auto epi_general = [&](int P) WS_INLINE {
#pragma unroll
        for (int c = 0; c < 2; ++c) {
            v16i& a = acc[P][c];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4i add4 = *reinterpret_cast<const v4i*>(wp.add + nl + 32 * c + 4 * q);
                const v4i s4 = *reinterpret_cast<const v4i*>(wp.s + nl + 32 * c + 4 * q);
                const v4i c04 = *reinterpret_cast<const v4i*>(wp.c0 + nl + 32 * c + 4 * q);
                const v4i cx4 = *reinterpret_cast<const v4i*>(wp.cx + nl + 32 * c + 4 * q);
                const v4i bs4 = *reinterpret_cast<const v4i*>(wp.bs + nl + 32 * c + 4 * q);
                a[q] = static_cast<int>(direct_requant4_general(a[q * 4], a[q * 4 + 1], a[q * 4 + 2], a[q * 4 + 3], add4, s4, c04, cx4, bs4, lo, hi));
                __builtin_amdgcn_sched_barrier(0);
            }
            store_group(P, c);
        }
    };

    int it = it0, h_c = h_first, cb_c = it0 / hx;  // the pair being computed
    int sc = 0;                                    // its ring slot

    // One piece: its two 32-row blocks one after the other, row block i into accumulator set i, each over all K steps with
    // the two column groups alternating. Behind the second MFMA of a K step the fragment four steps on is read, and beside
    // row block i the other set (row block 1 of the piece before, row block 0 of this one) is requantised, one value per
    // MFMA from the third MFMA on (its last MFMAs have left the pipe by then), and stored.
    // GEN: the column block takes the general requantisation, done right behind each row block, and its weight
    // fragments come from memory one K step at a time.
    // GEN keeps no weights in registers: fragment (column group, K step) of MFMA Z is fetched WD MFMAs ahead into a ring
    // (both row blocks of every piece of the column block take the same 2 * NKS fragments in the same order, so the
    // ring runs on across pieces; fetched at the MFMA that uses it, every MFMA waited for its own load from L2)
    constexpr int WD = 8;
    typedef unsigned v4u_w __attribute__((ext_vector_type(4)));
    v4u_w wq[WD];
    auto fetch_gen_weight = [&](int Zm) WS_INLINE {  // Zm: MFMA number within a row block, 0 .. NM - 1
        return __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, woff + ((Zm & 1) * NKS + (Zm >> 1)) * 1024, 0, 0);
    };
    auto do_piece = [&](auto gen_tag, auto first_tag) WS_INLINE {
        constexpr bool GEN = decltype(gen_tag)::value;
        piece_sync(first_tag);
        const int8_t* const tiles = stages + sc * (NKT * WS_STAGE);
        auto read_fragment = [&](int F) WS_INLINE {  // fragment F of the piece: row block F / NKS, K step F % NKS
            const int rb = F / NKS, s = F % NKS;
            af[F % AFS] = *reinterpret_cast<const v4i*>(tiles + (s >> 2) * WS_STAGE + rb * 32 * WS_BK + koff[s & 3]);
        };
#pragma unroll
        for (int F = 0; F < AFS; ++F) read_fragment(F);
        const int m0 = h_c * WS_ROWS;
        static_for<0, 2 * NM>([&](auto z_tag) WS_INLINE {
            constexpr int Z = decltype(z_tag)::value, i = Z / NM, z = Z % NM, s = z >> 1, c = z & 1;
            constexpr int F = i * NKS + s;  // the fragment both column groups of this K step take
            v4i a_op = af[F % AFS];
            if (A_UNSIGNED) a_op ^= static_cast<int>(0x80808080u);  // uint8 -> int8; 128 * colsum is in the start value
            if constexpr (GEN) {
                const v4u_w w = wq[Z % WD];
                wq[Z % WD] = fetch_gen_weight((z + WD) % NM);
                const v4i w_op = v4i{static_cast<int>(w[0]), static_cast<int>(w[1]), static_cast<int>(w[2]), static_cast<int>(w[3])};
                if constexpr (s == 0) acc[i][c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w_op, a_op, v16i{}, 0, 0, 0);
                else acc[i][c] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w_op, a_op, acc[i][c], 0, 0, 0);
            } else {
                if constexpr (s == 0) mfma_aw_from<A_UNSIGNED>(acc[i][c], bw[c][s], a_op, addv[c]);
                else mfma_aw<A_UNSIGNED>(acc[i][c], bw[c][s], a_op);
            }
            __builtin_amdgcn_sched_barrier(0);
            // one load of the piece two (or more) ahead every eight MFMAs
            if constexpr (Z % 8 == 5) {
                issue_tile(Z / 16, (Z / 8) & 1);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (c == 1 && F + AFS < 2 * NKS) {
                read_fragment(F + AFS);
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (!GEN) {
                constexpr int LEAD = NM > 2 ? 2 : NM - 1;
                static_for<0, 32>([&](auto v_tag) WS_INLINE {
                    if constexpr (LEAD + (decltype(v_tag)::value * (NM - LEAD)) / 32 == z) epi_value(i ^ 1, v_tag);
                });
                __builtin_amdgcn_sched_barrier(0);
            }
            if constexpr (z == NM - 1) {  // row block i is complete: these are its rows
                pend_m0[i] = m0 + 32 * i;
                pend_mend[i] = min(g.M, m0 + 32 * i + 32);
                if constexpr (GEN) {
                    mfma_drain();
                    epi_general(i);
                    pend_mend[i] = 0;
                }
            }
        });
        advance_issue();
        if (++sc == SLOTS) sc = 0;
        ++it;
        if (++h_c == hs1) {
            h_c = hs0;
            ++cb_c;
        }
    };

    bool first = true;
    while (it < it1) {
        // ---- one column block of the run. Everything its first piece needs is requested at once: column parameters, for
        // the run's first block the first pieces, and the weights.
        fetch_column_block(cb_c);
        if (first) {
#pragma unroll
            for (int r = 0; r < SLOTS - 1; ++r) issue_piece();
        }
        fetch_weights();
        park_column_block();
        if (first) A4G_STAMP(1);
        const int it_end = min(it1, (cb_c + 1) * hx);  // the run's pieces of this column block
        if (general) {
            // no weights stay in registers here: the general requantisation needs the room
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
#pragma unroll
            for (int q = 0; q < WD; ++q) wq[q] = fetch_gen_weight(q);
            while (it < it_end) do_piece(std::true_type{}, std::false_type{});
        } else {
            load_column_registers();
            pend_mend[0] = pend_mend[1] = 0;  // what set 1 holds beside the first row block is requantised and not stored
            // the first piece starts while the later weight fragments are still arriving
            do_piece(std::false_type{}, std::true_type{});
            if (it == it0 + 1) A4G_STAMP(2);
            while (it < it_end) do_piece(std::false_type{}, std::false_type{});
            // the block's last row block, with nothing to hide behind
            mfma_drain();
            static_for<0, 32>([&](auto v_tag) WS_INLINE { epi_value(1, v_tag); });
        }
        first = false;
    }
    A4G_STAMP(3);
    A4G_STAMP(4);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // the loads issued past the run's end have retired
    A4G_STAMP(5);
}

template <int NKT, bool A_UNSIGNED, int KIND>
hipError_t launch_wrow_kernel(const GemmArgs& g, hipStream_t stream) {
    auto kern = gemm_wrow_kernel<NKT, A_UNSIGNED, KIND>;
    static bool attr_set = false;  // benign race: the attribute is idempotent
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize, ws_lds_bytes(NKT));
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int pieces_m = (g.M + WS_ROWS - 1) / WS_ROWS, cbs = (g.N + WS_BN - 1) / WS_BN;
    const int sliced = pieces_m >= 16;
    const int64_t pairs = static_cast<int64_t>(pieces_m) * cbs;
    int grid = static_cast<int>(std::min<int64_t>(WS_WGS, pairs));
    if (sliced) grid &= ~7;
    const int a_bytes = static_cast<int>(static_cast<int64_t>(g.M - 1) * g.lda + g.K);
    kern<<<grid, WS_NT, ws_lds_bytes(NKT), stream>>>(g, pieces_m, cbs, sliced, a_bytes, static_cast<int>(rowpacked_bytes(g.N, g.K)));
    return hipGetLastError();
}
// One rounding kind's instances (K in one to six 128-byte tiles, signed and unsigned activations); each kind is compiled
// in a file of its own so that the library builds in parallel.
template <int KIND>
hipError_t launch_wrow_kind(const GemmArgs& g, hipStream_t stream) {
    switch ((g.K + 127) / 128) {
    case 1: return g.a_unsigned ? launch_wrow_kernel<1, true, KIND>(g, stream) : launch_wrow_kernel<1, false, KIND>(g, stream);
    case 2: return g.a_unsigned ? launch_wrow_kernel<2, true, KIND>(g, stream) : launch_wrow_kernel<2, false, KIND>(g, stream);
    case 3: return g.a_unsigned ? launch_wrow_kernel<3, true, KIND>(g, stream) : launch_wrow_kernel<3, false, KIND>(g, stream);
    case 4: return g.a_unsigned ? launch_wrow_kernel<4, true, KIND>(g, stream) : launch_wrow_kernel<4, false, KIND>(g, stream);
    case 5: return g.a_unsigned ? launch_wrow_kernel<5, true, KIND>(g, stream) : launch_wrow_kernel<5, false, KIND>(g, stream);
    case 6: return g.a_unsigned ? launch_wrow_kernel<6, true, KIND>(g, stream) : launch_wrow_kernel<6, false, KIND>(g, stream);
    default: return hipErrorInvalidValue;
    }
}

hipError_t launch_wrow_plain(const GemmArgs& g, hipStream_t stream);      // no tie bit: floor, ceil, positive_inf, negative_inf
hipError_t launch_wrow_sym_inf(const GemmArgs& g, hipStream_t stream);    // symmetric_inf
hipError_t launch_wrow_conv_even(const GemmArgs& g, hipStream_t stream);  // conv_even

}  // namespace a4g
