// The register-staged pipelined MFMA kernel, shared by the integer and the floating-point GEMM entry
// points. Tiles are handled as bytes: a fragment is 16 bytes of one operand row, and one K step is 32 (or 64)
// bytes per row, whatever the element type; a policy class supplies what depends on it:
//
//   acc_t                        16 accumulators of one 32 x 32 block (v16i or v16f)
//   MMAS                         MFMA instructions issued per pair of fragments
//   FIX_A, fix_a(v4i&)           optional fix-up of a 16-byte chunk of A before it is staged
//   mma(b, a, acc)               acc += the 32 x 32 block product of two fragments
//   KSTEP_BYTES                  bytes of K one mma() call consumes per operand row: 32 (one 16-byte fragment per lane)
//                                or 64 (two fragments per lane; the K tile then has two steps instead of four)
//   MAX_OUT_BYTES                widest output element (sizes the LDS image of the output tile)
//   SPLIT_A / split_a(x, y, extra, pair, live)
//                                A elements are two bytes wide: a thread loads 16 of them as two registers and
//                                turns them into their 16 high and 16 low bytes, which become two tile rows
//   SPLIT_B                      B^T comes as two byte planes (Bt, Bt_lo) that alternate in 32-row blocks of the tile
//   Extra                        per-thread state the policy carries from the staging to the epilogue
//   param_bytes<BN>()            LDS bytes of the per-column epilogue parameters
//   ColRegs, fetch_params<BN>, park_params<BN>   issue the loads of a thread's column parameters early,
//                                store them to LDS later (park_params contains a barrier and returns a
//                                workgroup-uniform code that the epilogue gets back)
//   epilogue<BM,BN,WTM,WTN,NT>   turns the accumulators into the output tile
#pragma once

#include <hip/hip_runtime.h>

#include <type_traits>

#include "common.hpp"

// Phase stamps for tuning builds (-DA4G_TIMING): thread 0 of every workgroup records the 100 MHz
// real-time counter at a few points of the pipelined kernel. Compiled out of the library.
#ifdef A4G_TIMING
__device__ unsigned long long a4g_stamps[8 * 65536];
#define A4G_STAMP(i)                                                                                  \
    do {                                                                                              \
        if (threadIdx.x == 0 && blockIdx.x < 65536) a4g_stamps[blockIdx.x * 8 + (i)] = __builtin_amdgcn_s_memrealtime(); \
    } while (0)
#else
#define A4G_STAMP(i) \
    do {             \
    } while (0)
#endif

namespace a4g {

// Sizes along K (K, lda, ldb, stride_a, stride_b) are in bytes for the floating-point element types;
// with one-byte elements that is the same thing. ldc / stride_c count output elements.
struct GemmArgs {
    const int8_t* A;
    const int8_t* Bt;
    void* C;
    const int32_t* bias;    // [N] or null
    const int32_t* colsum;  // [batch][N] or null (only read when a_unsigned)
    const int32_t* shifts;  // device shifts, entry n * shift_stride; null -> the scalar `shift`
    int64_t lda, stride_a, ldb, stride_b, ldc, stride_c, stride_colsum;
    int M, N, K;
    int shift;
    int shift_stride;  // 0: one device scalar for every column, 1: per output channel
    int a_unsigned;
    int relu;
    int out_kind;
    int mode;
    const int8_t* Bt_lo;    // second byte plane of B^T (policies with SPLIT_B), same pitch and strides as Bt
    // only read by the ragged form of the tiled int8 kernel: how a 16-byte chunk of an operand row may be fetched
    // (0 = one aligned load inside the row pitch, 1 = dwords, 2 = bytes); bytes at or past K always read as zero
    int ragged_a, ragged_b;
    // only read by the ragged forms of gemm_rs_kernel: 0, or the element size in bytes of an A that is stored transposed
    // ([K][lda]: lda, stride_a and K stay in bytes, K in bytes of a row of the untransposed operand)
    int trans_a_es;
    // the same weights in fragment order (a4g_rowpack_weights_i8) or null; only Dense kernels that keep weights in
    // registers read it
    const int8_t* Wf;
};

// Bytes of the fragment-order copy of an [N][K] int8 weight matrix: whole 32-column groups, whole 128-byte K tiles.
static inline int64_t rowpacked_bytes(int64_t N, int64_t K) { return (N + 31) / 32 * 32 * ((K + 127) / 128 * 128); }

// Workgroups per problem for tile_coord: whole ranges for the 8 XCDs (surplus workgroups exit at once), except that a
// problem of fewer than 8 tiles gets exactly its tiles: padding 768 one-tile problems to 8 workgroups each made the
// surplus ones queue for LDS they never use (88 us for 768 x 100 x 100 x 64).
static inline int grid_for_tiles(int64_t tiles) { return static_cast<int>(tiles < 8 ? tiles : (tiles + 7) / 8 * 8); }

struct TileCoord {
    int m0, n0, batch;
    bool valid;
};

// Workgroup -> tile mapping. Hardware deals consecutive workgroup ids round-robin over the 8 XCDs,
// each with a private L2, so id % 8 names the XCD: every XCD gets one contiguous range of tiles, and
// that range is ordered in bands of GROUP_M tile rows (row index fastest inside a band) so that the
// tiles resident on an XCD at one time share both activation and weight panels.
template <int BM, int BN>
__device__ __forceinline__ TileCoord tile_coord(const GemmArgs& g) {
    TileCoord tc;
    const int tiles_m = (g.M + BM - 1) / BM;
    const int tiles_n = (g.N + BN - 1) / BN;
    const int tiles = tiles_m * tiles_n;
    const int per_xcd = (tiles + 7) / 8;
    // fewer than 8 tiles per problem (many small problems): one workgroup per tile, no padding (grid_for_tiles)
    const int tile = tiles < 8 ? static_cast<int>(blockIdx.x) : (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    tc.valid = tile < tiles;
    constexpr int GROUP_M = 8;
    const int band = tile / (GROUP_M * tiles_n);
    const int band_rows = min(GROUP_M, tiles_m - band * GROUP_M);
    const int in_band = tile % (GROUP_M * tiles_n);
    tc.m0 = (band * GROUP_M + in_band % max(band_rows, 1)) * BM;
    tc.n0 = (in_band / max(band_rows, 1)) * BN;
    tc.batch = blockIdx.y;
    return tc;
}

// Copies the LDS image of an output tile (row pitch BN * obytes + 16) to global memory, whole rows in
// 16-byte pieces; pieces that cross the matrix edge or a misaligned pitch go byte by byte.
template <int BM, int BN, int NT>
__device__ __forceinline__ void store_tile_image(const GemmArgs& g, const TileCoord& tc, const int8_t* smem, int obytes, int tid) {
    const int cpitch = BN * obytes + 16;
    int8_t* Cb = static_cast<int8_t*>(g.C) + tc.batch * g.stride_c * obytes;
    const int cpr = BN * obytes / 16;  // 16-byte chunks per tile row
    const bool vec_ok = ((g.ldc * obytes) % 16 == 0) && ((reinterpret_cast<uintptr_t>(Cb) & 15) == 0);
    for (int idx = tid; idx < BM * cpr; idx += NT) {
        const int row = idx / cpr, ch = idx % cpr;
        const int m = tc.m0 + row;
        const int nb = tc.n0 * obytes + ch * 16;  // byte column in the output row
        if (m >= g.M || nb >= g.N * obytes) continue;
        const v4i v = *reinterpret_cast<const v4i*>(smem + row * cpitch + ch * 16);
        int8_t* dst = Cb + static_cast<int64_t>(m) * g.ldc * obytes + nb;
        if (vec_ok && nb + 16 <= g.N * obytes) {
            *reinterpret_cast<v4i*>(dst) = v;
        } else {
            const int nbytes = min(16, g.N * obytes - nb);
            const int8_t* srcb = smem + row * cpitch + ch * 16;
            for (int b = 0; b < nbytes; ++b) dst[b] = srcb[b];
        }
    }
}

__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xC07F); }

// -----------------------------------------------------------------------------------------------------
// Register-staged pipelined MFMA kernel (K % 128 == 0) — the kernel for large GEMMs.
//
// Measured on this part, 16-byte global loads into registers that cover whole 128-byte lines sustain
// about 1.75x the L2 throughput of the direct-to-LDS path, so tiles take the classic route: global ->
// VGPR (one K tile ahead) -> ds_write_b128 -> LDS (two stages) -> ds_read_b128 -> MFMA. BK = 128 makes
// every row segment one cache line. LDS layout and swizzle as in the direct-load kernel (BK = 128).
//
// Per K tile kt and wave, four K steps of TM*TN MFMAs each; the memory work is threaded between them:
//   step 0: MFMAs(kt,0) | reads(kt,1) | ds_write of the registers holding tile kt+1 -> stage (kt+1)%2
//   step 1: MFMAs(kt,1) | reads(kt,2) | global loads of tile kt+2 -> the same registers
//   step 2: MFMAs(kt,2) | reads(kt,3)
//   lgkmcnt(0); barrier        (tile kt+1 complete in LDS; nobody reads stage kt%2 after this point)
//   step 3: MFMAs(kt,3) | reads(kt+1,0)
// -----------------------------------------------------------------------------------------------------
template <class P, int BM, int BN, int WAVES_M, int WAVES_N>
struct RsCfg {
    static constexpr int BK = 128, CPR = 8;
    static constexpr int FR = P::KSTEP_BYTES / 32;      // 16-byte fragments per lane, operand row and K step
    static constexpr int KSTEPS = BK / P::KSTEP_BYTES;  // 4 or 2
    static_assert(P::KSTEP_BYTES == 32 || P::KSTEP_BYTES == 64, "K step of 32 or 64 bytes");
    static constexpr int NW = WAVES_M * WAVES_N;
    static constexpr int NT = NW * 64;
    static constexpr int WTM = BM / WAVES_M, WTN = BN / WAVES_N;
    static constexpr int TM = WTM / 32, TN = WTN / 32;
    static constexpr int ROWS_PER_PASS = NT / CPR;  // tile rows covered by one load per thread
    static constexpr int A_LOADS = BM / ROWS_PER_PASS, B_LOADS = BN / ROWS_PER_PASS;
    static constexpr int LOADS = A_LOADS + B_LOADS;
    static constexpr int STAGE_BYTES = (BM + BN) * BK;
    static constexpr int EPI_BYTES = BM * (P::MAX_OUT_BYTES * BN + 16);
    static constexpr int PARAM_OFF = 2 * STAGE_BYTES > EPI_BYTES ? 2 * STAGE_BYTES : EPI_BYTES;
    static constexpr int LDS_BYTES = PARAM_OFF + P::template param_bytes<BN>();
    static_assert(BM % ROWS_PER_PASS == 0 && BN % ROWS_PER_PASS == 0, "tile rows must divide over the threads");
    static_assert(WTM % 32 == 0 && WTN % 32 == 0, "wave tile must be whole 32x32 MFMA blocks");
    static_assert(TM * TN >= TM + TN, "one fragment read is issued behind each MFMA");
    static constexpr int EPM = (LOADS + TM * TN - 1) / (TM * TN);  // staging writes / global loads behind each MFMA
    static_assert(ROWS_PER_PASS % 16 == 0, "the swizzle term must not depend on the pass");
    static_assert((BM + BN) * BK <= 65536, "ds_write immediate offsets are 16 bits");
    static_assert(LDS_BYTES <= 160 * 1024, "LDS budget");
    // SPLIT_A: the tile's BM rows are BM/2 rows of two-byte elements seen as byte planes. Load 2j / 2j+1 of a thread
    // are the two halves of 16 elements of row lrow + j*ROWS_PER_PASS and land, split, in tile rows
    // lrow + 2j*ROWS_PER_PASS (high bytes) and lrow + (2j+1)*ROWS_PER_PASS (low bytes): runs of ROWS_PER_PASS tile
    // rows alternate between the high and the low plane of the same ROWS_PER_PASS rows of A, and a wave's
    // accumulator blocks i and i + ROWS_PER_PASS/32 (within each group of 2*ROWS_PER_PASS/32) belong together.
    static constexpr int RBM = P::SPLIT_A ? BM / 2 : BM;  // rows of A (and of the output) per tile
    static constexpr int RBN = P::SPLIT_B ? BN / 2 : BN;  // columns of the output per tile
    static_assert(!P::SPLIT_B || ROWS_PER_PASS == 64, "B planes alternate in 32-row blocks: 64 tile rows per pass");
    static_assert(!P::SPLIT_A || (A_LOADS % 2 == 0 && ROWS_PER_PASS % 32 == 0 && WTM % (2 * ROWS_PER_PASS) == 0),
                  "plane split: a wave's rows must hold whole high/low runs");
};

// How the ragged kernels may fetch 16-byte chunks of an operand's rows (see load_chunk_ragged).
static inline int ragged_mode(const void* p, int64_t ld, int64_t stride, int64_t K) {
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    if (ld % 16 == 0 && stride % 16 == 0 && a % 16 == 0 && ld >= (K + 15) / 16 * 16) return 0;
    if (ld % 4 == 0 && stride % 4 == 0 && a % 4 == 0) return 1;
    return 2;
}

// RAGGED: K need not fill its last tile and rows need not be aligned (chunk loads that respect the row ends).
// KTAIL: aligned rows, K in whole 16-byte chunks but not whole tiles: the aligned form's descriptor loads, with the
// chunks past K sent to an offset outside the descriptor (they read as zero) - no load sits in a branch, so the waits
// stay exact, which the ragged loads' branches do not allow (8192 x 784 -> 128: 17 us ragged, 9 us this way).
// KTAIL 2: the same for K off the 16-byte grid: rows of A 4-byte aligned (four dword loads per chunk, each inside K or
// sent outside the descriptor), rows of B 16-byte aligned with a pitch that holds K rounded up to 16; the bytes past K
// of the one dword or chunk that straddles it are cleared where the last K tile is staged. KTAIL 3: the same with rows
// of A 8-byte aligned, two 8-byte loads per chunk.
template <class P, int BM, int BN, int WAVES_M, int WAVES_N, bool EARLY = false, bool RAGGED = false, int KTAIL = 0>
__global__ __launch_bounds__(WAVES_M* WAVES_N * 64) void gemm_rs_kernel(GemmArgs g) {
    static_assert(KTAIL == 0 || (!RAGGED && !P::SPLIT_A && !P::SPLIT_B), "the K tail form serves the unsplit policies");
    using Cfg = RsCfg<P, BM, BN, WAVES_M, WAVES_N>;
    constexpr int BK = Cfg::BK, KSTEPS = Cfg::KSTEPS;
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;

    A4G_STAMP(0);
    const TileCoord tc = tile_coord<Cfg::RBM, Cfg::RBN>(g);
    if (!tc.valid) return;
    const int m0 = tc.m0, n0 = tc.n0;

    typename P::ColRegs col_regs;  // this thread's column parameters, in flight until they are parked
    typename P::Extra extra{};
    bool split_live = true;  // false while the staging registers hold a repeat of the last K tile
    P::template fetch_params<BN>(g, tc, tid, col_regs);

    // ---- global -> register staging: thread t owns chunk t%8 of rows t/8 + pass*ROWS_PER_PASS
    const int lrow = tid / Cfg::CPR, lchunk = tid % Cfg::CPR;
    const int8_t* __restrict__ Abase = g.A + tc.batch * g.stride_a + static_cast<int64_t>(m0) * g.lda;
    const int8_t* __restrict__ Bbase = ((P::SPLIT_B && (lrow & 32)) ? g.Bt_lo : g.Bt) + tc.batch * g.stride_b + static_cast<int64_t>(n0) * g.ldb;
    int offa[Cfg::A_LOADS], offb[Cfg::B_LOADS];  // 32-bit offsets from the tile's first row
#pragma unroll
    for (int i = 0; i < Cfg::A_LOADS; ++i) {
        if (P::SPLIT_A)
            offa[i] = min(lrow + (i >> 1) * Cfg::ROWS_PER_PASS, g.M - 1 - m0) * static_cast<int>(g.lda) + lchunk * 32 + (i & 1) * 16;
        else
            offa[i] = min(lrow + i * Cfg::ROWS_PER_PASS, g.M - 1 - m0) * static_cast<int>(g.lda) + lchunk * 16;
    }
#pragma unroll
    for (int i = 0; i < Cfg::B_LOADS; ++i) {
        // SPLIT_B: tile rows [64i, 64i + 32) are the first plane of columns [32i, 32i + 32), the next 32 the second
        const int brow = P::SPLIT_B ? i * 32 + (lrow & 31) : lrow + i * Cfg::ROWS_PER_PASS;
        offb[i] = min(brow, g.N - 1 - n0) * static_cast<int>(g.ldb) + lchunk * 16;
    }
    // LDS slot of that chunk; the swizzle term (row>>1)&7 is the same for every pass
    const int st_off = lrow * BK + ((lchunk ^ ((lrow >> 1) & 7)) * 16);

    v4i ra[Cfg::A_LOADS], rb[Cfg::B_LOADS];
    // The aligned form fetches through buffer descriptors of the tile's row bands, each ending with the last row that
    // exists (rows past it read as zero; their results are never stored): one vector offset per operand, formed once,
    // and everything that differs between the loads of a lane - the K tile, the pass over the rows - is a scalar.
    // With 64-bit pointers every load carried a vector address pair and a 64-bit add per K tile, and the wider-operand
    // policies, short of registers, reloaded address pairs from scratch inside the loop, each reload waiting for every
    // load in flight.
    constexpr int A_TILE_BYTES = P::SPLIT_A ? 2 * BK : BK;
    // KTAIL 2 reads the dword (A) or chunk (B) that straddles K whole: inside the row's pitch, which the host has checked
    const int64_t a_range = static_cast<int64_t>(g.M - 1 - m0) * g.lda +
                            (KTAIL == 3 ? (g.K + 7) / 8 * 8 : KTAIL == 2 ? (g.K + 3) / 4 * 4 : KTAIL ? g.K : static_cast<int64_t>(g.K / BK) * A_TILE_BYTES);
    const int64_t b_range = static_cast<int64_t>(g.N - 1 - n0) * g.ldb +
                            (KTAIL >= 2 ? (g.K + 15) / 16 * 16 : KTAIL ? g.K : static_cast<int64_t>(g.K / BK) * BK);
    const __amdgpu_buffer_rsrc_t rsrc_a = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<int8_t*>(Abase), 0, static_cast<int>(a_range < 0x7fffffff ? a_range : 0x7fffffff), 0x00020000);
    const __amdgpu_buffer_rsrc_t rsrc_b =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(g.Bt + tc.batch * g.stride_b + static_cast<int64_t>(n0) * g.ldb), 0,
                                          static_cast<int>(b_range < 0x7fffffff ? b_range : 0x7fffffff), 0x00020000);
    const int voff_a = lrow * static_cast<int>(g.lda) + lchunk * (P::SPLIT_A ? 32 : 16);
    const int voff_b = lrow * static_cast<int>(g.ldb) + lchunk * 16;
    auto load_one = [&](int kt, int idx) {
        if constexpr (KTAIL != 0) {
            constexpr unsigned NOWHERE = 0xfffffff0u;  // beyond every descriptor: reads as zero
            const bool inside = kt * BK + lchunk * 16 < g.K;
            if (idx < Cfg::A_LOADS) {
                const unsigned off = voff_a + kt * BK + idx * Cfg::ROWS_PER_PASS * static_cast<int>(g.lda);
                if constexpr (KTAIL == 3) {
                    typedef unsigned v2u_t __attribute__((ext_vector_type(2)));
                    const int rem = g.K - (kt * BK + lchunk * 16);
#pragma unroll
                    for (int j = 0; j < 2; ++j) {
                        const v2u_t w = __builtin_amdgcn_raw_buffer_load_b64(rsrc_a, 8 * j < rem ? off + 8 * j : NOWHERE, 0, 0);
                        ra[idx][2 * j] = static_cast<int>(w[0]);
                        ra[idx][2 * j + 1] = static_cast<int>(w[1]);
                    }
                    return;
                }
                if constexpr (KTAIL == 2) {
                    const int rem = g.K - (kt * BK + lchunk * 16);
#pragma unroll
                    for (int j = 0; j < 4; ++j)
                        ra[idx][j] = static_cast<int>(__builtin_amdgcn_raw_buffer_load_b32(rsrc_a, 4 * j < rem ? off + 4 * j : NOWHERE, 0, 0));
                    return;
                }
                ra[idx] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, inside ? off : NOWHERE, 0, 0));
            } else {
                const unsigned off = voff_b + kt * BK + (idx - Cfg::A_LOADS) * Cfg::ROWS_PER_PASS * static_cast<int>(g.ldb);
                rb[idx - Cfg::A_LOADS] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, inside ? off : NOWHERE, 0, 0));
            }
            return;
        }
        if constexpr (RAGGED) {
            // K (bytes here) need not fill its last tile and rows need not be aligned: bytes past K read as zero
            static_assert(!RAGGED || (!P::SPLIT_A && !P::SPLIT_B), "the ragged loads serve the unsplit policies");
            const int rem = g.K - (kt * BK + lchunk * 16);
            if (idx < Cfg::A_LOADS && g.trans_a_es) {
                // A stored transposed: the chunk's elements lie a row pitch apart, starting at column m of row k
                const int es = g.trans_a_es, m = m0 + min(lrow + idx * Cfg::ROWS_PER_PASS, g.M - 1 - m0);
                ra[idx] = load_chunk_transposed(g.A + tc.batch * g.stride_a + static_cast<int64_t>(m) * es, g.lda, (kt * BK + lchunk * 16) / es, g.K / es, es);
                return;
            }
            if (idx < Cfg::A_LOADS) ra[idx] = load_chunk_ragged(Abase + offa[idx] + static_cast<int64_t>(kt) * BK, rem, g.ragged_a);
            else rb[idx - Cfg::A_LOADS] = load_chunk_ragged(Bbase + offb[idx - Cfg::A_LOADS] + static_cast<int64_t>(kt) * BK, rem, g.ragged_b);
            return;
        }
        if constexpr (P::SPLIT_B) {
            // two weight planes are two tensors, so the weights' base differs by lane; with pointers for those loads
            // and descriptors for the activations' this policy measured 3 % slower than with pointers for both
            if (idx < Cfg::A_LOADS) ra[idx] = *reinterpret_cast<const v4i*>(Abase + offa[idx] + static_cast<int64_t>(kt) * A_TILE_BYTES);
            else rb[idx - Cfg::A_LOADS] = *reinterpret_cast<const v4i*>(Bbase + offb[idx - Cfg::A_LOADS] + static_cast<int64_t>(kt) * BK);
        } else if (idx < Cfg::A_LOADS) {
            const int pass = P::SPLIT_A ? (idx >> 1) * Cfg::ROWS_PER_PASS * static_cast<int>(g.lda) + (idx & 1) * 16
                                        : idx * Cfg::ROWS_PER_PASS * static_cast<int>(g.lda);
            ra[idx] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, voff_a, kt * A_TILE_BYTES + pass, 0));
        } else {
            const int pass = (idx - Cfg::A_LOADS) * Cfg::ROWS_PER_PASS * static_cast<int>(g.ldb);
            rb[idx - Cfg::A_LOADS] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, voff_b, kt * BK + pass, 0));
        }
    };
    const int ktiles = (RAGGED || KTAIL != 0) ? (g.K + BK - 1) / BK : g.K / BK;
    int stage_kt = 0;  // the K tile that the staging registers hold (KTAIL 2: its last tile is cleared past K)
    auto store_one = [&](int8_t* stage, int idx) {
        if constexpr (KTAIL >= 2) {
            if (stage_kt == ktiles - 1) {  // workgroup-uniform, and no load inside
                const int rem = g.K - (stage_kt * BK + lchunk * 16);
                v4i& r = idx < Cfg::A_LOADS ? ra[idx] : rb[idx - Cfg::A_LOADS];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int v = rem - 4 * j;  // bytes of this dword that belong to K
                    if (v <= 0) r[j] = 0;
                    else if (v < 4) r[j] &= static_cast<int>((1u << (8 * v)) - 1u);
                }
            }
        }
        if constexpr (P::SPLIT_A) {
            if (idx < Cfg::A_LOADS && (idx & 1) == 0)
                P::split_a(ra[idx], ra[idx + 1 < Cfg::A_LOADS ? idx + 1 : idx], extra, idx >> 1, split_live);
        }
        // the operand fix-up (uint8 -> int8) is made here, once per staged chunk: at the fragments every chunk would be
        // fixed again by each of the WAVES_N waves that read it
        if (P::FIX_A && idx < Cfg::A_LOADS) P::fix_a(ra[idx]);
        if (idx < Cfg::A_LOADS) *reinterpret_cast<v4i*>(stage + st_off + idx * Cfg::ROWS_PER_PASS * BK) = ra[idx];
        else *reinterpret_cast<v4i*>(stage + BM * BK + st_off + (idx - Cfg::A_LOADS) * Cfg::ROWS_PER_PASS * BK) = rb[idx - Cfg::A_LOADS];
    };

#pragma unroll
    for (int i = 0; i < Cfg::LOADS; ++i) load_one(0, i);

    const int epi_path = P::template park_params<BN>(g, smem + Cfg::PARAM_OFF, tid, col_regs);
    A4G_STAMP(1);

    // ---- fragment addressing: row = lane%32 of the block, 16-byte half of the 32-wide K step = lane/32
    const int frow = lane & 31;
    constexpr int FR = Cfg::FR;
    int koff[KSTEPS][FR];  // lane half h takes the chunks [FR * (2 * kk + h), + FR) of K step kk
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk)
#pragma unroll
        for (int f = 0; f < FR; ++f) koff[kk][f] = (((kk * 2 + (lane >> 5)) * FR + f) ^ ((frow >> 1) & 7)) * 16;
    const int a_off = (wm * Cfg::WTM + frow) * BK;
    // PERM_B: the lane supplies the weight row of another column of its 32-column block (direct_col_of_operand_row), so that
    // a lane's 16 accumulators of a block are 16 neighbouring columns, which the policy's epilogue requantises and
    // stores straight from registers
    const int brow = P::PERM_B ? direct_col_of_operand_row(frow) : frow;
    const int b_off = BM * BK + (wn * Cfg::WTN + brow) * BK;
    int koffb[KSTEPS][FR];
#pragma unroll
    for (int kk = 0; kk < KSTEPS; ++kk)
#pragma unroll
        for (int f = 0; f < FR; ++f) koffb[kk][f] = P::PERM_B ? (((kk * 2 + (lane >> 5)) * FR + f) ^ ((brow >> 1) & 7)) * 16 : koff[kk][f];

    typename P::acc_t acc[Cfg::TM][Cfg::TN];
#pragma unroll
    for (int i = 0; i < Cfg::TM; ++i)
#pragma unroll
        for (int j = 0; j < Cfg::TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
    if constexpr (P::PERM_B) P::template start_acc<BN, Cfg::WTN>(acc, smem + Cfg::PARAM_OFF, wn, lane);

    v4i af[2][Cfg::TM][FR], bf[2][Cfg::TN][FR];
    constexpr int NR = Cfg::TM + Cfg::TN, NM = Cfg::TM * Cfg::TN;
    auto read_one = [&](int set, const int8_t* base, int kk, int idx) {
        constexpr int TMIN = Cfg::TM < Cfg::TN ? Cfg::TM : Cfg::TN;
#pragma unroll
        for (int f = 0; f < FR; ++f) {
            if (idx < 2 * TMIN) {
                if (idx & 1) af[set][idx >> 1][f] = *reinterpret_cast<const v4i*>(base + a_off + (idx >> 1) * 32 * BK + koff[kk][f]);
                else bf[set][idx >> 1][f] = *reinterpret_cast<const v4i*>(base + b_off + (idx >> 1) * 32 * BK + koffb[kk][f]);
            } else if (Cfg::TM > Cfg::TN) {
                const int i = idx - TMIN;
                af[set][i][f] = *reinterpret_cast<const v4i*>(base + a_off + i * 32 * BK + koff[kk][f]);
            } else {
                const int j = idx - TMIN;
                bf[set][j][f] = *reinterpret_cast<const v4i*>(base + b_off + j * 32 * BK + koffb[kk][f]);
            }
        }
    };
    // EXTRA: 0 = nothing, 1 = staging writes into `stage_w`, 2 = global loads of tile `kt_load`
    auto step = [&](int cur, int nxt, const int8_t* next_base, int next_kk, auto extra_tag, int8_t* stage_w, int kt_load) {
        constexpr int EXTRA = decltype(extra_tag)::value;
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            const int i = m / Cfg::TN, j = m % Cfg::TN;
            // operands swapped: the block's first index (registers) runs over n, lanes over m
            acc[i][j] = P::mma(bf[cur][j], af[cur][i], acc[i][j]);
            if (m < NR) read_one(nxt, next_base, next_kk, m);
#pragma unroll
            for (int e = m * Cfg::EPM; e < (m + 1) * Cfg::EPM && e < Cfg::LOADS; ++e) {
                if (EXTRA == 1 || EXTRA == 3) store_one(stage_w, e);
                if (EXTRA == 2 || EXTRA == 3) load_one(kt_load, e);
            }
        }
#pragma unroll
        for (int m = 0; m < NM; ++m) {
            __builtin_amdgcn_sched_group_barrier(0x008, P::MMAS, 0);                              // one fragment pair
            if (m < NR) __builtin_amdgcn_sched_group_barrier(0x100, FR, 0);                         // one fragment's LDS reads
#pragma unroll
            for (int e = m * Cfg::EPM; e < (m + 1) * Cfg::EPM && e < Cfg::LOADS; ++e) {
                if (P::FIX_A && (EXTRA == 1 || EXTRA == 3) && e < Cfg::A_LOADS) __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);  // its fix-up
                if (EXTRA == 1 || EXTRA == 3) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // one LDS write
                if (EXTRA == 2 || EXTRA == 3) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one global load
            }
        }
    };
    using Tag0 = std::integral_constant<int, 0>;
    using Tag1 = std::integral_constant<int, 1>;
    using Tag2 = std::integral_constant<int, 2>;
    using Tag3 = std::integral_constant<int, 3>;

    // prologue: tile 0 -> stage 0, tile 1 -> registers, first fragments
#pragma unroll
    for (int i = 0; i < Cfg::LOADS; ++i) store_one(smem, i);
#pragma unroll
    for (int i = 0; i < Cfg::LOADS; ++i) load_one(min(1, ktiles - 1), i);
    __syncthreads();
#pragma unroll
    for (int r = 0; r < NR; ++r) read_one(0, smem, 0, r);
    A4G_STAMP(2);

    for (int kt = 0; kt < ktiles; ++kt) {
        int8_t* cur_base = smem + (kt & 1) * Cfg::STAGE_BYTES;
        int8_t* nxt_base = smem + ((kt + 1) & 1) * Cfg::STAGE_BYTES;
        split_live = kt + 1 < ktiles;
        stage_kt = min(kt + 1, ktiles - 1);
        if constexpr (KSTEPS == 2) {
            // two 64-byte steps per K tile: step 0 carries all the memory work, the barrier sits between the two
            if (EARLY) {
                step(0, 1, cur_base, 1, Tag3{}, nxt_base, min(kt + 2, ktiles - 1));
            } else {
                step(0, 1, cur_base, 1, Tag1{}, nxt_base, 0);
            }
            __builtin_amdgcn_sched_barrier(0);
            wait_lgkmcnt0();
            __builtin_amdgcn_s_barrier();
            __builtin_amdgcn_sched_barrier(0);
            if (EARLY) {
                step(1, 0, nxt_base, 0, Tag0{}, nullptr, 0);
            } else {
                step(1, 0, nxt_base, 0, Tag2{}, nullptr, min(kt + 2, ktiles - 1));
            }
            __builtin_amdgcn_sched_barrier(0);
        } else {
        if (EARLY) {
            step(0, 1, cur_base, 1, Tag3{}, nxt_base, min(kt + 2, ktiles - 1));
            __builtin_amdgcn_sched_barrier(0);
            step(1, 0, cur_base, 2, Tag0{}, nullptr, 0);
        } else {
            step(0, 1, cur_base, 1, Tag1{}, nxt_base, 0);
            __builtin_amdgcn_sched_barrier(0);
            step(1, 0, cur_base, 2, Tag2{}, nullptr, min(kt + 2, ktiles - 1));
        }
        __builtin_amdgcn_sched_barrier(0);
        step(0, 1, cur_base, 3, Tag0{}, nullptr, 0);
        __builtin_amdgcn_sched_barrier(0);
        wait_lgkmcnt0();               // own staging writes and fragment reads have completed
        __builtin_amdgcn_s_barrier();  // tile kt+1 complete in LDS; stage kt%2 is dead from here on
        __builtin_amdgcn_sched_barrier(0);
        step(1, 0, nxt_base, 0, Tag0{}, nullptr, 0);  // after the last tile this reads a stale stage: unused
        __builtin_amdgcn_sched_barrier(0);
        }
    }
    __syncthreads();  // every wave is past its last fragment read before the stages become the output image
    A4G_STAMP(3);

    P::template epilogue<BM, BN, Cfg::WTM, Cfg::WTN, Cfg::NT>(g, tc, acc, smem, smem + Cfg::PARAM_OFF, epi_path, wm, wn, lane, tid, extra);
    A4G_STAMP(5);
}

// Launches one workgroup per tile (padded to whole ranges for the 8 XCDs; surplus workgroups exit at once).
template <class P, int BM, int BN, int WAVES_M, int WAVES_N, bool EARLY = false, bool RAGGED = false, int KTAIL = 0>
static hipError_t launch_rs_policy(const GemmArgs& g, int batch, hipStream_t stream) {
    using Cfg = RsCfg<P, BM, BN, WAVES_M, WAVES_N>;
    auto kern = gemm_rs_kernel<P, BM, BN, WAVES_M, WAVES_N, EARLY, RAGGED, KTAIL>;
    static bool attr_set = false;  // benign race: the attribute is idempotent
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           Cfg::LDS_BYTES);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    const int tiles = ((g.M + Cfg::RBM - 1) / Cfg::RBM) * ((g.N + Cfg::RBN - 1) / Cfg::RBN);
    const int grid_x = grid_for_tiles(tiles);
    hipLaunchKernelGGL(kern, dim3(grid_x, batch), dim3(Cfg::NT), Cfg::LDS_BYTES, stream, g);
    return hipGetLastError();
}

// int16 activations x int8 weights on the pipelined kernel (defined beside the int8 policy, whose epilogue it
// shares). g.A points at the int16 matrix, g.lda / g.stride_a are in bytes, g.K counts elements (K % 128 == 0),
// g.colsum holds the column sums of the weights. False when the shape or the number of tiles does not suit it.
bool rs_i16i8_applicable(const GemmArgs& g, int batch);

// Dense with a short reduction on many rows: weights in registers, activations streamed (gemm_wreg.hip). One problem
// (no batch), int8 / uint8 activations and outputs.
bool wreg_applicable(const GemmArgs& g);
hipError_t launch_wreg(const GemmArgs& g, hipStream_t stream);
// The same shapes with the weights in fragment order as well (gemm_wrow.hip): 64-row pieces, requantisation overlapped.
bool wrow_applicable(const GemmArgs& g);
hipError_t launch_wrow(const GemmArgs& g, hipStream_t stream);

// Dense with a long reduction on 128 x 192 tiles, the reduction split inside an eight-wave workgroup (gemm_sk.hip). One
// problem (no batch), int8 / uint8 activations and outputs.
bool sk_applicable(const GemmArgs& g);
bool sk_preferred(const GemmArgs& g);
hipError_t launch_sk(const GemmArgs& g, hipStream_t stream);
hipError_t launch_rs_i16i8(const GemmArgs& g, int batch, hipStream_t stream);

}  // namespace a4g
