// Dense with int16 activations and int8 weights (the reference's (16, 8) width combination,
// op_impls/families/matmul/common.py:52, whose accumulator is acc32, op_impls/utils/precision.py:120-121):
//   acc32 = wrap32(bias[n] + sum_k a16[m,k] * w8[k,n]);  y = srs(acc32, shift);  optional ReLU
// (dense_bias_relu.cpp:112-163 with an int16 input type).
//
// The matrix cores multiply int8 x int8. An int16 activation is hi * 256 + lo with hi its signed upper byte
// and lo its unsigned lower byte; lo is fed as the signed byte lo - 128 (lo ^ 0x80). Two accumulator sets
// per output block then give  a.w = 256 * sum(hi.w) + sum((lo-128).w) + 128 * sum(w),  all in wrapping
// 32-bit arithmetic, which is exactly the acc32 the reference computes.
//
// Large problems with whole 128-element K tiles run on the software-pipelined kernel of gemm_rs.hpp with the
// planes as rows (and, for int16 weights, columns) of its tile: I16Policy beside the int8 policy whose epilogue
// it shares, I16x16Policy below. The kernels in this file take every other shape: K a multiple of 16 the
// double-buffered tiled ones, anything else one thread per output.
#include <cstdlib>
#include <algorithm>
#include "common.hpp"
#include "gemm_epilogue.hpp"
#include "gemm_rs.hpp"  // tile_coord (XCD-aware workgroup -> tile mapping) and the pipelined kernel template

namespace a4g {

// LDS of the tiled kernels below: one stage of either is 30720 bytes (K step 64, rows padded to 80 bytes), which
// the output image reuses. A reduction that fits one K tile takes a single stage, so more workgroups share a CU.
constexpr int TILED16_STAGE_BYTES = 30720;
static inline size_t tiled16_lds_bytes(int64_t K, int tile_rows) {
    const size_t stages = static_cast<size_t>(K > 64 ? 2 : 1) * TILED16_STAGE_BYTES;
    const size_t image = static_cast<size_t>(tile_rows) * (128 * 2 + 16);  // 128 two-byte outputs per row and its padding
    return stages > image ? stages : image;
}

struct Gemm16Args {
    const int16_t* A;
    const int8_t* Wt;        // [N][ldwt], K contiguous (a4g_pack_weights_i8)
    const int32_t* colsum;   // [N] sum_k W[k][n]
    const int32_t* bias;     // [N] or null
    const int32_t* shifts;   // device, one entry or N
    void* Y;
    int64_t lda, ldwt, ldy;  // lda, ldy in elements
    int M, N, K;
    int shift_stride, relu, out_kind, mode;
    // batched use (dynamic MatMul): element strides between consecutive problems, blockIdx.y = problem
    int64_t stride_a, stride_w, stride_colsum, stride_y;
    int shift;  // used when `shifts` is null (MatMul: one host-side shift)
    int ragged_a;  // RAGGED kernels: how chunks of A's rows may be fetched (load_chunk_ragged)
    int trans_a;   // RAGGED kernels: A is stored transposed, [K][lda]
};

// 128 x 128 output tile, K step 64, 4 waves (2 x 2) of 64 x 64, double-buffered LDS holding the two byte
// planes of A and the weight tile. Requires K % 8 == 0 and 16-byte aligned rows of A and Wt.
__device__ __forceinline__ void select_problem(Gemm16Args& g, int b) {
    const int obytes = (g.out_kind == A4G_I16 || g.out_kind == A4G_U16) ? 2 : 1;
    g.A += b * g.stride_a;
    g.Wt += b * g.stride_w;
    g.colsum += b * g.stride_colsum;
    g.Y = static_cast<int8_t*>(g.Y) + b * g.stride_y * obytes;
}

// RAGGED: K need not be a multiple of 16 nor A's rows 16-byte aligned (the packed weights always are, zero padded).
template <bool RAGGED>
__global__ __launch_bounds__(256, 2) void gemm_i16i8_kernel(Gemm16Args g) {
    constexpr int BM = 128, BN = 128, BK = 64, PITCH = BK + 16;
    select_problem(g, blockIdx.y);
    constexpr int PLANE = BM * PITCH, STAGE = 2 * PLANE + BN * PITCH;
    static_assert(STAGE == TILED16_STAGE_BYTES, "the launch sizes the LDS");
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];  // two stages, or one when K fits a single tile

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    GemmArgs shape{};
    shape.M = g.M;
    shape.N = g.N;
    const TileCoord tc = tile_coord<BM, BN>(shape);
    if (!tc.valid) return;
    const int m0 = tc.m0, n0 = tc.n0;

    // the epilogue of the int8 kernels, fed with this problem's pointers (select_problem has already moved them)
    GemmArgs eg{};
    eg.C = g.Y;
    eg.ldc = g.ldy;
    eg.M = g.M;
    eg.N = g.N;
    eg.bias = g.bias;
    eg.colsum = g.colsum;
    eg.shifts = g.shifts;
    eg.shift_stride = g.shift_stride;
    eg.shift = g.shift;
    eg.mode = g.mode;
    eg.relu = g.relu;
    eg.out_kind = g.out_kind;
    TileCoord here = tc;
    here.batch = 0;
    __shared__ __attribute__((aligned(16))) int8_t cp_mem[ColParams<BN>::BYTES];
    const ColParams<BN> cp(cp_mem);
    int col_add, col_shift;
    fetch_col_params<BN, true>(eg, here, tid, col_add, col_shift);

    // staging: A tile = 128 rows x 8 chunks of 8 int16 (4 per thread), W tile = 128 rows x 4 chunks of 16 int8 (2 per thread)
    v4i ra[4], rb[2];
    auto load_tile = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * 256, row = c >> 3, kc = (c & 7) * 8;
            const int gm = min(m0 + row, g.M - 1);
            if constexpr (RAGGED)
                ra[i] = g.trans_a ? load_chunk_transposed(reinterpret_cast<const int8_t*>(g.A + gm), g.lda * 2, k0 + kc, g.K, 2)
                                  : load_chunk_ragged(reinterpret_cast<const int8_t*>(g.A + static_cast<int64_t>(gm) * g.lda + k0 + kc),
                                                      (g.K - (k0 + kc)) * 2, g.ragged_a);
            else
                ra[i] = (k0 + kc < g.K) ? *reinterpret_cast<const v4i*>(g.A + static_cast<int64_t>(gm) * g.lda + k0 + kc)
                                        : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + i * 256, row = c >> 2, kc = (c & 3) * 16;
            const int gn = min(n0 + row, g.N - 1);
            rb[i] = (k0 + kc < g.K) ? *reinterpret_cast<const v4i*>(g.Wt + static_cast<int64_t>(gn) * g.ldwt + k0 + kc)
                                    : v4i{0, 0, 0, 0};
        }
    };
    auto store_tile = [&](int buf) {
        int8_t* st = smem + buf * STAGE;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * 256, row = c >> 3, kc = (c & 7) * 8;
            // eight int16 in four dwords -> their eight high bytes and eight low bytes
            const unsigned w0 = ra[i][0], w1 = ra[i][1], w2 = ra[i][2], w3 = ra[i][3];
            v2i hi = {static_cast<int>(__builtin_amdgcn_perm(w1, w0, 0x07050301u)), static_cast<int>(__builtin_amdgcn_perm(w3, w2, 0x07050301u))};
            v2i lo = {static_cast<int>(__builtin_amdgcn_perm(w1, w0, 0x06040200u) ^ 0x80808080u),
                      static_cast<int>(__builtin_amdgcn_perm(w3, w2, 0x06040200u) ^ 0x80808080u)};
            *reinterpret_cast<v2i*>(st + row * PITCH + kc) = hi;
            *reinterpret_cast<v2i*>(st + PLANE + row * PITCH + kc) = lo;
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + i * 256, row = c >> 2, kc = (c & 3) * 16;
            *reinterpret_cast<v4i*>(st + 2 * PLANE + row * PITCH + kc) = rb[i];
        }
    };

    v16i acc_hi[2][2], acc_lo[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc_hi[i][j][r] = acc_lo[i][j][r] = 0;

    const int frow = lane & 31, fk = (lane >> 5) * 16;
    const int a_off = (wm * 64 + frow) * PITCH + fk, b_off = 2 * PLANE + (wn * 64 + frow) * PITCH + fk;
    const int ktiles = (g.K + BK - 1) / BK;
    load_tile(0);
    const int round_path = park_col_params<BN>(eg, cp, tid, col_add, col_shift);  // contains barriers
    store_tile(0);
    __syncthreads();
    for (int kt = 0; kt < ktiles; ++kt) {
        const int8_t* st = smem + (kt & 1) * STAGE;
        if (kt + 1 < ktiles) load_tile((kt + 1) * BK);
#pragma unroll
        for (int kk = 0; kk < BK / 32; ++kk) {
            v4i ah[2], al[2], bf[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                ah[i] = *reinterpret_cast<const v4i*>(st + a_off + i * 32 * PITCH + kk * 32);
                al[i] = *reinterpret_cast<const v4i*>(st + PLANE + a_off + i * 32 * PITCH + kk * 32);
                bf[i] = *reinterpret_cast<const v4i*>(st + b_off + i * 32 * PITCH + kk * 32);
            }
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    // operands swapped: lanes run over rows m, accumulator registers over columns n
                    acc_hi[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[j], ah[i], acc_hi[i][j], 0, 0, 0);
                    acc_lo[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[j], al[i], acc_lo[i][j], 0, 0, 0);
                }
        }
        if (kt + 1 < ktiles) store_tile((kt + 1) & 1);
        __syncthreads();
    }

    // epilogue: lane owns row lane%32 of each block and, per register quad q, columns 8q + 4*(lane/32) .. +3
    // a.w = 256 * sum(hi.w) + sum((lo - 128).w) + 128 * sum(w): the last term is in the column's addend. The tile
    // leaves through the epilogue of the int8 kernels (the stages are dead: the loop ended on a barrier).
    v16i sum[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r)
                sum[i][j][r] = static_cast<int>((static_cast<unsigned>(acc_hi[i][j][r]) << 8) + static_cast<unsigned>(acc_lo[i][j][r]));
    epilogue_store<BM, BN, 64, 64, 256>(eg, here, sum, smem, cp, round_path, wm, wn, lane, tid);
}

// Any K / alignment: one thread per output element.
__global__ __launch_bounds__(256) void gemm_i16i8_generic_kernel(Gemm16Args g) {
    select_problem(g, blockIdx.y);
    const int64_t total = static_cast<int64_t>(g.M) * g.N;
    const int lo_b = g.relu ? max(kind_lo(g.out_kind), 0) : kind_lo(g.out_kind), hi_b = kind_hi(g.out_kind);
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total;
         idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int m = static_cast<int>(idx / g.N), n = static_cast<int>(idx % g.N);
        unsigned acc = g.bias ? static_cast<unsigned>(g.bias[n]) : 0u;
        const int16_t* ar = g.A + static_cast<int64_t>(m) * g.lda;
        const int8_t* wr = g.Wt + static_cast<int64_t>(n) * g.ldwt;
        for (int k = 0; k < g.K; ++k) acc += static_cast<unsigned>(static_cast<int>(ar[k]) * static_cast<int>(wr[k]));
        const int s = g.shifts ? g.shifts[static_cast<int64_t>(n) * g.shift_stride] : g.shift;
        const int y = clamp_i(apply_round(static_cast<int>(acc), make_round(g.mode, min(max(s, 0), 31))), lo_b, hi_b);
        store_kind(g.Y, static_cast<int64_t>(m) * g.ldy + n, g.out_kind, y);
    }
}

// -----------------------------------------------------------------------------------------------------
// Dense with int16 activations and int16 weights: the reference's (16, 16) combination, whose accumulator is
// acc64 (op_impls/utils/precision.py:122-123). Both operands are split into byte planes, both low planes are
// fed biased by 128:  a = a' + 128, w = w' + 128 with a' = 256 ah + al', w' = 256 wh + wl', so
//   sum a w = 65536 sum(ah wh) + 256 (sum(ah wl') + sum(al' wh)) + sum(al' wl')
//             + 128 sum_k a'[m,k] + 128 sum_k w'[k,n] + 16384 K.
// Four int32 accumulator sets per output block (each exact for K <= 32768), the column term from the packed
// weights, the row term from the A fragments the lanes hold anyway (v_dot4 against ones), all combined in
// 64-bit arithmetic in the epilogue.
// -----------------------------------------------------------------------------------------------------
struct Gemm16x16Args {
    const int16_t* A;
    const int8_t *Wh, *Wl;    // [N][ldwt] planes: signed high bytes, low bytes ^ 0x80
    const int32_t* colsum;    // [N] sum_k (w[k][n] - 128)
    const int32_t* bias;      // [N] or null
    const int32_t* shifts;
    void* Y;
    int64_t lda, ldwt, ldy;
    int M, N, K;
    int shift_stride, relu, out_kind, mode;
    int64_t stride_a, stride_w, stride_colsum, stride_y;  // batched use, as above
    int shift;                                            // used when `shifts` is null
    int trans_a;                                          // RAGGED kernels: A is stored transposed, [K][lda]
    int ragged_a;                                         // RAGGED kernels: how chunks of A's rows may be fetched
};

__device__ __forceinline__ long long round_shift64(long long v, int s, int mode) {
    if (s <= 0) return v;
    const long long q = v >> s;
    const unsigned long long r = static_cast<unsigned long long>(v) & ((1ull << s) - 1ull), h = 1ull << (s - 1);
    switch (mode) {
    case A4G_RND_FLOOR: return q;
    case A4G_RND_CEIL: return q + (r != 0ull);
    case A4G_RND_POSITIVE_INF: return q + (r >= h);
    case A4G_RND_NEGATIVE_INF: return q + (r > h);
    case A4G_RND_SYMMETRIC_INF: return q + ((r > h) | ((r == h) & (v >= 0)));
    case A4G_RND_SYMMETRIC_ZERO: return q + ((r > h) | ((r == h) & (v < 0)));
    case A4G_RND_CONV_EVEN: return q + ((r > h) | ((r == h) & ((q & 1) != 0)));
    default: return q + ((r > h) | ((r == h) & ((q & 1) == 0)));
    }
}

__device__ __forceinline__ int requant64(long long v, int s, int mode, int lo, int hi) {
    const long long y = round_shift64(v, s, mode);
    return static_cast<int>(y < lo ? lo : (y > hi ? hi : y));
}

// The same rounding as one add before the shift, for the tiled kernels: v + c0, plus a tie term of -1, 0 or 1
// that the mode takes from the sign of v or from bit s of v, then the shift and the saturation. c0 and en depend
// on the column's shift and on the mode only; en is 0 where the shift is 0 (nothing to round) and -1 elsewhere.
// |v| stays below 2^48 (K <= 32768) and c0 below 2^62, so the sum cannot overflow.
struct Round64 {
    long long c0;
    int s, en;
};

__device__ __forceinline__ Round64 make_round64(int shift, int mode) {
    Round64 r;
    r.s = min(max(shift, 0), 62);
    r.en = r.s > 0 ? -1 : 0;
    const long long h = (1ll << r.s) >> 1;
    switch (mode) {
    case A4G_RND_FLOOR: r.c0 = 0; break;
    case A4G_RND_CEIL: r.c0 = (1ll << r.s) - 1; break;
    case A4G_RND_POSITIVE_INF:
    case A4G_RND_SYMMETRIC_INF:
    case A4G_RND_CONV_ODD: r.c0 = h; break;
    default: r.c0 = h + r.en; break;  // ties go down unless the tie term says otherwise
    }
    return r;
}

template <int MODE>
__device__ __forceinline__ int requant64_m(long long v, long long c0, int s, int en, int lo, int hi) {
    long long t = v + c0;
    if constexpr (MODE == A4G_RND_SYMMETRIC_INF) t += static_cast<int>(v >> 63) & en;   // below zero: h - 1
    if constexpr (MODE == A4G_RND_SYMMETRIC_ZERO) t -= static_cast<int>(v >> 63) & en;  // below zero: h
    if constexpr (MODE == A4G_RND_CONV_EVEN) t += static_cast<int>(v >> s) & 1 & en;
    if constexpr (MODE == A4G_RND_CONV_ODD) t -= static_cast<int>(v >> s) & 1 & en;
    const long long q = t >> s;
    const int ql = static_cast<int>(q), qh = static_cast<int>(q >> 32);
    const int y = qh == (ql >> 31) ? ql : ((qh >> 31) ^ 0x7fffffff);  // beyond 32 bits: the bound on q's side
    return clamp_med3(y, lo, hi);
}

// Calls f with the rounding mode as a compile-time constant.
template <typename F>
__device__ __forceinline__ void with_round_mode(int mode, F&& f) {
    switch (mode) {
    case A4G_RND_FLOOR: f(std::integral_constant<int, A4G_RND_FLOOR>{}); break;
    case A4G_RND_CEIL: f(std::integral_constant<int, A4G_RND_CEIL>{}); break;
    case A4G_RND_POSITIVE_INF: f(std::integral_constant<int, A4G_RND_POSITIVE_INF>{}); break;
    case A4G_RND_NEGATIVE_INF: f(std::integral_constant<int, A4G_RND_NEGATIVE_INF>{}); break;
    case A4G_RND_SYMMETRIC_INF: f(std::integral_constant<int, A4G_RND_SYMMETRIC_INF>{}); break;
    case A4G_RND_SYMMETRIC_ZERO: f(std::integral_constant<int, A4G_RND_SYMMETRIC_ZERO>{}); break;
    case A4G_RND_CONV_EVEN: f(std::integral_constant<int, A4G_RND_CONV_EVEN>{}); break;
    default: f(std::integral_constant<int, A4G_RND_CONV_ODD>{}); break;
    }
}

// int16 x int16 on the software-pipelined kernel (K % 128 == 0, large problems). Both operands enter the tile as
// byte planes: the activations are split while they are staged (runs of 64 tile rows alternate between the high
// and the low plane of the same 64 rows), the weights come packed as two planes that alternate in 32-row blocks.
// A wave's 128 x 64 accumulator blocks are then, for each of its two 32-row blocks of outputs, the four partial
// products hh, hl, lh, ll of the same 32 x 32 outputs in the same lanes and registers. With the low planes
// biased by 128, sum a*w = 65536 hh + 256 (hl + lh) + ll + 128 sum_k a + 128 sum_k (w - 128): the column term
// comes with the packed weights, the row term is accumulated from the raw activations as they are split.
struct I16x16Policy {
    using acc_t = v16i;
    static constexpr int MMAS = 1, KSTEP_BYTES = 32;
    static constexpr bool FIX_A = false, SPLIT_A = true, SPLIT_B = true;
    static constexpr bool PERM_B = false;
    static constexpr int MAX_OUT_BYTES = 1;  // the output image holds 128 x 128 two-byte elements in a 256 x 256 one-byte frame
    static constexpr int MAX_ROWS = 128;
    struct Extra {
        int row_sum[2];  // sum over k of the activations of rows lrow and lrow + 64, this thread's 16 columns per K tile
    };
    struct ColRegs {
        int bias, colsum, shift;
    };
    struct Params {  // LDS: per output column of the tile, then per output row
        long long col_term[128];
        long long c0[128];  // Round64 of the column's shift
        int shift[128];
        int en[128];
        int row_sum[MAX_ROWS];
    };
    template <int BN>
    static constexpr int param_bytes() { return sizeof(Params); }
    __device__ static __forceinline__ void fix_a(v4i&) {}
    __device__ static __forceinline__ v16i mma(const v4i (&b)[1], const v4i (&a)[1], const v16i& c) {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(b[0], a[0], c, 0, 0, 0);
    }
    __device__ static __forceinline__ void split_a(v4i& x, v4i& y, Extra& e, int pair, bool live) {
        typedef short s2 __attribute__((ext_vector_type(2)));
        const s2 ones = live ? s2{1, 1} : s2{0, 0};
        int sum = 0;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const int xt = x[t], yt = y[t];  // copies: a bit cast applied to the vector element itself reads element 0
            sum = __builtin_amdgcn_sdot2(__builtin_bit_cast(s2, xt), ones, sum, false);
            sum = __builtin_amdgcn_sdot2(__builtin_bit_cast(s2, yt), ones, sum, false);
        }
        e.row_sum[pair] += sum;
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
        r.bias = r.colsum = r.shift = 0;
        if (tid < BN / 2) {
            const int nn = min(tc.n0 + tid, g.N - 1);
            r.bias = g.bias ? g.bias[nn] : 0;
            r.colsum = g.colsum[tc.batch * g.stride_colsum + nn];
            r.shift = g.shifts ? g.shifts[static_cast<int64_t>(nn) * g.shift_stride] : g.shift;
        }
    }
    template <int BN>
    __device__ static __forceinline__ int park_params(const GemmArgs& g, int8_t* lds, int tid, const ColRegs& r) {
        Params* p = reinterpret_cast<Params*>(lds);
        if (tid < BN / 2) {
            const Round64 rr = make_round64(r.shift, g.mode);
            p->col_term[tid] = 128ll * r.colsum + r.bias;
            p->c0[tid] = rr.c0;
            p->shift[tid] = rr.s;
            p->en[tid] = rr.en;
        }
        return 0;
    }
    template <int BM, int BN, int WTM, int WTN, int NT>
    __device__ static __forceinline__ void epilogue(const GemmArgs& g, const TileCoord& tc, v16i (&acc)[WTM / 32][WTN / 32],
                                                    int8_t* smem, int8_t* lds_params, int, int wm, int wn, int lane, int tid,
                                                    Extra& e) {
        static_assert(BM == 256 && BN == 256 && WTM == 128 && WTN == 64 && NT == 512, "written for the 256 x 256 tile of 8 waves");
        Params* p = reinterpret_cast<Params*>(lds_params);
        // the eight threads that staged one row (consecutive lanes) add up their shares of its sum
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            int v = e.row_sum[j];
            v += __shfl_xor(v, 1);
            v += __shfl_xor(v, 2);
            v += __shfl_xor(v, 4);
            if ((tid & 7) == 0) p->row_sum[(tid >> 3) + 64 * j] = v;
        }
        __syncthreads();
        const int lo_b = g.relu ? max(kind_lo(g.out_kind), 0) : kind_lo(g.out_kind), hi_b = kind_hi(g.out_kind);
        const int obytes = (g.out_kind == A4G_I16 || g.out_kind == A4G_U16) ? 2 : 1;
        const int cpitch = 128 * obytes + 16;
        with_round_mode(g.mode, [&](auto mode_tag) {
            constexpr int MODE = decltype(mode_tag)::value;
#pragma unroll
            for (int ri = 0; ri < 2; ++ri) {
                const int ml = wm * 64 + ri * 32 + (lane & 31);  // output row within the tile
                const long long row_term = 128ll * p->row_sum[ml];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const int nl = wn * 32 + 8 * q + 4 * (lane >> 5);
                    int y[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int r = 4 * q + t;
                        // hl + lh stays within 32 bits: each is at most K * 2^14 <= 2^29 in magnitude
                        const long long v = static_cast<long long>(acc[ri][0][r]) * 65536 +
                                            static_cast<long long>(acc[ri][1][r] + acc[ri + 2][0][r]) * 256 + acc[ri + 2][1][r] +
                                            row_term + p->col_term[nl + t];
                        y[t] = requant64_m<MODE>(v, p->c0[nl + t], p->shift[nl + t], p->en[nl + t], lo_b, hi_b);
                    }
                    if (obytes == 1) {
                        *reinterpret_cast<unsigned*>(smem + ml * cpitch + nl) = pack4_bytes(y[0], y[1], y[2], y[3]);
                    } else {
                        v2i o = {static_cast<int>(pack2_halves(y[0], y[1])), static_cast<int>(pack2_halves(y[2], y[3]))};
                        *reinterpret_cast<v2i*>(smem + ml * cpitch + nl * 2) = o;
                    }
                }
            }
        });
        __syncthreads();
        store_tile_image<128, 128, NT>(g, tc, smem, obytes, tid);
    }
};

static bool rs_i16i16_applicable(const GemmArgs& g, int batch) {
    // the pipelined kernel pays from K = 1024 on (3-10 % ahead of the tiled one; a few per cent behind at K <= 512),
    // and only when the tile's 128 columns are mostly used (N = 64: 299 us against 229 us)
    return g.K % 128 == 0 && g.K >= 1024 && g.N >= 192 && g.K <= 32768 && g.lda % 16 == 0 && g.stride_a % 16 == 0 && g.ldb % 16 == 0 &&
           g.stride_b % 16 == 0 && aligned16(g.A) && aligned16(g.Bt) && aligned16(g.Bt_lo) &&
           static_cast<int64_t>((g.M + 127) / 128) * ((g.N + 127) / 128) * batch >= 192;
}

// 64 x 128 output tile, K step 64, 4 waves (2 x 2) of 32 x 64, double-buffered LDS with the two byte planes
// of both operands. Requires K % 16 == 0, 16-byte aligned rows.
__device__ __forceinline__ void select_problem(Gemm16x16Args& g, int b) {
    const int obytes = (g.out_kind == A4G_I16 || g.out_kind == A4G_U16) ? 2 : 1;
    g.A += b * g.stride_a;
    g.Wh += b * g.stride_w;
    g.Wl += b * g.stride_w;
    g.colsum += b * g.stride_colsum;
    g.Y = static_cast<int8_t*>(g.Y) + b * g.stride_y * obytes;
}

template <bool RAGGED>
__global__ __launch_bounds__(256, 2) void gemm_i16i16_kernel(Gemm16x16Args g) {
    constexpr int BM = 64, BN = 128, BK = 64, PITCH = BK + 16;
    select_problem(g, blockIdx.y);
    constexpr int APLANE = BM * PITCH, WPLANE = BN * PITCH, STAGE = 2 * APLANE + 2 * WPLANE;
    static_assert(STAGE == TILED16_STAGE_BYTES, "the launch sizes the LDS");
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];  // two stages, or one when K fits a single tile

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    GemmArgs shape{};
    shape.M = g.M;
    shape.N = g.N;
    const TileCoord tc = tile_coord<BM, BN>(shape);
    if (!tc.valid) return;
    const int m0 = tc.m0, n0 = tc.n0;

    // per-column terms of the epilogue, parked in LDS while the first tile is on its way (the barriers of the
    // main loop order the writes before the reads)
    __shared__ struct {
        long long col_term[BN], c0[BN];
        int s[BN], en[BN];
    } cp;
    if (tid < BN) {
        const int nn = min(n0 + tid, g.N - 1);
        const Round64 rr = make_round64(g.shifts ? g.shifts[static_cast<int64_t>(nn) * g.shift_stride] : g.shift, g.mode);
        cp.col_term[tid] = 128ll * g.colsum[nn] + (g.bias ? g.bias[nn] : 0);
        cp.c0[tid] = rr.c0;
        cp.s[tid] = rr.s;
        cp.en[tid] = rr.en;
    }

    // staging: A tile = 64 rows x 8 chunks of 8 int16 (2 per thread); each W plane = 128 rows x 4 chunks (2 per thread)
    v4i ra[2], rh[2], rl[2];
    auto load_tile = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + i * 256, row = c >> 3, kc = (c & 7) * 8;
            const int gm = min(m0 + row, g.M - 1);
            if constexpr (RAGGED)
                ra[i] = g.trans_a ? load_chunk_transposed(reinterpret_cast<const int8_t*>(g.A + gm), g.lda * 2, k0 + kc, g.K, 2)
                                  : load_chunk_ragged(reinterpret_cast<const int8_t*>(g.A + static_cast<int64_t>(gm) * g.lda + k0 + kc),
                                                      (g.K - (k0 + kc)) * 2, g.ragged_a);
            else
                ra[i] = (k0 + kc < g.K) ? *reinterpret_cast<const v4i*>(g.A + static_cast<int64_t>(gm) * g.lda + k0 + kc)
                                        : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + i * 256, row = c >> 2, kc = (c & 3) * 16;
            const int gn = min(n0 + row, g.N - 1);
            const bool in = k0 + kc < g.K;
            // past the end of K the planes must contribute nothing: (0, 0) pairs with the zeroed A planes below
            rh[i] = in ? *reinterpret_cast<const v4i*>(g.Wh + static_cast<int64_t>(gn) * g.ldwt + k0 + kc) : v4i{0, 0, 0, 0};
            rl[i] = in ? *reinterpret_cast<const v4i*>(g.Wl + static_cast<int64_t>(gn) * g.ldwt + k0 + kc) : v4i{0, 0, 0, 0};
        }
    };
    auto store_tile = [&](int buf, int k0) {
        int8_t* st = smem + buf * STAGE;
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + i * 256, row = c >> 3, kc = (c & 7) * 8;
            const unsigned w0 = ra[i][0], w1 = ra[i][1], w2 = ra[i][2], w3 = ra[i][3];
            // beyond K both planes are zero, so the row sums stay exact: the low bytes are biased where k < K only
            const int live = min(max(g.K - (k0 + kc), 0), 8);  // elements of this chunk below K (0 or 8 unless RAGGED)
            const unsigned flip0 = live >= 4 ? 0x80808080u : (0x80808080u & ((1u << (8 * live)) - 1u));
            const unsigned flip1 = live >= 8 ? 0x80808080u : (live > 4 ? (0x80808080u & ((1u << (8 * (live - 4))) - 1u)) : 0u);
            v2i hi = {static_cast<int>(__builtin_amdgcn_perm(w1, w0, 0x07050301u)), static_cast<int>(__builtin_amdgcn_perm(w3, w2, 0x07050301u))};
            v2i lo = {static_cast<int>(__builtin_amdgcn_perm(w1, w0, 0x06040200u) ^ flip0),
                      static_cast<int>(__builtin_amdgcn_perm(w3, w2, 0x06040200u) ^ flip1)};
            *reinterpret_cast<v2i*>(st + row * PITCH + kc) = hi;
            *reinterpret_cast<v2i*>(st + APLANE + row * PITCH + kc) = lo;
        }
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            const int c = tid + i * 256, row = c >> 2, kc = (c & 3) * 16;
            *reinterpret_cast<v4i*>(st + 2 * APLANE + row * PITCH + kc) = rh[i];
            *reinterpret_cast<v4i*>(st + 2 * APLANE + WPLANE + row * PITCH + kc) = rl[i];
        }
    };

    v16i acc_hh[2], acc_hl[2], acc_lh[2], acc_ll[2];
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc_hh[j][r] = acc_hl[j][r] = acc_lh[j][r] = acc_ll[j][r] = 0;
    int rs_hi = 0, rs_lo = 0;  // this lane's share of sum_k ah[m,k] and sum_k al'[m,k] for row m = lane % 32

    const int frow = lane & 31, fk = (lane >> 5) * 16;
    const int a_off = (wm * 32 + frow) * PITCH + fk, b_off = 2 * APLANE + (wn * 64 + frow) * PITCH + fk;
    const int ktiles = (g.K + BK - 1) / BK;
    load_tile(0);
    store_tile(0, 0);
    __syncthreads();
    for (int kt = 0; kt < ktiles; ++kt) {
        const int8_t* st = smem + (kt & 1) * STAGE;
        if (kt + 1 < ktiles) load_tile((kt + 1) * BK);
#pragma unroll
        for (int kk = 0; kk < BK / 32; ++kk) {
            const v4i ah = *reinterpret_cast<const v4i*>(st + a_off + kk * 32);
            const v4i al = *reinterpret_cast<const v4i*>(st + APLANE + a_off + kk * 32);
            v4i bh[2], bl[2];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                bh[j] = *reinterpret_cast<const v4i*>(st + b_off + j * 32 * PITCH + kk * 32);
                bl[j] = *reinterpret_cast<const v4i*>(st + WPLANE + b_off + j * 32 * PITCH + kk * 32);
            }
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                rs_hi = __builtin_amdgcn_sdot4(ah[t], 0x01010101, rs_hi, false);
                rs_lo = __builtin_amdgcn_sdot4(al[t], 0x01010101, rs_lo, false);
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                acc_hh[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bh[j], ah, acc_hh[j], 0, 0, 0);
                acc_hl[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bl[j], ah, acc_hl[j], 0, 0, 0);
                acc_lh[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bh[j], al, acc_lh[j], 0, 0, 0);
                acc_ll[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bl[j], al, acc_ll[j], 0, 0, 0);
            }
        }
        if (kt + 1 < ktiles) store_tile((kt + 1) & 1, (kt + 1) * BK);
        __syncthreads();
    }
    // the other half of the row's k range sits in lane ^ 32
    rs_hi += __shfl_xor(rs_hi, 32);
    rs_lo += __shfl_xor(rs_lo, 32);
    const long long row_term = 128ll * (256ll * rs_hi + rs_lo) + 16384ll * g.K;

    const int lo_b = g.relu ? max(kind_lo(g.out_kind), 0) : kind_lo(g.out_kind), hi_b = kind_hi(g.out_kind);
    const int obytes = (g.out_kind == A4G_I16 || g.out_kind == A4G_U16) ? 2 : 1;
    // the tile leaves through an LDS image (the stages are dead: the loop ended on a barrier), then as whole rows
    const int cpitch = BN * obytes + 16;
    const int ml = wm * 32 + (lane & 31);
    with_round_mode(g.mode, [&](auto mode_tag) {
        constexpr int MODE = decltype(mode_tag)::value;
#pragma unroll
        for (int j = 0; j < 2; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int nl = wn * 64 + j * 32 + 8 * q + 4 * (lane >> 5);
                int y[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int r = q * 4 + t;
                    // hl + lh stays within 32 bits: each is at most K * 2^14 <= 2^29 in magnitude
                    const long long v = static_cast<long long>(acc_hh[j][r]) * 65536 +
                                        static_cast<long long>(acc_hl[j][r] + acc_lh[j][r]) * 256 + acc_ll[j][r] + row_term +
                                        cp.col_term[nl + t];
                    y[t] = requant64_m<MODE>(v, cp.c0[nl + t], cp.s[nl + t], cp.en[nl + t], lo_b, hi_b);
                }
                if (obytes == 1) {
                    *reinterpret_cast<unsigned*>(smem + ml * cpitch + nl) = pack4_bytes(y[0], y[1], y[2], y[3]);
                } else {
                    v2i o = {static_cast<int>(pack2_halves(y[0], y[1])), static_cast<int>(pack2_halves(y[2], y[3]))};
                    *reinterpret_cast<v2i*>(smem + ml * cpitch + nl * 2) = o;
                }
            }
        }
    });
    __syncthreads();
    GemmArgs img{};
    img.C = g.Y;
    img.ldc = g.ldy;
    img.M = g.M;
    img.N = g.N;
    TileCoord here = tc;
    here.batch = 0;  // select_problem has already moved the pointers to this problem
    store_tile_image<BM, BN, 256>(img, here, smem, obytes, tid);
}

// Any K / alignment: one thread per output element, straight from the planes (w = 256 wh + (wl ^ 0x80 as unsigned)).
__global__ __launch_bounds__(256) void gemm_i16i16_generic_kernel(Gemm16x16Args g) {
    select_problem(g, blockIdx.y);
    const int64_t total = static_cast<int64_t>(g.M) * g.N;
    const int lo_b = g.relu ? max(kind_lo(g.out_kind), 0) : kind_lo(g.out_kind), hi_b = kind_hi(g.out_kind);
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total;
         idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int m = static_cast<int>(idx / g.N), n = static_cast<int>(idx % g.N);
        long long acc = g.bias ? g.bias[n] : 0;
        const int16_t* ar = g.A + static_cast<int64_t>(m) * g.lda;
        const int8_t* wh = g.Wh + static_cast<int64_t>(n) * g.ldwt;
        const int8_t* wl = g.Wl + static_cast<int64_t>(n) * g.ldwt;
        for (int k = 0; k < g.K; ++k) {
            const int w = 256 * static_cast<int>(wh[k]) + static_cast<int>(static_cast<uint8_t>(wl[k]) ^ 0x80u);
            acc += static_cast<long long>(ar[k]) * w;
        }
        const int s = min(max(g.shifts ? g.shifts[static_cast<int64_t>(n) * g.shift_stride] : g.shift, 0), 62);
        store_kind(g.Y, static_cast<int64_t>(m) * g.ldy + n, g.out_kind, requant64(acc, s, g.mode, lo_b, hi_b));
    }
}

// Right operand of a 16-bit GEMM -> what the kernels above read: rows n with k contiguous (padded with zeros to
// ldt), plus the column sums. Element (k, n) of problem b sits at B[b * stride_b + (trans_b ? n * ldb + k : k * ldb + n)].
// WIDE: int16 operand -> the two byte planes (signed high byte; low byte ^ 0x80) and sum_k (w - 128); else
// int8 -> a transposed copy and sum_k w. Serves the constant weights (a4g_pack_weights_i16) and the dynamic
// operand of a4g_matmul_i16. One workgroup owns 64 columns and walks K in 64 x 64 tiles through LDS, so that
// both the reads and the writes are whole rows of a tile; a thread writes four consecutive k of one column as
// one dword and keeps that column's partial sum, which the 16 threads of a column add up at the end.
template <bool WIDE>
__global__ __launch_bounds__(256) void pack_rhs_kernel(const void* __restrict__ B, int64_t ldb, int64_t stride_b, int trans_b,
                                                       int8_t* __restrict__ hi, int8_t* __restrict__ lo, int64_t ldt,
                                                       int64_t stride_t, int32_t* __restrict__ colsum, int K, int N, int kspan) {
    __shared__ short tile[64][66];  // [k][n]
    const int tid = threadIdx.x, b = blockIdx.y, n0 = blockIdx.x * 64;
    // blockIdx.z picks a run of kspan (a multiple of 64) values of k; with more than one run the column sums are
    // added into a zeroed array
    const int k_begin = blockIdx.z * kspan, k_end = min(static_cast<int>(ldt), k_begin + kspan);
    const int kq = tid & 15;
    // an element past the edge packs to zero bytes and adds nothing to the sum: 128 has high byte 0 and low byte 0x80
    const short pad = WIDE ? 128 : 0;
    int col_acc[4] = {0, 0, 0, 0};
    for (int k0 = k_begin; k0 < k_end; k0 += 64) {
        for (int i = tid; i < 64 * 64; i += 256) {
            const int kk = trans_b ? (i & 63) : (i >> 6), nn = trans_b ? (i >> 6) : (i & 63);
            const int k = k0 + kk, n = n0 + nn;
            short v = pad;
            if (k < K && n < N) {
                const int64_t at = b * stride_b + (trans_b ? static_cast<int64_t>(n) * ldb + k : static_cast<int64_t>(k) * ldb + n);
                v = WIDE ? static_cast<const int16_t*>(B)[at] : static_cast<short>(static_cast<const int8_t*>(B)[at]);
            }
            tile[kk][nn] = v;
        }
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int nn = (tid >> 4) + 16 * j;
            int w[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) w[t] = tile[4 * kq + t][nn];
            const int64_t at = b * stride_t + static_cast<int64_t>(n0 + nn) * ldt + k0 + 4 * kq;
            const bool live = n0 + nn < N && k0 + 4 * kq < ldt;
            if (WIDE) {
                col_acc[j] += (w[0] - 128) + (w[1] - 128) + (w[2] - 128) + (w[3] - 128);
                if (live) {
                    *reinterpret_cast<unsigned*>(hi + at) = pack4_bytes(w[0] >> 8, w[1] >> 8, w[2] >> 8, w[3] >> 8);
                    *reinterpret_cast<unsigned*>(lo + at) = pack4_bytes(w[0], w[1], w[2], w[3]) ^ 0x80808080u;
                }
            } else {
                col_acc[j] += w[0] + w[1] + w[2] + w[3];
                if (live) *reinterpret_cast<unsigned*>(hi + at) = pack4_bytes(w[0], w[1], w[2], w[3]);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int v = col_acc[j];
        v += __shfl_xor(v, 1);
        v += __shfl_xor(v, 2);
        v += __shfl_xor(v, 4);
        v += __shfl_xor(v, 8);
        const int n = n0 + (tid >> 4) + 16 * j;
        if (kq == 0 && n < N) {
            if (gridDim.z == 1) colsum[static_cast<int64_t>(b) * N + n] = v;
            else atomicAdd(colsum + static_cast<int64_t>(b) * N + n, v);
        }
    }
}

__global__ __launch_bounds__(256) void zero_i32_kernel(int32_t* __restrict__ p, int64_t n) {
    const int64_t i = static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x;
    if (i < n) p[i] = 0;
}

// Launches the pack with K split into enough runs to give every CU several workgroups.
static hipError_t launch_pack_rhs(bool wide, const void* B, int64_t ldb, int64_t stride_b, int trans_b, int8_t* hi, int8_t* lo,
                                  int64_t ldt, int64_t stride_t, int32_t* colsum, int64_t batch, int K, int N, hipStream_t stream) {
    const int64_t groups = (N + 63) / 64 * batch, ktiles = (ldt + 63) / 64;
    int64_t runs = std::min<int64_t>(ktiles, std::max<int64_t>(1, 2048 / groups));
    const int kspan = static_cast<int>((ktiles + runs - 1) / runs) * 64;
    runs = (ldt + kspan - 1) / kspan;
    if (runs > 1) {
        const int64_t n = batch * N;
        zero_i32_kernel<<<static_cast<unsigned>((n + 255) / 256), 256, 0, stream>>>(colsum, n);
    }
    const dim3 grid(static_cast<unsigned>((N + 63) / 64), static_cast<unsigned>(batch), static_cast<unsigned>(runs));
    if (wide) pack_rhs_kernel<true><<<grid, 256, 0, stream>>>(B, ldb, stride_b, trans_b, hi, lo, ldt, stride_t, colsum, K, N, kspan);
    else pack_rhs_kernel<false><<<grid, 256, 0, stream>>>(B, ldb, stride_b, trans_b, hi, lo, ldt, stride_t, colsum, K, N, kspan);
    return hipGetLastError();
}

}  // namespace a4g

using namespace a4g;

extern "C" int a4g_dense_i16(const int16_t* A, int trans_a, int64_t lda, const int8_t* Wt, int64_t ldwt, const int32_t* colsum,
                             const int32_t* bias, const int32_t* shifts, int n_shift, int round_mode, int relu, int out_kind,
                             void* Y, int64_t ldy, int64_t M, int64_t N, int64_t K, a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "a4g_dense_i16";
    A4G_REQUIRE(M >= 0 && N >= 1 && K >= 1 && M <= INT32_MAX && N <= (1 << 24) && K <= (1 << 24), A4G_ERR_INVALID_ARGUMENT,
                "%s: bad shape M=%lld N=%lld K=%lld", who, (long long)M, (long long)N, (long long)K);
    A4G_REQUIRE(out_kind == A4G_I8 || out_kind == A4G_U8 || out_kind == A4G_I16, A4G_ERR_UNSUPPORTED,
                "%s: output kind %d is not int8/uint8/int16", who, out_kind);
    A4G_REQUIRE(valid_round(round_mode), A4G_ERR_INVALID_ARGUMENT, "%s: unknown rounding mode %d", who, round_mode);
    A4G_REQUIRE(n_shift == 1 || n_shift == N, A4G_ERR_INVALID_ARGUMENT, "%s: n_shift must be 1 or N=%lld, got %d", who,
                (long long)N, n_shift);
    A4G_REQUIRE(lda >= (trans_a ? M : K) && ldy >= N && ldwt >= K, A4G_ERR_INVALID_ARGUMENT, "%s: pitch smaller than the row", who);
    if (M == 0) return A4G_OK;
    A4G_REQUIRE(A && Wt && Y && shifts && colsum, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer (the packed colsum vector is required)",
                who);
    Gemm16Args g{};
    g.A = A; g.Wt = Wt; g.colsum = colsum; g.bias = bias; g.shifts = shifts; g.Y = Y;
    g.lda = lda; g.ldwt = ldwt; g.ldy = ldy;
    g.M = static_cast<int>(M); g.N = static_cast<int>(N); g.K = static_cast<int>(K);
    g.shift_stride = n_shift == 1 ? 0 : 1;
    g.relu = relu != 0;
    g.out_kind = out_kind;
    g.mode = round_mode;
    {
        // large problems with whole 128-element K tiles: the software-pipelined kernel with the plane split in its staging
        GemmArgs r{};
        r.A = reinterpret_cast<const int8_t*>(A); r.Bt = Wt; r.C = Y; r.bias = bias; r.colsum = colsum; r.shifts = shifts;
        r.lda = lda * 2; r.ldb = ldwt; r.ldc = ldy;
        r.M = g.M; r.N = g.N; r.K = g.K;
        r.shift_stride = g.shift_stride; r.relu = g.relu; r.out_kind = out_kind; r.mode = round_mode;
        if (!trans_a && rs_i16i8_applicable(r, 1)) return check_hip(launch_rs_i16i8(r, 1, stream), who);
    }
    const bool w_ok = ldwt % 16 == 0 && aligned16(Wt) && ldwt >= (K + 15) / 16 * 16;  // what a4g_pack_weights_i8 writes
    A4G_REQUIRE(!trans_a || w_ok, A4G_ERR_UNSUPPORTED, "%s: a transposed left operand needs weights as a4g_pack_weights_i8 writes them", who);
    g.trans_a = trans_a != 0;
    if (w_ok) {
        const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
        A4G_REQUIRE(tiles <= INT32_MAX, A4G_ERR_UNSUPPORTED, "%s: too many tiles", who);
        const dim3 grid(static_cast<unsigned>(grid_for_tiles(tiles)), 1);  // whole ranges for the 8 XCDs
        if (!trans_a && K % 16 == 0 && lda % 8 == 0 && aligned16(A)) {
            gemm_i16i8_kernel<false><<<grid, 256, tiled16_lds_bytes(g.K, 128), stream>>>(g);
        } else {
            g.ragged_a = ragged_mode(A, lda * 2, 0, K * 2);
            gemm_i16i8_kernel<true><<<grid, 256, tiled16_lds_bytes(g.K, 128), stream>>>(g);
        }
    } else {
        const int grid = static_cast<int>(std::min<int64_t>((M * N + 255) / 256, 256 * 32));
        gemm_i16i8_generic_kernel<<<grid, 256, 0, stream>>>(g);
    }
    return check_hip(hipGetLastError(), who);
}

extern "C" int a4g_pack_weights_i16(const int16_t* W, int64_t ldw, int64_t K, int64_t N, int8_t* Wt_hi, int8_t* Wt_lo,
                                    int32_t* colsum, a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "a4g_pack_weights_i16";
    A4G_REQUIRE(W && Wt_hi && Wt_lo && colsum, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    A4G_REQUIRE(K >= 1 && N >= 1 && K <= 32768 && N <= (1 << 24) && ldw >= N, A4G_ERR_INVALID_ARGUMENT,
                "%s: bad shape K=%lld (at most 32768) N=%lld ldw=%lld", who, (long long)K, (long long)N, (long long)ldw);
    const int64_t ldt = K <= 0 ? 16 : (K + 15) / 16 * 16;
    return check_hip(launch_pack_rhs(true, W, ldw, 0, 0, Wt_hi, Wt_lo, ldt, 0, colsum, 1, static_cast<int>(K), static_cast<int>(N), stream),
                     who);
}

extern "C" int a4g_dense_i16x16(const int16_t* A, int trans_a, int64_t lda, const int8_t* Wt_hi, const int8_t* Wt_lo, int64_t ldwt,
                                const int32_t* colsum, const int32_t* bias, const int32_t* shifts, int n_shift, int round_mode,
                                int relu, int out_kind, void* Y, int64_t ldy, int64_t M, int64_t N, int64_t K,
                                a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "a4g_dense_i16x16";
    A4G_REQUIRE(M >= 0 && N >= 1 && K >= 1 && M <= INT32_MAX && N <= (1 << 24) && K <= 32768, A4G_ERR_INVALID_ARGUMENT,
                "%s: bad shape M=%lld N=%lld K=%lld (K at most 32768)", who, (long long)M, (long long)N, (long long)K);
    A4G_REQUIRE(out_kind == A4G_I8 || out_kind == A4G_U8 || out_kind == A4G_I16, A4G_ERR_UNSUPPORTED,
                "%s: output kind %d is not int8/uint8/int16", who, out_kind);
    A4G_REQUIRE(valid_round(round_mode), A4G_ERR_INVALID_ARGUMENT, "%s: unknown rounding mode %d", who, round_mode);
    A4G_REQUIRE(n_shift == 1 || n_shift == N, A4G_ERR_INVALID_ARGUMENT, "%s: n_shift must be 1 or N=%lld, got %d", who,
                (long long)N, n_shift);
    A4G_REQUIRE(lda >= (trans_a ? M : K) && ldy >= N && ldwt >= K, A4G_ERR_INVALID_ARGUMENT, "%s: pitch smaller than the row", who);
    if (M == 0) return A4G_OK;
    A4G_REQUIRE(A && Wt_hi && Wt_lo && Y && shifts && colsum, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    Gemm16x16Args g{};
    g.A = A; g.Wh = Wt_hi; g.Wl = Wt_lo; g.colsum = colsum; g.bias = bias; g.shifts = shifts; g.Y = Y;
    g.lda = lda; g.ldwt = ldwt; g.ldy = ldy;
    g.M = static_cast<int>(M); g.N = static_cast<int>(N); g.K = static_cast<int>(K);
    g.shift_stride = n_shift == 1 ? 0 : 1;
    g.relu = relu != 0;
    g.out_kind = out_kind;
    g.mode = round_mode;
    {
        GemmArgs r{};
        r.A = reinterpret_cast<const int8_t*>(A); r.Bt = Wt_hi; r.Bt_lo = Wt_lo; r.C = Y; r.bias = bias; r.colsum = colsum;
        r.shifts = shifts;
        r.lda = lda * 2; r.ldb = ldwt; r.ldc = ldy;
        r.M = g.M; r.N = g.N; r.K = g.K;
        r.shift_stride = g.shift_stride; r.relu = g.relu; r.out_kind = out_kind; r.mode = round_mode;
        if (!trans_a && rs_i16i16_applicable(r, 1))
            return check_hip(launch_rs_policy<I16x16Policy, 256, 256, 2, 4, true>(r, 1, stream), who);
    }
    const bool w_ok = ldwt % 16 == 0 && aligned16(Wt_hi) && aligned16(Wt_lo) && ldwt >= (K + 15) / 16 * 16;  // a4g_pack_weights_i16
    A4G_REQUIRE(!trans_a || w_ok, A4G_ERR_UNSUPPORTED, "%s: a transposed left operand needs weights as a4g_pack_weights_i16 writes them", who);
    g.trans_a = trans_a != 0;
    if (w_ok) {
        const int64_t tiles = ((M + 63) / 64) * ((N + 127) / 128);
        A4G_REQUIRE(tiles <= INT32_MAX, A4G_ERR_UNSUPPORTED, "%s: too many tiles", who);
        const dim3 grid(static_cast<unsigned>(grid_for_tiles(tiles)), 1);
        if (!trans_a && K % 16 == 0 && lda % 8 == 0 && aligned16(A)) {
            gemm_i16i16_kernel<false><<<grid, 256, tiled16_lds_bytes(g.K, 64), stream>>>(g);
        } else {
            g.ragged_a = ragged_mode(A, lda * 2, 0, K * 2);
            gemm_i16i16_kernel<true><<<grid, 256, tiled16_lds_bytes(g.K, 64), stream>>>(g);
        }
    } else {
        const int grid = static_cast<int>(std::min<int64_t>((M * N + 255) / 256, 256 * 32));
        gemm_i16i16_generic_kernel<<<grid, 256, 0, stream>>>(g);
    }
    return check_hip(hipGetLastError(), who);
}

extern "C" size_t a4g_matmul_i16_workspace_bytes(int64_t batch, int64_t N, int64_t K, int b_kind) {
    if (batch <= 0 || N <= 0 || K <= 0) return 0;
    const int64_t ldt = (K + 15) / 16 * 16;
    const int64_t planes = b_kind == A4G_I16 ? 2 : 1;
    return static_cast<size_t>(batch * (planes * N * ldt + N * 4));
}

extern "C" int a4g_matmul_i16(const int16_t* A, int trans_a, int64_t lda, int64_t stride_a, const void* B, int b_kind, int64_t ldb,
                              int64_t stride_b, int trans_b, void* C, int64_t ldc, int64_t stride_c, int64_t batch, int64_t M,
                              int64_t N, int64_t K, int shift, int round_mode, int out_kind, void* workspace,
                              size_t workspace_bytes, a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "a4g_matmul_i16";
    A4G_REQUIRE(b_kind == A4G_I8 || b_kind == A4G_I16, A4G_ERR_INVALID_ARGUMENT, "%s: matmul RHS must use a signed integer precision", who);
    A4G_REQUIRE(batch >= 0 && batch <= 65535 && M >= 0 && N >= 1 && K >= 1 && M <= INT32_MAX && N <= (1 << 24) &&
                    K <= (b_kind == A4G_I16 ? 32768 : (1 << 24)),
                A4G_ERR_INVALID_ARGUMENT, "%s: bad shape batch=%lld M=%lld N=%lld K=%lld", who, (long long)batch, (long long)M,
                (long long)N, (long long)K);
    A4G_REQUIRE(out_kind == A4G_I8 || out_kind == A4G_U8 || out_kind == A4G_I16, A4G_ERR_UNSUPPORTED,
                "%s: output kind %d is not int8/uint8/int16", who, out_kind);
    A4G_REQUIRE(valid_round(round_mode), A4G_ERR_INVALID_ARGUMENT, "%s: unknown rounding mode %d", who, round_mode);
    A4G_REQUIRE(shift >= 0 && shift <= (b_kind == A4G_I16 ? 62 : 31), A4G_ERR_INVALID_ARGUMENT,
                "%s: matmul accumulator output shift %d out of range", who, shift);
    A4G_REQUIRE(lda >= (trans_a ? M : K) && ldc >= N && ldb >= (trans_b ? K : N), A4G_ERR_INVALID_ARGUMENT, "%s: pitch smaller than the row",
                who);
    if (M == 0 || batch == 0) return A4G_OK;
    A4G_REQUIRE(A && B && C, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    const size_t need = a4g_matmul_i16_workspace_bytes(batch, N, K, b_kind);
    A4G_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace), A4G_ERR_WORKSPACE,
                "%s: needs a 16-byte aligned workspace of %zu bytes (a4g_matmul_i16_workspace_bytes)", who, need);

    const int64_t ldt = (K + 15) / 16 * 16;
    const bool wide = b_kind == A4G_I16;
    int8_t* hi = static_cast<int8_t*>(workspace);
    int8_t* lo = wide ? hi + batch * N * ldt : nullptr;
    int32_t* colsum = reinterpret_cast<int32_t*>(hi + (wide ? 2 : 1) * batch * N * ldt);
    hipError_t e = launch_pack_rhs(wide, B, ldb, stride_b, trans_b, hi, lo, ldt, N * ldt, colsum, batch, (int)K, (int)N, stream);
    if (e != hipSuccess) return check_hip(e, who);

    const bool tiled = !trans_a && K % 16 == 0 && lda % 8 == 0 && stride_a % 8 == 0 && aligned16(A);
    const unsigned nb = static_cast<unsigned>(batch);
    if (wide) {
        Gemm16x16Args g{};
        g.A = A; g.Wh = hi; g.Wl = lo; g.colsum = colsum; g.bias = nullptr; g.shifts = nullptr; g.Y = C;
        g.lda = lda; g.ldwt = ldt; g.ldy = ldc;
        g.M = (int)M; g.N = (int)N; g.K = (int)K;
        g.out_kind = out_kind; g.mode = round_mode; g.shift = shift;
        g.stride_a = stride_a; g.stride_w = N * ldt; g.stride_colsum = N; g.stride_y = stride_c;
        GemmArgs r{};
        r.A = reinterpret_cast<const int8_t*>(A); r.Bt = hi; r.Bt_lo = lo; r.C = C; r.colsum = colsum;
        r.lda = lda * 2; r.stride_a = stride_a * 2; r.ldb = ldt; r.stride_b = N * ldt; r.ldc = ldc; r.stride_c = stride_c;
        r.stride_colsum = N;
        r.M = g.M; r.N = g.N; r.K = g.K;
        r.shift = shift; r.out_kind = out_kind; r.mode = round_mode;
        if (!trans_a && rs_i16i16_applicable(r, nb))
            return check_hip(launch_rs_policy<I16x16Policy, 256, 256, 2, 4, true>(r, nb, stream), who);
        g.trans_a = trans_a != 0;
        const int64_t tiles = ((M + 63) / 64) * ((N + 127) / 128);
        const dim3 grid(static_cast<unsigned>(grid_for_tiles(tiles)), nb);
        if (tiled) {
            gemm_i16i16_kernel<false><<<grid, 256, tiled16_lds_bytes(g.K, 64), stream>>>(g);
        } else {  // the packed planes in the workspace are always aligned and zero padded; A is fetched as its rows allow
            g.ragged_a = ragged_mode(A, lda * 2, stride_a * 2, K * 2);
            gemm_i16i16_kernel<true><<<grid, 256, tiled16_lds_bytes(g.K, 64), stream>>>(g);
        }
    } else {
        Gemm16Args g{};
        g.A = A; g.Wt = hi; g.colsum = colsum; g.bias = nullptr; g.shifts = nullptr; g.Y = C;
        g.lda = lda; g.ldwt = ldt; g.ldy = ldc;
        g.M = (int)M; g.N = (int)N; g.K = (int)K;
        g.out_kind = out_kind; g.mode = round_mode; g.shift = shift;
        g.stride_a = stride_a; g.stride_w = N * ldt; g.stride_colsum = N; g.stride_y = stride_c;
        GemmArgs r{};
        r.A = reinterpret_cast<const int8_t*>(A); r.Bt = hi; r.C = C; r.colsum = colsum;
        r.lda = lda * 2; r.stride_a = stride_a * 2; r.ldb = ldt; r.stride_b = N * ldt; r.ldc = ldc; r.stride_c = stride_c;
        r.stride_colsum = N;
        r.M = g.M; r.N = g.N; r.K = g.K;
        r.shift = shift; r.out_kind = out_kind; r.mode = round_mode;
        if (!trans_a && rs_i16i8_applicable(r, nb)) return check_hip(launch_rs_i16i8(r, nb, stream), who);
        g.trans_a = trans_a != 0;
        const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
        const dim3 grid(static_cast<unsigned>(grid_for_tiles(tiles)), nb);
        if (tiled) {
            gemm_i16i8_kernel<false><<<grid, 256, tiled16_lds_bytes(g.K, 128), stream>>>(g);
        } else {
            g.ragged_a = ragged_mode(A, lda * 2, stride_a * 2, K * 2);
            gemm_i16i8_kernel<true><<<grid, 256, tiled16_lds_bytes(g.K, 128), stream>>>(g);
        }
    }
    return check_hip(hipGetLastError(), who);
}
