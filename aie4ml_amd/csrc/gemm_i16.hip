// Dense with int16 activations and int8 weights (the reference's (16, 8) width combination,
// op_impls/families/matmul/common.py:52, whose accumulator is acc32, op_impls/utils/precision.py:120-121):
//   acc32 = wrap32(bias[n] + sum_k a16[m,k] * w8[k,n]);  y = srs(acc32, shift);  optional ReLU
// (dense_bias_relu.cpp:112-163 with an int16 input type).
//
// The matrix cores multiply int8 x int8. An int16 activation is hi * 256 + lo with hi its signed upper byte
// and lo its unsigned lower byte; lo is fed as the signed byte lo - 128 (lo ^ 0x80). Two accumulator sets
// per output block then give  a.w = 256 * sum(hi.w) + sum((lo-128).w) + 128 * sum(w),  all in wrapping
// 32-bit arithmetic, which is exactly the acc32 the reference computes.
#include "common.hpp"

namespace a4g {

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
};

// 128 x 128 output tile, K step 64, 4 waves (2 x 2) of 64 x 64, double-buffered LDS holding the two byte
// planes of A and the weight tile. Requires K % 8 == 0 and 16-byte aligned rows of A and Wt.
__global__ __launch_bounds__(256) void gemm_i16i8_kernel(Gemm16Args g) {
    constexpr int BM = 128, BN = 128, BK = 64, PITCH = BK + 16;
    constexpr int PLANE = BM * PITCH, STAGE = 2 * PLANE + BN * PITCH;
    __shared__ __attribute__((aligned(16))) int8_t smem[2 * STAGE];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int tiles_n = (g.N + BN - 1) / BN;
    const int m0 = (blockIdx.x / tiles_n) * BM, n0 = (blockIdx.x % tiles_n) * BN;

    // staging: A tile = 128 rows x 8 chunks of 8 int16 (4 per thread), W tile = 128 rows x 4 chunks of 16 int8 (2 per thread)
    v4i ra[4], rb[2];
    auto load_tile = [&](int k0) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int c = tid + i * 256, row = c >> 3, kc = (c & 7) * 8;
            const int gm = min(m0 + row, g.M - 1);
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
    const int lo_b = g.relu ? max(kind_lo(g.out_kind), 0) : kind_lo(g.out_kind), hi_b = kind_hi(g.out_kind);
    const int obytes = (g.out_kind == A4G_I16 || g.out_kind == A4G_U16) ? 2 : 1;
    int8_t* Yb = static_cast<int8_t*>(g.Y);
#pragma unroll
    for (int j = 0; j < 2; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int n = n0 + wn * 64 + j * 32 + 8 * q + 4 * (lane >> 5);
            unsigned add[4];
            RoundCfg rc[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const int nn = min(n + t, g.N - 1);
                add[t] = static_cast<unsigned>(g.bias ? g.bias[nn] : 0) + 128u * static_cast<unsigned>(g.colsum[nn]);
                const int s = g.shifts[static_cast<int64_t>(nn) * g.shift_stride];
                rc[t] = make_round(g.mode, min(max(s, 0), 31));
            }
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int m = m0 + wm * 64 + i * 32 + (lane & 31);
                if (m >= g.M) continue;
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    if (n + t >= g.N) continue;
                    const unsigned a = (static_cast<unsigned>(acc_hi[i][j][q * 4 + t]) << 8) +
                                       static_cast<unsigned>(acc_lo[i][j][q * 4 + t]) + add[t];
                    const int y = clamp_i(apply_round(static_cast<int>(a), rc[t]), lo_b, hi_b);
                    const int64_t at = static_cast<int64_t>(m) * g.ldy + n + t;
                    if (obytes == 1) Yb[at] = static_cast<int8_t>(y);
                    else reinterpret_cast<int16_t*>(Yb)[at] = static_cast<int16_t>(y);
                }
            }
        }
    }
}

// Any K / alignment: one thread per output element.
__global__ __launch_bounds__(256) void gemm_i16i8_generic_kernel(Gemm16Args g) {
    const int64_t total = static_cast<int64_t>(g.M) * g.N;
    const int lo_b = g.relu ? max(kind_lo(g.out_kind), 0) : kind_lo(g.out_kind), hi_b = kind_hi(g.out_kind);
    for (int64_t idx = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; idx < total;
         idx += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int m = static_cast<int>(idx / g.N), n = static_cast<int>(idx % g.N);
        unsigned acc = g.bias ? static_cast<unsigned>(g.bias[n]) : 0u;
        const int16_t* ar = g.A + static_cast<int64_t>(m) * g.lda;
        const int8_t* wr = g.Wt + static_cast<int64_t>(n) * g.ldwt;
        for (int k = 0; k < g.K; ++k) acc += static_cast<unsigned>(static_cast<int>(ar[k]) * static_cast<int>(wr[k]));
        const int s = g.shifts[static_cast<int64_t>(n) * g.shift_stride];
        const int y = clamp_i(apply_round(static_cast<int>(acc), make_round(g.mode, min(max(s, 0), 31))), lo_b, hi_b);
        store_kind(g.Y, static_cast<int64_t>(m) * g.ldy + n, g.out_kind, y);
    }
}

}  // namespace a4g

using namespace a4g;

extern "C" int a4g_dense_i16(const int16_t* A, int64_t lda, const int8_t* Wt, int64_t ldwt, const int32_t* colsum,
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
    A4G_REQUIRE(lda >= K && ldy >= N && ldwt >= K, A4G_ERR_INVALID_ARGUMENT, "%s: pitch smaller than the row", who);
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
    const bool tiled = K % 16 == 0 && lda % 8 == 0 && ldwt % 16 == 0 && aligned16(A) && aligned16(Wt);
    if (tiled) {
        const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
        A4G_REQUIRE(tiles <= INT32_MAX, A4G_ERR_UNSUPPORTED, "%s: too many tiles", who);
        gemm_i16i8_kernel<<<static_cast<unsigned>(tiles), 256, 0, stream>>>(g);
    } else {
        const int grid = static_cast<int>(std::min<int64_t>((M * N + 255) / 256, 256 * 32));
        gemm_i16i8_generic_kernel<<<grid, 256, 0, stream>>>(g);
    }
    return check_hip(hipGetLastError(), who);
}
