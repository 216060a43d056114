// HBM-bound row/stream operators: elementwise Add, integer LayerNorm (optionally with the residual
// add fused in front), and the table-driven integer Softmax (accurate exp and HCCS surrogate).
//
// Layout: plain row-major int8 rows. Fast paths stream each row exactly once as 16-byte chunks per
// lane (fully coalesced: 64 lanes x 16 B = 1 KiB per wave-load), keep the row in registers between
// the reduction and the normalisation, and reduce across lanes with DPP / ds_swizzle butterflies.
#include "common.hpp"

namespace a4g {

// =====================================================================================================
// Elementwise Add                                   (reference: elementwise_add.cpp:12-37)
// =====================================================================================================

// Saturating add of four packed int8 lanes. Even bytes are moved to the high byte of each 16-bit
// half so that the 16-bit saturating add clamps exactly where the int8 add would.
__device__ __forceinline__ unsigned sat_add_i8x4(unsigned a, unsigned b) {
    const v2s ae = __builtin_bit_cast(v2s, (a << 8) & 0xFF00FF00u);
    const v2s be = __builtin_bit_cast(v2s, (b << 8) & 0xFF00FF00u);
    const v2s ao = __builtin_bit_cast(v2s, a & 0xFF00FF00u);
    const v2s bo = __builtin_bit_cast(v2s, b & 0xFF00FF00u);
    const unsigned se = __builtin_bit_cast(unsigned, __builtin_elementwise_add_sat(ae, be));
    const unsigned so = __builtin_bit_cast(unsigned, __builtin_elementwise_add_sat(ao, bo));
    return (so & 0xFF00FF00u) | ((se >> 8) & 0x00FF00FFu);
}

__device__ __forceinline__ unsigned sat_add_u8x4(unsigned a, unsigned b) {
    const v2us ae = __builtin_bit_cast(v2us, a & 0x00FF00FFu);
    const v2us be = __builtin_bit_cast(v2us, b & 0x00FF00FFu);
    const v2us ao = __builtin_bit_cast(v2us, (a >> 8) & 0x00FF00FFu);
    const v2us bo = __builtin_bit_cast(v2us, (b >> 8) & 0x00FF00FFu);
    const v2us lim = {255, 255};
    const unsigned se = __builtin_bit_cast(unsigned, __builtin_elementwise_min(ae + be, lim));
    const unsigned so = __builtin_bit_cast(unsigned, __builtin_elementwise_min(ao + bo, lim));
    return se | (so << 8);
}

template <bool UNSIGNED>
__global__ __launch_bounds__(256) void add_sat8_kernel(const v4i* __restrict__ a, const v4i* __restrict__ b,
                                                        v4i* __restrict__ out, int64_t nvec) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += stride) {
        const v4i va = __builtin_nontemporal_load(a + i);
        const v4i vb = __builtin_nontemporal_load(b + i);
        v4i r;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            r[j] = UNSIGNED ? static_cast<int>(sat_add_u8x4(va[j], vb[j])) : static_cast<int>(sat_add_i8x4(va[j], vb[j]));
        }
        __builtin_nontemporal_store(r, out + i);
    }
}

__global__ __launch_bounds__(256) void add_generic_kernel(const void* __restrict__ a, const void* __restrict__ b,
                                                           void* __restrict__ out, int64_t first, int64_t n, int kind,
                                                           int shift, int mode) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    const int lo = kind_lo(kind), hi = kind_hi(kind);
    for (int64_t i = first + static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < n; i += stride) {
        const int s = load_kind(a, i, kind) + load_kind(b, i, kind);
        store_kind(out, i, kind, clamp_i(round_shift_rt(s, shift, mode), lo, hi));
    }
}

static int grid_for(int64_t work_items, int block, int max_blocks) {
    int64_t g = (work_items + block - 1) / block;
    if (g < 1) g = 1;
    if (g > max_blocks) g = max_blocks;
    return static_cast<int>(g);
}

}  // namespace a4g

using namespace a4g;

extern "C" int a4g_add(const void* a, const void* b, void* out, int64_t n, int kind, int shift, int round_mode,
                       a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    A4G_REQUIRE(n >= 0, A4G_ERR_INVALID_ARGUMENT, "a4g_add: negative element count %lld", (long long)n);
    if (n == 0) return A4G_OK;
    A4G_REQUIRE(a && b && out, A4G_ERR_INVALID_ARGUMENT, "a4g_add: null pointer");
    A4G_REQUIRE(kind == A4G_I8 || kind == A4G_U8 || kind == A4G_I16, A4G_ERR_UNSUPPORTED,
                "a4g_add: storage kind %d is not int8/uint8/int16", kind);
    A4G_REQUIRE(shift >= 0 && shift <= 15, A4G_ERR_INVALID_ARGUMENT, "a4g_add: shift %d outside [0,15]", shift);
    A4G_REQUIRE(valid_round(round_mode), A4G_ERR_INVALID_ARGUMENT, "a4g_add: unknown rounding mode %d", round_mode);

    int64_t done = 0;
    if (shift == 0 && (kind == A4G_I8 || kind == A4G_U8) && aligned16(a) && aligned16(b) && aligned16(out) && n >= 16) {
        const int64_t nvec = n / 16;
        const int grid = grid_for(nvec, 256, 256 * 16);
        if (kind == A4G_U8)
            add_sat8_kernel<true><<<grid, 256, 0, stream>>>(static_cast<const v4i*>(a), static_cast<const v4i*>(b),
                                                            static_cast<v4i*>(out), nvec);
        else
            add_sat8_kernel<false><<<grid, 256, 0, stream>>>(static_cast<const v4i*>(a), static_cast<const v4i*>(b),
                                                             static_cast<v4i*>(out), nvec);
        done = nvec * 16;
    }
    if (done < n) {
        const int grid = grid_for(n - done, 256, 256 * 8);
        add_generic_kernel<<<grid, 256, 0, stream>>>(a, b, out, done, n, kind, shift, round_mode);
    }
    return check_hip(hipGetLastError(), "a4g_add launch");
}

namespace a4g {

// =====================================================================================================
// Integer LayerNorm                                 (reference: layer_norm.cpp:14-121)
// =====================================================================================================

// Nearest Q15 of 1/sqrt(v), v >= 1, clamped to 32767: float seed, exact integer correction
// ((2q-1)^2 v <= 2^32 < (2q+1)^2 v).
__device__ __forceinline__ int rsqrt_q15(int v) {
    if (v < 1) v = 1;
    long long q = static_cast<long long>(32768.0f * __frsqrt_rn(static_cast<float>(v)) + 0.5f);
    if (q < 1) q = 1;
    const unsigned long long two32 = 1ull << 32;
    const unsigned long long uv = static_cast<unsigned long long>(v);
    while (q > 0 && static_cast<unsigned long long>((2 * q - 1) * (2 * q - 1)) * uv > two32) --q;
    while (static_cast<unsigned long long>((2 * q + 1) * (2 * q + 1)) * uv <= two32) ++q;
    return static_cast<int>(q > 32767 ? 32767 : q);
}

struct RowStats {
    int mu;
    int inv;
};

// layer_norm.cpp:22-34. log2c >= 0 when cols is a power of two (the reference's shift form); the
// floor divisions are the same numbers otherwise.
__device__ __forceinline__ RowStats row_stats(int sx, int sq, int cols, int log2c, int eps_q0) {
    RowStats st;
    int mu, var;
    if (log2c >= 0) {
        mu = (sx + (cols >> 1)) >> log2c;
        const int csq = static_cast<int>(static_cast<unsigned>(sq) - 2u * static_cast<unsigned>(mu) * static_cast<unsigned>(sx) +
                                         static_cast<unsigned>(cols) * static_cast<unsigned>(mu) * static_cast<unsigned>(mu));
        var = csq >> log2c;
    } else {
        mu = static_cast<int>(floordiv64(static_cast<int64_t>(sx) + (cols >> 1), cols));
        const int csq = static_cast<int>(static_cast<unsigned>(sq) - 2u * static_cast<unsigned>(mu) * static_cast<unsigned>(sx) +
                                         static_cast<unsigned>(cols) * static_cast<unsigned>(mu) * static_cast<unsigned>(mu));
        var = static_cast<int>(floordiv64(csq, cols));
    }
    if (var < 0) var = 0;
    st.mu = static_cast<int16_t>(mu);
    st.inv = rsqrt_q15(static_cast<int>(static_cast<unsigned>(var) + static_cast<unsigned>(eps_q0)));
    return st;
}

__device__ __forceinline__ int sext8(unsigned w, int j) { return static_cast<int>(w << (24 - 8 * j)) >> 24; }

// One wave per row; lane l owns the 16-byte chunks l, l+64, ... (NCH of them). gamma/beta for those
// columns stay in registers across the rows a wave processes.
template <int NCH, int MODE, bool FUSE_ADD>
__global__ __launch_bounds__(256) void layernorm_wave_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ x2,
                                                              const int16_t* __restrict__ gamma,
                                                              const int16_t* __restrict__ beta, int8_t* __restrict__ sum_out,
                                                              int8_t* __restrict__ out, int rows, int cols, int log2c,
                                                              int eps_q0, int gamma_shift, int final_shift) {
    const int lane = threadIdx.x & 63;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int nwaves = (gridDim.x * blockDim.x) >> 6;

    bool valid[NCH];
    v4i g[NCH][2], bt[NCH][2];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int col0 = (lane + 64 * i) * 16;
        valid[i] = col0 < cols;
        if (valid[i]) {
            g[i][0] = *reinterpret_cast<const v4i*>(gamma + col0);
            g[i][1] = *reinterpret_cast<const v4i*>(gamma + col0 + 8);
            bt[i][0] = *reinterpret_cast<const v4i*>(beta + col0);
            bt[i][1] = *reinterpret_cast<const v4i*>(beta + col0 + 8);
        } else {
            g[i][0] = g[i][1] = bt[i][0] = bt[i][1] = v4i{0, 0, 0, 0};
        }
    }

    for (int row = wave; row < rows; row += nwaves) {
        const int64_t base = static_cast<int64_t>(row) * cols;
        v4i xv[NCH];
        int sx = 0, sq = 0;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int col0 = (lane + 64 * i) * 16;
            xv[i] = v4i{0, 0, 0, 0};
            if (valid[i]) {
                xv[i] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(x + base + col0));
                if (FUSE_ADD) {
                    const v4i o = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(x2 + base + col0));
#pragma unroll
                    for (int j = 0; j < 4; ++j) xv[i][j] = static_cast<int>(sat_add_i8x4(xv[i][j], o[j]));
                    if (sum_out) __builtin_nontemporal_store(xv[i], reinterpret_cast<v4i*>(sum_out + base + col0));
                }
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                sx = __builtin_amdgcn_sdot4(xv[i][j], 0x01010101, sx, false);
                sq = __builtin_amdgcn_sdot4(xv[i][j], xv[i][j], sq, false);
            }
        }
        sx = group_allreduce<64>(sx, OpAdd());
        sq = group_allreduce<64>(sq, OpAdd());
        const RowStats st = row_stats(sx, sq, cols, log2c, eps_q0);

#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            if (!valid[i]) continue;
            const int col0 = (lane + 64 * i) * 16;
            v4i o;
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                int y4[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int e = w * 4 + j;  // element within the chunk
                    const int gw = g[i][e >> 3][(e & 7) >> 1];
                    const int bw = bt[i][e >> 3][(e & 7) >> 1];
                    const int gam = (e & 1) ? (gw >> 16) : static_cast<int>(static_cast<int16_t>(gw));
                    const int bet = (e & 1) ? (bw >> 16) : static_cast<int>(static_cast<int16_t>(bw));
                    const int vd = sext8(xv[i][w], j) - st.mu;
                    const int fs = clamp_i(round_shift<MODE>(st.inv * gam, gamma_shift), -32768, 32767);
                    const int acc = vd * fs + bet;
                    y4[j] = clamp_i(round_shift<MODE>(acc, final_shift), -128, 127);
                }
                o[w] = static_cast<int>(pack4_bytes(y4[0], y4[1], y4[2], y4[3]));
            }
            __builtin_nontemporal_store(o, reinterpret_cast<v4i*>(out + base + col0));
        }
    }
}

// Any column count / alignment / add shift: one 256-thread block per row, three passes over global
// memory, block reduction through LDS.
__global__ __launch_bounds__(256) void layernorm_generic_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ x2,
                                                                 int add_shift, int add_mode,
                                                                 const int16_t* __restrict__ gamma,
                                                                 const int16_t* __restrict__ beta, int8_t* __restrict__ sum_out,
                                                                 int8_t* __restrict__ out, int rows, int cols, int log2c,
                                                                 int eps_q0, int gamma_shift, int final_shift, int mode) {
    __shared__ int red[2][4];
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int row = blockIdx.x; row < rows; row += gridDim.x) {
        const int64_t base = static_cast<int64_t>(row) * cols;
        int sx = 0, sq = 0;
        for (int c = threadIdx.x; c < cols; c += blockDim.x) {
            int v = x[base + c];
            if (x2) v = clamp_i(round_shift_rt(v + x2[base + c], add_shift, add_mode), -128, 127);
            sx += v;
            sq += v * v;
        }
        sx = group_allreduce<64>(sx, OpAdd());
        sq = group_allreduce<64>(sq, OpAdd());
        __syncthreads();
        if (lane == 0) {
            red[0][wv] = sx;
            red[1][wv] = sq;
        }
        __syncthreads();
        sx = red[0][0] + red[0][1] + red[0][2] + red[0][3];
        sq = red[1][0] + red[1][1] + red[1][2] + red[1][3];
        const RowStats st = row_stats(sx, sq, cols, log2c, eps_q0);
        for (int c = threadIdx.x; c < cols; c += blockDim.x) {
            int v = x[base + c];
            if (x2) {
                v = clamp_i(round_shift_rt(v + x2[base + c], add_shift, add_mode), -128, 127);
                if (sum_out) sum_out[base + c] = static_cast<int8_t>(v);
            }
            const int fs = clamp_i(round_shift_rt(st.inv * gamma[c], gamma_shift, mode), -32768, 32767);
            const int acc = (v - st.mu) * fs + beta[c];
            out[base + c] = static_cast<int8_t>(clamp_i(round_shift_rt(acc, final_shift, mode), -128, 127));
        }
    }
}

template <int NCH, bool FUSE>
static void launch_ln_wave(int mode, int grid, hipStream_t stream, const int8_t* x, const int8_t* x2, const int16_t* gamma,
                           const int16_t* beta, int8_t* sum_out, int8_t* out, int rows, int cols, int log2c, int eps_q0,
                           int gamma_shift, int final_shift) {
#define A4G_LN_CASE(M)                                                                                                  \
    case M:                                                                                                             \
        layernorm_wave_kernel<NCH, M, FUSE><<<grid, 256, 0, stream>>>(x, x2, gamma, beta, sum_out, out, rows, cols, log2c, \
                                                                        eps_q0, gamma_shift, final_shift);               \
        break;
    switch (mode) {
        A4G_LN_CASE(0) A4G_LN_CASE(1) A4G_LN_CASE(2) A4G_LN_CASE(3) A4G_LN_CASE(4) A4G_LN_CASE(5) A4G_LN_CASE(6)
        A4G_LN_CASE(7)
    }
#undef A4G_LN_CASE
}

static int layernorm_dispatch(const int8_t* a, const int8_t* b, int add_shift, int add_mode, const int16_t* gamma,
                              const int16_t* beta, int8_t* sum_out, int8_t* out, int64_t rows, int64_t cols, int32_t eps_q0,
                              int gamma_shift, int out_shift, int mode, hipStream_t stream, const char* who) {
    A4G_REQUIRE(rows >= 0 && cols >= 1, A4G_ERR_INVALID_ARGUMENT, "%s: bad shape rows=%lld cols=%lld", who, (long long)rows,
                (long long)cols);
    A4G_REQUIRE(cols <= 65536 && rows <= INT32_MAX, A4G_ERR_UNSUPPORTED, "%s: cols %lld > 65536 or rows %lld too large", who,
                (long long)cols, (long long)rows);
    A4G_REQUIRE(eps_q0 >= 1 && eps_q0 <= (1 << 30), A4G_ERR_INVALID_ARGUMENT,
                "%s: eps_q0 must be positive (integer LayerNorm requires a positive variance floor), got %d", who, eps_q0);
    A4G_REQUIRE(out_shift >= 0 && out_shift <= 15, A4G_ERR_INVALID_ARGUMENT, "%s: out_shift=%d must be in [0, 15]", who,
                out_shift);
    A4G_REQUIRE(gamma_shift >= 0 && gamma_shift <= 15, A4G_ERR_INVALID_ARGUMENT, "%s: gamma_shift=%d must be in [0, 15]",
                who, gamma_shift);
    A4G_REQUIRE(valid_round(mode) && valid_round(add_mode), A4G_ERR_INVALID_ARGUMENT, "%s: unknown rounding mode", who);
    A4G_REQUIRE(add_shift >= 0 && add_shift <= 8, A4G_ERR_INVALID_ARGUMENT, "%s: add_shift %d outside [0,8]", who, add_shift);
    if (rows == 0) return A4G_OK;
    A4G_REQUIRE(a && gamma && beta && out, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);

    int log2c = -1;
    if ((cols & (cols - 1)) == 0) {
        log2c = 0;
        while ((1LL << log2c) < cols) ++log2c;
    }
    const int final_shift = 15 - out_shift;
    const bool fuse = b != nullptr;
    const bool fast = cols % 16 == 0 && cols <= 4096 && aligned16(a) && aligned16(out) && (!fuse || aligned16(b)) &&
                      (!sum_out || aligned16(sum_out)) && aligned16(gamma) && aligned16(beta) && (!fuse || add_shift == 0);
    if (fast) {
        const int nch = static_cast<int>((cols / 16 + 63) / 64);
        const int grid = grid_for(rows, 4, 256 * 8);
#define A4G_LN_NCH(N)                                                                                                        \
    if (fuse)                                                                                                                \
        launch_ln_wave<N, true>(mode, grid, stream, a, b, gamma, beta, sum_out, out, (int)rows, (int)cols, log2c, eps_q0,    \
                                gamma_shift, final_shift);                                                                   \
    else                                                                                                                     \
        launch_ln_wave<N, false>(mode, grid, stream, a, nullptr, gamma, beta, nullptr, out, (int)rows, (int)cols, log2c,     \
                                 eps_q0, gamma_shift, final_shift);
        if (nch <= 1) {
            A4G_LN_NCH(1)
        } else if (nch <= 2) {
            A4G_LN_NCH(2)
        } else {
            A4G_LN_NCH(4)
        }
#undef A4G_LN_NCH
    } else {
        const int grid = grid_for(rows, 1, 256 * 8);
        layernorm_generic_kernel<<<grid, 256, 0, stream>>>(a, b, add_shift, add_mode, gamma, beta, sum_out, out, (int)rows,
                                                           (int)cols, log2c, eps_q0, gamma_shift, final_shift, mode);
    }
    return check_hip(hipGetLastError(), who);
}

}  // namespace a4g

extern "C" int a4g_layernorm_i8(const int8_t* x, const int16_t* gamma, const int16_t* beta, int8_t* out, int64_t rows,
                                int64_t cols, int32_t eps_q0, int gamma_shift, int out_shift, int round_mode,
                                a4g_stream_t stream) {
    return layernorm_dispatch(x, nullptr, 0, 0, gamma, beta, nullptr, out, rows, cols, eps_q0, gamma_shift, out_shift,
                              round_mode, static_cast<hipStream_t>(stream), "a4g_layernorm_i8");
}

extern "C" int a4g_add_layernorm_i8(const int8_t* a, const int8_t* b, int add_shift, int add_round_mode,
                                    const int16_t* gamma, const int16_t* beta, int8_t* sum_out, int8_t* out, int64_t rows,
                                    int64_t cols, int32_t eps_q0, int gamma_shift, int out_shift, int round_mode,
                                    a4g_stream_t stream) {
    if (rows > 0 && !b) return fail(A4G_ERR_INVALID_ARGUMENT, "a4g_add_layernorm_i8: null second addend");
    return layernorm_dispatch(a, b, add_shift, add_round_mode, gamma, beta, sum_out, out, rows, cols, eps_q0, gamma_shift,
                              out_shift, round_mode, static_cast<hipStream_t>(stream), "a4g_add_layernorm_i8");
}

namespace a4g {

// =====================================================================================================
// Integer Softmax                                   (reference: softmax.cpp:19-127, 252-384)
// =====================================================================================================
// Both forms score an element from its gap d = max - x in [0,255] only, so the score is a 256-entry
// table built once per block in LDS: exp -> exp_score16(d, KQ); HCCS -> B - S*min(d, Dmax).

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

// Byte-wise max of four packed int8 as a scalar.
__device__ __forceinline__ int max_i8x4(unsigned w) {
    return max(max(sext8(w, 0), sext8(w, 1)), max(sext8(w, 2), sext8(w, 3)));
}

// L consecutive lanes share one row (64/L rows per wave pass); lane l of the group owns chunks
// l, l+L, ... (NCH of them), 16 int8 each.
template <int L, int NCH, bool NOCLAMP_U8>
__global__ __launch_bounds__(256) void softmax_lut_kernel(const int8_t* __restrict__ x, void* __restrict__ out, int rows,
                                                           int cols, SoftmaxParams p) {
    __shared__ int table[256];
    table[threadIdx.x] = table_entry(p, threadIdx.x);
    __syncthreads();

    constexpr int RPW = 64 / L;
    const int lane = threadIdx.x & 63;
    const int grp = lane / L, l = lane % L;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int nwaves = (gridDim.x * blockDim.x) >> 6;

    for (int row0 = wave * RPW; row0 < rows; row0 += nwaves * RPW) {
        const int row = row0 + grp;
        const bool row_ok = row < rows;
        const int64_t base = static_cast<int64_t>(row) * cols;
        v4i xv[NCH];
        bool valid[NCH];
        int m = -128;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            const int col0 = (l + L * i) * 16;
            valid[i] = row_ok && col0 < cols;
            xv[i] = v4i{(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
            if (valid[i]) xv[i] = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(x + base + col0));
#pragma unroll
            for (int j = 0; j < 4; ++j) m = max(m, max_i8x4(xv[i][j]));
        }
        m = group_allreduce<L>(m, OpMax());

        // gaps d = m - x per byte: with both biased to unsigned the word subtraction never borrows
        const unsigned mrep = static_cast<unsigned>((m ^ 0x80) & 0xFF) * 0x01010101u;
        int e[NCH][16];
        int sum = 0;
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                const unsigned d4 = mrep - (static_cast<unsigned>(xv[i][w]) ^ 0x80808080u);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int d = (d4 >> (8 * j)) & 0xFF;
                    const int s = valid[i] ? table[d] : 0;
                    e[i][w * 4 + j] = s;
                    sum += s;
                }
            }
        }
        sum = group_allreduce<L>(sum, OpAdd());
        const int inv = row_inverse(p, sum);

#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            if (!valid[i]) continue;
            const int col0 = (l + L * i) * 16;
            if (p.out_i16) {
                v4i o[2];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int y0 = sat16((e[i][2 * k] * inv) >> p.out_shift);
                    const int y1 = sat16((e[i][2 * k + 1] * inv) >> p.out_shift);
                    o[k >> 2][k & 3] = static_cast<int>(pack2_halves(y0, y1));
                }
                v4i* dst = reinterpret_cast<v4i*>(static_cast<int16_t*>(out) + base + col0);
                __builtin_nontemporal_store(o[0], dst);
                __builtin_nontemporal_store(o[1], dst + 1);
            } else {
                v4i o;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    int y4[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        y4[j] = (e[i][w * 4 + j] * inv) >> p.out_shift;
                        if (!NOCLAMP_U8) y4[j] = clamp_i(y4[j], 0, 255);
                    }
                    o[w] = static_cast<int>(pack4_bytes(y4[0], y4[1], y4[2], y4[3]));
                }
                __builtin_nontemporal_store(o, reinterpret_cast<v4i*>(static_cast<uint8_t*>(out) + base + col0));
            }
        }
    }
}

// Any column count / alignment: one block per row, three passes.
__global__ __launch_bounds__(256) void softmax_generic_kernel(const int8_t* __restrict__ x, void* __restrict__ out, int rows,
                                                               int cols, SoftmaxParams p) {
    __shared__ int table[256];
    __shared__ int red[4];
    table[threadIdx.x] = table_entry(p, threadIdx.x);
    __syncthreads();
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    for (int row = blockIdx.x; row < rows; row += gridDim.x) {
        const int64_t base = static_cast<int64_t>(row) * cols;
        int m = -128;
        for (int c = threadIdx.x; c < cols; c += blockDim.x) m = max(m, static_cast<int>(x[base + c]));
        m = group_allreduce<64>(m, OpMax());
        __syncthreads();
        if (lane == 0) red[wv] = m;
        __syncthreads();
        m = max(max(red[0], red[1]), max(red[2], red[3]));
        int sum = 0;
        for (int c = threadIdx.x; c < cols; c += blockDim.x) sum += table[m - x[base + c]];
        sum = group_allreduce<64>(sum, OpAdd());
        __syncthreads();
        if (lane == 0) red[wv] = sum;
        __syncthreads();
        sum = red[0] + red[1] + red[2] + red[3];
        const int inv = row_inverse(p, sum);
        for (int c = threadIdx.x; c < cols; c += blockDim.x) {
            const int y = (table[m - x[base + c]] * inv) >> p.out_shift;
            if (p.out_i16)
                static_cast<int16_t*>(out)[base + c] = static_cast<int16_t>(sat16(y));
            else
                static_cast<uint8_t*>(out)[base + c] = static_cast<uint8_t>(clamp_i(y, 0, 255));
        }
    }
}

template <int L, int NCH>
static void launch_softmax(bool noclamp, int grid, hipStream_t stream, const int8_t* x, void* out, int rows, int cols,
                           const SoftmaxParams& p) {
    if (noclamp)
        softmax_lut_kernel<L, NCH, true><<<grid, 256, 0, stream>>>(x, out, rows, cols, p);
    else
        softmax_lut_kernel<L, NCH, false><<<grid, 256, 0, stream>>>(x, out, rows, cols, p);
}

static int softmax_dispatch(const int8_t* x, void* out, int64_t rows, int64_t cols, const SoftmaxParams& p, bool noclamp,
                            hipStream_t stream, const char* who) {
    if (rows == 0) return A4G_OK;
    A4G_REQUIRE(x && out, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    const bool fast = cols % 16 == 0 && cols <= 4096 && aligned16(x) && aligned16(out);
    if (fast) {
        const int chunks = static_cast<int>(cols / 16);
        // lanes per row: smallest power of two >= chunks (capped at 64), then chunks per lane
        int L = 1;
        while (L < chunks && L < 64) L <<= 1;
        const int nch = (chunks + L - 1) / L;
        const int rpw = 64 / L;
        const int grid = grid_for((rows + rpw - 1) / rpw, 4, 256 * 8);
        const int r = static_cast<int>(rows), c = static_cast<int>(cols);
        if (nch > 1) {  // L == 64
            if (nch <= 2) launch_softmax<64, 2>(noclamp, grid, stream, x, out, r, c, p);
            else launch_softmax<64, 4>(noclamp, grid, stream, x, out, r, c, p);
        } else {
            switch (L) {
            case 1: launch_softmax<1, 1>(noclamp, grid, stream, x, out, r, c, p); break;
            case 2: launch_softmax<2, 1>(noclamp, grid, stream, x, out, r, c, p); break;
            case 4: launch_softmax<4, 1>(noclamp, grid, stream, x, out, r, c, p); break;
            case 8: launch_softmax<8, 1>(noclamp, grid, stream, x, out, r, c, p); break;
            case 16: launch_softmax<16, 1>(noclamp, grid, stream, x, out, r, c, p); break;
            case 32: launch_softmax<32, 1>(noclamp, grid, stream, x, out, r, c, p); break;
            default: launch_softmax<64, 1>(noclamp, grid, stream, x, out, r, c, p); break;
            }
        }
    } else {
        const int grid = grid_for(rows, 1, 256 * 8);
        softmax_generic_kernel<<<grid, 256, 0, stream>>>(x, out, static_cast<int>(rows), static_cast<int>(cols), p);
    }
    return check_hip(hipGetLastError(), who);
}

}  // namespace a4g

extern "C" int a4g_softmax_exp_i8(const int8_t* x, void* out, int64_t rows, int64_t cols, int exp_kq, int inv_shift,
                                  int out_kind, a4g_stream_t stream) {
    const char* who = "a4g_softmax_exp_i8";
    A4G_REQUIRE(rows >= 0 && cols >= 1 && cols <= 65536 && rows <= INT32_MAX, A4G_ERR_INVALID_ARGUMENT,
                "%s: bad shape rows=%lld cols=%lld", who, (long long)rows, (long long)cols);
    A4G_REQUIRE(out_kind == A4G_U8 || out_kind == A4G_I16, A4G_ERR_INVALID_ARGUMENT,
                "%s: requires uint8 or int16 output, got kind %d", who, out_kind);
    A4G_REQUIRE(exp_kq >= 1 && exp_kq <= 128, A4G_ERR_INVALID_ARGUMENT, "%s: exp Softmax needs 1 <= EXP_KQ <= 128, got %d",
                who, exp_kq);
    A4G_REQUIRE(inv_shift >= 1 && inv_shift <= 21, A4G_ERR_INVALID_ARGUMENT, "%s: inv_shift %d outside [1,21]", who,
                inv_shift);
    SoftmaxParams p{};
    p.is_hccs = 0;
    p.exp_kq = exp_kq;
    p.out_i16 = out_kind == A4G_I16;
    p.numer = p.out_i16 ? 32767 : (255 << inv_shift);
    p.inv_shift = inv_shift;
    p.use_clb = 0;
    p.out_shift = p.out_i16 ? 0 : inv_shift;
    // every score <= sum and inv = floor(numer/sum) fits int16, so score*inv >> shift <= 255
    return softmax_dispatch(x, out, rows, cols, p, /*noclamp=*/true, static_cast<hipStream_t>(stream), who);
}

extern "C" int a4g_softmax_hccs_i8(const int8_t* x, void* out, int64_t rows, int64_t cols, int B, int S, int Dmax,
                                   int inv_shift, int use_clb, int out_kind, a4g_stream_t stream) {
    const char* who = "a4g_softmax_hccs_i8";
    A4G_REQUIRE(rows >= 0 && cols >= 1 && cols <= 65536 && rows <= INT32_MAX, A4G_ERR_INVALID_ARGUMENT,
                "%s: bad shape rows=%lld cols=%lld", who, (long long)rows, (long long)cols);
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
    SoftmaxParams p{};
    p.is_hccs = 1;
    p.B = B;
    p.S = S;
    p.Dmax = Dmax;
    p.out_i16 = out_kind == A4G_I16;
    p.numer = p.out_i16 ? 32767 : (255 << inv_shift);
    p.inv_shift = inv_shift;
    p.use_clb = use_clb != 0;
    p.out_shift = p.out_i16 ? 0 : inv_shift;
    const bool noclamp = !p.use_clb && inv_shift <= 15;
    return softmax_dispatch(x, out, rows, cols, p, noclamp, static_cast<hipStream_t>(stream), who);
}
