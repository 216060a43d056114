// HBM-bound row/stream operators: elementwise Add, integer LayerNorm (optionally with the residual
// add fused in front), and the table-driven integer Softmax (accurate exp and HCCS surrogate).
//
// Layout: plain row-major int8 rows. Fast paths stream each row exactly once as 16-byte chunks per
// lane (fully coalesced: 64 lanes x 16 B = 1 KiB per wave-load), keep the row in registers between
// the reduction and the normalisation, and reduce across lanes with DPP / ds_swizzle butterflies.
#include <algorithm>
#include <type_traits>

#include "common.hpp"
#include "layernorm_common.hpp"
#include "softmax_common.hpp"

namespace a4g {

// =====================================================================================================
// Elementwise Add                                   (reference: elementwise_add.cpp:12-37)
// =====================================================================================================

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

// The row kernels of this file load with the default cache policy and store non-temporally. An operand that the launch
// before has written, or read, is then found in the 256 MB memory-side cache where it fits; loads marked non-temporal
// never are (measured on 16384 x 1024: LayerNorm 8.1 -> 6.5 us, Add 7.0 -> 6.5 us, Softmax on 134 MB 44.6 -> 39.8 us),
// while results that leave without allocating there do not push the operands out (Add with plain stores: 8.7 us).
template <bool UNSIGNED>
__global__ __launch_bounds__(256) void add_sat8_kernel(const v4i* __restrict__ a, const v4i* __restrict__ b,
                                                        v4i* __restrict__ out, int64_t nvec) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += stride) {
        const v4i va = a[i];
        const v4i vb = b[i];
        v4i r;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            r[j] = UNSIGNED ? static_cast<int>(sat_add_u8x4(va[j], vb[j])) : static_cast<int>(sat_add_i8x4(va[j], vb[j]));
        }
        __builtin_nontemporal_store(r, out + i);
    }
}

// Any shift, 8- and 16-bit kinds: 16 bytes per lane and turn, each element widened, added, rounded (the sum of two
// operands and the rounding constant stay far below 2^31, so the short form of the rounding applies), clamped and packed
// again. KIND: A4G_I8, A4G_U8 or A4G_I16.
template <int KIND>
__global__ __launch_bounds__(256) void add_vec_kernel(const v4i* __restrict__ a, const v4i* __restrict__ b, v4i* __restrict__ out,
                                                       int64_t nvec, FastRound fr, int lo, int hi) {
    const int64_t stride = static_cast<int64_t>(gridDim.x) * blockDim.x;
    for (int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; i < nvec; i += stride) {
        const v4i va = a[i];
        const v4i vb = b[i];
        v4i r;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const unsigned wa = static_cast<unsigned>(va[j]), wb = static_cast<unsigned>(vb[j]);
            if (KIND == A4G_I16) {
                const int s0 = static_cast<int16_t>(wa) + static_cast<int16_t>(wb);
                const int s1 = (va[j] >> 16) + (vb[j] >> 16);
                r[j] = static_cast<int>(pack2_halves(clamp_i(fast_round(s0, fr), lo, hi), clamp_i(fast_round(s1, fr), lo, hi)));
            } else {
                int y[4];
#pragma unroll
                for (int t = 0; t < 4; ++t) {
                    const int ea = KIND == A4G_I8 ? sext8(wa, t) : static_cast<int>((wa >> (8 * t)) & 0xffu);
                    const int eb = KIND == A4G_I8 ? sext8(wb, t) : static_cast<int>((wb >> (8 * t)) & 0xffu);
                    y[t] = clamp_i(fast_round(ea + eb, fr), lo, hi);
                }
                r[j] = static_cast<int>(pack4_bytes(y[0], y[1], y[2], y[3]));
            }
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
    } else if (aligned16(a) && aligned16(b) && aligned16(out) && n * (kind == A4G_I16 ? 2 : 1) >= 16) {
        const int per_vec = kind == A4G_I16 ? 8 : 16;
        const int64_t nvec = n / per_vec;
        const int grid = grid_for(nvec, 256, 256 * 16);
        const FastRound fr = make_fast_round(round_mode, shift);
        const int lo = kind == A4G_I8 ? -128 : (kind == A4G_I16 ? -32768 : 0), hi = kind == A4G_I8 ? 127 : (kind == A4G_I16 ? 32767 : 255);
        const v4i* va = static_cast<const v4i*>(a);
        const v4i* vb = static_cast<const v4i*>(b);
        v4i* vo = static_cast<v4i*>(out);
        if (kind == A4G_I8) add_vec_kernel<A4G_I8><<<grid, 256, 0, stream>>>(va, vb, vo, nvec, fr, lo, hi);
        else if (kind == A4G_U8) add_vec_kernel<A4G_U8><<<grid, 256, 0, stream>>>(va, vb, vo, nvec, fr, lo, hi);
        else add_vec_kernel<A4G_I16><<<grid, 256, 0, stream>>>(va, vb, vo, nvec, fr, lo, hi);
        done = nvec * per_vec;
    }
    if (done < n) {
        const int grid = grid_for(n - done, 256, 256 * 8);
        add_generic_kernel<<<grid, 256, 0, stream>>>(a, b, out, done, n, kind, shift, round_mode);
    }
    return check_hip(hipGetLastError(), "a4g_add launch");
}

// ---- transposes of 1-, 2- and 4-byte elements --------------------------------------------------------------
// 64 x 64 tiles through LDS (one element of padding per row): both the reads and the writes are rows of a tile.
template <typename T>
__global__ __launch_bounds__(256) void transpose_tiles_kernel(const T* __restrict__ src, int64_t ld_src, int64_t stride_src,
                                                               T* __restrict__ dst, int64_t ld_dst, int64_t stride_dst, int rows,
                                                               int cols) {
    __shared__ T tile[64][65];
    const int r0 = blockIdx.y * 64, c0 = blockIdx.x * 64;
    const T* s = src + static_cast<int64_t>(blockIdx.z) * stride_src;
    T* d = dst + static_cast<int64_t>(blockIdx.z) * stride_dst;
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int rr = i >> 6, cc = i & 63;
        if (r0 + rr < rows && c0 + cc < cols) tile[rr][cc] = s[static_cast<int64_t>(r0 + rr) * ld_src + c0 + cc];
    }
    __syncthreads();
    for (int i = threadIdx.x; i < 64 * 64; i += 256) {
        const int cc = i >> 6, rr = i & 63;
        if (r0 + rr < rows && c0 + cc < cols) d[static_cast<int64_t>(c0 + cc) * ld_dst + r0 + rr] = tile[rr][cc];
    }
}

extern "C" int a4g_transpose(const void* src, int elem_bytes, int64_t ld_src, int64_t stride_src, void* dst, int64_t ld_dst,
                             int64_t stride_dst, int64_t batch, int64_t rows, int64_t cols, a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "a4g_transpose";
    A4G_REQUIRE(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4, A4G_ERR_UNSUPPORTED, "%s: elements of %d bytes", who,
                elem_bytes);
    A4G_REQUIRE(batch >= 0 && batch <= 65535 && rows >= 0 && cols >= 0 && rows <= (1 << 30) && cols <= (1 << 30) &&
                    (rows + 63) / 64 <= 65535,
                A4G_ERR_INVALID_ARGUMENT, "%s: bad shape batch=%lld rows=%lld cols=%lld", who, (long long)batch, (long long)rows,
                (long long)cols);
    A4G_REQUIRE(ld_src >= cols && ld_dst >= rows, A4G_ERR_INVALID_ARGUMENT, "%s: pitch smaller than the row", who);
    if (batch == 0 || rows == 0 || cols == 0) return A4G_OK;
    A4G_REQUIRE(src && dst, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    const dim3 grid(static_cast<unsigned>((cols + 63) / 64), static_cast<unsigned>((rows + 63) / 64), static_cast<unsigned>(batch));
    const int r = static_cast<int>(rows), c = static_cast<int>(cols);
    if (elem_bytes == 1)
        transpose_tiles_kernel<uint8_t><<<grid, 256, 0, stream>>>(static_cast<const uint8_t*>(src), ld_src, stride_src,
                                                                  static_cast<uint8_t*>(dst), ld_dst, stride_dst, r, c);
    else if (elem_bytes == 2)
        transpose_tiles_kernel<uint16_t><<<grid, 256, 0, stream>>>(static_cast<const uint16_t*>(src), ld_src, stride_src,
                                                                   static_cast<uint16_t*>(dst), ld_dst, stride_dst, r, c);
    else
        transpose_tiles_kernel<uint32_t><<<grid, 256, 0, stream>>>(static_cast<const uint32_t*>(src), ld_src, stride_src,
                                                                   static_cast<uint32_t*>(dst), ld_dst, stride_dst, r, c);
    return check_hip(hipGetLastError(), who);
}

namespace a4g {

// =====================================================================================================
// Integer LayerNorm                                 (reference: layer_norm.cpp:14-121)
// =====================================================================================================


// L lanes per row, 64/L rows per wave at a time; a lane owns the 16-byte chunks l, l+L, ... (NCH of
// them) of its row. gamma/beta are widened to int32 once per block and kept in LDS, quad-major
// ([4][nchunks][4] ints) so that the lanes of a group read consecutive 16-byte words. x is read from
// HBM once: the statistics and the normalisation both work from registers, and the next rows' loads
// are issued before the current rows are normalised.
// FR >= 0 adds the float form of the normalisation, taken by a block whose gamma values allow it.
template <int L, int NCH, int BIT, bool FUSE_ADD, int FR>
__global__ __launch_bounds__(256, 2) void layernorm_rows_kernel(const int8_t* __restrict__ x, const int8_t* __restrict__ x2,
                                                              const int16_t* __restrict__ gamma,
                                                              const int16_t* __restrict__ beta, int8_t* __restrict__ sum_out,
                                                              int8_t* __restrict__ out, int rows, int cols, int log2c,
                                                              int eps_q0, LnRound rg, LnRound ro, LnFloat lf) {
    extern __shared__ int ln_lds[];
    const int nchunks = cols >> 4;
    int* lg = ln_lds;
    int* lb = ln_lds + nchunks * 16;

    constexpr int G = 64 / L;  // rows per wave and iteration
    const int lane = threadIdx.x & 63;
    const int grp = lane / L, sub = lane % L;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int nwaves = (gridDim.x * blockDim.x) >> 6;

    bool valid[NCH];
    int chunk_of[NCH];
#pragma unroll
    for (int i = 0; i < NCH; ++i) {
        const int chunk = sub + L * i;
        valid[i] = chunk < nchunks;
        chunk_of[i] = valid[i] ? chunk : 0;
    }

    // Rows travel through buffer descriptors that end where the tensors end: a chunk that does not exist (a row past the
    // end, a lane past the row's last chunk, a null sum_out) is an offset beyond the descriptor, reads as zero and is
    // dropped on a store, so that no load or store sits inside a branch. The compiler counts outstanding memory
    // operations from the youngest back; one conditional operation between a load and its use would turn every wait for
    // that load into a wait for everything, stores included.
    typedef unsigned v4u __attribute__((ext_vector_type(4)));
    constexpr unsigned NOWHERE = 0xfffffff0u;
    const int tensor_bytes = rows * cols;  // < 2^31: the host splits larger tensors over several launches
    const auto rsrc_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(x), 0, tensor_bytes, 0x00020000);
    const auto rsrc_x2 = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(x2), 0, FUSE_ADD ? tensor_bytes : 0, 0x00020000);
    const auto rsrc_sum = __builtin_amdgcn_make_buffer_rsrc(sum_out, 0, sum_out ? tensor_bytes : 0, 0x00020000);
    const auto rsrc_out = __builtin_amdgcn_make_buffer_rsrc(out, 0, tensor_bytes, 0x00020000);
    constexpr int NT = 2;     // stores: non-temporal
    constexpr int CACHED = 0;  // loads: default policy (see add_sat8_kernel)
    auto offset_of = [&](int row, int i) {
        return row < rows && valid[i] ? static_cast<unsigned>(row) * static_cast<unsigned>(cols) + chunk_of[i] * 16 : NOWHERE;
    };
    v4i nx[NCH], nx2[NCH];
    auto fetch = [&](int row) {
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            nx[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, offset_of(row, i), 0, CACHED));
            if (FUSE_ADD) nx2[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_x2, offset_of(row, i), 0, CACHED));
        }
    };
    auto put = [&](__amdgpu_buffer_rsrc_t rsrc, const v4i& v, int row, int i) {
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v), rsrc, offset_of(row, i), 0, NT);
    };

    // The parameter words are requested first and the first rows right behind them: loads return in issue
    // order, so the parameters (cache hits after the first blocks) are staged while the rows are in flight.
    const int n_half_chunks = 4 * nchunks;  // 8 int16 parameters each: gamma's, then beta's
    auto param_word = [&](int hc) {
        const bool is_beta = hc >= 2 * nchunks;
        return *reinterpret_cast<const v4i*>((is_beta ? beta : gamma) + (is_beta ? hc - 2 * nchunks : hc) * 8);
    };
    v4i first_word = v4i{0, 0, 0, 0};
    first_word = param_word(min(static_cast<int>(threadIdx.x), n_half_chunks - 1));  // unconditional: see the rows' loads
    int row0 = wave * G;
    // Rows of thousands of columns fill the registers by themselves (16 per 256 columns and operand): those forms fetch
    // a row when its turn comes instead of one turn ahead, and leave the overlap to the other waves of the CU.
    constexpr bool AHEAD = NCH <= 4 || (NCH <= 8 && !FUSE_ADD);
    if (AHEAD) fetch(row0 + grp);

    // half-chunk hc = 8 columns = quads 2*(hc&1), 2*(hc&1)+1 of chunk hc>>1.
    // as_float: gamma as float, beta scaled to the output's unit, biased and offset (the float form's operands)
    auto stage_word = [&](int hc, const v4i& raw, bool as_float) {
        int wide = 0;
        {
            const bool is_beta = hc >= 2 * nchunks;
            const int h = is_beta ? hc - 2 * nchunks : hc;
            int* dst = is_beta ? lb : lg;
            const int chunk = h >> 1, q0 = (h & 1) * 2;
            v4i q[2];
            q[0][0] = static_cast<int16_t>(raw[0]); q[0][1] = raw[0] >> 16; q[0][2] = static_cast<int16_t>(raw[1]); q[0][3] = raw[1] >> 16;
            q[1][0] = static_cast<int16_t>(raw[2]); q[1][1] = raw[2] >> 16; q[1][2] = static_cast<int16_t>(raw[3]); q[1][3] = raw[3] >> 16;
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                int* at = dst + (((q0 + k) * nchunks + chunk) << 2);
                if (as_float) {
                    v4f f;
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        if (!is_beta) wide |= abs(q[k][j]) > LN_FLOAT_MAX_GAMMA;
                        f[j] = is_beta ? fmaf(static_cast<float>(q[k][j]), lf.c, lf.h2) : static_cast<float>(q[k][j]);
                    }
                    *reinterpret_cast<v4f*>(at) = f;
                } else {
                    *reinterpret_cast<v4i*>(at) = q[k];
                }
            }
        }
        return wide;
    };
    // the word requested ahead is staged outside the loop over the others, so that no load stands between its request
    // and its use on any path
    auto stage_params = [&](bool as_float) {
        int wide = 0;
        if (static_cast<int>(threadIdx.x) < n_half_chunks) wide |= stage_word(threadIdx.x, first_word, as_float);
        for (int hc = threadIdx.x + blockDim.x; hc < n_half_chunks; hc += blockDim.x) wide |= stage_word(hc, param_word(hc), as_float);
        return wide;
    };
    bool in_float = false;
    if (FR >= 0) {
        // staged for the float form first; a block that meets a gamma beyond its range stages again as integers
        in_float = !__syncthreads_or(stage_params(true));
        if (!in_float) {
            stage_params(false);
            __syncthreads();
        }
    } else {
        stage_params(false);
        __syncthreads();
    }

    // One loop per form of the normalisation (the choice is the block's, made above): a loop with a single path lets the
    // compiler count the loads and stores in flight exactly.
    auto row_loop = [&](auto float_tag) {
        constexpr bool AS_FLOAT = decltype(float_tag)::value;
        for (; row0 < rows; row0 += nwaves * G) {
            const int row = row0 + grp;
            v4i xv[NCH];
            int sx = 0, sq = 0;
            if (!AHEAD) fetch(row);
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                xv[i] = nx[i];
                if (FUSE_ADD) {
#pragma unroll
                    for (int j = 0; j < 4; ++j) xv[i][j] = static_cast<int>(sat_add_i8x4(xv[i][j], nx2[i][j]));
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // every register of this group is taken over before the next loads may land
            if (AHEAD) fetch(row + nwaves * G);  // past the last row: zeros, never used
            if (FUSE_ADD) {
#pragma unroll
                for (int i = 0; i < NCH; ++i) put(rsrc_sum, xv[i], row, i);
            }
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    sx = __builtin_amdgcn_sdot4(xv[i][j], 0x01010101, sx, false);
                    sq = __builtin_amdgcn_sdot4(xv[i][j], xv[i][j], sq, false);
                }
            }
            sx = group_allreduce<L>(sx, OpAdd());
            sq = group_allreduce<L>(sq, OpAdd());
            const RowStats st = row_stats(sx, sq, cols, log2c, eps_q0);
            const float inv_s = static_cast<float>(st.inv) * lf.s1;
            const float nm = -static_cast<float>(st.mu + 128) * lf.c;
            // The float form clamps inv * gamma to int16 only in a wave that holds a row for which the product can leave
            // that range at all: |gamma| <= 511 there, so it takes 1/sigma above 64 (a variance below 16). The other
            // waves run the loop without the clamp, one instruction in seven fewer.
            const bool may_clip = AS_FLOAT && inv_s * static_cast<float>(LN_FLOAT_MAX_GAMMA) > 32766.f;  // (the floor and ceil forms add up to one)
            auto normalise = [&](auto clip_tag) __attribute__((always_inline)) {
                constexpr bool CLIP = decltype(clip_tag)::value;
#pragma unroll
            for (int i = 0; i < NCH; ++i) {
                v4i o;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    const int at = (w * nchunks + chunk_of[i]) << 2;
                    if (AS_FLOAT) {
                        const v4f g4 = *reinterpret_cast<const v4f*>(lg + at);
                        const v4f b4 = *reinterpret_cast<const v4f*>(lb + at);
                        const unsigned word = static_cast<unsigned>(xv[i][w]) ^ 0x80808080u;
                        unsigned packed = 0;
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const float vd = fmaf(static_cast<float>((word >> (8 * j)) & 0xffu), lf.c, nm);
                            float p = 0.f;
                            if (FR == 0) p = rintf(inv_s * g4[j]);
                            if (FR == 1) p = floorf(fmaf(inv_s, g4[j], lf.h1));
                            if (FR == 2) p = ceilf(fmaf(inv_s, g4[j], lf.h1));
                            const float fs = CLIP ? __builtin_amdgcn_fmed3f(p, -32768.f, 32767.f) : p;
                            float y = fmaf(vd, fs, b4[j]);
                            if (FR == 1) y = floorf(y);
                            if (FR == 2) y = ceilf(y);
                            packed = __builtin_amdgcn_cvt_pk_u8_f32(y, j, packed);
                        }
                        o[w] = static_cast<int>(packed ^ 0x80808080u);
                    } else {
                        const v4i g4 = *reinterpret_cast<const v4i*>(lg + at);
                        const v4i b4 = *reinterpret_cast<const v4i*>(lb + at);
                        int y4[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) {
                            const int vd = sext8(xv[i][w], j) - st.mu;
                            const int fs = clamp_i(ln_round<BIT>(__mul24(st.inv, g4[j]), rg), -32768, 32767);
                            y4[j] = clamp_i(ln_round<BIT>(__mul24(vd, fs) + b4[j], ro), -128, 127);
                        }
                        o[w] = static_cast<int>(pack4_bytes(y4[0], y4[1], y4[2], y4[3]));
                    }
                }
                put(rsrc_out, o, row, i);
            }
            };
            // (rows of sixteen chunks keep the one copy with the clamp: two copies of the loop cost them 42 spilled registers)
            if (!AS_FLOAT || NCH > 8 || __builtin_amdgcn_ballot_w64(may_clip) != 0) normalise(std::true_type{});
            else normalise(std::false_type{});
        }
    };
    if (FR >= 0 && in_float) row_loop(std::true_type{});
    else row_loop(std::false_type{});
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

// The rounding modes pair up as (BIT, FR): conv_even (3, 0), floor / positive_inf (0, 1), ceil / negative_inf (0, 2);
// the symmetric modes and conv_odd have no float form (FR -1).
template <int L, int NCH>
static hipError_t launch_ln_rows(int bit_kind, int fr, bool fuse, int grid, size_t lds, hipStream_t stream, const int8_t* x,
                           const int8_t* x2, const int16_t* gamma, const int16_t* beta, int8_t* sum_out, int8_t* out,
                           int rows, int cols, int log2c, int eps_q0, const LnRound& rg, const LnRound& ro,
                           const LnFloat& lf) {
    // rows of more than 4096 columns stage more than 32 KiB of parameters: the kernels that take them are allowed the
    // 128 KiB that 16384 columns need (not the whole LDS: the kernel has a few static bytes of its own; the attribute
    // is idempotent, the race on the flag benign)
#define A4G_LN_LDS(KERN)                                                                                                 \
    if (NCH > 4) {                                                                                                       \
        static bool attr_set = false;                                                                                    \
        if (!attr_set) {                                                                                                 \
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(KERN),                                \
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, 128 * 1024);            \
            if (e != hipSuccess) return e;                                                                               \
            attr_set = true;                                                                                             \
        }                                                                                                                \
    }
#define A4G_LN_CASE(B, F)                                                                                                \
    if (bit_kind == B && fr == F) {                                                                                      \
        if (fuse) {                                                                                                      \
            if constexpr (NCH <= 8) { /* the sixteen-chunk form with a second operand has no registers left */           \
                auto kern = layernorm_rows_kernel<L, NCH, B, true, F>;                                                   \
                A4G_LN_LDS(kern)                                                                                         \
                kern<<<grid, 256, lds, stream>>>(x, x2, gamma, beta, sum_out, out, rows, cols, log2c, eps_q0, rg, ro, lf); \
            }                                                                                                            \
        } else {                                                                                                         \
            auto kern = layernorm_rows_kernel<L, NCH, B, false, F>;                                                      \
            A4G_LN_LDS(kern)                                                                                             \
            kern<<<grid, 256, lds, stream>>>(x, nullptr, gamma, beta, nullptr, out, rows, cols, log2c, eps_q0, rg, ro,   \
                                             lf);                                                                        \
        }                                                                                                                \
        return hipSuccess;                                                                                               \
    }
    A4G_LN_CASE(3, 0) A4G_LN_CASE(0, 1) A4G_LN_CASE(0, 2) A4G_LN_CASE(1, -1) A4G_LN_CASE(2, -1) A4G_LN_CASE(4, -1)
#undef A4G_LN_CASE
#undef A4G_LN_LDS
    return hipErrorInvalidValue;  // no such pair of rounding forms
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
    const bool fast = cols % 16 == 0 && cols <= (fuse ? 8192 : 16384) && aligned16(a) && aligned16(out) && (!fuse || aligned16(b)) &&
                      (!sum_out || aligned16(sum_out)) && aligned16(gamma) && aligned16(beta) && (!fuse || add_shift == 0);
    if (fast) {
        const int nchunks = static_cast<int>(cols / 16);
        int bit_kind = 0, unused = 0;
        const LnRound rg = make_ln_round(mode, gamma_shift, &bit_kind);
        const LnRound ro = make_ln_round(mode, final_shift, &unused);
        int fr = -1;
        const LnFloat lf = make_ln_float(mode, gamma_shift, final_shift, &fr);
        const size_t lds = static_cast<size_t>(cols) * 8;
        // Three blocks per CU: every wave then normalises two or three groups of rows, so the loads of the next
        // group and the stores of the previous one overlap the arithmetic (one group per wave leaves the three
        // phases of all waves in step with each other). Measured on 16384 x 1024: 8.9 us against 9.5 us with four
        // blocks per CU and 10.2 us with 2.5.
        // (fewer where the staged parameters, 8 bytes a column, leave room for fewer)
        const int max_grid = 256 * static_cast<int>(std::min<size_t>(3, (160 * 1024) / lds));
        // the kernel addresses its tensors with 32-bit offsets: launches of less than 2 GiB each
        const int64_t rows_per_launch = std::max<int64_t>(1, ((int64_t{1} << 31) - 1) / cols);
        for (int64_t r0 = 0; r0 < rows; r0 += rows_per_launch) {
            const int nrows = static_cast<int>(std::min(rows_per_launch, rows - r0));
            const int64_t skip = r0 * cols;
            const int8_t* ac = a + skip;
            const int8_t* bc = b ? b + skip : nullptr;
            int8_t* sc = sum_out ? sum_out + skip : nullptr;
            int8_t* oc = out + skip;
#define A4G_LN_GO(L, NCH)                                                                                                \
    launched = launch_ln_rows<L, NCH>(bit_kind, fr, fuse, grid_for(nrows, 4 * (64 / L), max_grid), lds, stream, ac, bc,  \
                                      gamma, beta, sc, oc, nrows, (int)cols, log2c, eps_q0, rg, ro, lf)
            hipError_t launched = hipSuccess;
            if (nchunks <= 1) A4G_LN_GO(1, 1);
            else if (nchunks <= 2) A4G_LN_GO(2, 1);
            else if (nchunks <= 4) A4G_LN_GO(4, 1);
            else if (nchunks <= 8) A4G_LN_GO(4, 2);
            else if (nchunks <= 12) A4G_LN_GO(4, 3);
            else if (nchunks <= 16) A4G_LN_GO(8, 2);
            else if (nchunks <= 24) A4G_LN_GO(8, 3);
            else if (nchunks <= 32) A4G_LN_GO(16, 2);
            else if (nchunks <= 48) A4G_LN_GO(16, 3);
            else if (nchunks <= 64) A4G_LN_GO(32, 2);
            else if (nchunks <= 128) A4G_LN_GO(64, 2);
            else if (nchunks <= 256) A4G_LN_GO(64, 4);
            else if (nchunks <= 320) A4G_LN_GO(64, 5);
            else if (nchunks <= 384) A4G_LN_GO(64, 6);
            else if (nchunks <= 448) A4G_LN_GO(64, 7);
            else if (nchunks <= 512) A4G_LN_GO(64, 8);
            else A4G_LN_GO(64, 16);
#undef A4G_LN_GO
            if (launched != hipSuccess) return check_hip(launched, who);
        }
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

// Byte-wise max of four packed int8 as a scalar.
__device__ __forceinline__ int max_i8x4(unsigned w) {
    return max(max(sext8(w, 0), sext8(w, 1)), max(sext8(w, 2), sext8(w, 3)));
}

// L consecutive lanes share one row (64/L rows per wave pass); lane l of the group owns chunks
// l, l+L, ... (NCH of them), 16 int8 each.
// FASTP: uint8 output that needs no clamp with a shift of at most 16: the probability is read as byte 2 of
// score * (inv << (16 - shift)), which saves the shift. FULL: cols == L * NCH * 16, no chunk is ever masked.
// RAGGED (never with FULL): cols need not be a multiple of 16 nor rows 16-byte aligned; `ragged` says how a row's
// chunks may be fetched and stored (load_chunk_ragged), the last chunk of a row is cut at cols.
template <int L, int NCH, bool FASTP, bool FULL, bool RAGGED = false>
__global__ __launch_bounds__(256) void softmax_lut_kernel(const int8_t* __restrict__ x, void* __restrict__ out, int rows,
                                                           int cols, SoftmaxParams p, int ragged = 0) {
    static_assert(!(RAGGED && FULL), "a ragged row never fills its chunks");
    __shared__ int table[256];
    table[threadIdx.x] = table_entry(p, threadIdx.x);
    __syncthreads();

    constexpr int RPW = 64 / L;
    const int lane = threadIdx.x & 63;
    const int grp = lane / L, l = lane % L;
    const int wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const int nwaves = (gridDim.x * blockDim.x) >> 6;
    const char* tbytes = reinterpret_cast<const char*>(table);
    const unsigned two = 2;

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
            valid[i] = row_ok && (FULL || col0 < cols);
            xv[i] = v4i{(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
            if constexpr (RAGGED) {
                if (valid[i]) {
                    const int rem = cols - col0;
                    xv[i] = load_chunk_ragged(x + base + col0, rem, ragged);
#pragma unroll
                    for (int w = 0; w < 4; ++w) {  // bytes past the row's end: -128, which no maximum notices
                        const int n = rem - 4 * w;
                        if (n <= 0) xv[i][w] = static_cast<int>(0x80808080u);
                        else if (n < 4) xv[i][w] |= static_cast<int>(0x80808080u & ~((1u << (8 * n)) - 1u));
                    }
                }
            } else {
                if (valid[i]) xv[i] = *reinterpret_cast<const v4i*>(x + base + col0);
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) m = max(m, max_i8x4(xv[i][j]));
        }
        m = group_allreduce<L>(m, OpMax());

        // gaps d = m - x per byte: with both biased to unsigned the word subtraction never borrows
        const unsigned mrep = static_cast<unsigned>((m ^ 0x80) & 0xFF) * 0x01010101u;
        // Rows of up to 4096 columns keep their scores (16 registers a chunk) between the sum and the products; longer
        // rows have no room for that and look every score up a second time.
        constexpr bool KEEP = NCH <= 4;
        int e[KEEP ? NCH : 1][16];
        int sum = 0;
        auto scores_of = [&](int i, int w, int (&s4)[4]) {
            const unsigned d4 = mrep - (static_cast<unsigned>(xv[i][w]) ^ 0x80808080u);
            s4[0] = *reinterpret_cast<const int*>(tbytes + byte_x4<0>(d4, two));
            s4[1] = *reinterpret_cast<const int*>(tbytes + byte_x4<1>(d4, two));
            s4[2] = *reinterpret_cast<const int*>(tbytes + byte_x4<2>(d4, two));
            s4[3] = *reinterpret_cast<const int*>(tbytes + byte_x4<3>(d4, two));
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool in = RAGGED ? (l + L * i) * 16 + w * 4 + j < cols : valid[i];
                s4[j] = (FULL || (in && valid[i])) ? s4[j] : 0;
            }
        };
#pragma unroll
        for (int i = 0; i < NCH; ++i) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                int s4[4];
                scores_of(i, w, s4);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    if (KEEP) e[i][w * 4 + j] = s4[j];
                    sum += s4[j];
                }
            }
        }
        sum = group_allreduce<L>(sum, OpAdd());
        const int inv = row_inverse(p, sum);
        const unsigned inv16 = static_cast<unsigned>(inv) << (16 - p.out_shift);  // FASTP only

#pragma unroll
        for (int i = 0; i < NCH; ++i) {
            if (!valid[i]) continue;
            const int col0 = (l + L * i) * 16;
            int ei[16];
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                int s4[4];
                if (!KEEP) scores_of(i, w, s4);
#pragma unroll
                for (int j = 0; j < 4; ++j) ei[w * 4 + j] = KEEP ? e[i][w * 4 + j] : s4[j];
            }
            if (p.out_i16) {
                v4i o[2];
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    const int y0 = sat16(__mul24(ei[2 * k], inv) >> p.out_shift);
                    const int y1 = sat16(__mul24(ei[2 * k + 1], inv) >> p.out_shift);
                    o[k >> 2][k & 3] = static_cast<int>(pack2_halves(y0, y1));
                }
                if constexpr (RAGGED) {
                    int8_t* dst = reinterpret_cast<int8_t*>(static_cast<int16_t*>(out) + base + col0);
                    const int rem = (cols - col0) * 2;  // bytes
                    const int mode = ragged == 0 ? 1 : ragged;  // two-byte elements: an aligned byte row gives aligned dwords at best
                    store_chunk_ragged(dst, o[0], rem, (cols % 2 == 0 && mode == 1) ? 1 : 2);
                    store_chunk_ragged(dst + 16, o[1], rem - 16, (cols % 2 == 0 && mode == 1) ? 1 : 2);
                } else {
                    v4i* dst = reinterpret_cast<v4i*>(static_cast<int16_t*>(out) + base + col0);
                    __builtin_nontemporal_store(o[0], dst);
                    __builtin_nontemporal_store(o[1], dst + 1);
                }
            } else {
                v4i o;
#pragma unroll
                for (int w = 0; w < 4; ++w) {
                    if (FASTP) {
                        unsigned q[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) q[j] = __umul24(static_cast<unsigned>(ei[w * 4 + j]), inv16);
                        o[w] = static_cast<int>(__builtin_amdgcn_perm(q[1], q[0], 0x0c0c0602u) |
                                                __builtin_amdgcn_perm(q[3], q[2], 0x06020c0cu));
                    } else {
                        int y4[4];
#pragma unroll
                        for (int j = 0; j < 4; ++j) y4[j] = clamp_i(__mul24(ei[w * 4 + j], inv) >> p.out_shift, 0, 255);
                        o[w] = static_cast<int>(pack4_bytes(y4[0], y4[1], y4[2], y4[3]));
                    }
                }
                if constexpr (RAGGED)
                    store_chunk_ragged(static_cast<int8_t*>(out) + base + col0, o, cols - col0, ragged);
                else
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
                           const SoftmaxParams& p, int ragged) {
    const bool fastp = noclamp && !p.out_i16 && p.out_shift <= 16;
    if (ragged >= 0) {
        if constexpr (NCH <= 4) {  // the ragged form stops at 4096 columns
            if (fastp) softmax_lut_kernel<L, NCH, true, false, true><<<grid, 256, 0, stream>>>(x, out, rows, cols, p, ragged);
            else softmax_lut_kernel<L, NCH, false, false, true><<<grid, 256, 0, stream>>>(x, out, rows, cols, p, ragged);
        }
        return;
    }
    const bool full = cols == L * NCH * 16;
    if (fastp && full)
        softmax_lut_kernel<L, NCH, true, true><<<grid, 256, 0, stream>>>(x, out, rows, cols, p);
    else if (fastp)
        softmax_lut_kernel<L, NCH, true, false><<<grid, 256, 0, stream>>>(x, out, rows, cols, p);
    else if (full)
        softmax_lut_kernel<L, NCH, false, true><<<grid, 256, 0, stream>>>(x, out, rows, cols, p);
    else
        softmax_lut_kernel<L, NCH, false, false><<<grid, 256, 0, stream>>>(x, out, rows, cols, p);
}

static int softmax_dispatch(const int8_t* x, void* out, int64_t rows, int64_t cols, const SoftmaxParams& p, bool noclamp,
                            hipStream_t stream, const char* who) {
    if (rows == 0) return A4G_OK;
    A4G_REQUIRE(x && out, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    const bool aligned = cols % 16 == 0 && aligned16(x) && aligned16(out);
    if (cols <= 4096 || (aligned && cols <= 16384)) {
        // rows off the 16-byte grid: the same kernel with loads and stores that respect the row ends; the output has
        // the input's row offsets, so one mode serves both when both bases are equally aligned
        int ragged = -1;
        if (!aligned) {
            const uintptr_t both = reinterpret_cast<uintptr_t>(x) | reinterpret_cast<uintptr_t>(out);
            ragged = (cols % 4 == 0 && both % 4 == 0) ? 1 : 2;
        }
        const int chunks = static_cast<int>((cols + 15) / 16);
        // lanes per row: smallest power of two >= chunks (capped at 64), then chunks per lane
        int L = 1;
        while (L < chunks && L < 64) L <<= 1;
        const int nch = (chunks + L - 1) / L;
        const int rpw = 64 / L;
        // 32 blocks per CU measured best on 262144 x 512 (44.5 us; 8 per CU 47 us, 4 per CU 55 us, 128 per CU 46 us)
        const int grid = grid_for((rows + rpw - 1) / rpw, 4, 256 * 32);
        const int r = static_cast<int>(rows), c = static_cast<int>(cols);
        if (nch > 1) {  // L == 64
            if (nch <= 2) launch_softmax<64, 2>(noclamp, grid, stream, x, out, r, c, p, ragged);
            else if (nch <= 4) launch_softmax<64, 4>(noclamp, grid, stream, x, out, r, c, p, ragged);
            else if (nch <= 8) launch_softmax<64, 8>(noclamp, grid, stream, x, out, r, c, p, ragged);
            else launch_softmax<64, 16>(noclamp, grid, stream, x, out, r, c, p, ragged);
        } else {
            switch (L) {
            case 1: launch_softmax<1, 1>(noclamp, grid, stream, x, out, r, c, p, ragged); break;
            case 2: launch_softmax<2, 1>(noclamp, grid, stream, x, out, r, c, p, ragged); break;
            case 4: launch_softmax<4, 1>(noclamp, grid, stream, x, out, r, c, p, ragged); break;
            case 8: launch_softmax<8, 1>(noclamp, grid, stream, x, out, r, c, p, ragged); break;
            case 16: launch_softmax<16, 1>(noclamp, grid, stream, x, out, r, c, p, ragged); break;
            case 32: launch_softmax<32, 1>(noclamp, grid, stream, x, out, r, c, p, ragged); break;
            default: launch_softmax<64, 1>(noclamp, grid, stream, x, out, r, c, p, ragged); break;
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
    SoftmaxParams p{};
    bool noclamp = false;
    if (int rc = make_exp_params(who, exp_kq, inv_shift, out_kind, &p, &noclamp)) return rc;
    return softmax_dispatch(x, out, rows, cols, p, noclamp, static_cast<hipStream_t>(stream), who);
}

extern "C" int a4g_softmax_hccs_i8(const int8_t* x, void* out, int64_t rows, int64_t cols, int B, int S, int Dmax,
                                   int inv_shift, int use_clb, int out_kind, a4g_stream_t stream) {
    const char* who = "a4g_softmax_hccs_i8";
    A4G_REQUIRE(rows >= 0 && cols >= 1 && cols <= 65536 && rows <= INT32_MAX, A4G_ERR_INVALID_ARGUMENT,
                "%s: bad shape rows=%lld cols=%lld", who, (long long)rows, (long long)cols);
    SoftmaxParams p{};
    bool noclamp = false;
    if (int rc = make_hccs_params(who, cols, B, S, Dmax, inv_shift, use_clb, out_kind, &p, &noclamp)) return rc;
    return softmax_dispatch(x, out, rows, cols, p, noclamp, static_cast<hipStream_t>(stream), who);
}
