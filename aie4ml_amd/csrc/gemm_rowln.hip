// Dense whose output rows are normalised in the same launch:
//     out = LayerNorm(saturate_i8(Dense(x) + residual))                     (residual optional)
// the tail of a transformer sub-block (attention output projection or second feed-forward projection, then the
// residual Add, then the LayerNorm). Run as three launches the Dense result and the sum each make a round trip through
// memory and, at encoder sizes, each launch is a chain of latencies; LayerNorm needs whole rows, so the Dense kernels
// that tile the output columns over workgroups cannot normalise what they produce.
//
// Here a workgroup of eight waves owns 32 or 64 complete rows (RB blocks of 32; up to 768 columns):
//   * their activations, rows x K, are fetched once, straight into LDS (buffer loads with the LDS bit), and stay there;
//   * wave w computes, for all rows, the columns of up to three 32-wide blocks. Nobody else in the workgroup needs those weights, so
//     they go from memory (L2: every workgroup streams the same matrix) straight into registers, four K steps ahead
//     of the MFMAs that consume them, from a copy laid out in the order of the fragments (one fully coalesced 1 KiB
//     load per fragment, a4g_rowpack_weights_i8). After the activations have landed the main loop has no barrier;
//   * the accumulators are requantised in registers (weight rows permuted so that a lane holds 16 neighbouring bytes of
//     its output row), the residual is added, the row sums travel through LDS (one barrier) and the rows are normalised
//     and stored from registers.
// Every workgroup pulls the whole weight matrix out of L2, N x K bytes per 32 or 64 rows, and that traffic is what bounds
// the main loop (about 17 TB/s over the whole chip when every CU streams): 64 rows per workgroup halve it, at the price
// of half as many workgroups.
// Arithmetic: dense_bias_relu.cpp:112-163, elementwise_add.cpp:12-37, layer_norm.cpp:14-121, unchanged.
#include <algorithm>
#include <type_traits>

#include "gemm_direct.hpp"
#include "layernorm_common.hpp"

namespace a4g {

constexpr int RL_NT = 512, RL_WAVES = 8, RL_BPW = 3;
constexpr int RL_MAX_N = RL_WAVES * RL_BPW * 32;  // 768
constexpr int RL_MAX_K = 4096;                    // 128 KiB of activations in LDS at 32 rows
constexpr int RL_MAX_K2 = 2304;                   // 144 KiB at 64 rows
// LDS: the activations, then gamma, beta and the accumulators' start values (four bytes a column each), then the row
// sums [row][wave]{sum, sum of squares}, then one flag per wave
constexpr int rl_lds_bytes(int rows, int K, int N) { return rows * K + 12 * N + rows * RL_WAVES * 2 * 4 + RL_WAVES * 4; }

struct RowLnArgs {
    const int8_t* A;
    const int8_t* Wf;
    const int32_t* bias;
    const int32_t* colsum;
    const int8_t* res;
    const int16_t* gamma;
    const int16_t* beta;
    int8_t* out;
    int lda, ld_res, ld_out;
    int M, N, K;
    int a_unsigned, bpw;  // bpw: 32-column blocks per wave
    int a_bytes, w_bytes, res_bytes;
    ByteRequant dq;  // Dense requantisation: the quick form's constants ...
    RoundCfg drc;    // ... and the general form's
    int quick;       // the shift allows the quick form
    int lo, hi;
    int log2c, eps_q0, ln_mode, gamma_shift, final_shift;
    LnFloat lf;
    FastRound ln_rg, ln_ro;  // the integer form's two roundings (inv * gamma, then vd * fscale + beta) as data: one path for all modes
};

// FR: the float form of the normalisation (0 nearest even, 1 floor family, 2 ceil family), -1: integer form only.
template <int RB, int FR>
__global__ __launch_bounds__(RL_NT, 2) void gemm_rowln_kernel(RowLnArgs g) {
    constexpr int BM = 32 * RB, SLAB = BM * 128;
    extern __shared__ __attribute__((aligned(16))) int8_t rl_smem[];
    int8_t* const a_lds = rl_smem;  // K / 128 slabs of BM rows x 128 bytes
    int* const gamma_lds = reinterpret_cast<int*>(rl_smem + BM * g.K);  // floats for the float form, else int32
    int* const beta_lds = gamma_lds + g.N;
    int* const start_lds = beta_lds + g.N;
    int* const stat_lds = start_lds + g.N;
    int* const flag_lds = stat_lds + BM * RL_WAVES * 2;

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int frow = lane & 31, half = lane >> 5;
    const int m0 = blockIdx.x * BM;
    const int iters = g.K >> 7;  // slabs of 128 bytes = four K steps
    A4G_STAMP(0);

    // ---- activations: instruction q fills eight rows of a slab (4 RB instructions per slab); the 16-byte slot s of
    // row r holds K chunk s ^ ((r >> 1) & 7). Rows past the end of the matrix lie outside the descriptor and read as zero.
    {
        const auto rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(g.A), 0, g.a_bytes, 0x00020000);
        const int lrow8 = lane >> 3, slot = lane & 7;
        for (int q = wave; q < 4 * RB * iters; q += RL_WAVES) {
            const int row = 8 * (q % (4 * RB)) + lrow8;
            const int voff = (m0 + row) * g.lda + (q / (4 * RB)) * 128 + ((slot ^ ((row >> 1) & 7)) * 16);
            __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc_a, (__attribute__((address_space(3))) void*)(a_lds + q * 1024), 16, voff, 0, 0, 0);
        }
    }

    // gamma and beta wait in LDS for the epilogue: as the float form's operands (gamma as float, beta scaled to the
    // output's unit, biased and offset) or, where some gamma is beyond that form's range, as int32
    auto stage_params = [&](bool as_float) {
        int wide = 0;
        for (int c = tid; c < g.N / 4; c += RL_NT) {
            const bool is_beta = c >= g.N / 8;
            const int c8 = (is_beta ? c - g.N / 8 : c) * 8;
            const v4i raw = *reinterpret_cast<const v4i*>((is_beta ? g.beta : g.gamma) + c8);
            int* dst = (is_beta ? beta_lds : gamma_lds) + c8;
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int q[4] = {static_cast<int16_t>(raw[2 * h]), raw[2 * h] >> 16, static_cast<int16_t>(raw[2 * h + 1]), raw[2 * h + 1] >> 16};
                if (as_float) {
                    v4f f;
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        if (!is_beta) wide |= abs(q[t]) > LN_FLOAT_MAX_GAMMA;
                        f[t] = is_beta ? fmaf(static_cast<float>(q[t]), g.lf.c, g.lf.h2) : static_cast<float>(q[t]);
                    }
                    *reinterpret_cast<v4f*>(dst + 4 * h) = f;
                } else {
                    *reinterpret_cast<v4i*>(dst + 4 * h) = v4i{q[0], q[1], q[2], q[3]};
                }
            }
        }
        return wide;
    };
    // ---- this wave's blocks: columns 32 nb .. + 31, nb = wave * bpw + j; a lane ends up with columns 16 half .. + 15
    const auto rsrc_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(g.Wf), 0, g.w_bytes, 0x00020000);
    bool live[RL_BPW];
    int wv[RL_BPW], col0[RL_BPW];
#pragma unroll
    for (int j = 0; j < RL_BPW; ++j) {
        const int nb = wave * g.bpw + j;
        live[j] = j < g.bpw && nb * 32 < g.N;
        col0[j] = nb * 32 + 16 * half;
        // fragment (nb, ks) is the 1 KiB at ((nb * K / 32) + ks) * 1024; a dead block reads past the end: zeros
        wv[j] = live[j] ? nb * (g.K >> 5) * 1024 + lane * 16 : g.w_bytes;
    }
    auto wload = [&](int j, int ks) {
        return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, wv[j] + ks * 1024, 0, 0));
    };
    v4i wf[4][RL_BPW];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
        for (int j = 0; j < RL_BPW; ++j) wf[kk][j] = wload(j, kk);

    // ---- the residual, requested now so that it arrives with the first operands. Like the bias and the column sums
    // below it comes through a buffer descriptor that covers exactly what exists (nothing for a null pointer), so that
    // absent operands, rows past the end and dead blocks read as zero without a branch around any load: branches here
    // would put a wait behind every single load.
    constexpr int NOWHERE = 0x7ffffff0;  // beyond every descriptor
    const auto rsrc_res = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(g.res), 0, g.res ? g.res_bytes : 0, 0x00020000);
    v4i rw[RB][RL_BPW];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int j = 0; j < RL_BPW; ++j)
            rw[rb][j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                rsrc_res, live[j] ? (m0 + rb * 32 + frow) * g.ld_res + col0[j] : NOWHERE, 0, 0));

    // ---- the accumulators' start values, bias + 128 * colsum (int32 wraps like the sum it stands for), go through LDS:
    // fetched by every lane for its own columns they would be 24 load instructions per wave, and the vector memory
    // path takes 16 clocks per instruction however little it fetches
    if (tid < g.N / 4) {
        v4i st = {0, 0, 0, 0};
        if (g.bias) st = *reinterpret_cast<const v4i*>(g.bias + tid * 4);
        if (g.a_unsigned) st += 128 * *reinterpret_cast<const v4i*>(g.colsum + tid * 4);
        *reinterpret_cast<v4i*>(start_lds + tid * 4) = st;
    }

    // the parameter loads come last: their wait, inside the branch that issues them, then covers everything above
    const int wide_here = FR >= 0 ? stage_params(true) : (stage_params(false), 1);

    int koff[4];  // activation fragment of K step kk of a slab: row frow, chunk 2 kk + half
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) koff[kk] = frow * 128 + (((kk * 2 + half) ^ ((frow >> 1) & 7)) * 16);
    const int xmask = g.a_unsigned ? static_cast<int>(0x80808080u) : 0;  // uint8 -> int8

    if (lane == 0) flag_lds[wave] = __any(wide_here) ? 1 : 0;
    A4G_STAMP(1);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // own activation loads have landed ...
    __syncthreads();                                   // ... and everyone's
    const v4i fl0 = *reinterpret_cast<const v4i*>(flag_lds), fl1 = *reinterpret_cast<const v4i*>(flag_lds + 4);
    const bool in_float = ((fl0[0] | fl0[1] | fl0[2] | fl0[3] | fl1[0] | fl1[1] | fl1[2] | fl1[3]) == 0);  // every gamma fits the float form
    if (FR >= 0 && !in_float) {
        stage_params(false);
        __syncthreads();
    }
    // The compiler counts loads from the youngest back and, where two paths meet, lines them up at the youngest: a load
    // it believes outstanding on entry to the loop would look younger than everything the loop issues, and every wait
    // inside would become a wait for all loads. The first fragments have arrived with the wait above; passing them
    // through an empty asm makes the compiler wait for them here too, and the loop's waits then count exactly.
    v16i acc[RB][RL_BPW];
    bool small = true;
#pragma unroll
    for (int j = 0; j < RL_BPW; ++j) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const v4i st = live[j] ? *reinterpret_cast<const v4i*>(start_lds + col0[j] + 4 * q) : v4i{0, 0, 0, 0};
#pragma unroll
            for (int t = 0; t < 4; ++t) {
#pragma unroll
                for (int rb = 0; rb < RB; ++rb) acc[rb][j][q * 4 + t] = st[t];
                small = small && st[t] <= (1 << 30) && st[t] >= -(1 << 30);
            }
        }
    }
    const bool quick = g.quick && __all(small);
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
        for (int j = 0; j < RL_BPW; ++j) asm volatile("" : "+v"(wf[kk][j]));
#pragma unroll
    for (int rb = 0; rb < RB; ++rb)
#pragma unroll
        for (int j = 0; j < RL_BPW; ++j) asm volatile("" : "+v"(rw[rb][j]));

    auto slab = [&](int it, bool more) {
        const int8_t* base = a_lds + it * SLAB;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            v4i a_op[RB];
#pragma unroll
            for (int rb = 0; rb < RB; ++rb) a_op[rb] = *reinterpret_cast<const v4i*>(base + rb * 4096 + koff[kk]) ^ xmask;
#pragma unroll
            for (int rb = 0; rb < RB; ++rb)
#pragma unroll
                for (int j = 0; j < RL_BPW; ++j) acc[rb][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[kk][j], a_op[rb], acc[rb][j], 0, 0, 0);
            if (more) {
#pragma unroll
                for (int j = 0; j < RL_BPW; ++j) wf[kk][j] = wload(j, (it + 1) * 4 + kk);
            }
            __builtin_amdgcn_sched_barrier(0);  // the loads stay behind the MFMAs that free their registers
        }
    };
    A4G_STAMP(2);
    for (int it = 0; it < iters - 1; ++it) slab(it, true);

    slab(iters - 1, false);
    A4G_STAMP(3);

    // ---- Dense requantisation and the residual: word q of block j = columns col0[j] + 4 q .. + 3; the sums replace
    // the first four accumulators of their block
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        int sx = 0, sq = 0;
#pragma unroll
        for (int j = 0; j < RL_BPW; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                unsigned y;
                if (quick) {
                    y = requant4_bytes_rt(acc[rb][j][q * 4], acc[rb][j][q * 4 + 1], acc[rb][j][q * 4 + 2], acc[rb][j][q * 4 + 3], g.dq);
                } else {
                    int v[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) v[t] = clamp_i(apply_round(acc[rb][j][q * 4 + t], g.drc), g.lo, g.hi);
                    y = pack4_bytes(v[0], v[1], v[2], v[3]);
                }
                if (g.res) y = sat_add_i8x4(y, static_cast<unsigned>(rw[rb][j][q]));
                acc[rb][j][q] = static_cast<int>(y);
                if (live[j]) {
                    sx = __builtin_amdgcn_sdot4(static_cast<int>(y), 0x01010101, sx, false);
                    sq = __builtin_amdgcn_sdot4(static_cast<int>(y), static_cast<int>(y), sq, false);
                }
            }
        }
        sx += __shfl_xor(sx, 32);
        sq += __shfl_xor(sq, 32);
        if (half == 0) *reinterpret_cast<int2*>(stat_lds + ((rb * 32 + frow) * RL_WAVES + wave) * 2) = make_int2(sx, sq);
    }
    __syncthreads();

    A4G_STAMP(4);
    // ---- normalisation
    // one row block; written as a call per block because the integer form is too long for the unroller to duplicate
    auto normalise = [&](auto rb_tag) {
        constexpr int rb = decltype(rb_tag)::value;
        int sx = 0, sq = 0;
#pragma unroll
        for (int p = 0; p < RL_WAVES / 2; ++p) {
            const v4i t = *reinterpret_cast<const v4i*>(stat_lds + (rb * 32 + frow) * RL_WAVES * 2 + 4 * p);
            sx += t[0] + t[2];
            sq += t[1] + t[3];
        }
        const RowStats st = row_stats(sx, sq, g.N, g.log2c, g.eps_q0);
        const float inv_s = static_cast<float>(st.inv) * g.lf.s1;
        const float nm = -static_cast<float>(st.mu + 128) * g.lf.c;
        const int m = m0 + rb * 32 + frow;
#pragma unroll
        for (int j = 0; j < RL_BPW; ++j) {
            const int cj = live[j] ? col0[j] : 0;  // a dead block is computed on column 0's parameters and not stored
            v4i o;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                // columns 4 q .. + 3 of the lane's 16
                const unsigned sword = static_cast<unsigned>(acc[rb][j][q]);
                if (FR >= 0 && in_float) {
                    const v4f g4 = *reinterpret_cast<const v4f*>(gamma_lds + cj + 4 * q);
                    const v4f b4 = *reinterpret_cast<const v4f*>(beta_lds + cj + 4 * q);
                    const unsigned word = sword ^ 0x80808080u;
                    unsigned packed = 0;
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const float vd = fmaf(static_cast<float>((word >> (8 * t)) & 0xffu), g.lf.c, nm);
                        float p;
                        if (FR == 0) p = rintf(inv_s * g4[t]);
                        if (FR == 1) p = floorf(fmaf(inv_s, g4[t], g.lf.h1));
                        if (FR == 2) p = ceilf(fmaf(inv_s, g4[t], g.lf.h1));
                        const float fs = __builtin_amdgcn_fmed3f(p, -32768.f, 32767.f);
                        float y = fmaf(vd, fs, b4[t]);
                        if (FR == 1) y = floorf(y);
                        if (FR == 2) y = ceilf(y);
                        packed = __builtin_amdgcn_cvt_pk_u8_f32(y, t, packed);
                    }
                    o[q] = static_cast<int>(packed ^ 0x80808080u);
                } else {
                    const v4i g4 = *reinterpret_cast<const v4i*>(gamma_lds + cj + 4 * q);
                    const v4i b4 = *reinterpret_cast<const v4i*>(beta_lds + cj + 4 * q);
                    int y4[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int vd = sext8(sword, t) - st.mu;
                        // inv * gamma < 2^30 and |vd * fscale + beta| < 2^24: the short form of the rounding applies (the
                        // switch over the eight modes per element cost 10 us of the launch's 24)
                        const int fs = clamp_i(fast_round(st.inv * g4[t], g.ln_rg), -32768, 32767);
                        y4[t] = clamp_i(fast_round(vd * fs + b4[t], g.ln_ro), -128, 127);
                    }
                    o[q] = static_cast<int>(pack4_bytes(y4[0], y4[1], y4[2], y4[3]));
                }
            }
            if (live[j] && m < g.M) *reinterpret_cast<v4i*>(g.out + static_cast<int64_t>(m) * g.ld_out + col0[j]) = o;
        }
    };
    normalise(std::integral_constant<int, 0>{});
    if (RB > 1) normalise(std::integral_constant<int, RB - 1>{});
    A4G_STAMP(5);
}

// Wt [N][ldwt] (a4g_pack_weights_i8) -> fragments: the 16 bytes of lane l of fragment (nb, ks) are K chunk
// 32 ks + 16 (l / 32) of the weight row of column 32 nb + direct_col_of_operand_row(l % 32); columns past N and
// chunks past K are zero (whole 32-column groups, whole 128-byte K tiles: rowpacked_bytes).
__global__ __launch_bounds__(256) void rowpack_kernel(const int8_t* __restrict__ wt, int64_t ldwt, int N, int K, v4i* __restrict__ wf) {
    const int ksteps = (K + 127) / 128 * 4;
    const int64_t chunks = static_cast<int64_t>((N + 31) / 32) * ksteps * 64;
    for (int64_t c = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x; c < chunks; c += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int l = static_cast<int>(c & 63);
        const int64_t frag = c >> 6;
        const int ks = static_cast<int>(frag % ksteps), nb = static_cast<int>(frag / ksteps);
        const int n = nb * 32 + direct_col_of_operand_row(l & 31), k0 = ks * 32 + 16 * (l >> 5);
        v4i v = {0, 0, 0, 0};
        if (n < N && k0 < K) v = *reinterpret_cast<const v4i*>(wt + static_cast<int64_t>(n) * ldwt + k0);
        wf[c] = v;
    }
}

template <int RB, int FR>
static hipError_t launch_rowln(const RowLnArgs& g, hipStream_t stream) {
    auto kern = gemm_rowln_kernel<RB, FR>;
    static bool attr_set = false;  // benign race: the attribute is idempotent
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           rl_lds_bytes(32 * RB, RB == 1 ? RL_MAX_K : RL_MAX_K2, RL_MAX_N));
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    kern<<<(g.M + 32 * RB - 1) / (32 * RB), RL_NT, rl_lds_bytes(32 * RB, g.K, g.N), stream>>>(g);
    return hipGetLastError();
}
template <int RB>
static hipError_t launch_rowln_rb(const RowLnArgs& g, int fr, hipStream_t stream) {
    switch (fr) {
    case 0: return launch_rowln<RB, 0>(g, stream);
    case 1: return launch_rowln<RB, 1>(g, stream);
    case 2: return launch_rowln<RB, 2>(g, stream);
    default: return launch_rowln<RB, -1>(g, stream);
    }
}

}  // namespace a4g

using namespace a4g;

extern "C" int64_t a4g_rowpacked_bytes(int64_t N, int64_t K) { return N <= 0 || K <= 0 ? 0 : rowpacked_bytes(N, K); }

extern "C" int a4g_rowpack_weights_i8(const int8_t* Wt, int64_t ldwt, int64_t N, int64_t K, int8_t* Wf, a4g_stream_t stream_) {
    const char* who = "a4g_rowpack_weights_i8";
    A4G_REQUIRE(N >= 0 && K >= 0 && ldwt >= K, A4G_ERR_INVALID_ARGUMENT, "%s: bad shape N=%lld K=%lld ldwt=%lld", who, (long long)N,
                (long long)K, (long long)ldwt);
    A4G_REQUIRE(K % 16 == 0 && ldwt % 16 == 0 && N <= (1 << 24) && K <= (1 << 24) && rowpacked_bytes(N, K) < (int64_t{1} << 31),
                A4G_ERR_UNSUPPORTED, "%s: needs K %% 16 == 0, ldwt %% 16 == 0 and a result below 2 GiB (N=%lld K=%lld ldwt=%lld)", who,
                (long long)N, (long long)K, (long long)ldwt);
    if (N == 0 || K == 0) return A4G_OK;
    A4G_REQUIRE(Wt && Wf && aligned16(Wt) && aligned16(Wf), A4G_ERR_INVALID_ARGUMENT, "%s: null or misaligned pointer", who);
    const int64_t chunks = rowpacked_bytes(N, K) / 16;
    const int grid = static_cast<int>(std::min<int64_t>((chunks + 255) / 256, 2048));
    rowpack_kernel<<<grid, 256, 0, static_cast<hipStream_t>(stream_)>>>(Wt, ldwt, static_cast<int>(N), static_cast<int>(K),
                                                                        reinterpret_cast<v4i*>(Wf));
    return check_hip(hipGetLastError(), who);
}

extern "C" int a4g_dense_add_layernorm_i8(const void* A, int a_kind, int64_t lda, const int8_t* Wf, const int32_t* colsum,
                                          const int32_t* bias, int shift, int dense_round_mode, int relu, const int8_t* residual,
                                          int64_t ld_res, const int16_t* gamma, const int16_t* beta, int8_t* out, int64_t ld_out,
                                          int64_t M, int64_t N, int64_t K, int32_t eps_q0, int gamma_shift, int out_shift,
                                          int ln_round_mode, a4g_stream_t stream_) {
    const char* who = "a4g_dense_add_layernorm_i8";
    A4G_REQUIRE(M >= 0 && N >= 1 && K >= 1, A4G_ERR_INVALID_ARGUMENT, "%s: bad shape M=%lld N=%lld K=%lld", who, (long long)M,
                (long long)N, (long long)K);
    A4G_REQUIRE(a_kind == A4G_I8 || a_kind == A4G_U8, A4G_ERR_UNSUPPORTED, "%s: activations of kind %d", who, a_kind);
    A4G_REQUIRE(shift >= 0 && shift <= 31, A4G_ERR_INVALID_ARGUMENT, "%s: shift %d outside [0,31]", who, shift);
    A4G_REQUIRE(valid_round(dense_round_mode) && valid_round(ln_round_mode), A4G_ERR_INVALID_ARGUMENT, "%s: unknown rounding mode", who);
    A4G_REQUIRE(eps_q0 >= 1 && eps_q0 <= (1 << 30), A4G_ERR_INVALID_ARGUMENT,
                "%s: eps_q0 must be positive (integer LayerNorm requires a positive variance floor), got %d", who, eps_q0);
    A4G_REQUIRE(out_shift >= 0 && out_shift <= 15, A4G_ERR_INVALID_ARGUMENT, "%s: out_shift=%d must be in [0, 15]", who, out_shift);
    A4G_REQUIRE(gamma_shift >= 0 && gamma_shift <= 15, A4G_ERR_INVALID_ARGUMENT, "%s: gamma_shift=%d must be in [0, 15]", who,
                gamma_shift);
    A4G_REQUIRE(lda >= K && ld_out >= N && (!residual || ld_res >= N), A4G_ERR_INVALID_ARGUMENT, "%s: pitch smaller than the row", who);
    A4G_REQUIRE(N % 32 == 0 && N <= RL_MAX_N && K % 128 == 0 && K <= RL_MAX_K, A4G_ERR_UNSUPPORTED,
                "%s: needs N %% 32 == 0, N <= %d, K %% 128 == 0, K <= %d (N=%lld K=%lld); run a4g_dense_i8 and a4g_add_layernorm_i8",
                who, RL_MAX_N, RL_MAX_K, (long long)N, (long long)K);
    A4G_REQUIRE(lda % 16 == 0 && ld_out % 16 == 0 && (!residual || ld_res % 16 == 0) && (M + 64) * lda < (int64_t{1} << 31) &&
                    (!residual || (M + 64) * ld_res < (int64_t{1} << 31)),
                A4G_ERR_UNSUPPORTED, "%s: row pitches must be multiples of 16, activations and residual smaller than 2 GiB", who);
    if (M == 0) return A4G_OK;
    A4G_REQUIRE(A && Wf && gamma && beta && out, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    A4G_REQUIRE(a_kind != A4G_U8 || colsum, A4G_ERR_INVALID_ARGUMENT, "%s: uint8 activations need colsum", who);
    A4G_REQUIRE(aligned16(A) && aligned16(Wf) && aligned16(out) && aligned16(gamma) && aligned16(beta) && (!residual || aligned16(residual)) &&
                    (!bias || aligned16(bias)) && (!colsum || aligned16(colsum)),
                A4G_ERR_UNSUPPORTED, "%s: operands must be 16-byte aligned", who);

    RowLnArgs g{};
    g.A = static_cast<const int8_t*>(A);
    g.Wf = Wf;
    g.bias = bias;
    g.colsum = colsum;
    g.res = residual;
    g.gamma = gamma;
    g.beta = beta;
    g.out = out;
    g.lda = static_cast<int>(lda);
    g.ld_res = static_cast<int>(ld_res);
    g.ld_out = static_cast<int>(ld_out);
    g.M = static_cast<int>(M);
    g.N = static_cast<int>(N);
    g.K = static_cast<int>(K);
    g.a_unsigned = a_kind == A4G_U8;
    const int blocks = static_cast<int>(N / 32);
    g.bpw = (blocks + RL_WAVES - 1) / RL_WAVES;
    g.a_bytes = static_cast<int>((M - 1) * lda + K);
    g.w_bytes = static_cast<int>(N * K);
    g.res_bytes = residual ? static_cast<int>((M - 1) * ld_res + N) : 0;
    g.lo = relu ? 0 : -128;
    g.hi = 127;
    g.quick = shift <= 22;
    g.dq = make_byte_requant(make_fast_round(dense_round_mode, std::min(shift, 22)), g.lo, g.hi);
    g.drc = make_round(dense_round_mode, shift);
    g.log2c = -1;
    if ((N & (N - 1)) == 0) {
        g.log2c = 0;
        while ((int64_t{1} << g.log2c) < N) ++g.log2c;
    }
    g.eps_q0 = eps_q0;
    g.ln_mode = ln_round_mode;
    g.gamma_shift = gamma_shift;
    g.final_shift = 15 - out_shift;
    int fr = -1;
    g.lf = make_ln_float(ln_round_mode, gamma_shift, g.final_shift, &fr);
    g.ln_rg = make_fast_round(ln_round_mode, gamma_shift);
    g.ln_ro = make_fast_round(ln_round_mode, g.final_shift);

    hipStream_t stream = static_cast<hipStream_t>(stream_);
    // 64 rows per workgroup halve the weight traffic and double the epilogue's arithmetic per CU: taken when the
    // activations fit LDS and there are still enough workgroups for every CU (with 8192 rows, 128 workgroups of 64 rows
    // measured 20.9 us against 16.2 us for 256 of 32)
    // ... and also as soon as workgroups of 32 rows would need a second round on 256 CUs: 9216 / 12 288 rows measured
    // 23.3 / 24.2 us in two rounds of 32-row workgroups
    const bool two = K <= RL_MAX_K2 && (M + 31) / 32 > 256;
    const hipError_t e = two ? launch_rowln_rb<2>(g, fr, stream) : launch_rowln_rb<1>(g, fr, stream);
    return check_hip(e, who);
}
