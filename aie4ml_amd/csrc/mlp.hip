// Fused multi-layer perceptron: a chain of Dense(+ReLU) layers in ONE launch, every weight matrix
// resident in LDS, activations never leaving the CU. Same arithmetic, layer by layer, as the Dense
// kernel (dense_bias_relu.cpp:112-163): acc32 = bias + sum a*w; srs; ReLU.
//
// A workgroup of 256 threads owns 64 (or, for small batches, 16) samples. A lane works on one sample
// and four output neurons at a time; weights are read from LDS as (mostly) wave-uniform dwords,
// activations as per-lane dwords from a padded LDS row, and four MACs retire per v_dot4_i32_i8.
// uint8 activations are biased to int8 with x ^ 0x80 and corrected by 128 * colsum.
#include <type_traits>

#include "common.hpp"
#include "layernorm_common.hpp"

namespace a4g {

constexpr int MLP_MAX_LAYERS = 8;
constexpr int MLP_MAX_WIDTH = 256;
constexpr int MLP_ACT_PITCH = MLP_MAX_WIDTH + 4;     // bytes; 65 dwords -> conflict-free lane stride
constexpr int MLP_MAX_WEIGHT_BYTES = 96 * 1024;

struct MlpLayerDev {
    const int8_t* wt;
    const int32_t* colsum;
    const int32_t* bias;
    int ldwt;  // bytes per packed weight row (multiple of 16)
    int K, N;
    int shift, relu, out_kind;
    int w_off;  // byte offset of this layer's weights in LDS
    int b_off;  // byte offset of this layer's effective bias (int32 per neuron) in LDS
};

struct MlpArgs {
    MlpLayerDev layer[MLP_MAX_LAYERS];
    int n_layers;
    const int8_t* X;
    void* Y;
    int64_t ldx, ldy;
    int batch;
    int x_unsigned;
    int mode;
    int weight_bytes;
    int total_chunks;  // 16-byte chunks of packed weights over all layers
};

// SPW = samples per workgroup (64 or 16). A wave holds SPW samples x 64/SPW neuron slots: lane l works on
// sample l % SPW and, in each pass, on four neurons of its slot. Small batches use SPW = 16 so that the
// work spreads over four times as many CUs and each wave's serial chain is four times shorter.
template <int SPW>
__global__ __launch_bounds__(256) void mlp_fused_kernel(MlpArgs a) {
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];
    int8_t* sW = smem;
    int8_t* sAct0 = smem + a.weight_bytes;
    int8_t* sAct1 = sAct0 + SPW * MLP_ACT_PITCH;
    constexpr int SLOTS = 64 / SPW;   // neuron slots per wave
    constexpr int NPW = 4 * SLOTS;    // neurons in flight per workgroup and pass step

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int smp = lane % SPW, slot = lane / SPW;

    // Stage every layer's weights (16-byte chunks, LDS image = concatenation in layer order) and the
    // per-neuron accumulator start value: bias, plus 128 * column sum when the layer's input is uint8.
    // All global loads of a batch of chunks are issued before the first LDS store.
    for (int c0 = tid; c0 < a.total_chunks; c0 += 256 * 4) {
        v4i r[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = c0 + 256 * j;
            r[j] = v4i{0, 0, 0, 0};
            if (c < a.total_chunks) {
                int l = 0;
                while (l + 1 < a.n_layers && c * 16 >= a.layer[l + 1].w_off) ++l;
                r[j] = *reinterpret_cast<const v4i*>(a.layer[l].wt + (static_cast<int64_t>(c) * 16 - a.layer[l].w_off));
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int c = c0 + 256 * j;
            if (c < a.total_chunks) *reinterpret_cast<v4i*>(sW + c * 16) = r[j];
        }
    }
    {
        int in_u = a.x_unsigned;
        for (int l = 0; l < a.n_layers; ++l) {
            const MlpLayerDev& L = a.layer[l];
            int* sb = reinterpret_cast<int*>(sW + L.b_off);
            for (int n = tid; n < L.N; n += 256) {
                int b = L.bias ? L.bias[n] : 0;
                if (in_u) b += 128 * L.colsum[n];
                sb[n] = b;
            }
            in_u = L.out_kind == A4G_U8;
        }
    }

    const int K0 = a.layer[0].K, K0p = a.layer[0].ldwt;
    const bool vec_in = (K0 & 15) == 0 && (a.ldx & 15) == 0 && (reinterpret_cast<uintptr_t>(a.X) & 15) == 0;
    for (int s0 = blockIdx.x * SPW; s0 < a.batch; s0 += gridDim.x * SPW) {
        // input rows -> LDS, zero padded to the first layer's packed K
        __syncthreads();
        if (vec_in) {
            const int cpr = K0 >> 4;  // 16-byte chunks per row
            for (int i = tid; i < SPW * cpr; i += 256) {
                const int s = i / cpr, c = i % cpr;
                v4i v{0, 0, 0, 0};
                if (s0 + s < a.batch) v = *reinterpret_cast<const v4i*>(a.X + static_cast<int64_t>(s0 + s) * a.ldx + c * 16);
                int* d = reinterpret_cast<int*>(sAct0 + s * MLP_ACT_PITCH + c * 16);  // pitch is 4-byte aligned only
                d[0] = v[0]; d[1] = v[1]; d[2] = v[2]; d[3] = v[3];
            }
        } else {
            for (int i = tid; i < SPW * K0p; i += 256) {
                const int s = i / K0p, k = i % K0p;
                int8_t v = 0;
                if (k < K0 && s0 + s < a.batch) v = a.X[static_cast<int64_t>(s0 + s) * a.ldx + k];
                sAct0[s * MLP_ACT_PITCH + k] = v;
            }
        }
        __syncthreads();

        int8_t* in = sAct0;
        int8_t* out = sAct1;
        int in_unsigned = a.x_unsigned;
        for (int l = 0; l < a.n_layers; ++l) {
            const MlpLayerDev& L = a.layer[l];
            const bool last = l + 1 == a.n_layers;
            const int k4n = L.ldwt / 4;
            const int lo = L.relu ? max(kind_lo(L.out_kind), 0) : kind_lo(L.out_kind), hi = kind_hi(L.out_kind);
            const RoundCfg rc = make_round(a.mode, L.shift);
            const int xm = in_unsigned ? static_cast<int>(0x80808080u) : 0;
            const int* arow = reinterpret_cast<const int*>(in + smp * MLP_ACT_PITCH);
            const int next_kp = last ? 0 : a.layer[l + 1].ldwt;
            const int* sb = reinterpret_cast<const int*>(sW + L.b_off);
            // four neurons per lane and pass: one activation read feeds four dot products
            for (int n0 = wave * SLOTS + slot; n0 < L.N; n0 += 4 * NPW) {
                int acc[4];
                const int* wrow[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int n = min(n0 + NPW * j, L.N - 1);
                    wrow[j] = reinterpret_cast<const int*>(sW + L.w_off + n * L.ldwt);
                    acc[j] = sb[n];
                }
#pragma unroll 4
                for (int k4 = 0; k4 < k4n; ++k4) {
                    const int av = arow[k4] ^ xm;
#pragma unroll
                    for (int j = 0; j < 4; ++j) acc[j] = __builtin_amdgcn_sdot4(av, wrow[j][k4], acc[j], false);
                }
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int n = n0 + NPW * j;
                    if (n >= L.N) break;
                    const int y = clamp_i(apply_round(acc[j], rc), lo, hi);
                    if (last) {
                        if (s0 + smp < a.batch) {
                            if (L.out_kind == A4G_I16)
                                static_cast<int16_t*>(a.Y)[static_cast<int64_t>(s0 + smp) * a.ldy + n] = static_cast<int16_t>(y);
                            else
                                static_cast<int8_t*>(a.Y)[static_cast<int64_t>(s0 + smp) * a.ldy + n] = static_cast<int8_t>(y);
                        }
                    } else {
                        out[smp * MLP_ACT_PITCH + n] = static_cast<int8_t>(y);
                    }
                }
            }
            if (!last) {
                // zero the padding columns the next layer's dot products will touch
                for (int n = L.N + wave * SLOTS + slot; n < next_kp; n += NPW) out[smp * MLP_ACT_PITCH + n] = 0;
                __syncthreads();
                int8_t* t = in;
                in = out;
                out = t;
                in_unsigned = L.out_kind == A4G_U8;
            }
        }
    }
}


// =====================================================================================================
// The same chain on the matrix units, for batches large enough to be bound by arithmetic.
// =====================================================================================================
// A wave owns 32 samples at a time. Layer l computes, per block of 32 neurons, one 32x32x32 MFMA per 32 inputs with the
// weights as the first operand and the activations as the second: lane (m, half) supplies bytes [16 half, 16 half + 16)
// of sample m's 32 inputs, and receives 16 accumulators of sample m. The weight rows are handed over in the order
// direct_col_of_operand_row, which makes those 16 accumulators the neurons 32 nb + 16 half + 0..15 - requantised and
// packed they are exactly the lane's operand bytes for K step nb of the next layer, so the activations of a sample never
// leave the lane's registers between the first load and the last store. Weight fragments (1 KiB per 32 neurons x 32
// inputs, zero padded) and the accumulators' start values (bias + 128 * column sum for uint8 inputs) are staged in LDS
// once per workgroup.
struct MlpMfmaLayer {
    const int8_t* wt;
    const int32_t* colsum;
    const int32_t* bias;
    int ldwt, K, N;
    int Kb, Nb;   // blocks of 32 inputs / neurons
    int frag0;    // first fragment of the layer in LDS
    int start0;   // first start value of the layer (int32 index)
    int in_unsigned, out_kind;
    int quick;    // the shift allows the requantisation that clamps in front of the shift
    int fold;     // its rounding constant, added to the start values once instead of to every accumulator
    int lo, hi;
    ByteRequant dq;
    RoundCfg drc;
};

struct MlpMfmaArgs {
    MlpMfmaLayer layer[MLP_MAX_LAYERS];
    int n_layers;
    const int8_t* X;
    void* Y;
    int ldx, ldy;
    int batch;
    int x_bytes;      // bytes the launch may read from X on
    int x_aligned;    // rows start at multiples of 16 bytes
    int x_delta;      // else: X points to the dword below the first row, which starts this many bytes in
    int y_bytes;      // bytes of Y it may write
    int nfrag, nstart;
    int y_vec;        // rows of Y can be stored as 16-byte pieces
    int y_packed;     // at most 32 outputs in rows without gaps, Y 4-byte aligned: the tile store
    int y_magic;      // ceil(65536 / N): (j * y_magic) >> 16 == j / N for every j < 32 N
    // the form that adds a residual to the last layer's int8 result and normalises the row (LN kernels only)
    const int8_t* res;    // [batch][ld_res] int8, or null
    const int16_t* gamma; // [N] Q7
    const int16_t* beta;  // [N] Q15
    int ld_res, res_bytes;
    int ln_off;           // byte offset in LDS of gamma then beta widened to int32 (2 x 4 N bytes)
    int log2c, eps_q0;
    FastRound ln_rg, ln_ro;  // the two requantisations of the normalisation (gamma scale, output)
};

constexpr int64_t MLP_MFMA_MIN_BATCH = 512;

// MAXB: blocks of 32 that the widest layer has (2, 4 or 8: the loops over blocks are unrolled that far and guarded).
// BIT: what the rounding mode adds besides its constant (fast_round_kind: 0 nothing, 1 a bit of the accumulator,
// 2 minus that bit).
// YVEC: the result's rows can be stored as 16-byte pieces.
// LN: out = LayerNorm(saturate_i8(last layer + residual)) instead of the last layer's bytes (int8 result, N a multiple of
// 16, YVEC): a sample's row lies in the two lanes m and m + 32, so its sums are an in-lane sum and one exchange.
template <int MAXB, int BIT, bool YVEC, bool LN = false>
__global__ __launch_bounds__(1024) void mlp_mfma_kernel(MlpMfmaArgs a) {
    constexpr int MLP_MFMA_BLOCKS = MAXB;
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];
    int8_t* const frag = smem;
    int* const start = reinterpret_cast<int*>(smem + a.nfrag * 1024);
    int* const big = start + a.nstart;  // per layer: a start value too large for the quick requantisation
    const int tid = threadIdx.x, lane = tid & 63;
    const int m = lane & 31, half = lane >> 5;
    const int nthreads = blockDim.x;  // four to sixteen waves: as many as it takes to have sixteen on the CU
    int8_t* const zero_frag = frag + (a.nfrag - 1) * 1024;  // the last fragment is all zeros

    const auto rsrc_x = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.X), 0, a.x_bytes, 0x00020000);
    const int units = (a.batch + 31) >> 5;
    const int wpb = nthreads >> 6;
    const int nwaves = gridDim.x * wpb;
    const int Kb0 = a.layer[0].Kb;
    const int xm0 = a.layer[0].in_unsigned ? static_cast<int>(0x80808080u) : 0;
    // A sample's input bytes, one 16-byte piece per 32 inputs and lane; a piece the first layer does not have, and a
    // sample past the end of the batch, lie beyond the descriptor and read as zero, so that no load sits in a branch
    // and all of a unit's pieces are in flight together. Bytes past the row's end meet zero weights.
    const auto rsrc_y = __builtin_amdgcn_make_buffer_rsrc(static_cast<int8_t*>(a.Y), 0, a.y_bytes, 0x00020000);
    const int last_n = a.layer[a.n_layers - 1].N;
    // the packed store's tile, and where in it the four bytes of the lane's dwords come from (row * 32 + column of byte
    // j = 4 * dword + b of the unit's 32 N bytes; three 10-bit addresses in one register, the fourth in another)
    uint8_t* const tile = reinterpret_cast<uint8_t*>(big + MLP_MAX_LAYERS) + (tid >> 6) * 1024;
    unsigned tsrc[4] = {0, 0, 0, 0}, tsrc2[4] = {0, 0, 0, 0};
    if (!YVEC && a.y_packed) {
#pragma unroll
        for (int sl = 0; sl < 4; ++sl) {
            unsigned at[4];
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const int j = min((sl * 64 + lane) * 4 + b, 32 * last_n - 1);
                const int r = (j * a.y_magic) >> 16;  // j / last_n for j < 1024 (checked on the host for this N)
                at[b] = static_cast<unsigned>(r * 32 + (j - r * last_n));
            }
            tsrc[sl] = at[0] | (at[1] << 10) | (at[2] << 20);
            tsrc2[sl] = at[3];
        }
    }
    // Narrow chains request the next unit's input before this unit's layers (and stores); the wide ones have no
    // registers to spare for that (it cost them 10 %).
    constexpr bool AHEAD = MAXB <= 2;
    v4i nact[AHEAD ? MLP_MFMA_BLOCKS : 1];
    auto fetch = [&](int unit, v4i* dst) {
        const int r = unit * 32 + m;
        if (a.x_aligned) {
#pragma unroll
            for (int ks = 0; ks < MLP_MFMA_BLOCKS; ++ks)
                dst[ks] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                                                      rsrc_x, (ks < Kb0 && r < a.batch) ? r * a.ldx + ks * 32 + half * 16 : 0x7ffffff0, 0, 0));
        } else {
            // Rows at any address (57 inputs, a window of a wider matrix): the piece is cut out of the five dwords that
            // cover it. The descriptor starts at the dword below X (x_delta bytes), so every load is dword-aligned.
#pragma unroll
            for (int ks = 0; ks < MLP_MFMA_BLOCKS; ++ks) {
                const unsigned at = static_cast<unsigned>(r * a.ldx + ks * 32 + half * 16 + a.x_delta);
                const bool there = ks < Kb0 && r < a.batch;
                const unsigned sh = at & 3u;
                const v4i w = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_x, there ? (at & ~3u) : 0x7ffffff0u, 0, 0));
                const int w4 = static_cast<int>(__builtin_amdgcn_raw_buffer_load_b32(rsrc_x, there ? (at & ~3u) + 16u : 0x7ffffff0u, 0, 0));
                dst[ks][0] = static_cast<int>(__builtin_amdgcn_alignbyte(w[1], w[0], sh));
                dst[ks][1] = static_cast<int>(__builtin_amdgcn_alignbyte(w[2], w[1], sh));
                dst[ks][2] = static_cast<int>(__builtin_amdgcn_alignbyte(w[3], w[2], sh));
                dst[ks][3] = static_cast<int>(__builtin_amdgcn_alignbyte(w4, w[3], sh));
            }
        }
    };
    const int u0 = blockIdx.x * wpb + __builtin_amdgcn_readfirstlane(tid >> 6);
    if (AHEAD) fetch(u0, nact);  // the first unit's input travels while the fragments are staged

    int* const gamma_lds = reinterpret_cast<int*>(smem + a.ln_off);
    int* const beta_lds = gamma_lds + (LN ? a.layer[a.n_layers - 1].N : 0);
    if (LN) {
        const int n_ln = a.layer[a.n_layers - 1].N;
        for (int c = tid; c < n_ln; c += nthreads) {
            gamma_lds[c] = a.gamma[c];
            beta_lds[c] = a.beta[c];
        }
    }
    if (tid < MLP_MAX_LAYERS) big[tid] = 0;
    if (tid < 64) *reinterpret_cast<v4i*>(zero_frag + tid * 16) = v4i{0, 0, 0, 0};
    __syncthreads();
    for (int l = 0; l < a.n_layers; ++l) {
        const MlpMfmaLayer& L = a.layer[l];
        // Fragments, one 16-byte piece at a time per thread; where a layer has four rounds of pieces or more, four are
        // fetched together (a few round trips to L2 instead of one per piece). A piece that does not exist lies past the descriptor and reads as zero.
        const int pieces = L.Nb * L.Kb * 64;
        const int Kb_l = L.Kb, N_l = L.N, K_l = L.K, ldwt_l = L.ldwt, frag0_l = L.frag0;
        const auto rsrc_w = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(L.wt), 0, N_l * ldwt_l, 0x00020000);
        auto piece_from = [&](int p) -> int {  // byte offset of piece p in the packed weights, or nowhere
            const int f = p >> 6, ln = p & 63;
            const int nb = f / Kb_l, ks = f - nb * Kb_l;
            const int col = nb * 32 + direct_col_of_operand_row(ln & 31);
            const int k0 = ks * 32 + (ln >> 5) * 16;
            return (p < pieces && col < N_l && k0 < K_l) ? col * ldwt_l + k0 : 0x7ffffff0;
        };
        auto piece_store = [&](int p, v4i w) {
            const int f = p >> 6, ln = p & 63;
            const int k0 = (f - (f / Kb_l) * Kb_l) * 32 + (ln >> 5) * 16;
#pragma unroll
            for (int q = 0; q < 4; ++q) {  // inputs past K count nothing, whatever the packed rows hold there
                const int left = K_l - (k0 + 4 * q);
                if (left <= 0) w[q] = 0;
                else if (left < 4) w[q] &= static_cast<int>((1u << (8 * left)) - 1u);
            }
            if (p < pieces) *reinterpret_cast<v4i*>(frag + (frag0_l + f) * 1024 + ln * 16) = w;
        };
        int p = tid;
        for (; p - tid + 4 * nthreads <= pieces; p += 4 * nthreads) {  // (uniform: four whole rounds are left)
            v4i w[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) w[j] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, piece_from(p + j * nthreads), 0, 0));
#pragma unroll
            for (int j = 0; j < 4; ++j) piece_store(p + j * nthreads, w[j]);
        }
        for (; p < pieces; p += nthreads)
            piece_store(p, __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_w, piece_from(p), 0, 0)));
        for (int c = tid; c < L.Nb * 32; c += nthreads) {
            unsigned sv = 0;  // wraps like the int32 sum it stands for
            if (c < L.N) {
                if (L.bias) sv = static_cast<unsigned>(L.bias[c]);
                if (L.in_unsigned) sv += 128u * static_cast<unsigned>(L.colsum[c]);
            }
            const int sval = static_cast<int>(sv);
            start[L.start0 + c] = static_cast<int>(sv + static_cast<unsigned>(L.fold));
            if (sval > (1 << 30) || sval < -(1 << 30)) big[l] = 1;  // every writer writes the same value
        }
    }
    __syncthreads();

    for (int u = u0; u < units; u += nwaves) {
        const int row = u * 32 + m;
        const bool row_ok = row < a.batch;
        v4i act[MLP_MFMA_BLOCKS];
        if (AHEAD) {
#pragma unroll
            for (int ks = 0; ks < MLP_MFMA_BLOCKS; ++ks) act[ks] = nact[ks] ^ xm0;
            __builtin_amdgcn_sched_barrier(0);
            fetch(u + nwaves, nact);  // past the end: zeros, unused
        } else {
            fetch(u, act);
#pragma unroll
            for (int ks = 0; ks < MLP_MFMA_BLOCKS; ++ks) act[ks] ^= xm0;
        }
        // The residual's pieces are requested here, a whole chain ahead of their use, where the registers allow it: a unit
        // is one wave's work from end to end, and a load that starts after the last layer is waited for in full.
        constexpr bool RES_AHEAD = LN && MAXB <= 4;
        const auto rsrc_res = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.res), 0, (LN && a.res) ? a.res_bytes : 0, 0x00020000);
        auto residual_piece = [&](int nb) __attribute__((always_inline)) {
            const int col0 = nb * 32 + 16 * half;
            return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(
                                               rsrc_res, (row_ok && col0 < last_n) ? row * a.ld_res + col0 : 0x7ffffff0, 0, 0));
        };
        v4i rw_ahead[RES_AHEAD ? MLP_MFMA_BLOCKS : 1];
        if (RES_AHEAD) {
#pragma unroll
            for (int nb = 0; nb < MLP_MFMA_BLOCKS; ++nb) rw_ahead[nb] = residual_piece(nb);
        }
        for (int l = 0; l < a.n_layers; ++l) {
            const MlpMfmaLayer& L = a.layer[l];
            const bool last = l + 1 == a.n_layers;
            // The layer's constants live in the kernel's argument block, indexed by l: each is fetched once per layer and
            // pinned to a scalar register here (an empty asm that claims to modify it), or the compiler fetches it again
            // in every branch that uses it, with a wait each time.
            int Kb = L.Kb, Nb = L.Nb, frag0 = L.frag0, start0 = L.start0, width = L.N, okind = L.out_kind;
            int q_s = L.dq.fr.s, q_c0 = L.dq.fr.c0, q_pos = L.dq.fr.pos, q_lo = L.dq.lo_s, q_hi = L.dq.hi_s;
            int quick_l = L.quick;
            asm volatile("" : "+s"(Kb), "+s"(Nb), "+s"(frag0), "+s"(start0), "+s"(width), "+s"(okind), "+s"(quick_l));
            asm volatile("" : "+s"(q_s), "+s"(q_c0), "+s"(q_pos), "+s"(q_lo), "+s"(q_hi));
            ByteRequant dq;
            dq.fr = FastRound{q_s, q_c0, q_pos, 1, 0};
            dq.lo_s = q_lo;
            dq.hi_s = q_hi;
            const bool quick = quick_l != 0 && __builtin_amdgcn_readfirstlane(big[l]) == 0;
            v4i out[MLP_MFMA_BLOCKS];
            // one copy of the layer per form of the requantisation: the choice is made once, not per group of four values
            auto run_layer = [&](auto quick_tag) __attribute__((always_inline)) {
                constexpr bool QUICK = decltype(quick_tag)::value;
#pragma unroll
                for (int nb = 0; nb < MLP_MFMA_BLOCKS; ++nb) {
                    out[nb] = v4i{0, 0, 0, 0};
                    if (nb >= Nb) continue;
                    v16i acc;
                    {
                        const int* sp = start + start0 + nb * 32 + 16 * half;
#pragma unroll
                        for (int q = 0; q < 4; ++q) {
                            const v4i s4 = *reinterpret_cast<const v4i*>(sp + 4 * q);
#pragma unroll
                            for (int t = 0; t < 4; ++t) acc[4 * q + t] = s4[t];
                        }
                    }
                    // All MAXB fragments are requested before the first product, an absent one as the fragment of zeros (no
                    // branch between the loads: the compiler keeps them all in flight), and from four K steps on the products
                    // go to two accumulators in turn, which halves the chain of dependent MFMAs.
                    const int8_t* fp = frag + (frag0 + nb * Kb) * 1024 + lane * 16;
                    v4i wf[MLP_MFMA_BLOCKS];
#pragma unroll
                    for (int ks = 0; ks < MLP_MFMA_BLOCKS; ++ks)
                        wf[ks] = *reinterpret_cast<const v4i*>(ks < Kb ? fp + ks * 1024 : zero_frag + lane * 16);
                    if (MLP_MFMA_BLOCKS >= 4) {
                        v16i acc1 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
                        for (int ks = 0; ks < MLP_MFMA_BLOCKS; ++ks) {
                            if (ks & 1) acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[ks], act[ks], acc1, 0, 0, 0);
                            else acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[ks], act[ks], acc, 0, 0, 0);
                        }
                        acc += acc1;
                    } else {
#pragma unroll
                        for (int ks = 0; ks < MLP_MFMA_BLOCKS; ++ks) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(wf[ks], act[ks], acc, 0, 0, 0);
                    }
                    const int col0 = nb * 32 + 16 * half;
                    if (QUICK && BIT == 0) {
                        // This form's first readers of the accumulators are inline asm (v_med3), which the compiler's
                        // hazard recogniser does not look into: it would insert no wait states between the MFMA and them.
                        // One ordinary vector instruction reads the accumulator first (an identity DPP move, which gets
                        // the wait states), and nothing is scheduled across the barrier behind it.
                        acc[15] = __builtin_amdgcn_update_dpp(0, acc[15], 0xE4, 0xF, 0xF, false);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                    v4i o;
#pragma unroll
                    for (int q = 0; q < 4; ++q) {
                        if (QUICK) {
                            if (BIT == 0) {  // the rounding constant is in the start value already: clamp, shift into place
                                unsigned packed;  // byte 0 is written with the other bytes zeroed, bytes 1..3 are merged in
                                {
                                    const int v0 = clamp_med3(acc[4 * q], dq.lo_s, dq.hi_s);
                                    asm("v_ashrrev_i32_sdwa %0, %1, %2 dst_sel:BYTE_0 dst_unused:UNUSED_PAD src0_sel:DWORD src1_sel:DWORD"
                                        : "=v"(packed)
                                        : "v"(dq.fr.s), "v"(v0));
                                }
                                shift_into_byte<1>(packed, clamp_med3(acc[4 * q + 1], dq.lo_s, dq.hi_s), dq.fr.s);
                                shift_into_byte<2>(packed, clamp_med3(acc[4 * q + 2], dq.lo_s, dq.hi_s), dq.fr.s);
                                shift_into_byte<3>(packed, clamp_med3(acc[4 * q + 3], dq.lo_s, dq.hi_s), dq.fr.s);
                                o[q] = static_cast<int>(packed);
                            } else {
                                o[q] = static_cast<int>(requant4_bytes<BIT>(acc[4 * q], acc[4 * q + 1], acc[4 * q + 2], acc[4 * q + 3], dq));
                            }
                        } else {
                            int v[4];
#pragma unroll
                            for (int t = 0; t < 4; ++t)  // the folded constant is taken out again (wrapping, like the sum itself)
                                v[t] = clamp_i(apply_round(static_cast<int>(static_cast<unsigned>(acc[4 * q + t]) - static_cast<unsigned>(L.fold)), L.drc), L.lo, L.hi);
                            o[q] = static_cast<int>(pack4_bytes(v[0], v[1], v[2], v[3]));
                        }
                    }
                    // neurons past N have zero weights and a zero start value: they requantise to zero, and meet zero weights
                    // in the next layer; a uint8 result is biased to int8 for the next MFMA (the last layer's is kept as it is)
                    out[nb] = (!last && okind == A4G_U8) ? o ^ static_cast<int>(0x80808080u) : o;
                }
            };
            if (quick) run_layer(std::true_type{});
            else run_layer(std::false_type{});
#pragma unroll
            for (int nb = 0; nb < MLP_MFMA_BLOCKS; ++nb) act[nb] = out[nb];
        }
        // The last layer's bytes, stored outside the loop over the layers and without a branch: a byte (or 16-byte piece)
        // that does not exist gets an offset past the descriptor and is dropped. The compiler then knows how many stores
        // are in flight, and the wait for the next unit's input, requested before them, does not include their
        // acknowledgement.
        if (LN) {
            int sx = 0, sq = 0;
#pragma unroll
            for (int nb = 0; nb < MLP_MFMA_BLOCKS; ++nb) {
                const int col0 = nb * 32 + 16 * half;
                const bool there = col0 < last_n;  // N % 16 == 0: a piece of 16 columns exists as a whole or not at all
                const v4i rw = RES_AHEAD ? rw_ahead[RES_AHEAD ? nb : 0] : residual_piece(nb);
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    unsigned y = static_cast<unsigned>(act[nb][q]);
                    if (a.res) y = sat_add_i8x4(y, static_cast<unsigned>(rw[q]));
                    if (!there) y = 0;
                    act[nb][q] = static_cast<int>(y);
                    sx = __builtin_amdgcn_sdot4(static_cast<int>(y), 0x01010101, sx, false);
                    sq = __builtin_amdgcn_sdot4(static_cast<int>(y), static_cast<int>(y), sq, false);
                }
            }
            sx += __shfl_xor(sx, 32);
            sq += __shfl_xor(sq, 32);
            const RowStats st = row_stats(sx, sq, last_n, a.log2c, a.eps_q0);
#pragma unroll
            for (int nb = 0; nb < MLP_MFMA_BLOCKS; ++nb) {
                const int col0 = nb * 32 + 16 * half;
                if (nb * 32 >= last_n) continue;  // (uniform)
                const int cj = col0 < last_n ? col0 : 0;
                v4i o;
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const v4i g4 = *reinterpret_cast<const v4i*>(gamma_lds + cj + 4 * q);
                    const v4i b4 = *reinterpret_cast<const v4i*>(beta_lds + cj + 4 * q);
                    int y4[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int vd = sext8(static_cast<unsigned>(act[nb][q]), t) - st.mu;
                        // (both within fast_round's range: |inv * gamma| < 2^30, |vd * fs| < 2^23)
                        const int fs = clamp_i(fast_round(__mul24(st.inv, g4[t]), a.ln_rg), -32768, 32767);
                        y4[t] = clamp_i(fast_round(__mul24(vd, fs) + b4[t], a.ln_ro), -128, 127);
                    }
                    o[q] = static_cast<int>(pack4_bytes(y4[0], y4[1], y4[2], y4[3]));
                }
                act[nb] = o;
            }
        }
        if (!YVEC && a.y_packed && u * 32 + 32 <= a.batch) {
            // At most 32 neurons in rows that follow each other without a gap (a classifier's few outputs): the unit's
            // 32 rows are 32 N consecutive bytes. They go through a 1 KiB tile of the wave's own (no barrier: a wave's
            // LDS operations complete in order) and leave as whole dwords, instead of N byte stores per lane.
            *reinterpret_cast<v4i*>(tile + m * 32 + 16 * half) = act[0];
            const unsigned ubase = static_cast<unsigned>(u) * 32u * static_cast<unsigned>(last_n);
#pragma unroll
            for (int sl = 0; sl < 4; ++sl) {
                if (sl * 256 < 32 * last_n) {
                    const unsigned word = static_cast<unsigned>(tile[tsrc[sl] & 0x3ff]) | (static_cast<unsigned>(tile[(tsrc[sl] >> 10) & 0x3ff]) << 8) |
                                          (static_cast<unsigned>(tile[(tsrc[sl] >> 20) & 0x3ff]) << 16) |
                                          (static_cast<unsigned>(tile[tsrc2[sl]]) << 24);
                    __builtin_amdgcn_raw_buffer_store_b32(word, rsrc_y, (sl * 64 + lane) * 4 < 32 * last_n ? ubase + (sl * 64 + lane) * 4 : 0x7ffffff0u, 0, 0);
                }
            }
        } else {
            typedef unsigned v4u __attribute__((ext_vector_type(4)));
#pragma unroll
            for (int nb = 0; nb < MLP_MFMA_BLOCKS; ++nb) {
                const int col0 = nb * 32 + 16 * half;
                if (nb * 32 >= last_n) continue;  // (uniform)
                const unsigned y0 = static_cast<unsigned>(row) * static_cast<unsigned>(a.ldy) + col0;
                if (YVEC) {  // N % 16 == 0, rows 16-byte aligned
                    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, act[nb]), rsrc_y,
                                                           (row_ok && col0 < last_n) ? y0 : 0x7ffffff0u, 0, 0);
                } else {
#pragma unroll
                    for (int t = 0; t < 16; ++t)
                        __builtin_amdgcn_raw_buffer_store_b8(static_cast<unsigned char>(static_cast<unsigned>(act[nb][t >> 2]) >> (8 * (t & 3))),
                                                             rsrc_y, (row_ok && col0 + t < last_n) ? y0 + t : 0x7ffffff0u, 0, 0);
                }
            }
        }
    }
}

template <int MAXB, int BIT, bool YVEC, bool LN>
static hipError_t launch_mlp_mfma(int grid, int threads, size_t lds, hipStream_t stream, const MlpMfmaArgs& f) {
    auto kern = mlp_mfma_kernel<MAXB, BIT, YVEC, LN>;
    static bool attr_set = false;  // benign race: the attribute is idempotent
    if (!attr_set) {
        const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                                 144 * 1024);
        if (e != hipSuccess) return e;
        attr_set = true;
    }
    kern<<<grid, threads, lds, stream>>>(f);
    return hipGetLastError();
}

}  // namespace a4g

using namespace a4g;

namespace {
struct MlpLnExtra {  // what a4g_mlp_add_layernorm_i8 has beyond a4g_mlp_i8
    const int8_t* res;
    int64_t ld_res;
    const int16_t* gamma;
    const int16_t* beta;
    int eps_q0, gamma_shift, out_shift, ln_mode;
};
}  // namespace

static int mlp_entry(const a4g_mlp_layer* layers, int n_layers, const void* X, int x_kind, int64_t ldx, void* Y, int64_t ldy,
                     int64_t batch, int round_mode, const MlpLnExtra* ln, a4g_stream_t stream_, const char* who) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    A4G_REQUIRE(layers && n_layers >= 1, A4G_ERR_INVALID_ARGUMENT, "%s: no layers", who);
    A4G_REQUIRE(n_layers <= MLP_MAX_LAYERS, A4G_ERR_UNSUPPORTED, "%s: %d layers exceed the fused limit of %d", who, n_layers,
                MLP_MAX_LAYERS);
    A4G_REQUIRE(x_kind == A4G_I8 || x_kind == A4G_U8, A4G_ERR_UNSUPPORTED, "%s: input must be int8 or uint8", who);
    A4G_REQUIRE(valid_round(round_mode), A4G_ERR_INVALID_ARGUMENT, "%s: unknown rounding mode %d", who, round_mode);
    A4G_REQUIRE(batch >= 0 && batch <= INT32_MAX, A4G_ERR_INVALID_ARGUMENT, "%s: bad batch %lld", who, (long long)batch);

    MlpArgs a{};
    int off = 0;
    int in_kind = x_kind;
    for (int l = 0; l < n_layers; ++l) {
        const a4g_mlp_layer& s = layers[l];
        A4G_REQUIRE(s.K >= 1 && s.N >= 1, A4G_ERR_INVALID_ARGUMENT, "%s: layer %d has an empty shape", who, l);
        A4G_REQUIRE(s.K <= MLP_MAX_WIDTH && s.N <= MLP_MAX_WIDTH, A4G_ERR_UNSUPPORTED,
                    "%s: layer %d is %dx%d, wider than the fused limit of %d", who, l, s.K, s.N, MLP_MAX_WIDTH);
        A4G_REQUIRE(l == 0 || layers[l - 1].N == s.K, A4G_ERR_INVALID_ARGUMENT, "%s: layer %d input width %d != previous output %d",
                    who, l, s.K, l ? layers[l - 1].N : 0);
        A4G_REQUIRE(s.wt && aligned16(s.wt) && s.ldwt == a4g_packed_ld(s.K), A4G_ERR_INVALID_ARGUMENT,
                    "%s: layer %d weights must come from a4g_pack_weights_i8 (pitch %lld)", who, l,
                    (long long)a4g_packed_ld(s.K));
        A4G_REQUIRE(s.shift >= 0 && s.shift <= 31, A4G_ERR_INVALID_ARGUMENT,
                    "%s: layer %d accumulator output shift must be in [0,31], got %d", who, l, s.shift);
        const bool last = l + 1 == n_layers;
        A4G_REQUIRE(s.out_kind == A4G_I8 || s.out_kind == A4G_U8 || (last && s.out_kind == A4G_I16), A4G_ERR_UNSUPPORTED,
                    "%s: layer %d output kind %d unsupported", who, l, s.out_kind);
        A4G_REQUIRE(in_kind != A4G_U8 || s.colsum, A4G_ERR_INVALID_ARGUMENT, "%s: layer %d has uint8 input but no colsum", who, l);
        MlpLayerDev& d = a.layer[l];
        d.wt = s.wt;
        d.colsum = s.colsum;
        d.bias = s.bias;
        d.ldwt = static_cast<int>(s.ldwt);
        d.K = s.K;
        d.N = s.N;
        d.shift = s.shift;
        d.relu = s.relu != 0;
        d.out_kind = s.out_kind;
        d.w_off = off;
        off += d.N * d.ldwt;
        in_kind = s.out_kind;
    }
    const int weights_only = off;
    for (int l = 0; l < n_layers; ++l) {
        off = (off + 15) / 16 * 16;
        a.layer[l].b_off = off;
        off += a.layer[l].N * 4;
    }
    A4G_REQUIRE(weights_only <= MLP_MAX_WEIGHT_BYTES, A4G_ERR_UNSUPPORTED,
                "%s: %d bytes of packed weights exceed the LDS budget of %d", who, weights_only, MLP_MAX_WEIGHT_BYTES);
    if (batch == 0) return A4G_OK;
    A4G_REQUIRE(X && Y, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    A4G_REQUIRE(ldx >= layers[0].K && ldy >= layers[n_layers - 1].N, A4G_ERR_INVALID_ARGUMENT, "%s: pitch smaller than the row",
                who);
    a.n_layers = n_layers;
    a.X = static_cast<const int8_t*>(X);
    a.Y = Y;
    a.ldx = ldx;
    a.ldy = ldy;
    a.batch = static_cast<int>(batch);
    a.x_unsigned = x_kind == A4G_U8;
    a.mode = round_mode;
    a.weight_bytes = (off + 15) / 16 * 16;

    a.total_chunks = weights_only / 16;

    // Large batches: the chain on the matrix units, if its fragments fit the LDS and the rows can be fetched in 16-byte
    // pieces. (Small batches are a chain of latencies either way, and the kernel below spreads 16 samples per workgroup.)
    {
        MlpMfmaArgs f{};
        int nfrag = 0, nstart = 0, in_u = x_kind == A4G_U8;
        bool ok = (ln || batch >= MLP_MFMA_MIN_BATCH) && layers[n_layers - 1].out_kind != A4G_I16 && ldx <= INT32_MAX && ldy <= INT32_MAX &&
                  (batch - 1) * ldx + layers[0].K < (int64_t{1} << 31) - 64 &&
                  ((batch - 1) * ldy + layers[n_layers - 1].N) * 2 < (int64_t{1} << 31) - 64;
        const FastRound fr1 = make_fast_round(round_mode, 1);  // the kind of bit is the same for every shift >= 1
        for (int l = 0; l < n_layers && ok; ++l) {
            const a4g_mlp_layer& s = layers[l];
            MlpMfmaLayer& d = f.layer[l];
            d.wt = s.wt;
            d.colsum = s.colsum;
            d.bias = s.bias;
            d.ldwt = static_cast<int>(s.ldwt);
            d.K = s.K;
            d.N = s.N;
            d.Kb = (s.K + 31) / 32;
            d.Nb = (s.N + 31) / 32;
            d.frag0 = nfrag;
            d.start0 = nstart;
            d.in_unsigned = in_u;
            d.out_kind = s.out_kind;
            const int klo = s.out_kind == A4G_I8 ? -128 : (s.out_kind == A4G_I16 ? -32768 : 0);
            d.lo = s.relu ? std::max(klo, 0) : klo;
            d.hi = s.out_kind == A4G_I8 ? 127 : (s.out_kind == A4G_I16 ? 32767 : 255);
            const FastRound fr = make_fast_round(round_mode, s.shift);
            // |sum| <= 256 * 2^14: no overflow below 2^30 + 2^23; a shift of 0 rounds nothing, which the kernels that add
            // a bit of the accumulator do not know
            d.quick = byte_requant_ok(fr) && s.out_kind != A4G_I16 && (s.shift >= 1 || fast_round_kind(fr1) == 0);
            // modes that add a bit of the accumulator (its sign, or the parity of the quotient) need the accumulator as it
            // is: only the others fold their constant into the start values
            d.fold = d.quick && fast_round_kind(fr1) == 0 ? fr.c0 : 0;
            d.dq = make_byte_requant(fr, d.lo, d.hi);
            d.drc = make_round(round_mode, s.shift);
            nfrag += d.Nb * d.Kb;
            nstart += d.Nb * 32;
            in_u = s.out_kind == A4G_U8;
        }
        nfrag += 1;  // the fragment of zeros that absent K steps read
        // fragments, start values, one flag per layer (and, below, a 1 KiB tile per wave for the packed store)
        const size_t lds_core = static_cast<size_t>(nfrag) * 1024 + static_cast<size_t>(nstart) * 4 + MLP_MAX_LAYERS * 4;
        if (ok && ln) {  // the normalising form: int8 rows in whole 16-column pieces, 16-byte aligned on every side
            const a4g_mlp_layer& l_ = layers[n_layers - 1];
            ok = l_.out_kind == A4G_I8 && l_.N % 16 == 0 && ldy % 16 == 0 && aligned16(Y) &&
                 (!ln->res || (aligned16(ln->res) && ln->ld_res % 16 == 0 && ln->ld_res >= l_.N &&
                               (batch - 1) * ln->ld_res + l_.N < (int64_t{1} << 31) - 64));
        }
        if (ok && lds_core + (ln ? 8 * layers[n_layers - 1].N + 16 : 0) <= 128 * 1024) {
            const a4g_mlp_layer& lastl = layers[n_layers - 1];
            f.n_layers = n_layers;
            f.x_aligned = ldx % 16 == 0 && aligned16(X);
            f.x_delta = f.x_aligned ? 0 : static_cast<int>(reinterpret_cast<uintptr_t>(X) & 3);
            f.X = static_cast<const int8_t*>(X) - f.x_delta;
            f.Y = Y;
            f.ldx = static_cast<int>(ldx);
            f.ldy = static_cast<int>(ldy);
            f.batch = static_cast<int>(batch);
            // up to the end of the dword that holds the last byte: the range check is per dword, and a dword that
            // straddles the end of the descriptor would read as zero
            f.x_bytes = (static_cast<int>((batch - 1) * ldx + layers[0].K) + f.x_delta + 3) & ~3;
            f.y_bytes = static_cast<int>(((batch - 1) * ldy + lastl.N) * (lastl.out_kind == A4G_I16 ? 2 : 1));
            f.nfrag = nfrag;
            f.nstart = nstart;
            f.y_vec = lastl.out_kind != A4G_I16 && lastl.N % 16 == 0 && ldy % 16 == 0 && aligned16(Y);
            f.y_packed = !f.y_vec && lastl.N <= 32 && ldy == lastl.N && reinterpret_cast<uintptr_t>(Y) % 4 == 0;
            f.y_magic = (65536 + lastl.N - 1) / lastl.N;
            for (int j = 0; f.y_packed && j < 32 * lastl.N; ++j)
                if (((j * f.y_magic) >> 16) != j / lastl.N) f.y_packed = 0;  // (never, for N <= 32)
            int widest = 0;
            for (int l = 0; l < n_layers; ++l) widest = std::max(widest, std::max(f.layer[l].Kb, f.layer[l].Nb));
            const int bit_kind = fast_round_kind(fr1);
            // sixteen waves per CU (32 samples per wave and turn): four workgroups of four waves where the LDS holds four
            // copies of the fragments, fewer and larger workgroups otherwise
            const size_t tile_bytes = f.y_packed ? 16 * 1024 : 0;  // per CU, however its sixteen waves are grouped
            const int per_cu = static_cast<int>(std::max<size_t>(1, std::min<size_t>(4, (160 * 1024 - tile_bytes) / lds_core)));
            const int threads = per_cu >= 4 ? 256 : (per_cu >= 2 ? 512 : 1024);
            size_t lds_f = lds_core + (f.y_packed ? static_cast<size_t>(threads / 64) * 1024 : 0);
            if (ln) {
                f.res = ln->res;
                f.gamma = ln->gamma;
                f.beta = ln->beta;
                f.ld_res = static_cast<int>(ln->ld_res);
                f.res_bytes = ln->res ? static_cast<int>((batch - 1) * ln->ld_res + lastl.N) : 0;
                f.log2c = -1;
                if ((lastl.N & (lastl.N - 1)) == 0) {
                    f.log2c = 0;
                    while ((1 << f.log2c) < lastl.N) ++f.log2c;
                }
                f.eps_q0 = ln->eps_q0;
                f.ln_rg = make_fast_round(ln->ln_mode, ln->gamma_shift);
                f.ln_ro = make_fast_round(ln->ln_mode, 15 - ln->out_shift);
                f.ln_off = static_cast<int>((lds_f + 15) / 16 * 16);
                lds_f = static_cast<size_t>(f.ln_off) + 8 * static_cast<size_t>(lastl.N);
            }
            const int64_t wanted = (batch + (threads / 2) - 1) / (threads / 2);
            const int grid_f = static_cast<int>(std::min<int64_t>(wanted, 256 * per_cu));
            hipError_t e = hipErrorInvalidValue;
#define A4G_MLP_GO(MAXB, BIT)                                                                    \
    e = ln ? launch_mlp_mfma<MAXB, BIT, true, true>(grid_f, threads, lds_f, stream, f)            \
           : (f.y_vec ? launch_mlp_mfma<MAXB, BIT, true, false>(grid_f, threads, lds_f, stream, f) \
                      : launch_mlp_mfma<MAXB, BIT, false, false>(grid_f, threads, lds_f, stream, f))
#define A4G_MLP_BITS(MAXB)                                                  \
    if (bit_kind == 0) A4G_MLP_GO(MAXB, 0);                                  \
    else if (bit_kind == 1) A4G_MLP_GO(MAXB, 1);                             \
    else A4G_MLP_GO(MAXB, 2)
            if (widest <= 2) { A4G_MLP_BITS(2); }
            else if (widest <= 4) { A4G_MLP_BITS(4); }
            else { A4G_MLP_BITS(8); }
#undef A4G_MLP_BITS
#undef A4G_MLP_GO
            return check_hip(e, who);
        }
    }
    if (ln)
        return fail(A4G_ERR_UNSUPPORTED,
                    "%s: needs an int8 last layer of N %% 16 == 0 columns, 16-byte aligned rows of the result and the residual, "
                    "and weight fragments within 128 KiB of LDS", who);

    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(mlp_fused_kernel<64>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e == hipSuccess)
            e = hipFuncSetAttribute(reinterpret_cast<const void*>(mlp_fused_kernel<16>),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return check_hip(e, who);
        attr_set = true;
    }
    // 64 samples per workgroup once that fills the chip (2 workgroups per CU), 16 below
    const int spw = batch >= 64 * 512 ? 64 : 16;
    const int lds = a.weight_bytes + 2 * spw * MLP_ACT_PITCH;
    int grid = static_cast<int>((batch + spw - 1) / spw);
    if (grid > 256 * 4) grid = 256 * 4;
    if (spw == 64)
        hipLaunchKernelGGL(mlp_fused_kernel<64>, dim3(grid), dim3(256), lds, stream, a);
    else
        hipLaunchKernelGGL(mlp_fused_kernel<16>, dim3(grid), dim3(256), lds, stream, a);
    return check_hip(hipGetLastError(), who);
}

extern "C" int a4g_mlp_i8(const a4g_mlp_layer* layers, int n_layers, const void* X, int x_kind, int64_t ldx, void* Y,
                          int64_t ldy, int64_t batch, int round_mode, a4g_stream_t stream) {
    return mlp_entry(layers, n_layers, X, x_kind, ldx, Y, ldy, batch, round_mode, nullptr, stream, "a4g_mlp_i8");
}

extern "C" int a4g_mlp_add_layernorm_i8(const a4g_mlp_layer* layers, int n_layers, const void* X, int x_kind, int64_t ldx,
                                        const int8_t* residual, int64_t ld_res, const int16_t* gamma, const int16_t* beta,
                                        int8_t* Y, int64_t ldy, int64_t batch, int round_mode, int32_t eps_q0, int gamma_shift,
                                        int out_shift, int ln_round_mode, a4g_stream_t stream) {
    const char* who = "a4g_mlp_add_layernorm_i8";
    A4G_REQUIRE(eps_q0 >= 1 && eps_q0 <= (1 << 30), A4G_ERR_INVALID_ARGUMENT,
                "%s: eps_q0 must be positive (integer LayerNorm requires a positive variance floor), got %d", who, eps_q0);
    A4G_REQUIRE(out_shift >= 0 && out_shift <= 15, A4G_ERR_INVALID_ARGUMENT, "%s: out_shift=%d must be in [0, 15]", who, out_shift);
    A4G_REQUIRE(gamma_shift >= 0 && gamma_shift <= 15, A4G_ERR_INVALID_ARGUMENT, "%s: gamma_shift=%d must be in [0, 15]", who,
                gamma_shift);
    A4G_REQUIRE(valid_round(ln_round_mode), A4G_ERR_INVALID_ARGUMENT, "%s: unknown rounding mode", who);
    A4G_REQUIRE(batch == 0 || (gamma && beta), A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    const MlpLnExtra ln{residual, ld_res, gamma, beta, eps_q0, gamma_shift, out_shift, ln_round_mode};
    return mlp_entry(layers, n_layers, X, x_kind, ldx, Y, ldy, batch, round_mode, &ln, stream, who);
}
