// Fused multi-layer perceptron: a chain of Dense(+ReLU) layers in ONE launch, every weight matrix
// resident in LDS, activations never leaving the CU. Same arithmetic, layer by layer, as the Dense
// kernel (dense_bias_relu.cpp:112-163): acc32 = bias + sum a*w; srs; ReLU.
//
// A workgroup of 256 threads owns 64 (or, for small batches, 16) samples. A lane works on one sample
// and four output neurons at a time; weights are read from LDS as (mostly) wave-uniform dwords,
// activations as per-lane dwords from a padded LDS row, and four MACs retire per v_dot4_i32_i8.
// uint8 activations are biased to int8 with x ^ 0x80 and corrected by 128 * colsum.
#include "common.hpp"

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

}  // namespace a4g

using namespace a4g;

extern "C" int a4g_mlp_i8(const a4g_mlp_layer* layers, int n_layers, const void* X, int x_kind, int64_t ldx, void* Y,
                          int64_t ldy, int64_t batch, int round_mode, a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "a4g_mlp_i8";
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
