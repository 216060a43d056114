// Fused multi-layer perceptron: a chain of Dense(+ReLU) layers in ONE launch, every weight matrix
// resident in LDS, activations never leaving the CU. Same arithmetic, layer by layer, as the Dense
// kernel (dense_bias_relu.cpp:112-163): acc32 = bias + sum a*w; srs; ReLU.
//
// A workgroup of 256 threads owns 64 samples. Lane l of every wave works on sample l; the four waves
// split the output neurons of a layer between them. Weights are read from LDS as wave-uniform
// (broadcast) dwords, activations as per-lane dwords from a padded LDS row, and four MACs retire per
// v_dot4_i32_i8. uint8 activations are biased to int8 with x ^ 0x80 and corrected by 128 * colsum.
#include "common.hpp"

namespace a4g {

constexpr int MLP_MAX_LAYERS = 8;
constexpr int MLP_MAX_WIDTH = 256;
constexpr int MLP_SAMPLES = 64;                      // per workgroup
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
};

__global__ __launch_bounds__(256) void mlp_fused_kernel(MlpArgs a) {
    extern __shared__ __attribute__((aligned(16))) int8_t smem[];
    int8_t* sW = smem;
    int8_t* sAct0 = smem + a.weight_bytes;
    int8_t* sAct1 = sAct0 + MLP_SAMPLES * MLP_ACT_PITCH;

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;

    // stage all weights once (16-byte copies; rows are already zero padded to a multiple of 16)
    for (int l = 0; l < a.n_layers; ++l) {
        const MlpLayerDev& L = a.layer[l];
        const int chunks = L.N * L.ldwt / 16;
        for (int c = tid; c < chunks; c += 256)
            *reinterpret_cast<v4i*>(sW + L.w_off + c * 16) = *reinterpret_cast<const v4i*>(L.wt + static_cast<int64_t>(c) * 16);
    }

    for (int s0 = blockIdx.x * MLP_SAMPLES; s0 < a.batch; s0 += gridDim.x * MLP_SAMPLES) {
        // input rows -> LDS, zero padded to the first layer's packed K
        const int K0 = a.layer[0].K, K0p = a.layer[0].ldwt;
        __syncthreads();
        for (int i = tid; i < MLP_SAMPLES * K0p; i += 256) {
            const int s = i / K0p, k = i % K0p;
            int8_t v = 0;
            if (k < K0 && s0 + s < a.batch) v = a.X[static_cast<int64_t>(s0 + s) * a.ldx + k];
            sAct0[s * MLP_ACT_PITCH + k] = v;
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
            const int* arow = reinterpret_cast<const int*>(in + lane * MLP_ACT_PITCH);
            const int next_kp = last ? 0 : a.layer[l + 1].ldwt;
            for (int n = wave; n < L.N; n += 4) {
                const int* wrow = reinterpret_cast<const int*>(sW + L.w_off + n * L.ldwt);
                int acc = L.bias ? L.bias[n] : 0;
                if (in_unsigned) acc += 128 * L.colsum[n];
                for (int k4 = 0; k4 < k4n; ++k4) acc = __builtin_amdgcn_sdot4(arow[k4] ^ xm, wrow[k4], acc, false);
                const int y = clamp_i(apply_round(acc, rc), lo, hi);
                if (last) {
                    if (s0 + lane < a.batch) {
                        if (L.out_kind == A4G_I16)
                            static_cast<int16_t*>(a.Y)[static_cast<int64_t>(s0 + lane) * a.ldy + n] = static_cast<int16_t>(y);
                        else
                            static_cast<int8_t*>(a.Y)[static_cast<int64_t>(s0 + lane) * a.ldy + n] = static_cast<int8_t>(y);
                    }
                } else {
                    out[lane * MLP_ACT_PITCH + n] = static_cast<int8_t>(y);
                }
            }
            if (!last) {
                // zero the padding columns the next layer's dot products will touch
                for (int n = L.N + wave; n < next_kp; n += 4) out[lane * MLP_ACT_PITCH + n] = 0;
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
    A4G_REQUIRE(off <= MLP_MAX_WEIGHT_BYTES, A4G_ERR_UNSUPPORTED, "%s: %d bytes of packed weights exceed the LDS budget of %d",
                who, off, MLP_MAX_WEIGHT_BYTES);
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

    const int lds = a.weight_bytes + 2 * MLP_SAMPLES * MLP_ACT_PITCH;
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(mlp_fused_kernel),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        if (e != hipSuccess) return check_hip(e, who);
        attr_set = true;
    }
    int grid = static_cast<int>((batch + MLP_SAMPLES - 1) / MLP_SAMPLES);
    if (grid > 256 * 4) grid = 256 * 4;
    hipLaunchKernelGGL(mlp_fused_kernel, dim3(grid), dim3(256), lds, stream, a);
    return check_hip(hipGetLastError(), who);
}
