// Floating-point Dense / MatMul / Add: the reference's float compute path (bfloat16, float32 or fp8 e4m3
// operands, float32 accumulation, result converted to the operand format: round-to-nearest-even for bfloat16
// and float32, the conversion of the reference's own fp8 packer for fp8).
//   Dense   templates/nnet_utils/dense_bias_relu/dense_bias_relu.cpp:66-166 with acc_scalar_t = accfloat
//           (dense.py:105-127: shift 0, rounding conv_even, float32 bias as the accumulator's start value)
//   MatMul  templates/nnet_utils/matmul/matmul.cpp:31-118, same accumulator
//   Add     templates/nnet_utils/elementwise_add/elementwise_add.cpp:12-37
// The tiled path is the shared pipelined MFMA kernel with a float policy: a 16-byte fragment is eight
// bfloat16 (one v_mfma_f32_32x32x16_bf16), four float32 (four v_mfma_f32_32x32x2_f32) or sixteen fp8 (two
// v_mfma_f32_32x32x16_fp8_fp8); the order of the additions inside a dot product therefore differs from any
// sequential loop, as it does on the AI Engine.
#include <algorithm>

#include "gemm_rs.hpp"

namespace a4g {

typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));

__device__ __forceinline__ unsigned f32_to_bf16_bits(float f) {  // round to nearest even; NaN stays NaN
    const unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (u >> 16) | 0x40u;
    return (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
}
__device__ __forceinline__ float bf16_bits_to_f32(unsigned h) { return __uint_as_float(h << 16); }

// float32 -> fp8 e4m3 code, the integer recipe of the reference's packer (_float32_to_fp8_scalar,
// op_impls/families/matmul/common.py:262-276): round half away from zero at mantissa bit 20, exponent bias 7,
// gradual underflow below 2^-6, magnitudes from 480 up map to the code 0x7f.
__host__ __device__ __forceinline__ unsigned f32_bits_to_fp8(unsigned bits) {
    const unsigned h = bits + 0x00080000u;
    const unsigned e = (h & 0x7F800000u) >> 23, m = h & 0x007FFFFFu, sign = (h & 0x80000000u) >> 24;
    if (e > 135u) return sign | 0x7Fu;
    if (e > 120u) return sign | (((e - 120u) << 3) & 0x78u) | (m >> 20);
    if (e > 116u) return sign | ((((0x00780000u + m) >> (140u - e)) + 1u) >> 1);
    return sign;
}
__device__ __forceinline__ unsigned f32_to_fp8_bits(float f) { return f32_bits_to_fp8(__float_as_uint(f)) & 0xFFu; }
// fp8 e4m3 (OCP "fn": bias 7, no infinities, 0x7f / 0xff are NaN) -> float32, exact
__device__ __forceinline__ float fp8_bits_to_f32(unsigned c) {
    const unsigned sign = (c & 0x80u) << 24, e = (c >> 3) & 0xFu, m = c & 7u;
    if (e == 15u && m == 7u) return __uint_as_float(sign | 0x7FC00000u);
    if (e == 0u) return __uint_as_float(sign) + (sign ? -1.f : 1.f) * static_cast<float>(m) * 0.001953125f;  // m * 2^-9
    return __uint_as_float(sign | ((e + 120u) << 23) | (m << 20));
}

__device__ __forceinline__ float load_float(const void* p, int64_t i, int fmt) {
    if (fmt == A4G_F32) return static_cast<const float*>(p)[i];
    if (fmt == A4G_FP8) return fp8_bits_to_f32(static_cast<const uint8_t*>(p)[i]);
    return bf16_bits_to_f32(static_cast<const uint16_t*>(p)[i]);
}
__device__ __forceinline__ void store_float(void* p, int64_t i, int fmt, float v) {
    if (fmt == A4G_F32) static_cast<float*>(p)[i] = v;
    else if (fmt == A4G_FP8) static_cast<uint8_t*>(p)[i] = static_cast<uint8_t>(f32_to_fp8_bits(v));
    else static_cast<uint16_t*>(p)[i] = static_cast<uint16_t>(f32_to_bf16_bits(v));
}
static inline int fmt_bytes(int fmt) { return fmt == A4G_F32 ? 4 : (fmt == A4G_FP8 ? 1 : 2); }
static inline bool fmt_ok(int fmt) { return fmt == A4G_F32 || fmt == A4G_BF16 || fmt == A4G_FP8; }

template <int FMT>
struct FloatPolicy {
    using acc_t = v16f;
    static constexpr int ES = FMT == A4G_F32 ? 4 : (FMT == A4G_FP8 ? 1 : 2);
    // fp8 takes the 64-wide instruction (two 16-byte fragments per lane and operand), the others 32 bytes of K per call
    static constexpr int KSTEP_BYTES = FMT == A4G_FP8 ? 64 : 32;
    static constexpr int MMAS = FMT == A4G_F32 ? 4 : 1;
    static constexpr bool FIX_A = false;
    static constexpr bool SPLIT_A = false, SPLIT_B = false;
    static constexpr bool PERM_B = false;
    struct Extra {};
    static constexpr int MAX_OUT_BYTES = ES;
    template <int BN>
    static constexpr int param_bytes() { return 4 * BN; }
    struct ColRegs {
        float bias;
    };
    __device__ static __forceinline__ void fix_a(v4i&) {}
    __device__ static __forceinline__ v16f mma(const v4i (&b)[KSTEP_BYTES / 32], const v4i (&a)[KSTEP_BYTES / 32], v16f c) {
        if constexpr (FMT == A4G_F32) {
            const v4f bf = __builtin_bit_cast(v4f, b[0]), af = __builtin_bit_cast(v4f, a[0]);
#pragma unroll
            for (int t = 0; t < 4; ++t) c = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[t], af[t], c, 0, 0, 0);
            return c;
        } else if constexpr (FMT == A4G_FP8) {
            // v_mfma_f32_32x32x64_f8f6f4 with both operands fp8 e4m3 (format codes 0) and no block scaling: a lane
            // supplies 32 bytes of K per operand; which 32 is immaterial as long as both operands agree
            typedef int v8i __attribute__((ext_vector_type(8)));
            const v8i bw = {b[0][0], b[0][1], b[0][2], b[0][3], b[1][0], b[1][1], b[1][2], b[1][3]};
            const v8i aw = {a[0][0], a[0][1], a[0][2], a[0][3], a[1][0], a[1][1], a[1][2], a[1][3]};
            return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(bw, aw, c, 0, 0, 0, 0, 0, 0);
        } else {
            return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, b[0]), __builtin_bit_cast(v8bf, a[0]), c, 0, 0, 0);
        }
    }
    template <int BN>
    __device__ static __forceinline__ void fetch_params(const GemmArgs& g, const TileCoord& tc, int tid, ColRegs& r) {
        r.bias = 0.f;
        if (tid < BN && g.bias) r.bias = reinterpret_cast<const float*>(g.bias)[min(tc.n0 + tid, g.N - 1)];
    }
    template <int BN>
    __device__ static __forceinline__ int park_params(const GemmArgs&, int8_t* lds, int tid, const ColRegs& r) {
        if (tid < BN) reinterpret_cast<float*>(lds)[tid] = r.bias;
        __syncthreads();
        return 0;
    }
    // acc + bias -> ReLU -> operand format, through an LDS image of the tile, then whole-row stores
    template <int BM, int BN, int WTM, int WTN, int NT>
    __device__ static __forceinline__ void epilogue(const GemmArgs& g, const TileCoord& tc, v16f (&acc)[WTM / 32][WTN / 32],
                                                    int8_t* smem, int8_t* lds_params, int, int wm, int wn, int lane, int tid,
                                                    Extra&) {
        constexpr int TM = WTM / 32, TN = WTN / 32;
        constexpr int cpitch = BN * ES + 16;
        const float* bias = reinterpret_cast<const float*>(lds_params);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int nl = wn * WTN + j * 32 + 8 * q + 4 * (lane >> 5);  // column inside the tile
                const v4f b4 = *reinterpret_cast<const v4f*>(bias + nl);
#pragma unroll
                for (int i = 0; i < TM; ++i) {
                    const int ml = wm * WTM + i * 32 + (lane & 31);
                    float y[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        y[t] = acc[i][j][q * 4 + t] + b4[t];
                        if (g.relu) y[t] = fmaxf(y[t], 0.f);
                    }
                    if (FMT == A4G_F32) {
                        const v4f o = {y[0], y[1], y[2], y[3]};
                        *reinterpret_cast<v4f*>(smem + ml * cpitch + nl * 4) = o;
                    } else if (FMT == A4G_FP8) {
                        *reinterpret_cast<unsigned*>(smem + ml * cpitch + nl) =
                            f32_to_fp8_bits(y[0]) | (f32_to_fp8_bits(y[1]) << 8) | (f32_to_fp8_bits(y[2]) << 16) |
                            (f32_to_fp8_bits(y[3]) << 24);
                    } else {
                        v2i o;
                        o[0] = static_cast<int>(f32_to_bf16_bits(y[0]) | (f32_to_bf16_bits(y[1]) << 16));
                        o[1] = static_cast<int>(f32_to_bf16_bits(y[2]) | (f32_to_bf16_bits(y[3]) << 16));
                        *reinterpret_cast<v2i*>(smem + ml * cpitch + nl * 2) = o;
                    }
                }
            }
        }
        __syncthreads();
        store_tile_image<BM, BN, NT>(g, tc, smem, ES, tid);
    }
};

// The same policy with the epilogue of the register-requantising int8 kernels (I8DirectPolicy in gemm.hip): weight rows
// taken in the order that makes a lane's 16 accumulators of a block 16 neighbouring columns, which it converts and
// stores itself, 16 bytes at a time - no LDS image of the tile. bfloat16 outputs in whole 16-column pieces on 16-byte
// aligned rows (1183 -> 1204 TFLOP/s on 8192 x 4096 x 4096). The sum still meets its bias after the reduction, as in the reference (float addition does not
// associate, so the accumulators start from zero here).
template <int FMT>
struct FloatDirectPolicy : FloatPolicy<FMT> {
    static_assert(FMT == A4G_BF16 || FMT == A4G_FP8, "two- and one-byte outputs");  // (only bfloat16 is dispatched to it)
    static constexpr bool PERM_B = true;
    static constexpr int ES = FloatPolicy<FMT>::ES;
    using Extra = typename FloatPolicy<FMT>::Extra;
    template <int BN, int WTN, int TM, int TN>
    __device__ static __forceinline__ void start_acc(v16f (&)[TM][TN], int8_t*, int, int) {}
    template <int BM, int BN, int WTM, int WTN, int NT>
    __device__ static __forceinline__ void epilogue(const GemmArgs& g, const TileCoord& tc, v16f (&acc)[WTM / 32][WTN / 32],
                                                    int8_t*, int8_t* lds_params, int, int wm, int wn, int lane, int, Extra&) {
        constexpr int TM = WTM / 32, TN = WTN / 32;
        const float* bias = reinterpret_cast<const float*>(lds_params);
        const int half = lane >> 5, frow = lane & 31;
        int8_t* Cb = static_cast<int8_t*>(g.C) + tc.batch * g.stride_c * ES;
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const int nl = wn * WTN + j * 32 + 16 * half;  // the lane's 16 columns inside the tile
            v4f b4[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) b4[q] = *reinterpret_cast<const v4f*>(bias + nl + 4 * q);
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int m = tc.m0 + wm * WTM + i * 32 + frow, n = tc.n0 + nl;
                unsigned w[FMT == A4G_BF16 ? 8 : 4];
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    float y[4];
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        y[t] = acc[i][j][q * 4 + t] + b4[q][t];
                        if (g.relu) y[t] = fmaxf(y[t], 0.f);
                    }
                    if (FMT == A4G_BF16) {
                        w[2 * q] = f32_to_bf16_bits(y[0]) | (f32_to_bf16_bits(y[1]) << 16);
                        w[2 * q + 1] = f32_to_bf16_bits(y[2]) | (f32_to_bf16_bits(y[3]) << 16);
                    } else {
                        w[q] = f32_to_fp8_bits(y[0]) | (f32_to_fp8_bits(y[1]) << 8) | (f32_to_fp8_bits(y[2]) << 16) | (f32_to_fp8_bits(y[3]) << 24);
                    }
                }
                if (m < g.M && n + 16 <= g.N) {
                    int8_t* dst = Cb + (static_cast<int64_t>(m) * g.ldc + n) * ES;
#pragma unroll
                    for (int c = 0; c < (FMT == A4G_BF16 ? 2 : 1); ++c) {
                        const v4i o = {static_cast<int>(w[4 * c]), static_cast<int>(w[4 * c + 1]), static_cast<int>(w[4 * c + 2]), static_cast<int>(w[4 * c + 3])};
                        *reinterpret_cast<v4i*>(dst + 16 * c) = o;
                    }
                }
            }
        }
    }
};

// [K][ldb] -> [N][ldt] for 2- or 4-byte elements, 32 x 32 tiles through LDS; columns K..ldt-1 are zero filled.
template <typename T>
__global__ __launch_bounds__(256) void transpose_elems_kernel(const T* __restrict__ B, int64_t ldb, int64_t stride_b,
                                                              T* __restrict__ Bt, int64_t ldt, int64_t stride_t, int K, int N) {
    __shared__ T tile[32][33];
    const T* src = B + blockIdx.z * stride_b;
    T* dst = Bt + blockIdx.z * stride_t;
    const int k0 = blockIdx.x * 32, n0 = blockIdx.y * 32;
    const int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 32 x 8
    for (int r = ty; r < 32; r += 8) {
        const int k = k0 + r, n = n0 + tx;
        tile[r][tx] = (k < K && n < N) ? src[static_cast<int64_t>(k) * ldb + n] : T(0);
    }
    __syncthreads();
    for (int r = ty; r < 32; r += 8) {
        const int n = n0 + r, k = k0 + tx;
        if (n < N && k < ldt) dst[static_cast<int64_t>(n) * ldt + k] = tile[tx][r];
    }
}

__global__ __launch_bounds__(256) void add_float_kernel(const void* a, const void* b, void* out, int64_t n, int fmt) {
    for (int64_t i = blockIdx.x * 256ll + threadIdx.x; i < n; i += static_cast<int64_t>(gridDim.x) * 256)
        store_float(out, i, fmt, load_float(a, i, fmt) + load_float(b, i, fmt));
}

static inline int64_t round_up64(int64_t v, int64_t m) { return (v + m - 1) / m * m; }

// A is [batch][M][lda], Bt is [batch][N][ldb], both K-contiguous, element counts; C [batch][M][ldc].
static hipError_t launch_float_nt(const void* A, int trans_a, int64_t lda, int64_t stride_a, const void* Bt, int64_t ldb, int64_t stride_b,
                                  const float* bias, int relu, void* C, int64_t ldc, int64_t stride_c, int batch, int M, int N,
                                  int K, int fmt, hipStream_t stream) {
    const int es = fmt_bytes(fmt);
    const bool tiled = !trans_a && (static_cast<int64_t>(K) * es) % 128 == 0 && (lda * es) % 16 == 0 && (ldb * es) % 16 == 0 &&
                       (stride_a * es) % 16 == 0 && (stride_b * es) % 16 == 0 && aligned16(A) && aligned16(Bt);
    GemmArgs g{};
    g.A = static_cast<const int8_t*>(A);
    g.Bt = static_cast<const int8_t*>(Bt);
    g.C = C;
    g.bias = reinterpret_cast<const int32_t*>(bias);
    g.lda = lda * es;
    g.stride_a = stride_a * es;
    g.ldb = ldb * es;
    g.stride_b = stride_b * es;
    g.ldc = ldc;
    g.stride_c = stride_c;
    g.M = M;
    g.N = N;
    g.K = K * es;
    g.relu = relu != 0;
    const bool aligned_rows = !trans_a && (lda * es) % 16 == 0 && (ldb * es) % 16 == 0 && (stride_a * es) % 16 == 0 &&
                              (stride_b * es) % 16 == 0 && aligned16(A) && aligned16(Bt);
    if (!tiled && aligned_rows && g.K % 16 == 0 && g.K >= 256) {
        // K in whole 16-byte chunks but not whole tiles: the last tile's missing chunks come from outside the operands'
        // descriptors and read as zero on both sides (no load in a branch; 8192 x 1000 x 1000 bfloat16: 48 us with the
        // ragged loads)
        if (fmt == A4G_F32) return launch_rs_policy<FloatPolicy<A4G_F32>, 128, 128, 2, 2, false, false, true>(g, batch, stream);
        if (fmt == A4G_FP8) return launch_rs_policy<FloatPolicy<A4G_FP8>, 128, 128, 2, 2, false, false, true>(g, batch, stream);
        return launch_rs_policy<FloatPolicy<A4G_BF16>, 128, 128, 2, 2, false, false, true>(g, batch, stream);
    }
    if (!tiled) {
        // K that does not fill its last 128-byte tile, unaligned rows: the same kernel with loads that respect the row ends
        g.ragged_a = ragged_mode(g.A, g.lda, g.stride_a, g.K);
        g.ragged_b = ragged_mode(g.Bt, g.ldb, g.stride_b, g.K);
        g.trans_a_es = trans_a ? es : 0;  // A stored transposed: its chunks are gathered element by element
        if (!trans_a && g.K >= 256 && g.ragged_a <= 1 && g.ragged_b == 0 && g.lda >= (g.K + 3) / 4 * 4) {
            // 4-byte aligned activation rows, 16-byte aligned rows of the other operand that hold K rounded up to 16: the
            // descriptor loads without branches (K off the 16-byte grid; the bytes past K are cleared at the staging)
            if (fmt == A4G_F32) return launch_rs_policy<FloatPolicy<A4G_F32>, 128, 128, 2, 2, false, false, 2>(g, batch, stream);
            if (fmt == A4G_FP8) return launch_rs_policy<FloatPolicy<A4G_FP8>, 128, 128, 2, 2, false, false, 2>(g, batch, stream);
            return launch_rs_policy<FloatPolicy<A4G_BF16>, 128, 128, 2, 2, false, false, 2>(g, batch, stream);
        }
        if (fmt == A4G_F32) return launch_rs_policy<FloatPolicy<A4G_F32>, 128, 128, 2, 2, false, true>(g, batch, stream);
        if (fmt == A4G_FP8) return launch_rs_policy<FloatPolicy<A4G_FP8>, 128, 128, 2, 2, false, true>(g, batch, stream);
        return launch_rs_policy<FloatPolicy<A4G_BF16>, 128, 128, 2, 2, false, true>(g, batch, stream);
    }
    if (fmt == A4G_F32) return launch_rs_policy<FloatPolicy<A4G_F32>, 128, 128, 2, 2>(g, batch, stream);
    const int64_t tiles256 = static_cast<int64_t>((M + 255) / 256) * ((N + 255) / 256) * batch;
    const int64_t rounds256 = (tiles256 + 255) / 256;
    const bool big = M >= 256 && N >= 256 && K * es >= 512 && tiles256 * 100 >= rounds256 * 256 * 85;
    // whole 16-column pieces on 16-byte aligned rows: the epilogue that converts and stores from registers
    const bool direct = N % 16 == 0 && (ldc * es) % 16 == 0 && (stride_c * es) % 16 == 0 && aligned16(C);
    if (fmt == A4G_FP8) {  // (the register epilogue measured slower for fp8: 1474 against 1734 TFLOP/s on the 8192 x 4096 x 4096 shape)
        if (big) return launch_rs_policy<FloatPolicy<A4G_FP8>, 256, 256, 2, 4, true>(g, batch, stream);
        return launch_rs_policy<FloatPolicy<A4G_FP8>, 128, 128, 2, 2>(g, batch, stream);
    }
    if (big && direct) return launch_rs_policy<FloatDirectPolicy<A4G_BF16>, 256, 256, 2, 4, true>(g, batch, stream);
    if (big) return launch_rs_policy<FloatPolicy<A4G_BF16>, 256, 256, 2, 4, true>(g, batch, stream);
    if (direct) return launch_rs_policy<FloatDirectPolicy<A4G_BF16>, 128, 128, 2, 2>(g, batch, stream);
    return launch_rs_policy<FloatPolicy<A4G_BF16>, 128, 128, 2, 2>(g, batch, stream);
}

template <typename T>
static hipError_t launch_transpose(const void* B, int64_t ldb, int64_t stride_b, void* Bt, int64_t ldt, int64_t stride_t, int batch,
                                   int K, int N, hipStream_t stream) {
    dim3 grid(static_cast<unsigned>((ldt + 31) / 32), static_cast<unsigned>((N + 31) / 32), static_cast<unsigned>(batch));
    transpose_elems_kernel<T><<<grid, 256, 0, stream>>>(static_cast<const T*>(B), ldb, stride_b, static_cast<T*>(Bt), ldt, stride_t, K,
                                                        N);
    return hipGetLastError();
}

static hipError_t launch_transpose_fmt(int fmt, const void* B, int64_t ldb, int64_t stride_b, void* Bt, int64_t ldt,
                                       int64_t stride_t, int batch, int K, int N, hipStream_t stream) {
    if (fmt == A4G_F32) return launch_transpose<uint32_t>(B, ldb, stride_b, Bt, ldt, stride_t, batch, K, N, stream);
    if (fmt == A4G_FP8) return launch_transpose<uint8_t>(B, ldb, stride_b, Bt, ldt, stride_t, batch, K, N, stream);
    return launch_transpose<uint16_t>(B, ldb, stride_b, Bt, ldt, stride_t, batch, K, N, stream);
}

}  // namespace a4g

using namespace a4g;

extern "C" int64_t a4g_packed_ld_f(int64_t K, int fmt) {
    const int es = fmt_bytes(fmt);
    return K <= 0 ? 16 / es : round_up64(K * es, 16) / es;
}

extern "C" int a4g_pack_weights_f(const void* W, int fmt, int64_t ldw, int64_t K, int64_t N, void* Wt, a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "a4g_pack_weights_f";
    A4G_REQUIRE(fmt_ok(fmt), A4G_ERR_UNSUPPORTED, "%s: format %d is not bfloat16 / float32 / fp8 e4m3", who, fmt);
    A4G_REQUIRE(W && Wt, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    A4G_REQUIRE(K >= 1 && N >= 1 && K <= (1 << 24) && N <= (1 << 24) && ldw >= N, A4G_ERR_INVALID_ARGUMENT,
                "%s: bad shape K=%lld N=%lld ldw=%lld", who, (long long)K, (long long)N, (long long)ldw);
    const int64_t ldt = a4g_packed_ld_f(K, fmt);
    return check_hip(launch_transpose_fmt(fmt, W, ldw, 0, Wt, ldt, 0, 1, (int)K, (int)N, stream), who);
}

extern "C" int a4g_dense_f(const void* A, int fmt, int trans_a, int64_t lda, const void* Wt, int64_t ldwt, const float* bias, int relu, void* Y,
                           int64_t ldy, int64_t M, int64_t N, int64_t K, a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "a4g_dense_f";
    A4G_REQUIRE(fmt_ok(fmt), A4G_ERR_UNSUPPORTED, "%s: format %d is not bfloat16 / float32 / fp8 e4m3", who, fmt);
    A4G_REQUIRE(M >= 0 && N >= 1 && K >= 1 && M <= INT32_MAX && N <= (1 << 24) && K <= (1 << 24), A4G_ERR_INVALID_ARGUMENT,
                "%s: bad shape M=%lld N=%lld K=%lld", who, (long long)M, (long long)N, (long long)K);
    A4G_REQUIRE(lda >= (trans_a ? M : K) && ldy >= N && ldwt >= K, A4G_ERR_INVALID_ARGUMENT, "%s: pitch smaller than the row", who);
    if (M == 0) return A4G_OK;
    A4G_REQUIRE(A && Wt && Y, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    return check_hip(launch_float_nt(A, trans_a, lda, 0, Wt, ldwt, 0, bias, relu, Y, ldy, 0, 1, (int)M, (int)N, (int)K, fmt, stream), who);
}

extern "C" size_t a4g_matmul_f_workspace_bytes(int64_t batch, int64_t N, int64_t K, int trans_b, int fmt) {
    if (trans_b || batch <= 0 || N <= 0 || K <= 0) return 0;
    return static_cast<size_t>(batch) * N * a4g_packed_ld_f(K, fmt) * fmt_bytes(fmt);
}

extern "C" int a4g_matmul_f(const void* A, int fmt, int trans_a, int64_t lda, int64_t stride_a, const void* B, int64_t ldb, int64_t stride_b,
                            int trans_b, void* C, int64_t ldc, int64_t stride_c, int64_t batch, int64_t M, int64_t N, int64_t K,
                            void* workspace, size_t workspace_bytes, a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "a4g_matmul_f";
    A4G_REQUIRE(fmt_ok(fmt), A4G_ERR_UNSUPPORTED, "%s: format %d is not bfloat16 / float32 / fp8 e4m3", who, fmt);
    A4G_REQUIRE(batch >= 0 && batch <= 65535 && M >= 0 && N >= 1 && K >= 1 && M <= INT32_MAX && N <= (1 << 24) && K <= (1 << 24),
                A4G_ERR_INVALID_ARGUMENT, "%s: bad shape batch=%lld M=%lld N=%lld K=%lld", who, (long long)batch, (long long)M,
                (long long)N, (long long)K);
    A4G_REQUIRE(lda >= (trans_a ? M : K) && ldc >= N && ldb >= (trans_b ? K : N), A4G_ERR_INVALID_ARGUMENT, "%s: pitch smaller than the row",
                who);
    if (M == 0 || batch == 0) return A4G_OK;
    A4G_REQUIRE(A && B && C, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    if (trans_b)
        return check_hip(launch_float_nt(A, trans_a, lda, stride_a, B, ldb, stride_b, nullptr, 0, C, ldc, stride_c, (int)batch, (int)M, (int)N,
                                         (int)K, fmt, stream), who);
    const size_t need = a4g_matmul_f_workspace_bytes(batch, N, K, 0, fmt);
    A4G_REQUIRE(workspace && workspace_bytes >= need && aligned16(workspace), A4G_ERR_WORKSPACE,
                "%s: needs a 16-byte aligned workspace of %zu bytes (a4g_matmul_f_workspace_bytes)", who, need);
    const int64_t ldt = a4g_packed_ld_f(K, fmt);
    hipError_t e = launch_transpose_fmt(fmt, B, ldb, stride_b, workspace, ldt, N * ldt, (int)batch, (int)K, (int)N, stream);
    if (e != hipSuccess) return check_hip(e, who);
    return check_hip(launch_float_nt(A, trans_a, lda, stride_a, workspace, ldt, N * ldt, nullptr, 0, C, ldc, stride_c, (int)batch, (int)M, (int)N,
                                     (int)K, fmt, stream), who);
}

extern "C" int a4g_add_f(const void* a, const void* b, void* out, int64_t n, int fmt, a4g_stream_t stream_) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char* who = "a4g_add_f";
    A4G_REQUIRE(fmt_ok(fmt), A4G_ERR_UNSUPPORTED, "%s: format %d is not bfloat16 / float32 / fp8 e4m3", who, fmt);
    A4G_REQUIRE(n >= 0, A4G_ERR_INVALID_ARGUMENT, "%s: negative length", who);
    if (n == 0) return A4G_OK;
    A4G_REQUIRE(a && b && out, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    const int grid = static_cast<int>(std::min<int64_t>((n + 255) / 256, 256 * 16));
    add_float_kernel<<<grid, 256, 0, stream>>>(a, b, out, n, fmt);
    return check_hip(hipGetLastError(), who);
}
