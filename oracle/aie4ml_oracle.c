/*
 * TEST INFRASTRUCTURE — CPU oracle for the quantized operators aie4ml lowers.
 *
 * This file is a scalar, plain-C restatement of the arithmetic of the reference's AIE kernels
 * (src/aie4ml/templates/nnet_utils/...) and of the AIE-API primitives they call. It is the checker
 * the GPU library is compared against; it is never linked into, loaded by or called from the
 * product path. Only the tests, the smoke check and the CPU-baseline leg of the benchmark load it.
 *
 * Pinning status of each function (what fixes it beyond "it restates the source"):
 *   a4o_srs              closed forms for all 8 AIE rounding modes; brute-forced in the tests
 *                        against exact rational arithmetic (python fractions).
 *   a4o_dense / matmul   int64 numpy matmul + srs; identity / zero / tie / saturation cases.
 *   a4o_add              textbook saturating add.
 *   a4o_softmax_exp      all-integer in the reference; exhaustive 256xKQ table vs python ints;
 *                        reciprocal == python floor division.
 *   a4o_softmax_hccs     all-integer in the reference; python-int restatement + invariants.
 *                        use_clb branch: clb() semantics assumed = count-leading-bits of a positive
 *                        int32 (k = floor(log2 sum)) — PARITY UNPINNED for use_clb.
 *   a4o_layernorm        integer parts restated and checked against python ints; the reciprocal
 *                        standard deviation is float on the AIE (aie::invsqrt + aie::to_fixed,
 *                        layer_norm.cpp:33-34) and cannot be derived from the reference tree:
 *                        this oracle DEFINES it as round-to-nearest Q15 — PARITY UNPINNED for
 *                        inv_std16 (+-1 LSB against a real AIE is possible). Non-power-of-two
 *                        column counts are an extension (the reference rejects them,
 *                        layer_norm.py:169-170): mean/variance use exact floor division, which
 *                        equals the reference's shifts when cols is 2^k — PARITY UNPINNED for those.
 *
 * Build: see oracle/Makefile  (gcc -O3 -fopenmp -shared -fPIC).
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <math.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define A4O_EXPORT __attribute__((visibility("default")))

/* rounding modes: AIE-API aie::rounding_mode tokens, as emitted through
 * ROUNDING_TOKEN_MAP (src/aie4ml/op_impls/utils/precision.py:13-21). positive_inf / negative_inf /
 * conv_odd are AIE-API modes the reference never emits; positive_inf is "round half up". */
enum {
    A4O_RND_FLOOR = 0,
    A4O_RND_CEIL = 1,
    A4O_RND_POSITIVE_INF = 2,
    A4O_RND_NEGATIVE_INF = 3,
    A4O_RND_SYMMETRIC_INF = 4,
    A4O_RND_SYMMETRIC_ZERO = 5,
    A4O_RND_CONV_EVEN = 6,
    A4O_RND_CONV_ODD = 7,
};

/* element kinds for outputs / storage */
enum { A4O_I8 = 0, A4O_U8 = 1, A4O_I16 = 2, A4O_U16 = 3, A4O_I32 = 4 };

static inline int64_t kind_min(int kind) {
    switch (kind) {
    case A4O_I8: return -128;
    case A4O_U8: return 0;
    case A4O_I16: return -32768;
    case A4O_U16: return 0;
    default: return INT32_MIN;
    }
}
static inline int64_t kind_max(int kind) {
    switch (kind) {
    case A4O_I8: return 127;
    case A4O_U8: return 255;
    case A4O_I16: return 32767;
    case A4O_U16: return 65535;
    default: return INT32_MAX;
    }
}
static inline int kind_bytes(int kind) {
    return (kind == A4O_I8 || kind == A4O_U8) ? 1 : (kind == A4O_I32 ? 4 : 2);
}

static inline int32_t wrap32(int64_t v) { return (int32_t)(uint32_t)(uint64_t)v; }

/* Shift-round-saturate: aie::accum::to_vector<T>(shift) under aie::set_rounding(mode) and
 * saturation_mode::saturate (hard-wired in every variants/<op>/parameters.h.jinja, e.g.
 * dense_bias_relu/parameters.h.jinja:26-29). acc is the 32-bit accumulator value. */
static inline int64_t srs_round(int64_t acc, int s, int mode) {
    if (s <= 0) return acc;
    const int64_t one = (int64_t)1 << s;
    const int64_t h = one >> 1;
    const int64_t q = acc >> s;          /* arithmetic: floor */
    const int64_t r = acc & (one - 1);   /* 0 <= r < 2^s */
    switch (mode) {
    case A4O_RND_FLOOR: return q;
    case A4O_RND_CEIL: return q + (r != 0);
    case A4O_RND_POSITIVE_INF: return q + (r >= h);
    case A4O_RND_NEGATIVE_INF: return q + (r > h);
    case A4O_RND_SYMMETRIC_INF: /* nearest, ties away from zero */
        return q + ((r > h) || (r == h && acc >= 0));
    case A4O_RND_SYMMETRIC_ZERO: /* nearest, ties toward zero */
        return q + ((r > h) || (r == h && acc < 0));
    case A4O_RND_CONV_EVEN: return q + ((r > h) || (r == h && (q & 1)));
    case A4O_RND_CONV_ODD: return q + ((r > h) || (r == h && !(q & 1)));
    default: return q;
    }
}

static inline int64_t srs(int64_t acc, int s, int mode, int kind) {
    int64_t q = srs_round(acc, s, mode);
    const int64_t lo = kind_min(kind), hi = kind_max(kind);
    return q < lo ? lo : (q > hi ? hi : q);
}

A4O_EXPORT int32_t a4o_srs(int32_t acc, int shift, int mode, int kind) {
    return (int32_t)srs((int64_t)acc, shift, mode, kind);
}

static inline void store_kind(void* base, size_t idx, int kind, int64_t v) {
    switch (kind) {
    case A4O_I8: ((int8_t*)base)[idx] = (int8_t)v; break;
    case A4O_U8: ((uint8_t*)base)[idx] = (uint8_t)v; break;
    case A4O_I16: ((int16_t*)base)[idx] = (int16_t)v; break;
    case A4O_U16: ((uint16_t*)base)[idx] = (uint16_t)v; break;
    default: ((int32_t*)base)[idx] = (int32_t)v; break;
    }
}
static inline int64_t load_kind(const void* base, size_t idx, int kind) {
    switch (kind) {
    case A4O_I8: return ((const int8_t*)base)[idx];
    case A4O_U8: return ((const uint8_t*)base)[idx];
    case A4O_I16: return ((const int16_t*)base)[idx];
    case A4O_U16: return ((const uint16_t*)base)[idx];
    default: return ((const int32_t*)base)[idx];
    }
}

/* Dense: acc32 = bias[n] + sum_k a[m,k]*w[k,n]; y = srs(acc, SHIFT); relu = max(y, 0).
 * dense_bias_relu.cpp:112-163 (single tile) and :404-415 (cascade tail: bias added to the partial
 * sums before requantisation — numerically the same sum). Weights are the logical [K][N] matrix;
 * the reference's microtile packing (matmul/common.py:307-358) only reorders storage.
 * shifts: one value (n_shift == 1, the reference) or one per output column (n_shift == N, an
 * extension that reduces to the reference when all entries are equal).
 * a_kind: A4O_I8 or A4O_U8 activations (uint8 kept by resolve_storage_dtype, precision.py:48-61). */
A4O_EXPORT int a4o_dense_i8(const void* A, int a_kind, int64_t lda,
                            const int8_t* W, int64_t ldw,
                            const int32_t* bias,
                            const int32_t* shifts, int n_shift,
                            int mode, int relu, int out_kind,
                            void* Y, int64_t ldy,
                            int64_t M, int64_t N, int64_t K) {
    /* int16 activations: the reference's (16, 8) combination, also accumulated in acc32
     * (op_impls/families/matmul/common.py:52, op_impls/utils/precision.py:120-121) */
    if (!(a_kind == A4O_I8 || a_kind == A4O_U8 || a_kind == A4O_I16)) return -1;
    if (!(n_shift == 1 || n_shift == N)) return -1;
    /* transpose W once so the inner loop streams */
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        int32_t accrow[64];
        for (int64_t n0 = 0; n0 < N; n0 += 64) {
            const int64_t nb = (N - n0) < 64 ? (N - n0) : 64;
            for (int64_t j = 0; j < nb; ++j) accrow[j] = bias ? bias[n0 + j] : 0;
            for (int64_t k = 0; k < K; ++k) {
                const int32_t a = (int32_t)load_kind(A, (size_t)(m * lda + k), a_kind);
                const int8_t* wr = W + k * ldw + n0;
                for (int64_t j = 0; j < nb; ++j)
                    accrow[j] = (int32_t)((uint32_t)accrow[j] + (uint32_t)(a * (int32_t)wr[j]));
            }
            for (int64_t j = 0; j < nb; ++j) {
                const int s = shifts[n_shift == 1 ? 0 : (n0 + j)];
                int64_t y = srs((int64_t)accrow[j], s, mode, out_kind);
                if (relu && y < 0) y = 0;
                store_kind(Y, (size_t)(m * ldy + n0 + j), out_kind, y);
            }
        }
    }
    return 0;
}

/* Dense with int16 activations and int16 weights: the (16, 16) width combination, accumulated in acc64
 * (op_impls/families/matmul/common.py:52, op_impls/utils/precision.py:122-123); bias stays int32 at the
 * accumulator scale (matmul/resolver.py:147-157). Same kernel text as above, wider accumulator. */
A4O_EXPORT int a4o_dense_i16x16(const int16_t* A, int64_t lda, const int16_t* W, int64_t ldw, const int32_t* bias,
                                const int32_t* shifts, int n_shift, int mode, int relu, int out_kind, void* Y, int64_t ldy,
                                int64_t M, int64_t N, int64_t K) {
    if (!(n_shift == 1 || n_shift == N)) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        for (int64_t n = 0; n < N; ++n) {
            int64_t acc = bias ? bias[n] : 0;
            for (int64_t k = 0; k < K; ++k) acc += (int64_t)A[m * lda + k] * (int64_t)W[k * ldw + n];
            int64_t y = srs(acc, shifts[n_shift == 1 ? 0 : n], mode, out_kind);
            if (relu && y < 0) y = 0;
            store_kind(Y, (size_t)(m * ldy + n), out_kind, y);
        }
    }
    return 0;
}

/* MatMul: c = srs(wrap32(sum_k a[m,k]*b[k,n]), SHIFT); no bias, no ReLU. matmul.cpp:80-115.
 * trans_b: B is given as [N][K] (the last-two-axes transpose of the logical [K][N] operand, the
 * io_view perm of matmul.py:86-95 / TRANSPOSE_B matmul.cpp:70-76). batch > 1 = independent rank-2
 * products per leading index (the reference only accepts batch == 1 for the RHS,
 * matmul/resolver.py:440-463; batching is an extension with per-slice reference semantics). */
A4O_EXPORT int a4o_matmul_i8(const void* A, int a_kind, int64_t lda, int64_t stride_a,
                             const int8_t* B, int64_t ldb, int64_t stride_b, int trans_b,
                             void* C, int64_t ldc, int64_t stride_c,
                             int64_t batch, int64_t M, int64_t N, int64_t K,
                             int shift, int mode, int out_kind) {
    if (!(a_kind == A4O_I8 || a_kind == A4O_U8)) return -1;
    const int ob = kind_bytes(out_kind);
#pragma omp parallel for collapse(2) schedule(static)
    for (int64_t bi = 0; bi < batch; ++bi) {
        for (int64_t m = 0; m < M; ++m) {
            const uint8_t* Ab = (const uint8_t*)A + bi * stride_a;
            const int8_t* Bb = B + bi * stride_b;
            uint8_t* Cb = (uint8_t*)C + bi * stride_c * ob;
            for (int64_t n = 0; n < N; ++n) {
                uint32_t acc = 0;
                for (int64_t k = 0; k < K; ++k) {
                    const int32_t a = (int32_t)load_kind(Ab, (size_t)(m * lda + k), a_kind);
                    const int32_t b = trans_b ? Bb[n * ldb + k] : Bb[k * ldb + n];
                    acc += (uint32_t)(a * b);
                }
                store_kind(Cb, (size_t)(m * ldc + n), out_kind,
                           srs((int64_t)(int32_t)acc, shift, mode, out_kind));
            }
        }
    }
    return 0;
}

/* Elementwise add: out = to_vector<result_t>(acc32(a) + b, SHIFT). elementwise_add.cpp:28-35.
 * All three tensors share one storage type (elementwise/resolver.py:29-33). */
A4O_EXPORT int a4o_add(const void* a, const void* b, void* out, int64_t n, int kind, int shift, int mode) {
#pragma omp parallel for schedule(static)
    for (int64_t i = 0; i < n; ++i) {
        const int64_t s = load_kind(a, (size_t)i, kind) + load_kind(b, (size_t)i, kind);
        store_kind(out, (size_t)i, kind, srs(s, shift, mode, kind));
    }
    return 0;
}

/* round-to-nearest Q15 of 1/sqrt(v), v >= 1, clamped to [0, 32767]. Defined by this oracle (see the
 * header): q = floor(2^15/sqrt(v) + 1/2)  <=>  (2q-1)^2 v <= 2^32 < (2q+1)^2 v. */
A4O_EXPORT int32_t a4o_rsqrt_q15(int32_t v) {
    if (v < 1) v = 1;
    int64_t q = (int64_t)floor(32768.0 / sqrt((double)v) + 0.5);
    if (q < 1) q = 1;
    const uint64_t two32 = (uint64_t)1 << 32;
    while (q > 0 && (uint64_t)((2 * q - 1) * (2 * q - 1)) * (uint64_t)v > two32) --q;
    while ((uint64_t)((2 * q + 1) * (2 * q + 1)) * (uint64_t)v <= two32) ++q;
    return (int32_t)(q > 32767 ? 32767 : q);
}

/* Row statistics: layer_norm.cpp:14-40. int32 wraparound kept for the centred sum of squares.
 * For cols == 2^L the divisions below are exactly the reference's (sum + 2^(L-1)) >> L and
 * centered_sq >> L (both floor). */
static inline int64_t floordiv64(int64_t a, int64_t b) {
    int64_t q = a / b, r = a % b;
    return (r != 0 && ((r < 0) != (b < 0))) ? q - 1 : q;
}

static void ln_row(const int32_t* xrow, const int16_t* gamma, const int16_t* beta, int8_t* orow,
                   int64_t cols, int32_t eps_q0, int gamma_shift, int out_shift, int mode) {
    int32_t sx = 0, sq = 0;
    for (int64_t c = 0; c < cols; ++c) {
        sx = wrap32((int64_t)sx + xrow[c]);
        sq = wrap32((int64_t)sq + (int64_t)xrow[c] * xrow[c]);
    }
    const int32_t mu = (int32_t)floordiv64((int64_t)sx + (cols >> 1), cols);
    const int32_t csq = wrap32((int64_t)sq - 2 * (int64_t)mu * sx + (int64_t)cols * mu * mu);
    int32_t var = (int32_t)floordiv64((int64_t)csq, cols);
    if (var < 0) var = 0;
    const int32_t inv = a4o_rsqrt_q15(wrap32((int64_t)var + eps_q0));
    const int16_t mu16 = (int16_t)mu;
    for (int64_t c = 0; c < cols; ++c) {
        /* layer_norm.cpp:105-117 */
        const int64_t vd = srs((int64_t)xrow[c] - mu16, 0, mode, A4O_I16);
        const int64_t fs = srs((int64_t)inv * gamma[c], gamma_shift, mode, A4O_I16);
        const int64_t acc = (int64_t)wrap32(vd * fs + beta[c]);
        orow[c] = (int8_t)srs(acc, 15 - out_shift, mode, A4O_I8);
    }
}

/* LayerNorm int8 -> int8 over the last axis. layer_norm.cpp:44-121 (the microtile variant
 * :144-231 is the same arithmetic in another storage order). gamma is Q7 int16, beta Q15 int16
 * (layernorm/common.py:19-20); GAMMA_SHIFT = 7; final shift = 15 - OUT_SHIFT. */
A4O_EXPORT int a4o_layernorm_i8(const int8_t* x, const int16_t* gamma, const int16_t* beta, int8_t* out,
                                int64_t rows, int64_t cols, int32_t eps_q0, int gamma_shift,
                                int out_shift, int mode) {
    if (cols < 1 || cols > 65536 || out_shift < 0 || out_shift > 15 || eps_q0 < 1) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        int32_t tmp[1024];
        int32_t* xr = tmp;
        int32_t* heap = NULL;
        if (cols > 1024) { heap = (int32_t*)__builtin_malloc((size_t)cols * 4); xr = heap; }
        for (int64_t c = 0; c < cols; ++c) xr[c] = x[r * cols + c];
        ln_row(xr, gamma, beta, out + r * cols, cols, eps_q0, gamma_shift, out_shift, mode);
        if (heap) __builtin_free(heap);
    }
    return 0;
}

/* Residual add followed by LayerNorm; the intermediate is the saturating int8 add of a4o_add
 * (shift add_shift), so this equals a4o_add -> a4o_layernorm_i8. sum_out (nullable) receives the
 * int8 sum. The reference runs them as two kernels. */
A4O_EXPORT int a4o_add_layernorm_i8(const int8_t* a, const int8_t* b, int add_shift, int add_mode,
                                    const int16_t* gamma, const int16_t* beta, int8_t* sum_out, int8_t* out,
                                    int64_t rows, int64_t cols, int32_t eps_q0, int gamma_shift,
                                    int out_shift, int mode) {
    if (cols < 1 || cols > 65536 || out_shift < 0 || out_shift > 15 || eps_q0 < 1) return -1;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        int32_t* xr = (int32_t*)__builtin_malloc((size_t)cols * 4);
        for (int64_t c = 0; c < cols; ++c) {
            xr[c] = (int32_t)srs((int64_t)a[r * cols + c] + b[r * cols + c], add_shift, add_mode, A4O_I8);
            if (sum_out) sum_out[r * cols + c] = (int8_t)xr[c];
        }
        ln_row(xr, gamma, beta, out + r * cols, cols, eps_q0, gamma_shift, out_shift, mode);
        __builtin_free(xr);
    }
    return 0;
}

/* exp_score16: softmax.cpp:252-273. Q14 value of 2^(-d*KQ/256) for a logit gap d in [0,255].
 * All to_vector<int16>() calls run under rounding_mode::floor (softmax/parameters.h.jinja:23-27)
 * and saturate. Constants: EXP_A2=2811, EXP_B1=-11004, EXP_C0=16384, EXP_ZF=8
 * (softmax/parameters.h.jinja:19-22). */
A4O_EXPORT int32_t a4o_exp_score16(int32_t d, int32_t kq) {
    const int64_t z = srs((int64_t)d * kq, 0, A4O_RND_FLOOR, A4O_I16);
    const int64_t zint = z >> 8;
    const int64_t zfrac = z & 255;
    const int64_t t = srs(zfrac * 2811, 8, A4O_RND_FLOOR, A4O_I16);
    const int64_t inner = srs(t - 11004, 0, A4O_RND_FLOOR, A4O_I16); /* aie::add on int16 vectors */
    const int64_t t2 = srs(inner * zfrac, 8, A4O_RND_FLOOR, A4O_I16);
    int64_t e = (int16_t)(t2 + 16384);
    for (int b = 0; b < 4; ++b)
        if ((zint & (1 << b)) >= (1 << b)) e = e >> (1 << b); /* aie::downshift: arithmetic */
    if (zint >= 16) e = 0;
    return (int32_t)e;
}

/* Accurate integer-exp softmax over the last axis, int8 -> uint8 (A4O_U8) or int16 (A4O_I16).
 * softmax.cpp:333-384 (linear) / :279-329 (microtile, same arithmetic); reciprocal
 * softmax.cpp:108-127 == floor(NUMER / max(sum,1)); NUMER per softmax.h:22;
 * OUT_SHIFT = INV_SHIFT for uint8, 0 for int16 (softmax.h:144). */
A4O_EXPORT int a4o_softmax_exp_i8(const int8_t* x, void* out, int64_t rows, int64_t cols,
                                  int exp_kq, int inv_shift, int out_kind) {
    if (!(out_kind == A4O_U8 || out_kind == A4O_I16)) return -1;
    if (exp_kq < 1 || exp_kq > 128 || inv_shift < 1 || inv_shift > 23 || cols < 1 || cols > 65536) return -1;
    int16_t table[256];
    for (int d = 0; d < 256; ++d) table[d] = (int16_t)a4o_exp_score16(d, exp_kq);
    const int64_t numer = out_kind == A4O_I16 ? 32767 : ((int64_t)255 << inv_shift);
    const int out_shift = out_kind == A4O_I16 ? 0 : inv_shift;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const int8_t* xr = x + r * cols;
        int m = -128;
        for (int64_t c = 0; c < cols; ++c) if (xr[c] > m) m = xr[c];
        int64_t sum = 0;
        for (int64_t c = 0; c < cols; ++c) sum += table[m - xr[c]];
        const int64_t s = sum > 0 ? sum : 1;
        const int64_t q = numer / s;
        const int16_t inv16 = (int16_t)q; /* (int16_t)rinv[row], softmax.cpp:375 */
        for (int64_t c = 0; c < cols; ++c) {
            const int64_t prod = (int64_t)wrap32((int64_t)table[m - xr[c]] * inv16);
            store_kind(out, (size_t)(r * cols + c), out_kind, srs(prod, out_shift, A4O_RND_FLOOR, out_kind));
        }
    }
    return 0;
}

/* HCCS clipped-linear surrogate softmax, int8 -> uint8 / int16. softmax.cpp:19-88.
 * d = min(max - x, Dmax); score = B - S*d (acc32 -> int16 saturate); sum; inv = (255<<INV_SHIFT)/sum
 * or 32767/sum (C integer division), narrowed to int16 by the broadcast (softmax.cpp:79);
 * out = to_vector<out_t>(score*inv, OUT_SHIFT) under floor + saturate. */
A4O_EXPORT int a4o_softmax_hccs_i8(const int8_t* x, void* out, int64_t rows, int64_t cols,
                                   int B, int S, int Dmax, int inv_shift, int use_clb, int out_kind) {
    if (!(out_kind == A4O_U8 || out_kind == A4O_I16)) return -1;
    if (B < 0 || B > 32767 || S < 0 || S > 127 || Dmax < 0 || Dmax > 127) return -1;
    if (inv_shift < 1 || inv_shift > 23 || cols < 1 || cols > 65536) return -1;
    if (B - S * Dmax < 0) return -1;
    const int out_shift = out_kind == A4O_I16 ? 0 : inv_shift;
    int status = 0;
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        const int8_t* xr = x + r * cols;
        int m = -128;
        for (int64_t c = 0; c < cols; ++c) if (xr[c] > m) m = xr[c];
        int64_t sum = 0;
        for (int64_t c = 0; c < cols; ++c) {
            int d = (uint8_t)((uint8_t)m - (uint8_t)xr[c]);
            if (d > Dmax) d = Dmax;
            sum += srs((int64_t)B - (int64_t)S * d, 0, A4O_RND_FLOOR, A4O_I16);
        }
        if (sum <= 0) { status = -2; continue; }
        int64_t inv;
        if (use_clb) {
            int k = 31 - __builtin_clz((uint32_t)sum);
            if (out_kind == A4O_I16) inv = 32767 >> k;
            else inv = k <= inv_shift ? ((int64_t)255 << (inv_shift - k)) : 0;
        } else {
            inv = out_kind == A4O_I16 ? 32767 / sum : (((int64_t)255 << inv_shift) / sum);
        }
        const int16_t inv16 = (int16_t)inv;
        for (int64_t c = 0; c < cols; ++c) {
            int d = (uint8_t)((uint8_t)m - (uint8_t)xr[c]);
            if (d > Dmax) d = Dmax;
            const int64_t score = srs((int64_t)B - (int64_t)S * d, 0, A4O_RND_FLOOR, A4O_I16);
            const int64_t prod = (int64_t)wrap32(score * inv16);
            store_kind(out, (size_t)(r * cols + c), out_kind, srs(prod, out_shift, A4O_RND_FLOOR, out_kind));
        }
    }
    return status;
}

A4O_EXPORT int a4o_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

A4O_EXPORT void a4o_set_num_threads(int n) {
#ifdef _OPENMP
    if (n > 0) omp_set_num_threads(n);
#else
    (void)n;
#endif
}
