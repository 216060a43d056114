/*
 * aie4ml_gfx950.h — C ABI of libaie4ml_gfx950.so: the quantized operators aie4ml lowers
 * (Dense/GEMM + ReLU, dynamic MatMul, elementwise Add, integer LayerNorm, integer Softmax in its
 * accurate and HCCS-surrogate forms), executed on one AMD Instinct MI355X (gfx950).
 *
 * Conventions
 *  - Every pointer is a DEVICE pointer owned by the caller unless the comment says "host".
 *    The library never allocates, frees or copies to the host. Work is enqueued on `stream`
 *    (a hipStream_t passed as void*; NULL = the default stream) and the call returns without
 *    synchronising.
 *  - Tensors are plain row-major; `ld*` are row pitches in ELEMENTS, `stride_*` batch pitches in
 *    elements.
 *  - Return value: A4G_OK (0) or a negative a4g_status. a4g_last_error() returns a host string
 *    describing the last failure on the calling thread. Arguments are validated before any launch.
 *  - Results are bit-exact restatements of the reference's AIE kernels under
 *    aie::saturation_mode::saturate and the given aie::rounding_mode.
 *
 * The reference interface each entry point replaces is cited as file:line under
 * src/aie4ml/ of dimdano/aie4ml.
 */
#ifndef AIE4ML_GFX950_H
#define AIE4ML_GFX950_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Interface revision. Revisions 2xx and 3xx changed signatures that existed before (2xx: `trans_a` in a4g_dense_i8 and
 * a4g_matmul_i8; 3xx: `trans_a` in the 16-bit and floating-point Dense and MatMul), so a caller compiled against an
 * older header must not bind a newer library: compare a4g_version() with the header's value at load time. */
#define A4G_VERSION 300

#if defined(__GNUC__)
#define A4G_API __attribute__((visibility("default")))
#else
#define A4G_API
#endif

typedef void* a4g_stream_t; /* hipStream_t */

enum a4g_status {
    A4G_OK = 0,
    A4G_ERR_INVALID_ARGUMENT = -1, /* the reference would raise ValueError */
    A4G_ERR_UNSUPPORTED = -2,      /* the reference would raise NotImplementedError */
    A4G_ERR_WORKSPACE = -3,        /* workspace missing or too small */
    A4G_ERR_HIP = -4               /* a HIP runtime call failed (RuntimeError) */
};

/* aie::rounding_mode tokens, as produced by ROUNDING_TOKEN_MAP (op_impls/utils/precision.py:13-21).
 * positive_inf ("round half up"), negative_inf and conv_odd are AIE-API modes the reference
 * never emits; they are accepted for completeness. */
enum a4g_rounding {
    A4G_RND_FLOOR = 0,
    A4G_RND_CEIL = 1,
    A4G_RND_POSITIVE_INF = 2,
    A4G_RND_NEGATIVE_INF = 3,
    A4G_RND_SYMMETRIC_INF = 4,
    A4G_RND_SYMMETRIC_ZERO = 5,
    A4G_RND_CONV_EVEN = 6,
    A4G_RND_CONV_ODD = 7
};

/* storage kinds (AIEDataType.format, aie_types.py:42-90) */
enum a4g_kind { A4G_I8 = 0, A4G_U8 = 1, A4G_I16 = 2, A4G_U16 = 3, A4G_I32 = 4 };

A4G_API int a4g_version(void);
A4G_API const char* a4g_last_error(void);

/* Dynamic MatMul with an int16 left operand: the (16, 8) and (16, 16) width combinations of the matmul family
 * (op_impls/families/matmul/common.py:52; docs/support.md: "Dynamic MatMul: Int8/int16"), acc32 and acc64 as for
 * Dense. B is int8 or int16 (b_kind), [batch][K][ldb] or, with trans_b, [batch][N][ldb]; it is repacked per call
 * into the workspace (a4g_matmul_i16_workspace_bytes). Other arguments as a4g_matmul_i8, `trans_a` included: the left
 * operand stored as [batch][K][lda], lda >= M (TRANSPOSE_A, matmul.cpp:60-66), gathered while its tiles are staged. */
A4G_API size_t a4g_matmul_i16_workspace_bytes(int64_t batch, int64_t N, int64_t K, int b_kind);
A4G_API int a4g_matmul_i16(const int16_t* A, int trans_a, int64_t lda, int64_t stride_a, const void* B, int b_kind, int64_t ldb,
                   int64_t stride_b, int trans_b, void* C, int64_t ldc, int64_t stride_c, int64_t batch, int64_t M,
                   int64_t N, int64_t K, int shift, int round_mode, int out_kind, void* workspace, size_t workspace_bytes,
                   a4g_stream_t stream);

/* ---- Elementwise Add ---------------------------------------------------------------------------
 * out[i] = srs(a[i] + b[i], shift, round_mode) saturated to `kind` (int8 / uint8 / int16).
 * Replaces elementwise_add_kernel<Cfg>::run, templates/nnet_utils/elementwise_add/
 * elementwise_add.cpp:12-37, configured by AddOpImplVariant.resolve
 * (op_impls/families/elementwise/add.py:57-164: SHIFT, ROUNDING). */
A4G_API int a4g_add(const void* a, const void* b, void* out, int64_t n, int kind, int shift, int round_mode,
            a4g_stream_t stream);

/* ---- Dense weights -----------------------------------------------------------------------------
 * Packs a logical [K][N] int8 weight matrix (row pitch ldw) into the layout the GEMM consumes:
 * Wt[N][ldwt] with the reduction axis contiguous and zero-padded to ldwt = a4g_packed_ld(K), plus
 * colsum[n] = sum_k W[k][n] (needed when the activations are uint8). Device-side; replaces
 * pack_mmul_rhs_matrix (op_impls/families/matmul/common.py:307-358), which lays the same matrix
 * out in aie::mmul microtiles. */
A4G_API int64_t a4g_packed_ld(int64_t K);
A4G_API int a4g_pack_weights_i8(const int8_t* W, int64_t ldw, int64_t K, int64_t N, int8_t* Wt, int32_t* colsum,
                        a4g_stream_t stream);

/* ---- Dense (GEMM + bias + requantise + ReLU) ----------------------------------------------------
 * acc32 = bias[n] + sum_k A[m][k] * W[k][n];  y = saturate(round(acc >> shift));  relu: y = max(y,0).
 * Replaces dense_single/first/middle/last<Cfg>::run, templates/nnet_utils/dense_bias_relu/
 * dense_bias_relu.cpp:66-430, configured by _DenseVariantBase.resolve
 * (op_impls/families/matmul/dense.py:94-133) through variants/dense_bias_relu/parameters.h.jinja.
 *   A       [M][lda]  int8 or uint8 (a_kind); with trans_a != 0 the operand is stored transposed, [K][lda] with
 *           lda >= M, and is transposed inside the kernel while its tiles are staged (TRANSPOSE_A,
 *           dense_bias_relu.cpp:95-101, set from an io_view permutation of the input, dense.py:94-133)
 *   Wt      packed weights from a4g_pack_weights_i8, pitch ldwt
 *   colsum  [N] from a4g_pack_weights_i8; required iff a_kind == A4G_U8, else may be NULL
 *   bias    [N] int32 at accumulator scale, or NULL (USE_BIAS = false)
 *   shifts  [n_shift] int32 on the device; n_shift == 1 (the reference's scalar SHIFT) or == N
 *           (per-output-channel extension; identical to the reference when all entries are equal)
 *   Y       [M][ldy]  out_kind in {A4G_I8, A4G_U8, A4G_I16} */
A4G_API int a4g_dense_i8(const void* A, int a_kind, int trans_a, int64_t lda, const int8_t* Wt, int64_t ldwt,
                 const int32_t* colsum, const int32_t* bias, const int32_t* shifts, int n_shift,
                 int round_mode, int relu, int out_kind, void* Y, int64_t ldy, int64_t M, int64_t N,
                 int64_t K, a4g_stream_t stream);

/* The same Dense for a caller that also holds the weights in fragment order (the layout a matrix-core operand has
 * in registers; the counterpart of the microtile order pack_mmul_rhs_matrix gives the AIE kernels,
 * op_impls/families/matmul/common.py:307-358). Same arguments and results as a4g_dense_i8, plus
 *   Wf      a4g_rowpack_weights_i8 applied to Wt (a4g_rowpacked_bytes(N, K) bytes, 16-byte aligned), or NULL
 * With Wf, reductions of up to 768 with 16-byte aligned rows on both sides take a kernel that keeps a column block's
 * weights in registers and fetches them with whole-line loads (csrc/gemm_wrow.hip); every other shape, and a NULL Wf,
 * runs exactly as a4g_dense_i8. That kernel overlaps the requantisation with its matrix work where a block of 256
 * columns has every shift in 1..15 and every bias + 128 * colsum within +-2^30; other blocks take a form that refetches
 * the weights per row block and runs at about half the rate, below that of a4g_dense_i8: a caller that knows a layer's
 * shifts to lie outside 1..15 passes NULL. */
A4G_API int a4g_dense_i8_wf(const void* A, int a_kind, int trans_a, int64_t lda, const int8_t* Wt, int64_t ldwt,
                    const int8_t* Wf, const int32_t* colsum, const int32_t* bias, const int32_t* shifts, int n_shift,
                    int round_mode, int relu, int out_kind, void* Y, int64_t ldy, int64_t M, int64_t N,
                    int64_t K, a4g_stream_t stream);

/* Dense with int16 activations and int8 weights: the reference's (16, 8) width combination
 * (op_impls/families/matmul/common.py:52), accumulated in acc32 like the 8-bit case
 * (op_impls/utils/precision.py:120-121). Same arguments as a4g_dense_i8 with A [M][lda] int16 (lda in
 * elements); colsum (from a4g_pack_weights_i8) is always required: the low bytes of A are fed to the
 * matrix cores biased by 128. trans_a != 0: A is stored transposed, [K][lda] with lda >= M, and gathered while its
 * tiles are staged (TRANSPOSE_A, dense_bias_relu.cpp:95-101); the weights must then be a4g_pack_weights_i8's. */
A4G_API int a4g_dense_i16(const int16_t* A, int trans_a, int64_t lda, const int8_t* Wt, int64_t ldwt, const int32_t* colsum,
                  const int32_t* bias, const int32_t* shifts, int n_shift, int round_mode, int relu, int out_kind,
                  void* Y, int64_t ldy, int64_t M, int64_t N, int64_t K, a4g_stream_t stream);

/* Dense with int16 activations and int16 weights: the reference's (16, 16) combination, accumulated in acc64
 * (op_impls/families/matmul/common.py:52, op_impls/utils/precision.py:122-123), bias int32 at the accumulator
 * scale. a4g_pack_weights_i16 turns W [K][ldw] int16 into two byte planes [N][ld] (ld = K rounded up to 16:
 * signed high bytes; low bytes ^ 0x80) and colsum[n] = sum_k (W[k][n] - 128); K <= 32768 keeps every partial
 * sum exact. Shifts up to 62. Other arguments as a4g_dense_i16. */
A4G_API int a4g_pack_weights_i16(const int16_t* W, int64_t ldw, int64_t K, int64_t N, int8_t* Wt_hi, int8_t* Wt_lo,
                         int32_t* colsum, a4g_stream_t stream);
A4G_API int a4g_dense_i16x16(const int16_t* A, int trans_a, int64_t lda, const int8_t* Wt_hi, const int8_t* Wt_lo, int64_t ldwt,
                     const int32_t* colsum, const int32_t* bias, const int32_t* shifts, int n_shift, int round_mode,
                     int relu, int out_kind, void* Y, int64_t ldy, int64_t M, int64_t N, int64_t K, a4g_stream_t stream);

/* ---- Dynamic MatMul (both operands activations) --------------------------------------------------
 * C[b] = saturate(round((A[b] x B[b]) >> shift)), no bias, no ReLU, for b in [0, batch).
 * Replaces matmul_single/first/middle/last<Cfg>::run, templates/nnet_utils/matmul/matmul.cpp:31-390,
 * configured by _MatmulVariantBase.resolve (op_impls/families/matmul/matmul.py:47-98).
 *   A  [batch][M][lda]  int8 or uint8 (a_kind; uint8 = softmax probabilities). trans_a != 0: stored as
 *      [batch][K][lda], lda >= M — the left operand arrives as the last-two-axes transpose of its producer
 *      (TRANSPOSE_A, matmul.cpp:60-66; flag from matmul.py:78-81) and is transposed in-kernel, tile by tile.
 *   B  signed int8 (matmul.py:96-98). trans_b == 0: [batch][K][ldb] (logical K x N).
 *      trans_b == 1: [batch][N][ldb] — the operand arrives as the last-two-axes transpose of the
 *      producer tensor (io_view perm, matmul.py:86-95 / TRANSPOSE_B, matmul.cpp:70-76).
 *   C  [batch][M][ldc]  out_kind in {A4G_I8, A4G_U8, A4G_I16}
 * The reference accepts only batch == 1 for B (matmul/resolver.py:440-463); larger batches are
 * independent per-slice products. `workspace` must hold a4g_matmul_i8_workspace_bytes(...) bytes
 * (0 for some argument combinations, in which case it may be NULL). */
A4G_API size_t a4g_matmul_i8_workspace_bytes(int64_t batch, int64_t M, int64_t N, int64_t K, int trans_b, int a_kind);
A4G_API int a4g_matmul_i8(const void* A, int a_kind, int trans_a, int64_t lda, int64_t stride_a, const int8_t* B, int64_t ldb,
                  int64_t stride_b, int trans_b, void* C, int64_t ldc, int64_t stride_c, int64_t batch,
                  int64_t M, int64_t N, int64_t K, int shift, int round_mode, int out_kind, void* workspace,
                  size_t workspace_bytes, a4g_stream_t stream);

/* The same MatMul for callers that cannot allocate device memory or carry a workspace: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference. Arguments
 * and results are those of a4g_matmul_i8 without the workspace pair: the repacked right operand and its column sums
 * go to a fixed array of A4G_MATMUL_I8_STATIC_MAX_BYTES bytes of device memory that every GPU the library is used on
 * holds until the process ends. The call allocates and frees nothing. A problem whose
 * a4g_matmul_i8_workspace_bytes() exceeds the array returns A4G_ERR_WORKSPACE (shapes that need no workspace are
 * never rejected). All calls on one GPU share that GPU's array: calls that may overlap on one GPU (different
 * streams, different threads) race; the array keeps the last call's contents and nothing in it needs clearing. The
 * array's address is resolved on the first call on each device, which should be made outside stream capture. */
#define A4G_MATMUL_I8_STATIC_MAX_BYTES (16u << 20)
A4G_API int a4g_matmul_i8_static(const void* A, int a_kind, int trans_a, int64_t lda, int64_t stride_a, const int8_t* B, int64_t ldb,
                         int64_t stride_b, int trans_b, void* C, int64_t ldc, int64_t stride_c, int64_t batch,
                         int64_t M, int64_t N, int64_t K, int shift, int round_mode, int out_kind, a4g_stream_t stream);

/* ---- Integer LayerNorm, int8 -> int8, over the last axis -------------------------------------------
 * Replaces layernorm_i8<Cfg>::run / layernorm_i8_tiled<Cfg>::run and
 * layernorm_base<Cfg>::row_statistics, templates/nnet_utils/layer_norm/layer_norm.cpp:14-231,
 * configured by _LayerNormVariantBase.resolve (op_impls/families/layernorm/layer_norm.py:94-167).
 *   gamma  [cols] int16 Q7, beta [cols] int16 Q15 (layernorm/common.py:19-20)
 *   eps_q0 >= 1; gamma_shift = 7; out_shift in [0,15] = the output's fractional bits.
 * cols need not be a power of two (the reference requires it): mean and variance use exact floor
 * division, equal to the reference's shifts when cols is 2^k. */
A4G_API int a4g_layernorm_i8(const int8_t* x, const int16_t* gamma, const int16_t* beta, int8_t* out, int64_t rows,
                     int64_t cols, int32_t eps_q0, int gamma_shift, int out_shift, int round_mode,
                     a4g_stream_t stream);

/* Residual add fused in front of the LayerNorm: s = saturate_i8(round((a + b) >> add_shift));
 * out = layernorm(s). sum_out (nullable) receives s. Equals a4g_add followed by a4g_layernorm_i8
 * (the reference runs the two kernels back to back through a memory tile). */
A4G_API int a4g_add_layernorm_i8(const int8_t* a, const int8_t* b, int add_shift, int add_round_mode,
                         const int16_t* gamma, const int16_t* beta, int8_t* sum_out, int8_t* out, int64_t rows,
                         int64_t cols, int32_t eps_q0, int gamma_shift, int out_shift, int round_mode,
                         a4g_stream_t stream);

/* Dense, residual Add and LayerNorm in one launch: out = layernorm(saturate_i8(dense(A) + residual)), the tail of a
 * transformer sub-block. Equals a4g_dense_i8 (scalar shift, int8 output) followed by a4g_add_layernorm_i8 with
 * add_shift 0; the reference runs dense_bias_relu.cpp:66-166, elementwise_add.cpp:12-37 and layer_norm.cpp:14-121 as
 * three kernels with memory tiles between them. A workgroup computes complete output rows, so neither the Dense result
 * nor the sum is written to memory.
 *   Wf        the weights in fragment order: a4g_rowpack_weights_i8 applied to the Wt of a4g_pack_weights_i8
 *             (a4g_rowpacked_bytes(N, K) bytes, = N * K within this call's limits); colsum, bias as for a4g_dense_i8
 *   residual  [M][ld_res] int8 or NULL (LayerNorm of the Dense output itself)
 *   gamma, beta, eps_q0, gamma_shift, out_shift, ln_round_mode as for a4g_layernorm_i8 (cols = N)
 * Limits: N a multiple of 32 up to 768, K a multiple of 128 up to 4096, pitches multiples of 16, operands 16-byte
 * aligned; outside them the call returns A4G_ERR_UNSUPPORTED and the caller runs the two calls above. */
/* Fragment order: N is taken in groups of 32 columns and K in 128-byte tiles (both zero padded); the 1 KiB fragment
 * of (column group nb, K step ks of 32 bytes) lies at ((nb * (tiles * 4)) + ks) * 1024, 16 bytes per wavefront lane.
 * K a multiple of 16. Device-side, like a4g_pack_weights_i8. */
A4G_API int64_t a4g_rowpacked_bytes(int64_t N, int64_t K);
A4G_API int a4g_rowpack_weights_i8(const int8_t* Wt, int64_t ldwt, int64_t N, int64_t K, int8_t* Wf, a4g_stream_t stream);
A4G_API int a4g_dense_add_layernorm_i8(const void* A, int a_kind, int64_t lda, const int8_t* Wf, const int32_t* colsum,
                               const int32_t* bias, int shift, int dense_round_mode, int relu, const int8_t* residual,
                               int64_t ld_res, const int16_t* gamma, const int16_t* beta, int8_t* out, int64_t ld_out,
                               int64_t M, int64_t N, int64_t K, int32_t eps_q0, int gamma_shift, int out_shift,
                               int ln_round_mode, a4g_stream_t stream);

/* ---- Integer Softmax over the last axis, int8 -> uint8 (scale 1/256) or int16 -----------------------
 * Accurate form: 2nd-order integer exp. Replaces softmax_exp_i8<Cfg>::run /
 * softmax_exp_i8_tiled<Cfg>::run, exp_score16 and softmax_base<Cfg>::batched_reciprocal,
 * templates/nnet_utils/softmax/softmax.cpp:108-127,252-384, configured by
 * _SoftmaxExpBase._resolve_params (op_impls/families/softmax/softmax.py:309-349).
 *   exp_kq in [1,128]; inv_shift in [1,21] (the reference always uses 15). */
A4G_API int a4g_softmax_exp_i8(const int8_t* x, void* out, int64_t rows, int64_t cols, int exp_kq, int inv_shift,
                       int out_kind, a4g_stream_t stream);

/* HCCS clipped-linear surrogate: score = B - S*min(max-x, Dmax). Replaces
 * softmax_i8<Cfg>::softmax_row/run and softmax_i8_tiled<Cfg>::run,
 * templates/nnet_utils/softmax/softmax.cpp:19-239, configured by _SoftmaxHccsBase._resolve_params
 * (op_impls/families/softmax/softmax.py:258-283) under the constraints of validate_hccs_params
 * (op_impls/families/softmax/common.py:59-89), which this call re-checks. inv_shift in [1,23]. */
A4G_API int a4g_softmax_hccs_i8(const int8_t* x, void* out, int64_t rows, int64_t cols, int B, int S, int Dmax,
                        int inv_shift, int use_clb, int out_kind, a4g_stream_t stream);

/* ---- Fused multi-layer perceptron ---------------------------------------------------------------------
 * A chain of Dense layers evaluated in one launch with every weight matrix resident in LDS; same
 * arithmetic as calling a4g_dense_i8 per layer (scalar shift per layer). Replaces the chain of
 * dense_bias_relu_graph instances the reference wires for an hls4ml MLP
 * (templates/nnet_utils/dense_bias_relu/dense_bias_relu_graph.h:12-134).
 * `layers` is a HOST array. Limits: n_layers <= 8, every K and N <= 256, packed weights <= 96 KiB in
 * total; beyond them the call returns A4G_ERR_UNSUPPORTED and the caller runs layer by layer.
 * Two forms behind the one call, the same integers from both: batches below 512 samples (a chain of
 * latencies) take dot-product instructions on 16 or 64 samples per workgroup; from 512 samples the chain
 * runs on the matrix units, 32 samples per wave, the activations in registers from the first layer to the
 * last (rows at any address and pitch; fastest with ldx and X multiples of 16 bytes). A single narrow layer on a long batch (n_layers == 1, say
 * a million rows of 16 -> 64) is served by that form at the speed of its rows' traffic, 1.5 to 2 times
 * faster than a4g_dense_i8 up to 64 outputs (from 128 outputs on a4g_dense_i8 is ahead). */
typedef struct a4g_mlp_layer {
    const int8_t* wt;      /* packed weights (a4g_pack_weights_i8), pitch ldwt */
    int64_t ldwt;
    const int32_t* colsum; /* required iff the layer's input is uint8 */
    const int32_t* bias;   /* nullable */
    int32_t K, N;
    int32_t shift;
    int32_t relu;
    int32_t out_kind;      /* A4G_I8 or A4G_U8; becomes the next layer's input kind */
} a4g_mlp_layer;

A4G_API int a4g_mlp_i8(const a4g_mlp_layer* layers, int n_layers, const void* X, int x_kind, int64_t ldx, void* Y,
               int64_t ldy, int64_t batch, int round_mode, a4g_stream_t stream);

/* The same chain with the block's tail in the same launch:
 *   Y = LayerNorm(saturate_i8(chain(X) + residual))
 * i.e. a4g_mlp_i8 (int8 last layer) -> a4g_add (shift 0) -> a4g_layernorm_i8, the integers of those three calls. It is
 * what a small transformer block ends its two halves with: the attention output projection, or the pair of
 * feed-forward layers, then the residual Add (elementwise_add.cpp:12-37) and the LayerNorm (layer_norm.cpp:14-121) -
 * three kernels connected through memtile buffers in the reference's graph. A sample's row lies in two lanes of
 * the chain kernel, so the row sums cost one exchange. residual may be NULL; gamma int16 Q7, beta int16 Q15 as in
 * a4g_layernorm_i8, ln_round_mode its rounding, round_mode the layers'.
 * Limits: those of the chain's matrix-unit form (weight fragments within 128 KiB of LDS, any batch), an int8
 * last layer of N % 16 == 0 columns (N <= 256), Y and residual 16-byte aligned with pitches that are multiples
 * of 16; otherwise A4G_ERR_UNSUPPORTED, and the caller issues the three calls. */
A4G_API int a4g_mlp_add_layernorm_i8(const a4g_mlp_layer* layers, int n_layers, const void* X, int x_kind, int64_t ldx,
                             const int8_t* residual, int64_t ld_res, const int16_t* gamma, const int16_t* beta,
                             int8_t* Y, int64_t ldy, int64_t batch, int round_mode, int32_t eps_q0, int gamma_shift,
                             int out_shift, int ln_round_mode, a4g_stream_t stream);

/* ---- Fused attention core -----------------------------------------------------------------------------
 * O[b,h] = srs( softmax( srs(Q[b,h] x K[b,h]^T, logit_shift) ) x V[b,h], out_shift ) in one launch: the
 * chain MatMul (TRANSPOSE_B, matmul.cpp:70-115) -> Softmax (softmax.cpp:19-127 or 252-384) -> MatMul with
 * a uint8 left operand that the reference builds from three kernels (the graph of
 * scripts/check_onnx_bit_exact.py's attention models after fold_views.py / fold_scale.py). Same integer
 * operations in the same order as a4g_matmul_i8 -> a4g_softmax_*_i8 -> a4g_matmul_i8; the int8 logits and
 * the uint8 probabilities are never written to memory.
 *   Q [batch][heads][sq][d], K and V [batch][heads][sk][d], O [batch][heads][sq][d], all int8, feature
 *   axis contiguous. strides: 12 byte strides {batch, head, row} for Q, K, V, O in that order, so head
 *   slices of a packed QKV projection and a concatenated output need no copies.
 *   softmax_kind 0: accurate exp (exp_kq, inv_shift); 1: HCCS (hccs_B, hccs_S, hccs_Dmax, inv_shift,
 *   use_clb), same parameter rules as the stand-alone entries; probabilities are uint8.
 * Covered shapes: d a multiple of 16, up to 64 with 1 <= sk <= 512 and up to 128 with 1 <= sk <= 256 (head
 * dimensions 16, 48, 80, 96 and 112 run the 32-, 64- and 128-wide kernels with the missing 16-byte pieces of a row
 * masked; any key count: kernels exist for 1, 2, 4, 8 and 16 tiles of 32 keys, for head dimensions 48 and 64 also for
 * 3, 5, 6 and 12, and a count in between, e.g. 100 tokens, runs the next of them with the missing keys masked out),
 * any sq, pointers and strides multiples of 16 bytes, the keys of one head within 2 GiB; anything else returns A4G_ERR_UNSUPPORTED and the caller runs the three operators separately. */
A4G_API int a4g_attention_i8(const int8_t* Q, const int8_t* K, const int8_t* V, int8_t* O, int64_t batch, int64_t heads,
                     int64_t sq, int64_t sk, int64_t d, const int64_t* strides, int logit_shift,
                     int logit_round_mode, int softmax_kind, int exp_kq, int hccs_B, int hccs_S, int hccs_Dmax,
                     int inv_shift, int use_clb, int out_shift, int out_round_mode, a4g_stream_t stream);

/* ---- Floating-point compute path ------------------------------------------------------------------
 * The reference's float mode (FloatIntent tensors, passes/force_float_mode.py): bfloat16, float32 or fp8
 * e4m3 operands, float32 accumulation (acc_scalar_t = accfloat), results converted to the operand format:
 * round-to-nearest-even for bfloat16 / float32 (dense.py:105-127: shift 0, rounding_mode 'conv_even'), the
 * integer recipe of the reference's own packer for fp8 (matmul/common.py:262-276). Operands, weights and
 * results of one call share one format (resolver.py:125-129). Sizes and pitches count elements. */
enum a4g_float_format { A4G_BF16 = 16, A4G_F32 = 17, A4G_FP8 = 18 /* e4m3, bias 7, as the matrix cores read it */ };

/* Row pitch (elements) of a packed float weight matrix: rows start 16-byte aligned. */
A4G_API int64_t a4g_packed_ld_f(int64_t K, int fmt);
/* W [K][ldw] (the reference's [n_in][n_out], after pack_as_float, matmul/common.py:253-284)
 * -> Wt [N][a4g_packed_ld_f(K, fmt)], padding zero filled. */
A4G_API int a4g_pack_weights_f(const void* W, int fmt, int64_t ldw, int64_t K, int64_t N, void* Wt, a4g_stream_t stream);
/* Y = fmt(relu?(bias + A x W)). Replaces dense_single<Cfg>::run with float types,
 * templates/nnet_utils/dense_bias_relu/dense_bias_relu.cpp:66-166 (the bias is the accumulator's start
 * value, :112-124). A [M][lda] (trans_a != 0: stored transposed, [K][lda] with lda >= M, TRANSPOSE_A of
 * dense_bias_relu.cpp:95-101, gathered while its tiles are staged), Wt packed, bias float32 [N] or null, Y [M][ldy]. */
A4G_API int a4g_dense_f(const void* A, int fmt, int trans_a, int64_t lda, const void* Wt, int64_t ldwt, const float* bias, int relu, void* Y,
                int64_t ldy, int64_t M, int64_t N, int64_t K, a4g_stream_t stream);
/* C[b] = fmt(A[b] x B[b]). Replaces matmul_single<Cfg>::run with float types,
 * templates/nnet_utils/matmul/matmul.cpp:31-118. trans_b != 0: B is [batch][N][ldb] (the io_view swap of
 * matmul.py:84-98); otherwise B is [batch][K][ldb] and a workspace of a4g_matmul_f_workspace_bytes()
 * holds its transpose. trans_a != 0: A is [batch][K][lda], lda >= M (TRANSPOSE_A, matmul.cpp:60-66). */
A4G_API size_t a4g_matmul_f_workspace_bytes(int64_t batch, int64_t N, int64_t K, int trans_b, int fmt);
A4G_API int a4g_matmul_f(const void* A, int fmt, int trans_a, int64_t lda, int64_t stride_a, const void* B, int64_t ldb, int64_t stride_b,
                 int trans_b, void* C, int64_t ldc, int64_t stride_c, int64_t batch, int64_t M, int64_t N, int64_t K,
                 void* workspace, size_t workspace_bytes, a4g_stream_t stream);
/* out[i] = fmt(a[i] + b[i]). Replaces elementwise_add_kernel<Cfg>::run with float types,
 * templates/nnet_utils/elementwise_add/elementwise_add.cpp:12-37. */
A4G_API int a4g_add_f(const void* a, const void* b, void* out, int64_t n, int fmt, a4g_stream_t stream);

/* ---- Transposed operands of any width ------------------------------------------------------------------
 * dst[b][c][r] = src[b][r][c] for elements of 1, 2 or 4 bytes; pitches and batch strides in elements.
 * The kernels of the reference read a transposed operand through a transposing load
 * (templates/nnet_utils/matmul/matmul.cpp:60-66, dense_bias_relu.cpp:95-101, selected by transpose_lhs / transpose_rhs of
 * op_impls/families/matmul/matmul.py:78-98), and so does every Dense and MatMul entry point here (`trans_a`, `trans_b`).
 * This call is for a caller that wants the transposed copy itself, on the device and in memory it owns. */
A4G_API int a4g_transpose(const void* src, int elem_bytes, int64_t ld_src, int64_t stride_src, void* dst, int64_t ld_dst,
                  int64_t stride_dst, int64_t batch, int64_t rows, int64_t cols, a4g_stream_t stream);

/* ---- Concatenated results --------------------------------------------------------------------------------
 * rows windows of row_bytes bytes, pitches ld_src and ld_dst in bytes, copied device to device (the runtime's 2-D
 * copy; a memcpy node under stream capture). The reference never copies for Concat: its producers write their slices
 * of one memtile buffer (docs/support.md:13-15, passes/fold_views.py). A graph executor whose producers return tensors
 * of their own places each one in its slice of the concatenated tensor with this call. */
A4G_API int a4g_copy_2d(const void* src, int64_t ld_src, void* dst, int64_t ld_dst, int64_t rows, int64_t row_bytes,
                a4g_stream_t stream);

#ifdef __cplusplus
}
#endif
#endif /* AIE4ML_GFX950_H */
