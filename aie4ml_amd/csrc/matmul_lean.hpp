// LDS-light batched MatMul kernels for the two attention shapes: a short reduction (K <= 128) with the
// right operand given transposed, and a narrow result (N <= 128) with the right operand in [K][N] order.
// Both keep one operand's fragments in registers and stream the other, so a workgroup has no K-loop
// barriers; the tiled GEMM's fixed per-tile cost dominates exactly these shapes.
#pragma once

#include "common.hpp"

namespace a4g {

struct LeanArgs {
    const int8_t* A;
    const int8_t* B;
    int8_t* C;  // int8 or uint8 elements
    int64_t lda, stride_a, ldb, stride_b, ldc, stride_c;
    int M, N, K, batch;
    int a_unsigned;
    int lo, hi;  // saturation bounds of the output kind
    FastRound fr;
    ByteRequant br;  // fr with the clamp bounds moved in front of the shift (transposed-B kernel)
    float fscale;    // 2^-shift when the transposed-B kernel may requantise in float (nearest even), else 0
};

// C = srs(A x B^T): B is [N][ldb], K in {32,64,96,128}, N % 32 == 0. Returns false when not applicable.
bool lean_nt_applicable(const LeanArgs& a);
hipError_t launch_lean_nt(const LeanArgs& a, hipStream_t stream);

// C = srs(A x B): B is [K][ldb], N in {32,64,128}, K % 128 == 0, N * (K + 16) <= 60 KiB.
bool lean_nn_applicable(const LeanArgs& a);
hipError_t launch_lean_nn(const LeanArgs& a, hipStream_t stream);

}  // namespace a4g
