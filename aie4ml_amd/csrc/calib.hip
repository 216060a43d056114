// Calibration kernels: what the int8 matrix cores of this GPU sustain with no memory traffic at all, and the clock
// they run at while doing so. bench.py times them beside the GEMM so that "fraction of the 5.0 POP/s data-sheet peak"
// can be read next to "fraction of what this box sustains". A measurement aid with no counterpart in the reference:
// it is built into a library of its own (libaie4ml_bench_gfx950.so), not into the one an integrator ships.
#include "common.hpp"

namespace a4g {

// Every wave keeps TM x TN = 4 x 2 accumulator blocks (the GEMM kernel's wave tile) in registers and issues
// v_mfma_i32_32x32x32_i8 back to back on operands that never leave registers. Two operand sets alternate so that the
// multiplier inputs toggle the way streamed operands do. clocks[2*block] = shader-clock ticks, [2*block+1] = ticks of
// the 100 MHz constant counter over the same interval (wave 0 of each workgroup).
// `zero`: all-zero operands instead (the same instruction stream with nothing toggling in the multipliers: what the
// power limit leaves when the data costs nothing).
__global__ __launch_bounds__(256) void calib_mfma_i8_kernel(int iters, int zero, int* __restrict__ sink,
                                                            unsigned long long* __restrict__ clocks) {
    const unsigned seed = zero ? 0u : (blockIdx.x * 256u + threadIdx.x) * 2654435761u;
    v4i a[2][4], b[2][2];
#pragma unroll
    for (int s = 0; s < 2; ++s) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) a[s][i][r] = zero ? 0 : static_cast<int>((seed ^ (0x9E3779B9u * (s * 16 + i * 4 + r + 1))) * 0x85EBCA6Bu);
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) b[s][j][r] = zero ? 0 : static_cast<int>((seed ^ (0xC2B2AE35u * (s * 8 + j * 4 + r + 1))) * 0x27D4EB2Fu);
    }
    v16i acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;

    const unsigned long long c0 = __builtin_amdgcn_s_memtime();
    const unsigned long long r0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(b[s][j], a[s][i], acc[i][j], 0, 0, 0);
    }
    int x = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) x ^= acc[i][j][r];
    const unsigned long long c1 = __builtin_amdgcn_s_memtime();
    const unsigned long long r1 = __builtin_amdgcn_s_memrealtime();
    if (x == 0x7fffffff) sink[0] = x;  // keeps the accumulators alive; practically never taken
    if (threadIdx.x == 0 && clocks) {
        clocks[2 * blockIdx.x] = c1 - c0;
        clocks[2 * blockIdx.x + 1] = r1 - r0;
    }
}

}  // namespace a4g

using namespace a4g;

#define A4G_BENCH_API extern "C" __attribute__((visibility("default")))

// operations of one launch: per wave and iteration 2 operand sets x 8 MFMAs x 2 * 32 * 32 * 32; 4 waves per workgroup
A4G_BENCH_API int64_t a4g_calib_mfma_i8_ops(int blocks, int iters) { return static_cast<int64_t>(blocks) * 4 * iters * 16 * 65536; }

// 0, or -1 for arguments out of range, or a HIP error code. clocks (nullable, 2 * blocks entries) receives per workgroup
// the shader-clock ticks and the 100 MHz counter ticks over the loop; sink: one int of device memory (never written in
// practice).
A4G_BENCH_API int a4g_calib_mfma_i8(int blocks, int iters, int zero, int* sink, unsigned long long* clocks, void* stream) {
    if (blocks < 1 || blocks > (1 << 20) || iters < 1 || iters > (1 << 24) || sink == nullptr) return -1;
    calib_mfma_i8_kernel<<<blocks, 256, 0, static_cast<hipStream_t>(stream)>>>(iters, zero, sink, clocks);
    return static_cast<int>(hipGetLastError());
}
