// See matmul_lean.hpp. Arithmetic is that of matmul.cpp:80-115: int32 accumulation, shift / round /
// saturate; a uint8 left operand is read as int8 after ^0x80 and corrected by 128 * column sum.
//
// Shared conventions (MFMA operands swapped, so lanes are rows): lane (m, half) supplies bytes
// [16*half, 16*half+16) of each 32-wide k step of row m, and receives 16 results of row m. The lane that
// supplies column j of the right operand may load any actual column: it loads column
// 16*h' + 4*g + i for j = 8*g + 4*h' + i, which makes a lane's 16 results 16 CONTIGUOUS output bytes.
#include "matmul_lean.hpp"

namespace a4g {

typedef unsigned v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ int lean_col(int j) { return ((j >> 2) & 1) * 16 + (j >> 3) * 4 + (j & 3); }

// ---- A x B^T, short K ----------------------------------------------------------------------------------
// grid: (row blocks of 128, column chunks of 512, batch); 4 waves x 32 rows; A fragments live in registers.
// Columns are processed in groups of TG tiles of 32. Within a group the lane that supplies MFMA column
// j = 8*g + 4*h' + i of tile T loads actual column (16*TG)*h' + 16*T + 4*g + i, so that lane (m, half) ends
// the group with 16*TG contiguous output bytes of row m (a whole 128-byte line per row for TG = 4).
template <int DT, int TG>
__device__ __forceinline__ void lean_nt_load(const LeanArgs& a, __amdgpu_buffer_rsrc_t rsrc_b, v4i (&bf)[TG][DT], int col0, int m, int half) {
    const int g = m >> 3, hp = (m >> 2) & 1, i = m & 3;
#pragma unroll
    for (int T = 0; T < TG; ++T) {
        const int col = col0 + 16 * TG * hp + 16 * T + 4 * g + i;
        // a column past the matrix lies past the descriptor and reads as zero: no branch around the load
#pragma unroll
        for (int ks = 0; ks < DT; ++ks)
            bf[T][ks] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_b, col * static_cast<int>(a.ldb) + ks * 32 + half * 16, 0, 0));
    }
}

// A group of four tiles (128 columns) leaves lane (m, half) with bytes [64*half, 64*half + 64) of row m. Stored
// as they are, every 16-byte piece is a write request of its own to L2; a round trip through a wave-private
// LDS patch (32 rows x 128 bytes, rows padded to 144 for conflict-free access) regroups them so that eight
// consecutive lanes write one whole 128-byte line.
constexpr int LEAN_PATCH_PITCH = 144;
constexpr int LEAN_PATCH_BYTES = 32 * LEAN_PATCH_PITCH;

template <int DT, int TG, int RB, int BIT, bool UOUT>
__device__ __forceinline__ void lean_nt_compute(const LeanArgs& a, __amdgpu_buffer_rsrc_t rsrc_c, const v4i (&af)[RB][DT], const v4i (&bf)[TG][DT],
                                                int col0, int lane, const int (&row)[RB], const bool (&row_ok)[RB],
                                                int8_t* patch, int row_base) {
    const int m = lane & 31, half = lane >> 5;
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        v4i o[TG];
#pragma unroll
        for (int T = 0; T < TG; ++T) {
            // BIT == 3: the sums start from the bit pattern of the float 1.5 * 2^23. Floats of that binade are one apart,
            // so adding an integer x (|x| <= K * 2^14 <= 2^21 here) to the pattern gives the pattern of 1.5 * 2^23 + x:
            // the accumulators leave the matrix unit already converted, and one fused multiply-add with the constant
            // bias - 1.5 * 2^23 * 2^-s yields x * 2^-s + bias exactly (every term a multiple of 2^-s below 2^24).
            constexpr int START = BIT == 3 ? 0x4B400000 : 0;
            v16i acc = {START, START, START, START, START, START, START, START, START, START, START, START, START, START, START, START};
#pragma unroll
            for (int ks = 0; ks < DT; ++ks) acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[T][ks], af[rb][ks], acc, 0, 0, 0);
#pragma unroll
            for (int gg = 0; gg < 4; ++gg) {
                if (BIT == 3) {
                    // v_cvt_pk_u8_f32 rounds to nearest even, saturates to 0..255 and places the byte
                    const float bias = (UOUT ? 0.f : 128.f) - 12582912.f * a.fscale;
                    unsigned w = 0;
#pragma unroll
                    for (int t = 0; t < 4; ++t) {
                        const int sum_bits = acc[4 * gg + t];  // (a bit cast applied to the vector's element reads element 0)
                        const float v = fmaf(__builtin_bit_cast(float, sum_bits), a.fscale, bias);
                        if (t == 0) w = __builtin_amdgcn_cvt_pk_u8_f32(v, 0, w);
                        if (t == 1) w = __builtin_amdgcn_cvt_pk_u8_f32(v, 1, w);
                        if (t == 2) w = __builtin_amdgcn_cvt_pk_u8_f32(v, 2, w);
                        if (t == 3) w = __builtin_amdgcn_cvt_pk_u8_f32(v, 3, w);
                    }
                    o[T][gg] = static_cast<int>(UOUT ? w : w ^ 0x80808080u);
                } else {
                    o[T][gg] = static_cast<int>(requant4_bytes<BIT>(acc[4 * gg], acc[4 * gg + 1], acc[4 * gg + 2], acc[4 * gg + 3], a.br));
                }
            }
        }
        if (TG == 4) {
#pragma unroll
            for (int T = 0; T < TG; ++T)
                *reinterpret_cast<v4i*>(patch + m * LEAN_PATCH_PITCH + 64 * half + 16 * T) = o[T];
            const int r0 = row_base + rb * 32;
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4) {
                const int r = 8 * s4 + (lane >> 3), c = lane & 7;
                const v4i v = *reinterpret_cast<const v4i*>(patch + r * LEAN_PATCH_PITCH + 16 * c);
                // a row past the matrix lies past the descriptor: the store is dropped, again without a branch
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, v), rsrc_c, (r0 + r) * static_cast<int>(a.ldc) + col0 + 16 * c, 0, 0);
            }
        } else {
#pragma unroll
            for (int T = 0; T < TG; ++T)
                __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, o[T]), rsrc_c,
                                                       row[rb] * static_cast<int>(a.ldc) + col0 + 16 * TG * half + 16 * T, 0, 0);
        }
    }
}

// RB = 32-row blocks per wave: 2 (256 rows per workgroup) halves how often B is re-read.
template <int DT, int RB, int BIT, bool UOUT>
__global__ __launch_bounds__(256, 2) void matmul_lean_nt_kernel(LeanArgs a) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = lane & 31, half = lane >> 5;
    __shared__ __attribute__((aligned(16))) int8_t patches[4 * LEAN_PATCH_BYTES];
    int8_t* patch = patches + wave * LEAN_PATCH_BYTES;
    const int row_base = blockIdx.x * (128 * RB) + wave * RB * 32;
    const int8_t* Ap = a.A + blockIdx.z * a.stride_a;
    // B and C of this problem behind descriptors that end with the matrices. The compiler counts outstanding memory
    // operations from the youngest back, and a load or store inside a branch makes every later wait a wait for
    // everything: with them the prefetch of the next column group was waited for at once, before the arithmetic it was
    // meant to overlap.
    const auto rsrc_b = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.B + blockIdx.z * a.stride_b), 0,
                                                          (a.N - 1) * static_cast<int>(a.ldb) + a.K, 0x00020000);
    const auto rsrc_c = __builtin_amdgcn_make_buffer_rsrc(a.C + blockIdx.z * a.stride_c, 0, (a.M - 1) * static_cast<int>(a.ldc) + a.N,
                                                          0x00020000);
    const int c0 = blockIdx.y * 512, c1 = min(c0 + 512, a.N);

    int row[RB];
    bool row_ok[RB];
    v4i af[RB][DT];
#pragma unroll
    for (int rb = 0; rb < RB; ++rb) {
        row[rb] = blockIdx.x * (128 * RB) + (wave * RB + rb) * 32 + m;
        row_ok[rb] = row[rb] < a.M;
        const int64_t rowc = row_ok[rb] ? row[rb] : a.M - 1;
#pragma unroll
        for (int ks = 0; ks < DT; ++ks) af[rb][ks] = *reinterpret_cast<const v4i*>(Ap + rowc * a.lda + ks * 32 + half * 16);
    }
    int col = c0;
    if (col + 128 <= c1) {
        v4i bf[4][DT], nbf[4][DT];
        lean_nt_load<DT, 4>(a, rsrc_b, bf, col, m, half);
        for (; col + 128 <= c1; col += 128) {
            lean_nt_load<DT, 4>(a, rsrc_b, nbf, col + 128, m, half);  // in flight during the arithmetic below (zeros past the end)
            lean_nt_compute<DT, 4, RB, BIT, UOUT>(a, rsrc_c, af, bf, col, lane, row, row_ok, patch, row_base);
#pragma unroll
            for (int T = 0; T < 4; ++T)
#pragma unroll
                for (int ks = 0; ks < DT; ++ks) bf[T][ks] = nbf[T][ks];
        }
    }
    for (; col < c1; col += 32) {
        v4i bf[1][DT];
        lean_nt_load<DT, 1>(a, rsrc_b, bf, col, m, half);
        lean_nt_compute<DT, 1, RB, BIT, UOUT>(a, rsrc_c, af, bf, col, lane, row, row_ok, patch, row_base);
    }
}

// ---- A x B, narrow N -----------------------------------------------------------------------------------
// grid: (row blocks of 128, batch); B^T is staged once per workgroup in LDS ([N][K + 16] bytes, natural k
// order); a lane streams 64 contiguous bytes of its A row per group of 128 k (k order inside a group is
// permuted identically for both operands, which an integer dot product cannot see).
template <int NTL>
__global__ __launch_bounds__(256, 2) void matmul_lean_nn_kernel(LeanArgs a, int row_blocks) {
    extern __shared__ __attribute__((aligned(16))) int8_t lean_smem[];
    constexpr int N = NTL * 32;
    const int pitch = a.K + 16;
    int8_t* bt = lean_smem;
    int* colsum = reinterpret_cast<int*>(lean_smem + N * pitch);

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, half = lane >> 5;
    const int8_t* Ap = a.A + blockIdx.y * a.stride_a;
    const int8_t* Bp = a.B + blockIdx.y * a.stride_b;
    int8_t* Cp = a.C + blockIdx.y * a.stride_c;
    // a workgroup transposes B once and then takes `row_blocks` consecutive blocks of 128 rows
    int row = blockIdx.x * row_blocks * 128 + wave * 32 + m;
    // A and C of this problem behind descriptors that end with the matrices: a row past the end reads as zero and its
    // store is dropped, so that neither the prefetch of the next group nor a store sits inside a branch (the compiler
    // would otherwise wait for the prefetch at once, see matmul_lean_nt_kernel)
    constexpr unsigned NOWHERE = 0x80000000u;
    const int lda = static_cast<int>(a.lda), ldc = static_cast<int>(a.ldc);
    const auto rsrc_a = __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(Ap), 0, (a.M - 1) * lda + a.K, 0x00020000);
    const auto rsrc_c = __builtin_amdgcn_make_buffer_rsrc(Cp, 0, (a.M - 1) * ldc + N, 0x00020000);
    unsigned aoff = row < a.M ? static_cast<unsigned>(row * lda + half * 64) : NOWHERE;
    auto load_a = [&](unsigned off) { return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_a, off, 0, 0)); };

    const int groups = a.K >> 7;
    v4i af[4], af_next[4];  // the group being multiplied and the one in flight
#pragma unroll
    for (int s = 0; s < 4; ++s) af[s] = load_a(aoff + s * 16);

    if (tid < N) colsum[tid] = 0;
    __syncthreads();
    {
        // 4x4 byte blocks of B transposed through registers; 256 % (N/4) == 0 keeps a thread on its columns
        const int nb = (a.K >> 2) * (N / 4);
        const int n0 = (tid % (N / 4)) * 4;
        int part[4] = {0, 0, 0, 0};
        // four blocks' loads are issued before the first is transposed: one exposed load latency per four blocks
        for (int blk0 = tid; blk0 < nb; blk0 += 4 * 256) {
            unsigned av[4][4];
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int blk = blk0 + u * 256;
                const int k0 = (min(blk, nb - 1) / (N / 4)) * 4;
#pragma unroll
                for (int i = 0; i < 4; ++i) av[u][i] = *reinterpret_cast<const unsigned*>(Bp + static_cast<int64_t>(k0 + i) * a.ldb + n0);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const int blk = blk0 + u * 256;
                if (blk >= nb) break;
                const int k0 = (blk / (N / 4)) * 4;
                unsigned cv[4];
                const unsigned lo01 = __builtin_amdgcn_perm(av[u][1], av[u][0], 0x05010400u);
                const unsigned hi01 = __builtin_amdgcn_perm(av[u][1], av[u][0], 0x07030602u);
                const unsigned lo23 = __builtin_amdgcn_perm(av[u][3], av[u][2], 0x05010400u);
                const unsigned hi23 = __builtin_amdgcn_perm(av[u][3], av[u][2], 0x07030602u);
                cv[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
                cv[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
                cv[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
                cv[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    *reinterpret_cast<unsigned*>(bt + (n0 + j) * pitch + k0) = cv[j];
                    part[j] = __builtin_amdgcn_sdot4(static_cast<int>(cv[j]), 0x01010101, part[j], false);
                }
            }
        }
        if (a.a_unsigned) {
#pragma unroll
            for (int j = 0; j < 4; ++j) atomicAdd(&colsum[n0 + j], part[j]);
        }
    }
    __syncthreads();

    const int xm = a.a_unsigned ? static_cast<int>(0x80808080u) : 0;
    const int8_t* brow = bt + lean_col(m) * pitch + half * 64;
    for (int rbk = 0; rbk < row_blocks; ++rbk) {
    v16i acc[NTL];
#pragma unroll
    for (int u = 0; u < NTL; ++u) acc[u] = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    auto multiply = [&](const v4i (&grp)[4], int G) {
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            v4i av = grp[s];
            av[0] ^= xm; av[1] ^= xm; av[2] ^= xm; av[3] ^= xm;
#pragma unroll
            for (int u = 0; u < NTL; ++u) {
                const v4i bv = *reinterpret_cast<const v4i*>(brow + u * 32 * pitch + G * 128 + s * 16);
                acc[u] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bv, av, acc[u], 0, 0, 0);
            }
        }
    };
    // the next block's first group is requested while this block's last group is multiplied
    const int next_row = row + 128;
    const bool more = rbk + 1 < row_blocks && (blockIdx.x * row_blocks + rbk + 1) * 128 < a.M;
    const unsigned next_aoff = more && next_row < a.M ? static_cast<unsigned>(next_row * lda + half * 64) : NOWHERE;
    for (int G = 0; G < groups; ++G) {
        // One group ahead; three groups ahead through a ring of four register sets measured the same (C3 P x V: 29.0 us
        // either way, the rate of a plain copy on that box).
        const unsigned pre = G + 1 < groups ? aoff + (G + 1) * 128 : next_aoff;
#pragma unroll
        for (int s = 0; s < 4; ++s) af_next[s] = load_a(pre + s * 16);
        __builtin_amdgcn_sched_barrier(0);  // the requests stay in front of the arithmetic they are meant to overlap
        multiply(af, G);
#pragma unroll
        for (int s = 0; s < 4; ++s) af[s] = af_next[s];
    }

#pragma unroll
    for (int u = 0; u < NTL; ++u) {
        v4i o;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const v4i cs = *reinterpret_cast<const v4i*>(colsum + 32 * u + 16 * half + 4 * g);
            int y[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) y[i] = clamp_i(fast_round(acc[u][4 * g + i] + 128 * cs[i], a.fr), a.lo, a.hi);
            o[g] = static_cast<int>(pack4_bytes(y[0], y[1], y[2], y[3]));
        }
        __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(v4u, o), rsrc_c,
                                               row < a.M ? static_cast<unsigned>(row * ldc + 32 * u + 16 * half) : NOWHERE, 0, 0);
    }
    if (!more) break;
    row = next_row;
    aoff = next_aoff;
    }  // row blocks
}

static bool lean_common_ok(const LeanArgs& a) {
    return aligned16(a.A) && aligned16(a.B) && aligned16(a.C) && a.lda % 16 == 0 && a.ldb % 16 == 0 && a.ldc % 16 == 0 &&
           a.stride_a % 16 == 0 && a.stride_b % 16 == 0 && a.stride_c % 16 == 0 && a.fr.s <= 24 && a.batch <= 65535 && a.M >= 1;
}

bool lean_nt_applicable(const LeanArgs& a) {
    return lean_common_ok(a) && !a.a_unsigned && a.K % 32 == 0 && a.K <= 128 && a.N % 32 == 0 && a.N <= 512 * 65535 &&
           byte_requant_ok(a.fr) && (static_cast<int64_t>(a.N) + 128) * a.ldb < (int64_t{1} << 31) &&
           (static_cast<int64_t>(a.M) + 512) * a.ldc < (int64_t{1} << 31);  // 32-bit offsets inside one problem
}

template <int DT, int RB>
static void launch_lean_nt_cfg(const LeanArgs& a, dim3 grid, hipStream_t stream) {
    const int bit = a.fscale > 0.f ? 3 : fast_round_kind(a.fr);  // 3: nearest even in float arithmetic
    const bool uo = a.lo == 0;
#define A4G_NT(B)                                                                          \
    if (uo)                                                                                \
        matmul_lean_nt_kernel<DT, RB, B, true><<<grid, 256, 0, stream>>>(a);               \
    else                                                                                   \
        matmul_lean_nt_kernel<DT, RB, B, false><<<grid, 256, 0, stream>>>(a);
    if (bit == 0) { A4G_NT(0) } else if (bit == 1) { A4G_NT(1) } else if (bit == 2) { A4G_NT(2) } else { A4G_NT(3) }
#undef A4G_NT
}

template <int RB>
static void launch_lean_nt_rb(const LeanArgs& a, hipStream_t stream) {
    const dim3 grid(static_cast<unsigned>((a.M + 128 * RB - 1) / (128 * RB)), static_cast<unsigned>((a.N + 511) / 512),
                    static_cast<unsigned>(a.batch));
    switch (a.K / 32) {
    case 1: launch_lean_nt_cfg<1, RB>(a, grid, stream); break;
    case 2: launch_lean_nt_cfg<2, RB>(a, grid, stream); break;
    case 3: launch_lean_nt_cfg<3, RB>(a, grid, stream); break;
    default: launch_lean_nt_cfg<4, RB>(a, grid, stream); break;
    }
}

hipError_t launch_lean_nt(const LeanArgs& a, hipStream_t stream) {
    if (a.M > 128)
        launch_lean_nt_rb<2>(a, stream);
    else
        launch_lean_nt_rb<1>(a, stream);
    return hipGetLastError();
}

bool lean_nn_applicable(const LeanArgs& a) {
    return lean_common_ok(a) && (a.N == 32 || a.N == 64 || a.N == 128) && a.K % 128 == 0 &&
           static_cast<int64_t>(a.N) * (a.K + 16) + a.N * 4 <= 60 * 1024 &&
           (static_cast<int64_t>(a.M) + 128) * a.lda < (int64_t{1} << 31) &&
           (static_cast<int64_t>(a.M) + 128) * a.ldc < (int64_t{1} << 31);  // 32-bit offsets inside one problem
}

hipError_t launch_lean_nn(const LeanArgs& a, hipStream_t stream) {
    // Transposing B into LDS is a fixed cost per workgroup: with many 128-row blocks per problem a workgroup takes
    // several of them, as long as two workgroups per CU remain (C3: one workgroup per head, 29.0 us against 34.6 us
    // with one 128-row block each).
    const int64_t blocks = (a.M + 127) / 128;
    int row_blocks = 1;
    while (row_blocks < 8 && blocks % (row_blocks * 2) == 0 && (blocks / (row_blocks * 2)) * a.batch >= 512) row_blocks *= 2;
    const dim3 grid(static_cast<unsigned>((blocks + row_blocks - 1) / row_blocks), static_cast<unsigned>(a.batch));
    const size_t lds = static_cast<size_t>(a.N) * (a.K + 16) + a.N * 4;
    switch (a.N / 32) {
    case 1: matmul_lean_nn_kernel<1><<<grid, 256, lds, stream>>>(a, row_blocks); break;
    case 2: matmul_lean_nn_kernel<2><<<grid, 256, lds, stream>>>(a, row_blocks); break;
    default: matmul_lean_nn_kernel<4><<<grid, 256, lds, stream>>>(a, row_blocks); break;
    }
    return hipGetLastError();
}

}  // namespace a4g
