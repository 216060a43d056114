// Fused attention core: O = srs( softmax_int( srs(Q K^T) ) V ) for every (batch, head), in ONE launch.
// It performs exactly the integer operations of the three reference kernels it replaces, in the same
// order — MatMul (matmul.cpp:80-115) with the K operand transposed, Softmax in either form
// (softmax.cpp:19-127 / 252-384), MatMul with a uint8 left operand — so the result is bit-identical to
// running them one after another; the int8 logits and uint8 probabilities simply never leave the CU.
//
// A wave owns 32 query rows. With the MFMA operands swapped (lanes = rows), lane (m, half) ends each
// 32x32 logit tile with 16 values of row m: columns 32t + 8g + 4*half + i. They are requantised and packed
// to four dwords per tile and stay in registers: the row maximum and the score sum are in-lane reductions
// plus one exchange between the two lanes of a row. The probabilities are then fed to the second MFMA
// straight from those registers: integer dot products do not care about the order of k, so step t uses the
// k-set a lane already holds, and V^T is laid out in LDS in the matching order.
#include <algorithm>

#include "common.hpp"
#include "softmax_common.hpp"

namespace a4g {

struct AttnArgs {
    const int8_t* Q;
    const int8_t* K;
    const int8_t* V;
    int8_t* O;
    int64_t q_sb, q_sh, q_ss;  // byte strides: batch, head, row (the feature axis is contiguous)
    int64_t k_sb, k_sh, k_ss;
    int64_t v_sb, v_sh, v_ss;
    int64_t o_sb, o_sh, o_ss;
    int heads, sq;
    int d;      // head dimension that exists, a multiple of 16 up to the kernel's width: the 16-byte pieces of a row past it do not
    int sk;     // key / value rows that exist (the ragged form; the kernel's tiles cover the next tile count that has an instance)
    int items;  // (batch, head, block of query rows) triples in all
    FastRound lr, orr;  // logits and output requantisation
    SoftmaxParams sm;
    int noclamp;
    float lscale;  // 2^-logit_shift, for the float form of the logit requantisation
};

// 4x4 byte transpose: in a[i] byte j  ->  out c[j] byte i.
__device__ __forceinline__ void transpose4x4(const unsigned a[4], unsigned c[4]) {
    const unsigned lo01 = __builtin_amdgcn_perm(a[1], a[0], 0x05010400u);
    const unsigned hi01 = __builtin_amdgcn_perm(a[1], a[0], 0x07030602u);
    const unsigned lo23 = __builtin_amdgcn_perm(a[3], a[2], 0x05010400u);
    const unsigned hi23 = __builtin_amdgcn_perm(a[3], a[2], 0x07030602u);
    c[0] = __builtin_amdgcn_perm(lo23, lo01, 0x05040100u);
    c[1] = __builtin_amdgcn_perm(lo23, lo01, 0x07060302u);
    c[2] = __builtin_amdgcn_perm(hi23, hi01, 0x05040100u);
    c[3] = __builtin_amdgcn_perm(hi23, hi01, 0x07060302u);
}

// NT = key/value rows / 32, DT = head dimension / 32. 256 threads = 4 waves = 128 query rows of one head.
// BIT: rounding kind of the logits (fast_round_kind), or 3: round to nearest even done in float arithmetic -
// |acc| <= D * 2^14 and the bias 2^(7+shift) stay below 2^24, so (acc + 128 * 2^s) * 2^-s is exact in a float and
// v_cvt_pk_u8_f32 (nearest even, saturating to 0..255, writing one byte of a dword) is the rounding, the int8
// saturation (biased by 128) and the packing at once. FASTP: the probabilities need no clamp and their shift is
// at most 16, so p = (e * inv) >> shift is read as byte 2 of e * (inv << (16 - shift)).
// RAGGED: fewer keys exist than the NT tiles cover (any count >= 1). K and V rows past the end load as zero; their
// logits are forced to the minimum (they cannot raise the row maximum), their scores
// to zero (they add nothing to the row sum, and a zero probability times a zero V row nothing to the output).
// NW = waves per workgroup. 4: two workgroups share a CU. 8: one workgroup of 256 query rows per CU, which
// leaves room to store the score table once per LDS bank (entry d for lane c at dword d * 64 + c, byte address
// (d << 8) | (c << 2) built by one v_perm): with a single copy, lanes that gather different gaps from one bank
// serialise, and those conflicts were two thirds of this kernel's LDS cycles.
template <int NT, int DT, int BIT, bool FASTP, int NW = 4, bool RAGGED = false>
__global__ __launch_bounds__(NW * 64, (NW == 8 || NW == 6) ? 1 : 2) void attention_kernel(AttnArgs a) {
    constexpr int SK = NT * 32, D = DT * 32, PITCH = SK + 16;
    constexpr bool BANKED = NW == 8 || NW == 6;  // 6: the same form on 192 query rows (384 queries are two such blocks)
    constexpr int THREADS = NW * 64, ROWS = NW * 32;
    // The score table is a static array: its LDS address is then a compile-time constant that folds into the
    // offset field of the gathers (an array inside the dynamic block costs one address add per gather).
    __shared__ int table[BANKED ? 256 * 64 : 256];                 // score of a gap d in [0,255]
    extern __shared__ __attribute__((aligned(16))) int8_t attn_smem[];
    int8_t* vt = attn_smem;                                        // V^T, k-permuted: [D][PITCH]
    int* colsum = reinterpret_cast<int*>(attn_smem + D * PITCH);   // sum_k V[k][n]
    // The 512-key form holds 64 logit and up to 128 score registers per lane at once; with everything else that is
    // a handful more than the 256 a lane has, and the compiler's spills went to scratch memory (18 MB of extra HBM
    // writes per launch). The scores of the last PARK tiles wait in LDS instead: slot s of thread t at dword
    // s * THREADS + t, so every access is conflict free.
    constexpr int PARK = (NT >= 16 && BANKED) ? 3 : 0;
    unsigned* parked = reinterpret_cast<unsigned*>(colsum + D);

    const int nblk = (a.sq + ROWS - 1) / ROWS;
    // The eight-wave form is persistent: one workgroup per CU takes a contiguous run of items (the blocks of query rows
    // of one head are neighbours, so its K and V are fetched once), builds the 64 KiB replicated score table once
    // instead of once per item.
    constexpr bool PERSIST = BANKED;
    // One item per workgroup: workgroups go to the eight XCDs round robin, so the items are renumbered to give an XCD
    // consecutive ones. Neighbouring heads of a packed projection share cache lines (a head's row is 64 bytes of a 128-byte
    // line); on one XCD, launched one after the other, the second finds in L2 what the first fetched.
    const int spread = (gridDim.x & 7) == 0 ? static_cast<int>((blockIdx.x & 7) * (gridDim.x >> 3) + (blockIdx.x >> 3)) : static_cast<int>(blockIdx.x);
    const int item_begin = PERSIST ? static_cast<int>(static_cast<int64_t>(blockIdx.x) * a.items / gridDim.x) : spread;
    const int item_end = PERSIST ? static_cast<int>(static_cast<int64_t>(blockIdx.x + 1) * a.items / gridDim.x) : item_begin + 1;

    // operand fragments straight from global memory: lane (m, half) holds bytes [16*half, 16*half+16) of
    // each 32-wide k step of its row. V is requested with them: a thread owns the 4x4 byte blocks blk = tid,
    // tid + THREADS, ... (rows k0..k0+3, its four columns n0..n0+3).
    constexpr int NB = (SK / 4) * (D / 4);
    constexpr int VB = (NB + THREADS - 1) / THREADS;
    const int wave_uniform = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // The items of a workgroup are taken head by head. A head's V^T and column sums are laid down once, between two
    // barriers; the blocks of query rows that follow touch nothing in LDS that another wave writes (the parked scores are
    // a thread's own), so their waves do not meet again until the next head and may drift a block apart meanwhile.
    for (int head_item = item_begin; head_item < item_end;) {
    const int bh = head_item / nblk;
    const int run_end = PERSIST ? min(item_end, (bh + 1) * nblk) : head_item + 1;
    // The thread's indices are formed again for every head from an opaque copy of its id: derived from the id itself,
    // the dozens of per-thread addresses below would be kept in registers across the whole loop, which the 512-key form
    // has none to spare for.
    int tid = threadIdx.x;
    if (PERSIST) {  // wave number from a scalar register, lane number counted afresh: no vector register is carried
        int lane_now;
        asm volatile("v_mbcnt_lo_u32_b32 %0, -1, 0\n\tv_mbcnt_hi_u32_b32 %0, -1, %0" : "=v"(lane_now));
        tid = wave_uniform * 64 + lane_now;
    }
    const int lane = tid & 63, wave = tid >> 6;
    const int m = lane & 31, half = lane >> 5;
    // A head dimension below the kernel's width (16 on the 32-wide kernel, 48 on the 64-wide, 80 .. 112 on the 128-wide):
    // the lanes whose 16-byte piece of a row does not exist fetch the row's first piece for Q (no access leaves the row)
    // and put zeros in its place, so that whatever the K fragment holds there counts nothing; K is read through a
    // descriptor that ends with the last row that exists; V columns past the dimension load as zero and output pieces
    // past it are not stored.
    const int hoff = half * 16;
    const int n0 = (tid % (D / 4)) * 4;  // THREADS % (D/4) == 0: a thread keeps its four columns
    const int b = bh / a.heads, h = bh - b * a.heads;
    // K fragments run KD - 1 tiles ahead of the matrix unit (a slot is fetched again as soon as its tile has been
    // multiplied): a tile's worth of work is a quarter of what a fetch from the L2 takes, and with one tile in flight the
    // first pass spent most of its time waiting for it
    constexpr int KD = NT < 4 ? NT : 4;
    v4i qf[DT], kf[KD][DT];
    const int k_ss = static_cast<int>(a.k_ss);  // the host has checked that a head's keys span less than 2 GiB
    // K through a buffer descriptor of this head: the lane's offset is formed once, a tile adds a scalar and a
    // constant, and rows past the last key read as zero
    const __amdgpu_buffer_rsrc_t rsrc_k =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<int8_t*>(a.K + b * a.k_sb + h * a.k_sh), 0, (a.sk - 1) * k_ss + a.d, 0x00020000);
    const int kvoff = m * k_ss + hoff;
    auto load_k = [&](int t, int ks) __attribute__((always_inline)) {
        return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(rsrc_k, kvoff + ks * 32, t * 32 * k_ss, 0));
    };
    // the query rows of a block and the first K tiles
    auto request = [&](int item) __attribute__((always_inline)) {
        const int8_t* Qp = a.Q + b * a.q_sb + h * a.q_sh;
        const int row = (item - bh * nblk) * ROWS + wave * 32 + m;
        const int rowc = row < a.sq ? row : a.sq - 1;
#pragma unroll
        for (int ks = 0; ks < DT; ++ks) {
            const bool missing = a.d < D && ks * 32 + hoff >= a.d;
            qf[ks] = *reinterpret_cast<const v4i*>(Qp + rowc * a.q_ss + (missing ? 0 : ks * 32 + hoff));
            if (missing) qf[ks] = v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int t = 0; t < KD; ++t) {
#pragma unroll
            for (int ks = 0; ks < DT; ++ks) kf[t][ks] = load_k(t, ks);
        }
    };
    {
    // V is requested before anything is done with LDS, so that (first head) building the score table hides the latency;
    // the first block's operands follow it
    unsigned av[VB][4];
    const int8_t* Vp = a.V + b * a.v_sb + h * a.v_sh;
#pragma unroll
    for (int it = 0; it < VB; ++it) {
        const int blk = tid + it * THREADS;
        const int k0 = (blk / (D / 4)) * 4;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            av[it][i] = blk < NB && (!RAGGED || k0 + i < a.sk) && n0 < a.d
                            ? *reinterpret_cast<const unsigned*>(Vp + (k0 + i) * a.v_ss + n0) : 0u;
    }
    request(head_item);
    if (head_item == item_begin) {
        if (BANKED) {
            // each entry is computed once, parked in the (still unused) V^T area, then copied to its 64 slots, four
            // slots per 16-byte store
            int* once = reinterpret_cast<int*>(vt);
            if (tid < 256) once[tid] = table_entry(a.sm, tid);
            __syncthreads();
            for (int i = tid * 4; i < 256 * 64; i += THREADS * 4) {
                const int e = once[i >> 6];
                *reinterpret_cast<v4i*>(table + i) = v4i{e, e, e, e};
            }
        } else {
            for (int i = tid; i < 256; i += THREADS) table[i] = table_entry(a.sm, i);
        }
    }
    // everybody is done with the previous head's V^T and column sums (first head: with the table's staging area)
    __syncthreads();
    if (tid < D) colsum[tid] = 0;
    __syncthreads();

    // V -> LDS, transposed in 4x4 byte blocks. Within each group of 32 k, position 16*half + 4*g + i holds
    // k = 8*g + 4*half + i: the order in which a lane's probability registers run.
    {
        int part[4] = {0, 0, 0, 0};
#pragma unroll
        for (int it = 0; it < VB; ++it) {
            const int blk = tid + it * THREADS;
            if (blk < NB) {
                const int k0 = (blk / (D / 4)) * 4;
                unsigned cv[4];
                transpose4x4(av[it], cv);
                const int kk = k0 & 31;
                const int pos = (k0 & ~31) + ((kk >> 2) & 1) * 16 + (kk >> 3) * 4;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    *reinterpret_cast<unsigned*>(vt + (n0 + j) * PITCH + pos) = cv[j];
                    part[j] = __builtin_amdgcn_sdot4(static_cast<int>(cv[j]), 0x01010101, part[j], false);
                }
            }
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) atomicAdd(&colsum[n0 + j], part[j]);
    }
    }
    // A persistent workgroup meets here, once per head; one with a single item does after its first pass, which then
    // hides the wait.
    if (PERSIST) __syncthreads();  // V^T, column sums and the score table are complete

    for (int item = head_item; item < run_end; ++item) {
    // ---- pass A: logits = srs(Q K^T), packed int8 in registers; running row maximum -----------------
    unsigned lg[NT][4];  // biased by 128: byte = logit ^ 0x80
    int mx = -128;
    float mxf = 0.f;
    // (1.5 * 2^23 + x) * 2^-s + (128 - 1.5 * 2^23 * 2^-s) = x * 2^-s + 128, exactly: every term is a multiple of 2^-s
    // below 2^24, and a fused multiply-add rounds once
    const float lbias = 128.f - 12582912.f * a.lscale;
    constexpr int START = 0x4B400000;
    const v16i start16 = {START, START, START, START, START, START, START, START, START, START, START, START, START, START, START, START};
    // BIT == 3: the sums start from the bit pattern of the float 1.5 * 2^23. Floats of that binade are one apart, so
    // adding an integer x (|x| <= D * 2^14 < 2^22) to the pattern gives the pattern of the float 1.5 * 2^23 + x: the
    // accumulators come out of the matrix unit already converted.
    auto logits_of_tile = [&](int t) __attribute__((always_inline)) {
        v16i sums = BIT == 3 ? start16 : v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int ks = 0; ks < DT; ++ks) sums = __builtin_amdgcn_mfma_i32_32x32x32_i8(kf[t % KD][ks], qf[ks], sums, 0, 0, 0);
        return sums;
    };
    // The matrix unit works a tile ahead of the requantisation: its products of tile t + 1 are under way while the
    // vector unit packs tile t.
    v16i acc_next = logits_of_tile(0);
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const v16i acc = acc_next;
        if (t + 1 < NT) acc_next = logits_of_tile(t + 1);
        if (KD > 1 && t + KD < NT) {
#pragma unroll
            for (int ks = 0; ks < DT; ++ks) kf[(t + KD) % KD][ks] = load_k(t + KD, ks);
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            // accumulator 4 g + i belongs to key 32 t + 8 g + 4 half + i: `left` of this group's four keys exist
            const int left = RAGGED ? a.sk - (t * 32 + 8 * g + 4 * half) : 4;
            if (BIT == 3) {
                float f[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int sum_bits = acc[4 * g + i];
                    f[i] = fmaf(__builtin_bit_cast(float, sum_bits), a.lscale, lbias);
                    if (RAGGED) f[i] = i < left ? f[i] : 0.f;
                }
                // two three-operand maxima
                mxf = __builtin_fmaxf(__builtin_fmaxf(mxf, f[0]), f[1]);
                mxf = __builtin_fmaxf(__builtin_fmaxf(mxf, f[2]), f[3]);
                unsigned w = __builtin_amdgcn_cvt_pk_u8_f32(f[0], 0, 0u);
                w = __builtin_amdgcn_cvt_pk_u8_f32(f[1], 1, w);
                w = __builtin_amdgcn_cvt_pk_u8_f32(f[2], 2, w);
                lg[t][g] = __builtin_amdgcn_cvt_pk_u8_f32(f[3], 3, w);
            } else {
                int y[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    y[i] = clamp_i(fast_round_k<BIT>(acc[4 * g + i], a.lr), -128, 127);
                    if (RAGGED) y[i] = i < left ? y[i] : -128;
                }
                mx = max(max(mx, y[0]), max(y[1], max(y[2], y[3])));
                lg[t][g] = pack4_bytes(y[0], y[1], y[2], y[3]) ^ 0x80808080u;
            }
        }
        // The packed logits are pinned here: left to itself, the compiler moves the packing down to where the second
        // pass reads them and keeps four floats alive per register it would have packed.
#pragma unroll
        for (int g = 0; g < 4; ++g) asm volatile("" : "+v"(lg[t][g]));
        if (NT >= 16) __builtin_amdgcn_sched_barrier(0);  // KD - 1 tiles of K fragments in flight, not all sixteen
    }
    // the row maximum as a biased byte; rounding and saturation are monotone, so they commute with the maximum
    unsigned mxb;
    if (BIT == 3) {
        mxf = __builtin_fmaxf(mxf, __builtin_bit_cast(float, lane_xor<32>(__builtin_bit_cast(int, mxf))));
        mxb = __builtin_amdgcn_cvt_pk_u8_f32(mxf, 0, 0u);
    } else {
        mx = max(mx, lane_xor<32>(mx));  // lanes m and m+32 share a row
        mxb = static_cast<unsigned>((mx ^ 0x80) & 0xFF);
    }

    // the operands of the head's next block of rows travel while this block goes through its second and third pass
    if (PERSIST && item + 1 < run_end) request(item + 1);
    if (!PERSIST) __syncthreads();  // V^T, column sums and the score table are complete

    // ---- pass B: scores by table lookup on the gap to the maximum; row sum ----------------------------
    const unsigned mrep = mxb * 0x01010101u;
    const char* tbytes = reinterpret_cast<const char*>(table);
    const unsigned two = 2;
    const unsigned lane4 = static_cast<unsigned>(lane) << 2;  // BANKED: this lane's copy of the table
    unsigned ep[NT][8];  // two 16-bit scores per register
    unsigned sum_even = 0, sum_odd = 0;
    auto sum_and_keep = [&](int t, const unsigned (&pr)[8]) __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < 8; ++r) {
            // scores are at most 32767: both halves of a pair are summed by one dot product with (1, 1)
            // (into two sums in turn: a dot product that waits for the one before it costs an idle slot)
            unsigned& part = (r & 1) ? sum_odd : sum_even;
            part = __builtin_amdgcn_udot2(__builtin_bit_cast(v2us, pr[r]), __builtin_bit_cast(v2us, 0x00010001u), part, false);
            if (t >= NT - PARK) parked[((t - (NT - PARK)) * 8 + r) * THREADS + tid] = pr[r];
            else ep[t][r] = pr[r];
        }
    };
    {
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            unsigned pr[8];
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                const unsigned d4 = mrep - lg[t][g];  // per byte, never borrows
                int e0, e1, e2, e3;
                if (BANKED) {
                    e0 = *reinterpret_cast<const int*>(tbytes + __builtin_amdgcn_perm(d4, lane4, 0x0c0c0400u));
                    e1 = *reinterpret_cast<const int*>(tbytes + __builtin_amdgcn_perm(d4, lane4, 0x0c0c0500u));
                    e2 = *reinterpret_cast<const int*>(tbytes + __builtin_amdgcn_perm(d4, lane4, 0x0c0c0600u));
                    e3 = *reinterpret_cast<const int*>(tbytes + __builtin_amdgcn_perm(d4, lane4, 0x0c0c0700u));
                } else {
                    e0 = *reinterpret_cast<const int*>(tbytes + byte_x4<0>(d4, two));
                    e1 = *reinterpret_cast<const int*>(tbytes + byte_x4<1>(d4, two));
                    e2 = *reinterpret_cast<const int*>(tbytes + byte_x4<2>(d4, two));
                    e3 = *reinterpret_cast<const int*>(tbytes + byte_x4<3>(d4, two));
                }
                if (RAGGED) {
                    const int left = a.sk - (t * 32 + 8 * g + 4 * half);
                    e0 = left > 0 ? e0 : 0;
                    e1 = left > 1 ? e1 : 0;
                    e2 = left > 2 ? e2 : 0;
                    e3 = left > 3 ? e3 : 0;
                }
                pr[2 * g] = pack2_halves(e0, e1);
                pr[2 * g + 1] = pack2_halves(e2, e3);
            }
            sum_and_keep(t, pr);
            // keep the scheduler from hoisting many tiles' lookups at once (their results would spill)
            if (NT >= 16 && (t & 1)) __builtin_amdgcn_sched_barrier(0);
        }
    }
    int sum = static_cast<int>(sum_even + sum_odd);
    sum += lane_xor<32>(sum);
    const int inv = row_inverse(a.sm, sum);

    // ---- pass C: probabilities (uint8, read as int8 after ^0x80) feed the second MFMA from registers ----
    v16i oacc[DT];
#pragma unroll
    for (int u = 0; u < DT; ++u) oacc[u] = v16i{0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
    const unsigned inv16 = static_cast<unsigned>(inv) << (16 - a.sm.out_shift);  // FASTP only: 0 <= inv, shift <= 16
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        v4i pf;
        if (t >= NT - PARK) {  // own slots only: no barrier needed
#pragma unroll
            for (int r = 0; r < 8; ++r) ep[t][r] = parked[((t - (NT - PARK)) * 8 + r) * THREADS + tid];
        }
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            if (FASTP) {
                unsigned q[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    // score (one half of its register, picked by the instruction) times inv16, which is below 2^16 whenever
                    // no clamp is needed (255 * 65536 / the smallest possible row sum): p in bits 16..23, nothing above
                    const unsigned pair = ep[t][2 * g + (i >> 1)];
                    if (i & 1) asm("v_mad_u32_u16 %0, %1, %2, 0 op_sel:[1,0,0,0]" : "=v"(q[i]) : "v"(pair), "v"(inv16));
                    else asm("v_mad_u32_u16 %0, %1, %2, 0" : "=v"(q[i]) : "v"(pair), "v"(inv16));
                }
                const unsigned lo = __builtin_amdgcn_perm(q[1], q[0], 0x0c0c0602u);
                const unsigned hi = __builtin_amdgcn_perm(q[3], q[2], 0x06020c0cu);
                pf[g] = static_cast<int>((lo | hi) ^ 0x80808080u);
            } else {
                int p[4];
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const unsigned pair = ep[t][2 * g + (i >> 1)];
                    const int e = (i & 1) ? static_cast<int>(pair >> 16) : static_cast<int>(pair & 0xFFFFu);
                    p[i] = clamp_i(__mul24(e, inv) >> a.sm.out_shift, 0, 255);
                }
                pf[g] = static_cast<int>(pack4_bytes(p[0], p[1], p[2], p[3]) ^ 0x80808080u);
            }
        }
#pragma unroll
        for (int u = 0; u < DT; ++u) {
            const v4i vf = *reinterpret_cast<const v4i*>(vt + (32 * u + m) * PITCH + t * 32 + half * 16);
            oacc[u] = __builtin_amdgcn_mfma_i32_32x32x32_i8(vf, pf, oacc[u], 0, 0, 0);
        }
        if (NT >= 16 && (t & 1)) __builtin_amdgcn_sched_barrier(0);  // products of later tiles stay packed until needed
    }

    // ---- epilogue: + 128 * colsum (undoes the ^0x80), requantise, 16 contiguous bytes per lane ---------
    int8_t* Op = a.O + b * a.o_sb + h * a.o_sh;
    const int row = (item - bh * nblk) * ROWS + wave * 32 + m;
    const bool row_ok = row < a.sq;
#pragma unroll
    for (int u = 0; u < DT; ++u) {
        unsigned ow[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const v4i cs = *reinterpret_cast<const v4i*>(colsum + 32 * u + 8 * g + 4 * half);
            int y[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) y[i] = clamp_i(fast_round(oacc[u][4 * g + i] + 128 * cs[i], a.orr), -128, 127);
            ow[g] = pack4_bytes(y[0], y[1], y[2], y[3]);
        }
        // lane m holds dwords 0,2,4,6 of the row's 32 bytes, lane m+32 dwords 1,3,5,7: two half-wave swaps
        // give lane m bytes 0-15 and lane m+32 bytes 16-31
        const auto s02 = __builtin_amdgcn_permlane32_swap(ow[0], ow[2], false, false);
        const auto s13 = __builtin_amdgcn_permlane32_swap(ow[1], ow[3], false, false);
        const v4i o = {static_cast<int>(s02[0]), static_cast<int>(s02[1]), static_cast<int>(s13[0]),
                       static_cast<int>(s13[1])};
        if (row_ok && 32 * u + 16 * half < a.d) *reinterpret_cast<v4i*>(Op + row * a.o_ss + 32 * u + 16 * half) = o;
    }
    }  // blocks of query rows
    head_item = run_end;
    }  // heads
}

constexpr int ATTN_CUS = 256;

template <int NT, int DT, int BIT, bool FASTP, int NW = 8>
static void launch_attention_wide(int grid8, size_t lds, hipStream_t stream, const AttnArgs& a) {
    auto kern = attention_kernel<NT, DT, BIT, FASTP, NW>;
    static bool attr_set = false;  // benign race: the attribute is idempotent
    if (!attr_set) {
        (void)hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                  static_cast<int>(lds));
        attr_set = true;
    }
    kern<<<std::min(grid8, ATTN_CUS), NW * 64, lds, stream>>>(a);  // persistent: at most one workgroup per CU
}

// grid: workgroups of 128 query rows; grid8: workgroups of 256 (0 = do not use the eight-wave form), or, when
// `six`, of 192 in the six-wave form.
template <int NT, int DT>
static void launch_attention_nt(int grid, int grid8, size_t lds, hipStream_t stream, const AttnArgs& a, bool six = false) {
    const bool fastp = a.noclamp && a.sm.out_shift <= 16;
    const bool ragged = a.sk != NT * 32;  // always in workgroups of four waves (grid8 == 0)
#define A4G_ATTN(B)                                                                  \
    if (ragged) {                                                                    \
        if (fastp) attention_kernel<NT, DT, B, true, 4, true><<<grid, 256, lds, stream>>>(a);   \
        else attention_kernel<NT, DT, B, false, 4, true><<<grid, 256, lds, stream>>>(a);        \
    } else if (NT >= 8 && DT == 2 && grid8 > 0) {                                           \
        if constexpr (NT >= 8 && DT == 2) {                                                     \
            if (six) {                                                                          \
                if (fastp) launch_attention_wide<NT, DT, B, true, 6>(grid8, lds, stream, a);    \
                else launch_attention_wide<NT, DT, B, false, 6>(grid8, lds, stream, a);         \
            } else if (fastp) launch_attention_wide<NT, DT, B, true>(grid8, lds, stream, a); \
            else launch_attention_wide<NT, DT, B, false>(grid8, lds, stream, a);      \
        }                                                                            \
    } else if (fastp)                                                                \
        attention_kernel<NT, DT, B, true><<<grid, 256, lds, stream>>>(a);            \
    else                                                                             \
        attention_kernel<NT, DT, B, false><<<grid, 256, lds, stream>>>(a);
    switch (a.lscale > 0.f ? 3 : fast_round_kind(a.lr)) {
    case 0: A4G_ATTN(0) break;
    case 1: A4G_ATTN(1) break;
    case 2: A4G_ATTN(2) break;
    default: A4G_ATTN(3) break;
    }
#undef A4G_ATTN
}

// Seven key tiles, seven waves (224 x 224 covers a head of 193 .. 224 tokens), always in the ragged form.
static void launch_attention_seven(int grid, hipStream_t stream, const AttnArgs& a) {
    const size_t lds = static_cast<size_t>(64) * (7 * 32 + 16) + 64 * 4;
    const bool fastp = a.noclamp && a.sm.out_shift <= 16;
#define A4G_ATTN7(B)                                                                       \
    if (fastp) attention_kernel<7, 2, B, true, 7, true><<<grid, 448, lds, stream>>>(a);    \
    else attention_kernel<7, 2, B, false, 7, true><<<grid, 448, lds, stream>>>(a);
    switch (a.lscale > 0.f ? 3 : fast_round_kind(a.lr)) {
    case 0: A4G_ATTN7(0) break;
    case 1: A4G_ATTN7(1) break;
    case 2: A4G_ATTN7(2) break;
    default: A4G_ATTN7(3) break;
    }
#undef A4G_ATTN7
}

template <int DT>
static int launch_attention(int nt, int grid, int grid8, hipStream_t stream, const AttnArgs& a, bool six = false) {
    size_t lds = static_cast<size_t>(DT * 32) * (nt * 32 + 16) + DT * 32 * 4;  // V^T + column sums
    if (nt >= 16 && grid8 > 0) lds += 3 * 8 * 512 * sizeof(unsigned);            // + three parked score tiles per thread
    switch (nt) {
    case 1: launch_attention_nt<1, DT>(grid, 0, lds, stream, a); break;
    case 2: launch_attention_nt<2, DT>(grid, 0, lds, stream, a); break;
    case 4: launch_attention_nt<4, DT>(grid, 0, lds, stream, a); break;
    case 8: launch_attention_nt<8, DT>(grid, grid8, lds, stream, a, six); break;
    // tile counts between the powers of two, for the 64-wide heads only (96, 160, 192 and 384 keys: a kernel of the next
    // power of two would spend a quarter to three eighths of its three passes on keys that do not exist)
    case 3:
        if constexpr (DT == 2) launch_attention_nt<3, DT>(grid, 0, lds, stream, a);
        else return 1;
        break;
    case 5:
        if constexpr (DT == 2) launch_attention_nt<5, DT>(grid, 0, lds, stream, a);
        else return 1;
        break;
    case 6:
        if constexpr (DT == 2) launch_attention_nt<6, DT>(grid, 0, lds, stream, a);
        else return 1;
        break;
    case 12:
        if constexpr (DT == 2) launch_attention_nt<12, DT>(grid, grid8, lds, stream, a, six);
        else return 1;
        break;
    case 16:
        if constexpr (DT <= 2) launch_attention_nt<16, DT>(grid, grid8, lds, stream, a, six);
        else return 1;
        break;
    default: return 1;
    }
    return 0;
}

}  // namespace a4g

using namespace a4g;

extern "C" int a4g_attention_i8(const int8_t* Q, const int8_t* K, const int8_t* V, int8_t* O, int64_t batch, int64_t heads,
                                int64_t sq, int64_t sk, int64_t d, const int64_t* strides, int logit_shift,
                                int logit_round_mode, int softmax_kind, int exp_kq, int hccs_B, int hccs_S, int hccs_Dmax,
                                int inv_shift, int use_clb, int out_shift, int out_round_mode, a4g_stream_t stream_) {
    const char* who = "a4g_attention_i8";
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    A4G_REQUIRE(batch >= 0 && heads >= 1 && sq >= 1 && sk >= 1 && d >= 1, A4G_ERR_INVALID_ARGUMENT,
                "%s: bad shape batch=%lld heads=%lld sq=%lld sk=%lld d=%lld", who, (long long)batch, (long long)heads,
                (long long)sq, (long long)sk, (long long)d);
    A4G_REQUIRE(valid_round(logit_round_mode) && valid_round(out_round_mode), A4G_ERR_INVALID_ARGUMENT,
                "%s: unknown rounding mode", who);
    A4G_REQUIRE(logit_shift >= 0 && logit_shift <= 24 && out_shift >= 0 && out_shift <= 24, A4G_ERR_INVALID_ARGUMENT,
                "%s: accumulator output shift must be in [0,24], got %d and %d", who, logit_shift, out_shift);
    A4G_REQUIRE(softmax_kind == 0 || softmax_kind == 1, A4G_ERR_INVALID_ARGUMENT, "%s: softmax_kind must be 0 (exp) or 1 (hccs)",
                who);
    AttnArgs a{};
    bool noclamp = false;
    if (softmax_kind == 0) {
        if (int rc = make_exp_params(who, exp_kq, inv_shift, A4G_U8, &a.sm, &noclamp)) return rc;
    } else {
        if (int rc = make_hccs_params(who, sk, hccs_B, hccs_S, hccs_Dmax, inv_shift, use_clb, A4G_U8, &a.sm, &noclamp))
            return rc;
    }
    A4G_REQUIRE(d % 16 == 0 && d <= 128 && sk <= (d > 64 ? 256 : 512), A4G_ERR_UNSUPPORTED,
                "%s: fused path covers head dimensions that are multiples of 16, up to 64 with up to 512 keys and up to 128 with up "
                "to 256, got d=%lld sk=%lld", who, (long long)d, (long long)sk);
    const int width = d <= 32 ? 32 : (d <= 64 ? 64 : 128);  // of the kernel: narrower heads run with their missing pieces masked
    // tiles of 32 keys the kernel is instantiated for: the powers of two, and for 64-wide heads also 3, 5, 6 and 12
    static const int tile_counts_64[] = {1, 2, 3, 4, 5, 6, 8, 12, 16};
    static const int tile_counts[] = {1, 2, 4, 8, 16};
    int nt = 16;
    if (width == 64) {
        for (int i = 8; i >= 0; --i)
            if (tile_counts_64[i] * 32 >= sk) nt = tile_counts_64[i];
    } else {
        for (int i = 4; i >= 0; --i)
            if (tile_counts[i] * 32 >= sk) nt = tile_counts[i];
    }
    const bool ragged = nt * 32 != sk;
    A4G_REQUIRE(batch * heads * ((sq + 127) / 128) <= INT32_MAX && sq <= (1 << 24), A4G_ERR_UNSUPPORTED, "%s: too many rows", who);
    if (batch == 0) return A4G_OK;
    A4G_REQUIRE(Q && K && V && O && strides, A4G_ERR_INVALID_ARGUMENT, "%s: null pointer", who);
    bool ok = aligned16(Q) && aligned16(K) && aligned16(V) && aligned16(O);
    for (int i = 0; i < 12; ++i) ok = ok && strides[i] % 16 == 0 && strides[i] >= 0;
    A4G_REQUIRE(ok, A4G_ERR_UNSUPPORTED, "%s: pointers and strides must be multiples of 16 bytes", who);
    A4G_REQUIRE(strides[2] >= d && strides[5] >= d && strides[8] >= d && strides[11] >= d, A4G_ERR_INVALID_ARGUMENT,
                "%s: row stride smaller than the head dimension", who);
    A4G_REQUIRE((sk + 32) * strides[5] < (int64_t{1} << 31), A4G_ERR_UNSUPPORTED,
                "%s: the keys of one head must span less than 2 GiB (row stride %lld bytes)", who, (long long)strides[5]);
    a.Q = Q; a.K = K; a.V = V; a.O = O;
    a.q_sb = strides[0]; a.q_sh = strides[1]; a.q_ss = strides[2];
    a.k_sb = strides[3]; a.k_sh = strides[4]; a.k_ss = strides[5];
    a.v_sb = strides[6]; a.v_sh = strides[7]; a.v_ss = strides[8];
    a.o_sb = strides[9]; a.o_sh = strides[10]; a.o_ss = strides[11];
    a.heads = static_cast<int>(heads);
    a.sq = static_cast<int>(sq);
    a.sk = static_cast<int>(sk);
    a.d = static_cast<int>(d);
    a.lr = make_fast_round(logit_round_mode, logit_shift);
    a.orr = make_fast_round(out_round_mode, out_shift);
    a.noclamp = noclamp;
    // nearest-even logits take the float form: d * 2^14 + 2^(7 + shift) < 2^24 for the head dimensions covered
    a.lscale = (logit_round_mode == A4G_RND_CONV_EVEN && logit_shift >= 1 && logit_shift <= 15 && d <= 512)
                   ? ldexpf(1.f, -logit_shift) : 0.f;
    const int grid = static_cast<int>(batch * heads * ((sq + 127) / 128));
    // eight waves per workgroup (256 query rows, bank-replicated score table) once every CU gets at least one
    const int64_t wg8 = batch * heads * ((sq + 255) / 256);
    int grid8 = (!ragged && d == 64 && sq >= 256 && wg8 >= 256) ? static_cast<int>(wg8) : 0;
    // blocks of 192 rows where they leave fewer rows empty than blocks of 256 (384 queries: two full blocks against one
    // full and one half)
    const int64_t wg6 = batch * heads * ((sq + 191) / 192);
    const bool six = grid8 > 0 && wg6 >= 256 && (sq + 191) / 192 * 192 < (sq + 255) / 256 * 256;
    if (six) grid8 = static_cast<int>(wg6);
    a.items = grid8 > 0 ? grid8 : grid;
    if (d == 64 && sq > 192 && sq <= 224 && sk > 192 && sk <= 224) {
        // 193 .. 224 queries and keys (the 197 tokens of a vision transformer): seven key tiles instead of eight, and one
        // workgroup of seven waves per head instead of two of four, so that a head's V^T and score table are built once
        a.items = static_cast<int>(batch * heads);
        launch_attention_seven(a.items, stream, a);
        return check_hip(hipGetLastError(), who);
    }
    const int no_kernel = width == 64 ? launch_attention<2>(nt, grid, grid8, stream, a, six)
                          : (width == 32 ? launch_attention<1>(nt, grid, 0, stream, a) : launch_attention<4>(nt, grid, 0, stream, a));
    if (no_kernel) return fail(A4G_ERR_UNSUPPORTED, "%s: no kernel for sk=%lld", who, (long long)sk);
    return check_hip(hipGetLastError(), who);
}
