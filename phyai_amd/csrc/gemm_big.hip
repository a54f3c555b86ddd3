// MFMA-bound fp8 GEMM for large M (prefix prefill, batched serving): 256 x 256 output tile
// per workgroup, 128 x 128 per wavefront.
//
// Why this shape.  One v_mfma_f32_32x32x64_f8f6f4 takes 64 cycles and consumes two 2 KB
// operand blocks.  A wavefront that owns TM x TN blocks reads (TM + TN) blocks from LDS per
// TM*TN MFMAs; LDS delivers 128 bytes per clock to the whole CU, so four wavefronts with
// 4 x 4 blocks each ask for 64 bytes per clock (half of what LDS can give) while 2 x 2 blocks
// would ask for 256.  4 x 4 blocks of 16 accumulators are 256 registers: the accumulators
// live in AGPRs, one wavefront per SIMD, and latency is hidden inside the wavefront:
//
//  * global -> LDS copies bypass the register file (global_load_lds_dwordx4): lane i of a
//    wavefront fetches one 16-byte chunk and the hardware deposits chunk i at LDS base + 16*i.
//    The XOR swizzle that keeps the 128-bit operand reads conflict-free is therefore applied
//    on the global side: lane i (row i/4 of a 16-row group, slot i%4 of the 64-byte row)
//    fetches chunk (i%4) ^ ((row/2)%4) of its row.
//  * K is consumed in 64-byte slabs through a ring of four 32 KB LDS stages: the copies of
//    slab s+3 are issued while slab s is being multiplied, so a copy has three slab times
//    (about 1.3 us of MFMA work) to arrive.  One barrier per slab: it tells every wavefront
//    that slab s has landed everywhere and that the stage about to be refilled is no longer
//    being read.
//  * inside a slab the A block of the next row group is read from LDS before the current
//    group's four MFMAs are issued, so ds_read latency overlaps MFMA time.
//
// Gated epilogues use the same trick as the smaller tile kernel: within a wavefront's 128
// columns the first 64 are gate columns and the last 64 the matching up columns.
// Requires K % 128 == 0 and K >= 256 (slabs are never partial and come in pairs).
#include "fp8_device.h"
#include "launch.h"
#include <stdlib.h>

namespace phyai {

constexpr int BIG_BM = 256, BIG_BN = 256, BIG_BK = 64;
constexpr int BIG_STAGES = 4;
constexpr int BIG_TILE_BYTES = (BIG_BM + BIG_BN) * BIG_BK;  // 32 KB per K slab

struct BigArgs {
    const uint8_t* __restrict__ a;   // xq [M, K]
    const uint8_t* __restrict__ b;   // w  [N, K]
    const float* __restrict__ a_scale;
    const float* __restrict__ b_scale;
    const uint16_t* __restrict__ bias;
    uint16_t* __restrict__ out;
    int64_t ldo;
    int M, N, K;
    int a_scale_scalar;
};

// One 16-byte chunk per lane from global memory straight into LDS: lane i's chunk lands at
// lds_wave_base + 16*i.  Issued as inline assembly so that the compiler does not order its own
// LDS reads behind copies that are still in flight; the waits are placed by hand below.
__device__ __forceinline__ void copy16_to_lds(const uint8_t* base, uint32_t lane_offset, uint32_t lds_wave_base) {
    asm volatile("s_mov_b32 m0, %2\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(lane_offset), "s"(base), "s"(lds_wave_base) : "memory", "m0");
}

// Operand block of v_mfma_f32_32x32x64: lane (l32, h) reads bytes [32h, 32h+32) of its row,
// i.e. chunks 2h and 2h+1, from their swizzled places.
__device__ __forceinline__ v8i big_frag(const uint8_t* buf, int row, int h) {
    const int sw = (row >> 1) & 3;
    const uint8_t* r = buf + row * BIG_BK;
    const v4i lo = *reinterpret_cast<const v4i*>(r + (((2 * h) ^ sw) << 4));
    const v4i hi = *reinterpret_cast<const v4i*>(r + (((2 * h + 1) ^ sw) << 4));
    v8i f;
    f[0] = lo[0]; f[1] = lo[1]; f[2] = lo[2]; f[3] = lo[3];
    f[4] = hi[0]; f[5] = hi[1]; f[6] = hi[2]; f[7] = hi[3];
    return f;
}

template <int EPI>
__global__ __launch_bounds__(256, 1) void gemm_fp8_big_kernel(const BigArgs p) {
    constexpr bool GATED = epi_is_gated(EPI);
    __shared__ __attribute__((aligned(1024))) uint8_t lds[BIG_STAGES * BIG_TILE_BYTES];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int l32 = lane & 31, h = lane >> 5;
    const int half_n = p.N / 2;
    const int m0 = blockIdx.y * BIG_BM;
    const int n0 = GATED ? blockIdx.x * (BIG_BN / 2) : blockIdx.x * BIG_BN;

    // ---- copy geometry: wavefront w moves 16-row groups w*4 .. w*4+3 of A and of B ----------
    const int crow = lane >> 2;                                   // row inside the 16-row group
    const int cchunk = ((lane & 3) ^ ((crow >> 1) & 3)) << 4;     // swizzled 16-byte chunk of that row
    uint32_t aoff[4], boff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int jj = (wave * 4 + i) * 16 + crow;    // row of the A tile / column of the output tile
        int r = m0 + jj;
        r = r < p.M ? r : p.M - 1;
        aoff[i] = (uint32_t)r * (uint32_t)p.K + cchunk;
        int rb;
        if constexpr (GATED) {
            const int w_ = jj >> 7, j = jj & 127;
            int g = n0 + w_ * 64 + (j & 63);
            g = g < half_n ? g : half_n - 1;
            rb = (j >> 6) * half_n + g;
        } else {
            rb = n0 + jj;
            rb = rb < p.N ? rb : p.N - 1;
        }
        boff[i] = (uint32_t)rb * (uint32_t)p.K + cchunk;
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
    auto issue = [&](int stage, int k) {
        const uint32_t dst = __builtin_amdgcn_readfirstlane(lds_base + stage * BIG_TILE_BYTES + wave * 4096);
#pragma unroll
        for (int i = 0; i < 4; ++i) copy16_to_lds(p.a + k, aoff[i], dst + i * 1024);
#pragma unroll
        for (int i = 0; i < 4; ++i) copy16_to_lds(p.b + k, boff[i], dst + BIG_BM * BIG_BK + i * 1024);
    };

    v16f acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // One slab = four row groups of four MFMAs.  To keep the MFMA pipe fed across slabs:
    //  * the barrier that publishes slab s+1 sits in the MIDDLE of slab s (after group 1), where
    //    all wavefronts arrive at about the same time and still have MFMAs queued;
    //  * the operand blocks that open slab s+1 (four B blocks, first A block) are read from LDS
    //    during the last group of slab s, into a second register set.
    const int n_slabs = p.K / BIG_BK;
    const int arow = wm * 128 + l32, brow = wn * 128 + l32;
    auto stage_ptr = [&](int s) -> const uint8_t* { return lds + (s % BIG_STAGES) * BIG_TILE_BYTES; };
#define PHYAI_MFMA_GROUP(I, FA, FB0, FB1, FB2, FB3)                                                            \
    acc[I][0] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(FA, FB0, acc[I][0], 0, 0, 0, 0, 0, 0);            \
    acc[I][1] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(FA, FB1, acc[I][1], 0, 0, 0, 0, 0, 0);            \
    acc[I][2] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(FA, FB2, acc[I][2], 0, 0, 0, 0, 0, 0);            \
    acc[I][3] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(FA, FB3, acc[I][3], 0, 0, 0, 0, 0, 0);            \
    __builtin_amdgcn_sched_barrier(0);

// S: slab index; FA0/FB*: opening blocks of slab S (in registers); NFA0/NFB*: receive those of
// slab S+1.  NEXT: slab S+1 exists; NEXT2: slab S+2 exists (its copies may still be in flight);
// ISSUE: slab S+3 exists and is requested here.  The flags are literals, so the steady-state
// loop body is straight-line code.
#define PHYAI_RUN_SLAB(S, NEXT, NEXT2, ISSUE, FA0, FB0, FB1, FB2, FB3, NFA0, NFB0, NFB1, NFB2, NFB3)               \
    {                                                                                                             \
        const int s_ = (S);                                                                                       \
        const uint8_t* abuf_ = stage_ptr(s_);                                                                     \
        const v8i fa1_ = big_frag(abuf_, arow + 32, h);                                                           \
        PHYAI_MFMA_GROUP(0, FA0, FB0, FB1, FB2, FB3)                                                              \
        const v8i fa2_ = big_frag(abuf_, arow + 64, h);                                                           \
        PHYAI_MFMA_GROUP(1, fa1_, FB0, FB1, FB2, FB3)                                                             \
        if (NEXT) {                                                                                               \
            /* my copies of slab s+1 are done (slab s+2, if any, may still be in flight) ... */                   \
            if (NEXT2) asm volatile("s_waitcnt vmcnt(8)" ::: "memory");                                           \
            else asm volatile("s_waitcnt vmcnt(0)" ::: "memory");                                                 \
            __syncthreads(); /* ... and so are everybody's; nobody reads slab s-1 any more */                      \
            if (ISSUE) issue((s_ + BIG_STAGES - 1) % BIG_STAGES, (s_ + BIG_STAGES - 1) * BIG_BK);                 \
        }                                                                                                         \
        const v8i fa3_ = big_frag(abuf_, arow + 96, h);                                                           \
        PHYAI_MFMA_GROUP(2, fa2_, FB0, FB1, FB2, FB3)                                                             \
        if (NEXT) {                                                                                               \
            const uint8_t* nbuf_ = stage_ptr(s_ + 1);                                                             \
            NFB0 = big_frag(nbuf_ + BIG_BM * BIG_BK, brow, h);                                                    \
            NFB1 = big_frag(nbuf_ + BIG_BM * BIG_BK, brow + 32, h);                                               \
            NFB2 = big_frag(nbuf_ + BIG_BM * BIG_BK, brow + 64, h);                                               \
            NFB3 = big_frag(nbuf_ + BIG_BM * BIG_BK, brow + 96, h);                                               \
            NFA0 = big_frag(nbuf_, arow, h);                                                                      \
        }                                                                                                         \
        PHYAI_MFMA_GROUP(3, fa3_, FB0, FB1, FB2, FB3)                                                             \
    }

    // prologue: slabs 0..2 in flight, slab 0 published, its opening blocks in registers.
    // n_slabs is even and at least 4 (K is a multiple of 128 and at least 256).
    issue(0, 0);
    issue(1, BIG_BK);
    issue(2, 2 * BIG_BK);
    asm volatile("s_waitcnt vmcnt(16)" ::: "memory");
    __syncthreads();
    v8i a0, b0, b1, b2, b3, na0, nb0, nb1, nb2, nb3;
    b0 = big_frag(lds + BIG_BM * BIG_BK, brow, h);
    b1 = big_frag(lds + BIG_BM * BIG_BK, brow + 32, h);
    b2 = big_frag(lds + BIG_BM * BIG_BK, brow + 64, h);
    b3 = big_frag(lds + BIG_BM * BIG_BK, brow + 96, h);
    a0 = big_frag(lds, arow, h);
    int s = 0;
    for (; s < n_slabs - 4; s += 2) {
        PHYAI_RUN_SLAB(s, 1, 1, 1, a0, b0, b1, b2, b3, na0, nb0, nb1, nb2, nb3)
        PHYAI_RUN_SLAB(s + 1, 1, 1, 1, na0, nb0, nb1, nb2, nb3, a0, b0, b1, b2, b3)
    }
    PHYAI_RUN_SLAB(s, 1, 1, 1, a0, b0, b1, b2, b3, na0, nb0, nb1, nb2, nb3)        // slab n-4 requests n-1
    PHYAI_RUN_SLAB(s + 1, 1, 1, 0, na0, nb0, nb1, nb2, nb3, a0, b0, b1, b2, b3)    // slab n-3
    PHYAI_RUN_SLAB(s + 2, 1, 0, 0, a0, b0, b1, b2, b3, na0, nb0, nb1, nb2, nb3)    // slab n-2
    PHYAI_RUN_SLAB(s + 3, 0, 0, 0, na0, nb0, nb1, nb2, nb3, a0, b0, b1, b2, b3)    // slab n-1
#undef PHYAI_RUN_SLAB
#undef PHYAI_MFMA_GROUP

    // ---- epilogue ------------------------------------------------------------------------
    // The accumulator layout gives a lane one column and 16 scattered rows, which would mean
    // 2-byte stores.  Instead each wavefront stages its bf16 output tile (128 rows x 128 or 64
    // columns) in its own 32 KB slice of the now idle LDS and writes it out row-wise, 16 bytes
    // per lane, whole 256- or 128-byte row segments per instruction.  Neighbouring lanes swap
    // one value first (DPP) so that every LDS write is a packed pair of columns.
    constexpr int TNO = GATED ? 2 : 4;
    constexpr int ROWB = TNO * 64;                       // staged row length in bytes
    const int n_lim = GATED ? half_n : p.N;
    const int nbase = n0 + (GATED ? wn * 64 : wn * 128);
    float sg[TNO], bg[TNO], su[TNO], bu[TNO];
#pragma unroll
    for (int j = 0; j < TNO; ++j) {
        const int n = nbase + j * 32 + l32;
        const int n_safe = n < n_lim ? n : 0;
        sg[j] = p.b_scale[n_safe];
        bg[j] = p.bias ? bf16_bits_to_f32(p.bias[n_safe]) : 0.f;
        su[j] = 0.f; bu[j] = 0.f;
        if constexpr (GATED) {
            su[j] = p.b_scale[half_n + n_safe];
            bu[j] = p.bias ? bf16_bits_to_f32(p.bias[half_n + n_safe]) : 0.f;
        }
    }
    __syncthreads();  // every wavefront is done reading operands from LDS
    uint8_t* stg = lds + wave * 32768;
    const int odd = lane & 1;
    // Row scales of this lane: rows mrow0 + i*32 + 8*g + (0..3), g = 0..3.
    const int mrow0 = m0 + wm * 128 + 4 * h;
    const bool vec_rows = !p.a_scale_scalar && m0 + BIG_BM <= p.M &&
                          (reinterpret_cast<uintptr_t>(p.a_scale) & 15) == 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        v4f sa[4];
        if (vec_rows) {
#pragma unroll
            for (int g = 0; g < 4; ++g) sa[g] = *reinterpret_cast<const v4f*>(p.a_scale + mrow0 + i * 32 + 8 * g);
        } else {
#pragma unroll
            for (int g = 0; g < 4; ++g)
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int m = mrow0 + i * 32 + 8 * g + e;
                    sa[g][e] = p.a_scale[p.a_scale_scalar ? 0 : (m < p.M ? m : p.M - 1)];
                }
        }
#pragma unroll
        for (int j = 0; j < TNO; ++j) {
#pragma unroll
            for (int t = 0; t < 8; ++t) {
                uint32_t b[2];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const int r = 2 * t + e;
                    const float s_a = sa[r / 4][r % 4];
                    float v = acc[i][j][r] * (s_a * sg[j]) + bg[j];
                    if constexpr (GATED) {
                        const float u = acc[i][j + 2][r] * (s_a * su[j]) + bu[j];
                        v = apply_act<EPI>(round_bf16(v)) * round_bf16(u);
                    } else if constexpr (EPI != EPI_NONE) {
                        v = apply_act<EPI>(round_bf16(v));
                    }
                    b[e] = f32_to_bf16_bits(v);
                }
                // even lane keeps row r0 and receives the neighbour's r0 value (column n+1);
                // odd lane keeps row r1 and receives the neighbour's r1 value (column n-1).
                const uint32_t send = odd ? b[0] : b[1];
                const uint32_t recv = (uint32_t)__builtin_amdgcn_mov_dpp((int)send, 0xB1, 0xF, 0xF, true);
                const uint32_t word = odd ? (recv | (b[1] << 16)) : (b[0] | (recv << 16));
                const int row = i * 32 + 8 * (t / 2) + 4 * h + 2 * (t % 2) + odd;
                const int col = j * 32 + (l32 & ~1);
                *reinterpret_cast<uint32_t*>(stg + row * ROWB + col * 2) = word;
            }
        }
    }
    // write the staged tile out: 1 KB (4 or 8 whole rows) per instruction
#pragma unroll 4
    for (int qd = 0; qd < 128 * ROWB / 1024; ++qd) {
        const int byte = qd * 1024 + lane * 16;
        const int row = byte / ROWB, colb = byte % ROWB;
        const uint4 v = *reinterpret_cast<const uint4*>(stg + byte);
        const int m = m0 + wm * 128 + row;
        const int n = nbase + (colb >> 1);
        if (m < p.M && n < n_lim) *reinterpret_cast<uint4*>(p.out + (int64_t)m * p.ldo + n) = v;
    }
}

// ---- host side ---------------------------------------------------------------------------

static int big_ceil_div(int a, int b) { return (a + b - 1) / b; }

// Worth it when the tile grid fills the chip at least once.
bool big_applicable(int M, int N, int K, int epilogue) {
    if (K % 128 != 0 || K < 256) return false;
    if (const char* e = getenv("PHYAI_FP8_BIG")) {   // "0": never, "2": whenever the shape allows (tests)
        if (e[0] == '0') return false;
        if (e[0] == '2') return true;
    }
    if (M < 192) return false;
    const int n_eff = epi_is_gated(epilogue) ? N / 2 : N;
    const int bn_eff = epi_is_gated(epilogue) ? BIG_BN / 2 : BIG_BN;
    return big_ceil_div(M, BIG_BM) * big_ceil_div(n_eff, bn_eff) >= 200;
}

template <int EPI>
static void big_launch(const BigArgs& a, dim3 grid, hipStream_t st) {
    hipLaunchKernelGGL((gemm_fp8_big_kernel<EPI>), grid, dim3(256), 0, st, a);
}

int launch_gemm_big(const GemmProblem& g, hipStream_t st) {
    // the epilogue writes 16 bytes per lane
    if (g.ldo % 8 != 0 || (reinterpret_cast<uintptr_t>(g.out) & 15) != 0) return -2;
    BigArgs a;
    a.a = g.xq; a.b = g.w; a.a_scale = g.x_scale; a.b_scale = g.w_scale; a.bias = g.bias;
    a.out = g.out; a.ldo = g.ldo; a.M = g.M; a.N = g.N; a.K = g.K;
    a.a_scale_scalar = g.x_scale_is_scalar;
    const bool gated = epi_is_gated(g.epilogue);
    const int n_eff = gated ? g.N / 2 : g.N;
    const dim3 grid(big_ceil_div(n_eff, gated ? BIG_BN / 2 : BIG_BN), big_ceil_div(g.M, BIG_BM));
    switch (g.epilogue) {
    case EPI_NONE: big_launch<EPI_NONE>(a, grid, st); return 0;
    case EPI_GEGLU_TANH: big_launch<EPI_GEGLU_TANH>(a, grid, st); return 0;
    case EPI_GEGLU_ERF: big_launch<EPI_GEGLU_ERF>(a, grid, st); return 0;
    case EPI_SWIGLU: big_launch<EPI_SWIGLU>(a, grid, st); return 0;
    case EPI_GELU_TANH: big_launch<EPI_GELU_TANH>(a, grid, st); return 0;
    case EPI_GELU_ERF: big_launch<EPI_GELU_ERF>(a, grid, st); return 0;
    default: return -2;
    }
}

}  // namespace phyai
