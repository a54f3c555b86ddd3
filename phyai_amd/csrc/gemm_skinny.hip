// Weight-streaming fp8 GEMM for small token counts (the M = 50 action-chunk regime, and the
// batched M = 100 .. 400 cases where the weights still dominate the bytes).
//
// At these sizes a whole weight matrix (2-8 MB) is less than what the chip holds
// in flight, so the kernel is built around latency, not throughput:
//
//  * No cross-workgroup reduction.  A workgroup owns 16*NT output columns over the
//    WHOLE K range; its eight wavefronts split K between them (wavefront w takes
//    the 128-byte K steps w, w+8, w+16, ...) and meet once, in LDS, to add their
//    partial sums in wavefront order (fixed order: reproducible results).  A
//    device-wide split-K would need three dependent trips to memory (publish
//    partials, bump a counter, read partials back); this needs none.
//  * Few output columns (N = 1024) would leave most CUs idle, and every workgroup has to
//    read the activations of all its token rows, so such shapes are also split along M
//    (grid.y): a workgroup then owns 16*NT columns x 16*MB token rows.  Workgroups that
//    share a weight tile differ only in blockIdx.y, and with a multiple of 8 tiles they land
//    on the same XCD, so the tile comes from HBM once and from that XCD's L2 afterwards.
//  * Every wavefront requests all of its bytes first - weights and quantized activations,
//    together with the scales and bias the epilogue will want - and only then starts to
//    compute.  The operands go global -> LDS (the wavefront's own slice, see STAGED below) ->
//    VGPRs in MFMA operand layout; nobody else reads that slice, so there is no barrier
//    between the loads and the math.
//  * v_mfma_f32_16x16x128_f8f6f4: lane l supplies operand row (l % 16) and 32 of
//    the 128 K bytes of a step.  Which 32 is free as long as both operands agree;
//    lane group q = l / 16 takes bytes [16q, 16q+16) and [64+16q, 64+16q+16), so
//    one 128-bit load instruction reads 64 contiguous bytes of each of 16 rows.
//    w is the "A" operand (rows = output columns n), x the "B" operand (columns =
//    token rows m): accumulator register r of lane l is
//    out[m = 16*mb + l%16][n = n0 + 4*(l/16) + r].
//  * Gated epilogues (GeGLU / SwiGLU): the 16 operand rows of a tile are 8 gate
//    columns and the 8 up columns that pair with them, so gate and up of one output
//    sit 32 lanes apart in the same accumulator and meet in the LDS reduction.
//  * After the reduction one thread owns four consecutive output columns of one
//    token: scale, bias, activation, one 64-bit bf16x4 store.
#include "fp8_device.h"
#include "launch.h"
#include "tuning.h"
#include "weight_layout.h"
#include <stdio.h>
#include <stdlib.h>

namespace phyai {

struct SkinnyArgs {
    const uint8_t* __restrict__ xq;  // [M, K]
    const uint8_t* __restrict__ w;   // [N, K]
    const float* __restrict__ x_scale;
    const float* __restrict__ w_scale;
    const uint16_t* __restrict__ bias;
    uint16_t* __restrict__ out;
    int64_t ldo;
    int M, N, K;
    int x_scale_scalar;
    int rounds;  // K steps are consumed in rounds of SK_WAVES * KPW
    int stream_w;  // weights with non-temporal loads
    int operand_w; // weights in MFMA operand order (weight_layout.h; the gated form for gated epilogues)
    ResidualArgs res;
};

constexpr int SK_WAVES = 8;
constexpr int SK_THREADS = SK_WAVES * kWave;

__device__ __forceinline__ v8i join(v4i lo, v4i hi) {
    v8i f;
    f[0] = lo[0]; f[1] = lo[1]; f[2] = lo[2]; f[3] = lo[3];
    f[4] = hi[0]; f[5] = hi[1]; f[6] = hi[2]; f[7] = hi[3];
    return f;
}

// MB: 16-row token blocks per workgroup (grid.y workgroups cover M); NT: 16-row weight
// tiles per workgroup; KPW: K steps per wavefront per round.
//
// STAGED: the operands reach the MFMA layout through the wavefront's own slice of LDS instead of
// directly.  A direct load gives each operand row 64 contiguous bytes per instruction (4 lanes
// per row); the copy into LDS is free to give it the whole 128-byte step (8 lanes per row), i.e.
// one L2 line per request.  A CU pulls about twice the bytes per second that way, and the load
// phase of this kernel is bound by exactly that rate (every workgroup needs its weight tiles
// AND all of the activation codes of its token rows).  Nobody but the wavefront itself reads
// what it staged, so there is still no barrier before the math: copies, s_waitcnt, ds_read.
//
// Kernel arguments are plain scalars, ordered so that what the first instructions need (operand
// pointers, sizes) sits in the first 16 dwords: the library is built with kernel-argument
// preloading, which delivers those in SGPRs at wavefront start instead of through a scalar load
// from memory at the head of every launch.  They are gathered into a SkinnyArgs right away.
template <int MB, int NT, int KPW, int EPI, bool STAGED>
__global__ __launch_bounds__(SK_THREADS) void gemm_fp8_skinny_kernel(
    const uint8_t* __restrict__ a_w, const uint8_t* __restrict__ a_xq, const float* __restrict__ a_x_scale,
    const float* __restrict__ a_w_scale, const uint16_t* __restrict__ a_bias, int a_K, int a_N, int a_m_flags,
    uint16_t* __restrict__ a_out, int64_t a_ldo, const ResidualArgs a_res) {
    // 13 preloaded dwords: everything the operand requests and the early epilogue loads need.
    // a_m_flags = M | operand-order weights << 28 | stream_weights << 29 | x_scale_is_scalar << 30; the
    // rounds follow from K.
    SkinnyArgs p;
    p.xq = a_xq; p.w = a_w; p.x_scale = a_x_scale; p.w_scale = a_w_scale; p.bias = a_bias; p.out = a_out;
    p.ldo = a_ldo; p.M = a_m_flags & 0x0FFFFFFF; p.N = a_N; p.K = a_K; p.x_scale_scalar = (a_m_flags >> 30) & 1;
    // weights read with non-temporal loads: a matrix that the caller does not want to displace
    // others from the Infinity Cache (STAGED form only; the hint is ignored otherwise)
    const bool stream_w = __builtin_amdgcn_readfirstlane((a_m_flags >> 29) & 1) != 0;
    (void)stream_w;
    // Weights in operand order: tile nt of this workgroup is unit blockIdx.x * NT + nt of the matrix (for
    // gated epilogues the gated order is exactly the row order of a gated tile); a K step is 2 KB away
    // instead of 128 bytes, a 16-byte chunk 256 bytes instead of 16.
    const bool operand_w = __builtin_amdgcn_readfirstlane((a_m_flags >> 28) & 1) != 0;
    const int w_step_shift = operand_w ? 11 : 7;
    const uint32_t w_units = (uint32_t)a_N >> 4;
    auto w_unit = [&](int nt) -> uint32_t {
        const uint32_t u = blockIdx.x * NT + nt;
        return u < w_units ? u : w_units - 1;
    };
    p.rounds = (((a_K >> 7) + SK_WAVES - 1) / SK_WAVES + KPW - 1) / KPW;
    p.res = a_res;
    constexpr bool GATED = epi_is_gated(EPI);
    constexpr int COLS_PER_TILE = GATED ? 8 : 16;  // output columns per 16-row weight tile
    constexpr int BLOCKS = NT + MB;                // 16-row operand blocks (2 KB each) per K step
    constexpr int RED_PER_WAVE = NT * MB * kWave * (int)sizeof(v4f);
    constexpr int STAGE_PER_WAVE = KPW * BLOCKS * 2048;
    constexpr int PER_WAVE = STAGED ? (STAGE_PER_WAVE > RED_PER_WAVE ? STAGE_PER_WAVE : RED_PER_WAVE) : RED_PER_WAVE;
    static_assert(SK_WAVES * PER_WAVE <= 160 * 1024, "staging does not fit the LDS");

    // per wavefront: staging of its K steps, later its partial sums (red[wave][nt][mb][lane])
    __shared__ __attribute__((aligned(1024))) uint8_t smem[SK_WAVES * PER_WAVE];
    auto red = [&](int w, int nt, int mb, int l) -> v4f& {
        return reinterpret_cast<v4f*>(smem + w * PER_WAVE)[(nt * MB + mb) * kWave + l];
    };

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    const int half_n = p.N / 2;
    const int n_out_total = GATED ? half_n : p.N;
    const int col0 = blockIdx.x * (COLS_PER_TILE * NT);  // first output column of the workgroup
    const int total_steps = p.K >> 7;
    const int m_base = blockIdx.y * (MB * 16);

    // ---- epilogue roles of this thread and their operands (requested first) --------------------
    // A role is (tile e_nt, token block e_mb): the thread finishes token m = 16*e_mb + lane%16
    // and output columns e_n .. e_n+3 of it.  The eight wavefronts cover eight roles at a time;
    // workgroup shapes with more blocks than that (NT * MB > 8) go round twice.
    constexpr int ROLE_ROUNDS = (NT * MB + SK_WAVES - 1) / SK_WAVES;
    const int e_lane = tid & 63;
    const int e_q = e_lane >> 4;
    int e_mb[ROLE_ROUNDS], e_nt[ROLE_ROUNDS], e_m[ROLE_ROUNDS], e_n[ROLE_ROUNDS];
    bool e_role[ROLE_ROUNDS], e_live[ROLE_ROUNDS];
    v4f sw4[ROLE_ROUNDS], su4[ROLE_ROUNDS];
    uint2 bw2[ROLE_ROUNDS], bu2[ROLE_ROUNDS];
    float sa[ROLE_ROUNDS];
#pragma unroll
    for (int rr = 0; rr < ROLE_ROUNDS; ++rr) {
        const int role = rr * SK_WAVES + (tid >> 6);
        e_mb[rr] = role % MB;
        e_nt[rr] = role / MB;
        e_role[rr] = e_nt[rr] < NT;
        e_m[rr] = m_base + e_mb[rr] * 16 + (e_lane & 15);
        e_n[rr] = col0 + (e_nt[rr] < NT ? e_nt[rr] : 0) * COLS_PER_TILE + (GATED ? 2 : 4) * e_q;
        e_live[rr] = e_role[rr] && e_m[rr] < p.M && e_n[rr] < n_out_total;
        const int e_n_safe = e_live[rr] ? e_n[rr] : 0;
        su4[rr] = v4f{0.f, 0.f, 0.f, 0.f};
        bw2[rr] = make_uint2(0, 0); bu2[rr] = make_uint2(0, 0);
        if constexpr (GATED) {   // two output columns per lane: two scales and two bias values of each half
            const float2 sg = *reinterpret_cast<const float2*>(p.w_scale + e_n_safe);
            const float2 su = *reinterpret_cast<const float2*>(p.w_scale + half_n + e_n_safe);
            sw4[rr] = v4f{sg.x, sg.y, 0.f, 0.f};
            su4[rr] = v4f{su.x, su.y, 0.f, 0.f};
            if (p.bias) {
                bw2[rr].x = *reinterpret_cast<const uint32_t*>(p.bias + e_n_safe);
                bu2[rr].x = *reinterpret_cast<const uint32_t*>(p.bias + half_n + e_n_safe);
            }
        } else {
            sw4[rr] = *reinterpret_cast<const v4f*>(p.w_scale + e_n_safe);
            if (p.bias) bw2[rr] = *reinterpret_cast<const uint2*>(p.bias + e_n_safe);
        }
        sa[rr] = p.x_scale[(p.x_scale_scalar || !e_live[rr]) ? 0 : e_m[rr]];
    }
    // gated residual: requested once the operand requests are out (its arguments are not among
    // the preloaded ones, and nothing before the operand requests should wait for a scalar load)
    uint2 res2[ROLE_ROUNDS], gate2[ROLE_ROUNDS];
#pragma unroll
    for (int rr = 0; rr < ROLE_ROUNDS; ++rr) { res2[rr] = make_uint2(0, 0); gate2[rr] = make_uint2(0, 0); }
    auto request_residual = [&]() {
        if constexpr (EPI == EPI_NONE) {
#pragma unroll
            for (int rr = 0; rr < ROLE_ROUNDS; ++rr) {
                if (p.res.residual != nullptr && e_live[rr]) {
                    res2[rr] = *reinterpret_cast<const uint2*>(p.res.residual + (int64_t)e_m[rr] * p.res.ld_res + e_n[rr]);
                    gate2[rr] = *reinterpret_cast<const uint2*>(
                        p.res.gate + (int64_t)(e_m[rr] / p.res.gate_group) * p.res.ld_gate + e_n[rr]);
                }
            }
        }
    };

    // ---- operand rows ----------------------------------------------------------------------
    // weight row of operand row r16 (0..15) of tile nt, token row of operand row r16 of block mb
    auto w_row = [&](int nt, int r16) -> int {
        if constexpr (GATED) {
            // rows 4p .. 4p+3 of a gated tile: gate columns 2p, 2p+1, then up columns 2p, 2p+1, so that
            // an MFMA lane (which owns four consecutive tile rows) holds both halves of two output
            // columns: no exchange between lanes, and all 64 lanes take part in the epilogue
            const int g = col0 + nt * 8 + 2 * (r16 >> 2) + (r16 & 1);
            return ((r16 & 2) ? half_n : 0) + (g < half_n ? g : half_n - 1);
        } else {
            const int r = col0 + nt * 16 + r16;
            return r < p.N ? r : p.N - 1;
        }
    };
    auto x_row = [&](int mb, int r16) -> int {
        const int r = m_base + mb * 16 + r16;
        return r < p.M ? r : p.M - 1;  // rows past M only feed outputs that are never stored
    };

    v4f acc[NT][MB];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[nt][mb] = v4f{0.f, 0.f, 0.f, 0.f};

    if constexpr (!STAGED) {
        const uint8_t* wrow[NT];
#pragma unroll
        for (int nt = 0; nt < NT; ++nt)
            wrow[nt] = operand_w ? p.w + operand_row_offset(w_unit(nt), l16, p.K) + q * kOperandChunkBytes
                                 : p.w + (size_t)w_row(nt, l16) * p.K + q * 16;
        const int w_hi = operand_w ? 4 * (int)kOperandChunkBytes : 64;   // chunk 4 + q
        const uint8_t* xrow[MB];
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) xrow[mb] = p.xq + (size_t)x_row(mb, l16) * p.K + q * 16;

        for (int rnd = 0; rnd < p.rounds; ++rnd) {
            v4i wlo[KPW][NT], whi[KPW][NT], xlo[KPW][MB], xhi[KPW][MB];
            bool live[KPW];
            // ---- 1. request every byte of this round ------------------------------------
#pragma unroll
            for (int j = 0; j < KPW; ++j) {
                const int s = (rnd * KPW + j) * SK_WAVES + wave;  // wave-uniform
                live[j] = s < total_steps;
                const int off = (live[j] ? s : total_steps - 1) << 7;
                const int woff_s = (live[j] ? s : total_steps - 1) << w_step_shift;
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    wlo[j][nt] = *reinterpret_cast<const v4i*>(wrow[nt] + woff_s);
                    whi[j][nt] = *reinterpret_cast<const v4i*>(wrow[nt] + woff_s + w_hi);
                }
#pragma unroll
                for (int mb = 0; mb < MB; ++mb) {
                    xlo[j][mb] = *reinterpret_cast<const v4i*>(xrow[mb] + off);
                    xhi[j][mb] = *reinterpret_cast<const v4i*>(xrow[mb] + off + 64);
                }
            }
            if (rnd == 0) request_residual();
            // ---- 2. MFMA ---------------------------------------------------------------------
#pragma unroll
            for (int j = 0; j < KPW; ++j) {
#pragma unroll
                for (int nt = 0; nt < NT; ++nt) {
                    v8i a = join(wlo[j][nt], whi[j][nt]);
                    if (!live[j]) a = v8i{0, 0, 0, 0, 0, 0, 0, 0};  // a step past K adds nothing
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
                        acc[nt][mb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                            a, join(xlo[j][mb], xhi[j][mb]), acc[nt][mb], 0, 0, 0, 0, 0, 0);
                }
            }
        }
    } else {
        // Copy geometry: one instruction moves 8 operand rows x 128 bytes; lane i fills slot i%8 of
        // row i/8 with chunk (i%8) ^ swz(row), swz(r) = (r/2)%8, which keeps the 128-bit reads of
        // the MFMA layout (lane (l16, q): chunks q and 4+q of row l16) off each other's banks.
        const int c_row = lane >> 3, c_slot = lane & 7;
        uint32_t woff[NT][2], xoff[MB][2];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const int r16 = hf * 8 + c_row;
            const uint32_t chunk = (uint32_t)((c_slot ^ ((r16 >> 1) & 7)) << 4);
#pragma unroll
            // rows and K are below 2^24 and their product below 2^32 (checked by the launcher): the
            // 24-bit multiply is a full-rate instruction, the general one is not
            // operand order: a unit's K step is copied as it lies, 1 KB per instruction (a copy that gathers it
            // into the row-major staging layout asks for 16 bytes of four different lines per four lanes
            // and runs at a quarter of the rate: measured 6.9 against 6.0 us for 50 x 1024 x 4096)
            for (int nt = 0; nt < NT; ++nt)
                woff[nt][hf] = operand_w ? operand_row_offset(w_unit(nt), 0, p.K) + hf * 1024 + lane * 16
                                         : __umul24((uint32_t)w_row(nt, r16), (uint32_t)p.K) + chunk;
#pragma unroll
            for (int mb = 0; mb < MB; ++mb) xoff[mb][hf] = __umul24((uint32_t)x_row(mb, r16), (uint32_t)p.K) + chunk;
        }
        const uint32_t lds_wave = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem + wave * PER_WAVE);
        const uint8_t* my_stage = smem + wave * PER_WAVE;
        const int swz = (l16 >> 1) & 7;
        const int rd_lo = l16 * 128 + ((q ^ swz) << 4), rd_hi = l16 * 128 + (((4 + q) ^ swz) << 4);
        // a staged unit in operand order: chunk q of row l16 at (16 q + l16) * 16 = 16 * lane, chunk 4 + q 1 KB on
        const int wrd_lo = operand_w ? lane * 16 : rd_lo, wrd_hi = operand_w ? 1024 + lane * 16 : rd_hi;

        for (int rnd = 0; rnd < p.rounds; ++rnd) {
            if (rnd > 0) asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // last round's reads have landed
            // ---- 1. request every byte of this round ------------------------------------
#pragma unroll
            for (int j = 0; j < KPW; ++j) {
                const int s = __builtin_amdgcn_readfirstlane((rnd * KPW + j) * SK_WAVES + wave);
                if (s < total_steps) {
                    const uint32_t dst = lds_wave + j * (BLOCKS * 2048);
                    // one branch per K step: the weights of this call either pass the caches by or not
                    if (stream_w) {
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                            for (int hf = 0; hf < 2; ++hf)
                                copy16_to_lds_nt(p.w + ((size_t)s << w_step_shift), woff[nt][hf], dst + (nt * 2 + hf) * 1024);
                    } else {
#pragma unroll
                        for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                            for (int hf = 0; hf < 2; ++hf)
                                copy16_to_lds(p.w + ((size_t)s << w_step_shift), woff[nt][hf], dst + (nt * 2 + hf) * 1024);
                    }
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
                        for (int hf = 0; hf < 2; ++hf)
                            copy16_to_lds(p.xq + ((size_t)s << 7), xoff[mb][hf], dst + ((NT + mb) * 2 + hf) * 1024);
                }
            }
            if (rnd == 0) request_residual();
            wait_copies<0>();   // everything this wavefront asked for (epilogue operands included)
            // ---- 2. MFMA ---------------------------------------------------------------------
#pragma unroll
            for (int j = 0; j < KPW; ++j) {
                const int s = __builtin_amdgcn_readfirstlane((rnd * KPW + j) * SK_WAVES + wave);
                if (s < total_steps) {
                    const uint8_t* blk = my_stage + j * (BLOCKS * 2048);
                    v8i xb[MB];
#pragma unroll
                    for (int mb = 0; mb < MB; ++mb)
                        xb[mb] = join(*reinterpret_cast<const v4i*>(blk + (NT + mb) * 2048 + rd_lo),
                                      *reinterpret_cast<const v4i*>(blk + (NT + mb) * 2048 + rd_hi));
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        const v8i a = join(*reinterpret_cast<const v4i*>(blk + nt * 2048 + wrd_lo),
                                           *reinterpret_cast<const v4i*>(blk + nt * 2048 + wrd_hi));
#pragma unroll
                        for (int mb = 0; mb < MB; ++mb)
                            acc[nt][mb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(
                                a, xb[mb], acc[nt][mb], 0, 0, 0, 0, 0, 0);
                    }
                }
            }
        }
        // the partial sums below overwrite this wavefront's own staging: its reads must be done
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    }

    // ---- 3. add the eight wavefronts' partial sums, in wavefront order -------------------
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) red(wave, nt, mb, lane) = acc[nt][mb];
    __syncthreads();
#pragma unroll
    for (int rr = 0; rr < ROLE_ROUNDS; ++rr) {
        if (e_nt[rr] >= NT) continue;   // wavefront-uniform: this wavefront has no block in this round
        v4f g = red(0, e_nt[rr], e_mb[rr], e_lane);
#pragma unroll
        for (int w = 1; w < SK_WAVES; ++w) g += red(w, e_nt[rr], e_mb[rr], e_lane);
        if (!e_role[rr]) continue;

        // ---- 4. epilogue --------------------------------------------------------------------
        const float bwf[4] = {bf16_bits_to_f32(bw2[rr].x & 0xFFFFu), bf16_bits_to_f32(bw2[rr].x >> 16),
                              bf16_bits_to_f32(bw2[rr].y & 0xFFFFu), bf16_bits_to_f32(bw2[rr].y >> 16)};
        if constexpr (GATED) {
            // g[0], g[1]: gate sums of this lane's two columns; g[2], g[3]: their up sums
            const float buf[2] = {bf16_bits_to_f32(bu2[rr].x & 0xFFFFu), bf16_bits_to_f32(bu2[rr].x >> 16)};
            float vf[2];
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                float v = __builtin_fmaf(g[r], sa[rr] * sw4[rr][r], bwf[r]);   // one rounding, like the tile kernels
                float up = __builtin_fmaf(g[2 + r], sa[rr] * su4[rr][r], buf[r]);
                round_bf16_pair(v, up);
                vf[r] = apply_act<EPI>(v) * up;
            }
            if (e_live[rr])
                *reinterpret_cast<uint32_t*>(p.out + (int64_t)e_m[rr] * p.ldo + e_n[rr]) = pack_bf16x2(vf[0], vf[1]);
        } else {
            float vf[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float v = __builtin_fmaf(g[r], sa[rr] * sw4[rr][r], bwf[r]);   // one rounding, like the tile kernels
                if constexpr (EPI != EPI_NONE) v = apply_act<EPI>(round_bf16(v));
                vf[r] = v;
            }
            if constexpr (EPI == EPI_NONE) {
                if (p.res.residual != nullptr) addcmul4(vf, res2[rr], gate2[rr]);
            }
            if (e_live[rr])
                *reinterpret_cast<uint2*>(p.out + (int64_t)e_m[rr] * p.ldo + e_n[rr]) =
                    make_uint2(pack_bf16x2(vf[0], vf[1]), pack_bf16x2(vf[2], vf[3]));
        }
    }
}

// ---- host side -------------------------------------------------------------------------

static int sk_ceil_div(int a, int b) { return (a + b - 1) / b; }

// Widths are multiples of 8 so that four consecutive output columns are valid together.
// Largest M served here.  Every group of token rows re-reads the weight tiles from L2, so with
// enough output tiles the LDS-staged tile kernels win; the dispatcher prefers those as soon as
// their grid is large enough (see launch_gemm) and falls back to this kernel up to here
// (N = 1024: ahead of the 128 x 128 tile kernel up to M = 1000, 11.0 against 17.5 us at 800 x 1024 x 4096).
static int skinny_max_m() {
    if (const char* e = tuning_env("PHYAI_FP8_SKINNY_MAXM")) return atoi(e);
    return 1024;
}

bool skinny_applicable(int M, int N, int K, int epilogue, int64_t ldo) {
    if (M > skinny_max_m() || K % 128 != 0 || ldo % 4 != 0) return false;
    if (epi_is_gated(epilogue)) return (N / 2) % 8 == 0;
    return N % 8 == 0;
}

// K steps a wavefront stages per round: up to 4, as many as K offers and the LDS holds
static int skinny_steps_per_round(int K, int nt, int mb) {
    const int per_wave = sk_ceil_div(K / 128, SK_WAVES);
    int kpw = per_wave >= 4 ? 4 : (per_wave >= 2 ? 2 : 1);
    while (kpw > 1 && SK_WAVES * kpw * (nt + mb) * 2048 > 160 * 1024) kpw /= 2;
    return kpw;
}

SkinnyPlan skinny_plan(int M, int N, int K, int epilogue) {
    const bool gated = epi_is_gated(epilogue);
    const int cols = gated ? N / 2 : N;
    const int per_tile = gated ? 8 : 16;
    SkinnyPlan pl;
    const int blocks = sk_ceil_div(M, 16);  // 16-row token blocks in all
    // Workgroup shape: nt weight tiles x mb token blocks.  A workgroup's time is set by the operand
    // blocks it pulls through its CU's vector cache (nt + mb per K step) and the launch takes as
    // many rounds as the workgroups need on 256 CUs: take the shape with the smallest product
    // (ties: the smaller workgroup).  The product orders the shapes as the clock does - at M = 50
    // (2560 columns: 2x2 3.49 us, 1x1 3.66, 1x4 3.73, 2x4 4.04 for products 4, 4, 5, 6; 1024
    // columns: 1x1 with four workgroups along M; gate_up: 2x4) as at M = 100 .. 1000
    // (800 x 1024 x 4096: 4x4 11.0 us, 2x4 13.6, 4x3 15.8, 2x3 16.4, 2x2 17.9 for products 8, 12,
    // 14, 15, 16), where the winner beats a fixed 1 x 4 by 10-50 % and, on the 1024-wide
    // projections, the 128 x 128 tile kernel (17.5 us).
    {
        int best_cost = 1 << 30;
        pl.nt = 1; pl.mb = 1;
        static const int shapes[][2] = {{1, 1}, {1, 2}, {1, 3}, {1, 4}, {2, 1}, {2, 2}, {2, 3}, {2, 4}, {4, 3}, {4, 4}};
        for (const auto& sh : shapes) {
            const int nt = sh[0], mb = sh[1];
            if (mb > blocks && mb > 1) continue;   // token blocks that do not exist
            const int wgs = sk_ceil_div(cols, per_tile * nt) * sk_ceil_div(blocks, mb);
            const int cost = sk_ceil_div(wgs, 256) * (nt + mb);
            if (cost < best_cost || (cost == best_cost && nt + mb < pl.nt + pl.mb)) {
                best_cost = cost; pl.nt = nt; pl.mb = mb;
            }
        }
        pl.tiles = sk_ceil_div(cols, per_tile * pl.nt);
        pl.msplit = sk_ceil_div(blocks, pl.mb);
    }
    if (const char* e = tuning_env("PHYAI_FP8_SKINNY_PLAN")) {  // "nt,mb" tuning override
        int nt = 0, mb = 0;
        if (sscanf(e, "%d,%d", &nt, &mb) == 2 && (nt == 1 || nt == 2 || (nt == 4 && mb >= 3)) && mb >= 1 && mb <= 4) {
            pl.nt = nt; pl.tiles = sk_ceil_div(cols, per_tile * nt); pl.mb = mb; pl.msplit = sk_ceil_div(blocks, mb);
        }
    }
    // staging of 8 wavefronts x kpw steps x (nt + mb) blocks of 2 KB must fit the 160 KB of LDS:
    // more rounds of fewer steps beat the unstaged form (down 50..400 x 1024 x 4096: 12 -> 7 us)
    pl.kpw = skinny_steps_per_round(K, pl.nt, pl.mb);
    pl.rounds = sk_ceil_div(sk_ceil_div(K / 128, SK_WAVES), pl.kpw);
    return pl;
}

// The staged form wherever its LDS fits (8 wavefronts x KPW steps x (NT + MB) blocks of 2 KB).
template <int MB, int NT, int KPW, int EPI>
static void sk_launch_one(const SkinnyArgs& a, const dim3& grid, hipStream_t st) {
    constexpr bool fits = SK_WAVES * KPW * (NT + MB) * 2048 <= 160 * 1024;
    static const bool want = []() { const char* e = tuning_env("PHYAI_FP8_SKINNY_STAGED"); return !(e && atoi(e) == 0); }();
    if constexpr (fits) {
        if (want && a.K * (int64_t)(a.N > a.M ? a.N : a.M) < ((int64_t)1 << 32) && a.K < (1 << 24) && a.N < (1 << 24)) {
            hipLaunchKernelGGL((gemm_fp8_skinny_kernel<MB, NT, KPW, EPI, true>), grid, dim3(SK_THREADS), 0, st,
                               a.w, a.xq, a.x_scale, a.w_scale, a.bias, a.K, a.N, a.M | (a.x_scale_scalar ? 1 << 30 : 0) | (a.stream_w ? 1 << 29 : 0) | (a.operand_w ? 1 << 28 : 0),
                               a.out, a.ldo, a.res);
            return;
        }
    }
    hipLaunchKernelGGL((gemm_fp8_skinny_kernel<MB, NT, KPW, EPI, false>), grid, dim3(SK_THREADS), 0, st,
                       a.w, a.xq, a.x_scale, a.w_scale, a.bias, a.K, a.N, a.M | (a.x_scale_scalar ? 1 << 30 : 0) | (a.stream_w ? 1 << 29 : 0) | (a.operand_w ? 1 << 28 : 0),
                       a.out, a.ldo, a.res);
}

template <int MB, int NT, int EPI>
static int sk_launch_kpw(const SkinnyArgs& a, const SkinnyPlan& pl, hipStream_t st) {
    const dim3 grid(pl.tiles, pl.msplit);
    switch (pl.kpw) {
    case 1: sk_launch_one<MB, NT, 1, EPI>(a, grid, st); return 0;
    case 2: sk_launch_one<MB, NT, 2, EPI>(a, grid, st); return 0;
    case 4: sk_launch_one<MB, NT, 4, EPI>(a, grid, st); return 0;
    default: return -2;
    }
}

template <int EPI>
static int sk_launch_epi(const SkinnyArgs& a, const SkinnyPlan& pl, hipStream_t st) {
    if (pl.nt == 4) {   // four weight tiles: 3 or 4 token blocks, one K step per wavefront per round
        if (pl.kpw != 1) return -2;
        const dim3 grid(pl.tiles, pl.msplit);
        if (pl.mb == 3) { sk_launch_one<3, 4, 1, EPI>(a, grid, st); return 0; }
        if (pl.mb == 4) { sk_launch_one<4, 4, 1, EPI>(a, grid, st); return 0; }
        return -2;
    }
    switch (pl.mb * 2 + (pl.nt - 1)) {
    case 2: return sk_launch_kpw<1, 1, EPI>(a, pl, st);
    case 3: return sk_launch_kpw<1, 2, EPI>(a, pl, st);
    case 4: return sk_launch_kpw<2, 1, EPI>(a, pl, st);
    case 5: return sk_launch_kpw<2, 2, EPI>(a, pl, st);
    case 6: return sk_launch_kpw<3, 1, EPI>(a, pl, st);
    case 7: return sk_launch_kpw<3, 2, EPI>(a, pl, st);
    case 8: return sk_launch_kpw<4, 1, EPI>(a, pl, st);
    case 9: return sk_launch_kpw<4, 2, EPI>(a, pl, st);
    default: return -2;
    }
}

int launch_gemm_skinny(const GemmProblem& g, const SkinnyPlan& pl, hipStream_t st) {
    SkinnyArgs a;
    a.xq = g.xq; a.w = g.w; a.x_scale = g.x_scale; a.w_scale = g.w_scale; a.bias = g.bias;
    a.out = g.out; a.ldo = g.ldo; a.M = g.M; a.N = g.N; a.K = g.K;
    a.x_scale_scalar = g.x_scale_is_scalar;
    a.rounds = pl.rounds;
    a.stream_w = g.stream_weights;
    a.operand_w = g.weight_layout != W_ROW_MAJOR;
    a.res = residual_of(g);
    switch (g.epilogue) {
    case EPI_NONE: return sk_launch_epi<EPI_NONE>(a, pl, st);
    case EPI_GEGLU_TANH: return sk_launch_epi<EPI_GEGLU_TANH>(a, pl, st);
    case EPI_GEGLU_ERF: return sk_launch_epi<EPI_GEGLU_ERF>(a, pl, st);
    case EPI_SWIGLU: return sk_launch_epi<EPI_SWIGLU>(a, pl, st);
    case EPI_GELU_TANH: return sk_launch_epi<EPI_GELU_TANH>(a, pl, st);
    case EPI_GELU_ERF: return sk_launch_epi<EPI_GELU_ERF>(a, pl, st);
    default: return -2;
    }
}

}  // namespace phyai
