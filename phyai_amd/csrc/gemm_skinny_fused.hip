// The whole quantized linear for small token counts in ONE launch: every workgroup quantizes the
// activation rows it multiplies, then runs the weight-streaming GEMM of gemm_skinny.hip on them.
//
// Two launches (row-wise quantizer, then GEMM) cost two kernel-node floors per linear, and at
// M = 50 a node floor is as long as the work.  Quantizing inside the GEMM repeats the conversion in
// every workgroup that shares token rows, so the shape of a workgroup is chosen for that cost:
//
//  * total conversions = (column tiles) x M x K, so a workgroup owns MANY weight tiles (NT up to 8:
//    128 output columns) and FEW token rows (ROWS = 8, 16 or 32), the opposite of the
//    two-launch kernel's choice; the chip is filled along M instead (grid.y), weight tiles shared
//    between the workgroups of a tile column come from L2;
//  * a wavefront converts only the K steps it multiplies (w, w + 8, ...): the bf16 rows of those
//    steps go global -> VGPR with loads whose arrival is awaited by hand, so that the wait leaves
//    the younger global -> LDS copies of the weights in flight; conversion then runs while the
//    weights are still landing;
//  * the row maximum needs all of K: per-wavefront maxima (packed 16-bit max, then DPP inside the 16
//    lanes that share a row) meet in a small LDS table, one barrier, and every wavefront derives all
//    row scales itself (lane l: row l), handing them to the converting lanes with ds_bpermute;
//  * arithmetic is that of the stand-alone quantizer (quant_device.h): bit-equal codes and scales,
//    so the output equals quantizer + GEMM bit for bit.
//
// Codes are written into the wavefront's own LDS staging slice in the layout the weight-streaming
// kernel's copies produce (128-byte rows, 16-byte chunks XOR-swizzled by row), and from there on
// the kernel is that kernel: MFMA over the wavefront's K steps, partial sums through LDS in
// wavefront order, epilogue of four output columns per lane.
#include "fp8_device.h"
#include "launch.h"
#include <type_traits>

#include "quant_device.h"
#include "stamps.h"
#include "tuning.h"
#include "weight_layout.h"
#include <stdio.h>

namespace phyai {

constexpr int FQ_WAVES = 8;
constexpr int FQ_THREADS = FQ_WAVES * kWave;
// (debug build only: the kernel's time stamps - 1 rows landed, 2 row scales known, 3 codes written, 4 MFMAs done,
// 5 partial sums exchanged, 6 stores issued)
PHYAI_STAMP_SINK(g_fq_stamps)

// A 16-byte load whose arrival the compiler does not track: the value may be used only after
// landed() has waited for it.
__device__ __forceinline__ v4i fq_load16_async(const uint8_t* base, uint32_t lane_offset) {
    v4i v;
    asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(v) : "v"(lane_offset), "s"(base) : "memory");
    return v;
}
// At most YOUNGER memory instructions of this wavefront issued after the load are still in flight;
// ties the register to the wait so that no use can move above it.
template <int YOUNGER>
__device__ __forceinline__ void fq_landed(v4i& a) {
    static_assert(YOUNGER >= 0 && YOUNGER < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%1)" : "+v"(a) : "n"(YOUNGER) : "memory");
}
__device__ __forceinline__ uint4 fq_as_uint4(v4i v) {
    return make_uint4((uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]);
}
__device__ __forceinline__ v8i fq_join(v4i lo, v4i hi) {
    v8i f;
    f[0] = lo[0]; f[1] = lo[1]; f[2] = lo[2]; f[3] = lo[3];
    f[4] = hi[0]; f[5] = hi[1]; f[6] = hi[2]; f[7] = hi[3];
    return f;
}
// m / group for the token rows of this kernel (0 <= m < 128, 1 <= group <= 128) without the integer
// division sequence: (m + 0.5) / group is at least 0.5 / 128 away from an integer, and the float
// product with the hardware reciprocal is off by less than 128.5 * 2^-22.
__device__ __forceinline__ int gate_row_of(int m, int group) {
    return group == 1 ? m : (int)(((float)m + 0.5f) * __builtin_amdgcn_rcpf((float)group));
}
__device__ __forceinline__ float fq_bpermute(float v, int src_lane) {
    return __uint_as_float((uint32_t)__builtin_amdgcn_ds_bpermute(src_lane << 2, (int)__float_as_uint(v)));
}

// Row maxima handed from one linear to the next (the gate | up projection of an MLP to its down
// projection): table[M][64] of bf16 bit patterns of |value| maxima, one slot per workgroup column of
// the producer; the consumer takes the maximum over the first `parts` slots of a row.  Plain stores
// and loads, no atomics, nothing to reset between calls.
constexpr int kAmaxSlots = 64;   // slots (16-bit) per token row: 128 bytes
struct AmaxOut {
    uint16_t* table;   // null: do not produce
};

// ROWS: token rows per workgroup (8, 16 or 32; grid.y workgroups cover M); NT: 16-row weight tiles
// per workgroup; KPW: K steps per wavefront (K <= 128 * 8 * KPW, one round).
//
// Between the row loads and the wait for them the code is straight-line on purpose: the loaded
// registers are live behind the compiler's back, and any branch there lets it merge values with
// copies that would read them too early.  Hence the weight requests are issued for every K step slot
// (a slot past the end fetches the last step again; it is never multiplied), which also keeps the
// number of requests younger than the row loads a compile-time constant, and the cache policy of the
// weight requests (STREAM: non-temporal) is a template parameter, not a run-time branch.
//
// DIRECT: the weights are in MFMA operand order (weight_layout.h): lane i of a wavefront wants bytes
// [16 i, 16 i + 16) and [1024 + 16 i, ...) of a 2 KB unit, so every request is 1 KB in a row and goes
// straight into registers; LDS then holds only the activation codes.  Otherwise the weights are
// row-major and are staged through the wavefront's LDS slice.
//
// AMAX_IN: the row maxima come from the producer of the activations (AmaxOut of an earlier launch)
// instead of being found here: no table of per-wavefront maxima, no barrier before the conversions.
template <int ROWS, int NT, int KPW, int EPI, bool STREAM, bool DIRECT, bool AMAX_IN>
__global__ __launch_bounds__(FQ_THREADS) void gemm_fp8_fusedq_kernel(
    const uint8_t* __restrict__ a_w, const uint8_t* __restrict__ a_x, int a_K, int a_N, int a_M, int a_ldx_bytes,
    const uint8_t* __restrict__ a_amax_in, int a_amax_parts, const float* __restrict__ a_w_scale,
    const uint16_t* __restrict__ a_bias, uint16_t* __restrict__ a_out, int64_t a_ldo, const ResidualArgs a_res,
    const AmaxOut a_amax_out) {
    constexpr bool GATED = epi_is_gated(EPI);
    constexpr int MB = (ROWS + 15) / 16;              // 16-row token blocks (the last one may be half used)
    constexpr int COLS_PER_TILE = GATED ? 8 : 16;
    // One K step of staging: NT weight blocks of 2 KB (16 rows x 128 bytes; none when they go straight to
    // registers) and the codes of the token rows; an 8-row workgroup keeps only the 1 KB of its 8 rows
    // (the MFMA's other 8 columns re-read them).
    constexpr int XB = ROWS < 16 ? ROWS * 128 : 2048;
    constexpr int WB = DIRECT ? 0 : NT * 2048;        // staged weight bytes per K step
    constexpr int STEP_BYTES = WB + MB * XB;
    constexpr int RED_PER_WAVE = NT * MB * kWave * (int)sizeof(v4f);
    constexpr int STAGE_PER_WAVE = KPW * STEP_BYTES;
    constexpr int PER_WAVE = STAGE_PER_WAVE > RED_PER_WAVE ? STAGE_PER_WAVE : RED_PER_WAVE;
    // The table of row maxima (one word per wavefront and row) has its own 2 KB unless the staging
    // leaves no room: then it lies over the first wavefront's code block of K step 0, which nobody
    // writes before a second barrier has seen every wavefront read the table.
    constexpr int TBL_ROWS = ROWS < 64 ? ROWS : 64;
    constexpr bool TBL_ALIASED = !AMAX_IN && FQ_WAVES * PER_WAVE + FQ_WAVES * 64 * 4 > 160 * 1024;
    static_assert(!TBL_ALIASED || FQ_WAVES * TBL_ROWS * 4 <= XB, "aliased table does not fit a code block");
    static_assert(ROWS == 8 || ROWS % 16 == 0, "token rows per workgroup");   // (4-row workgroups were measured: slower)
    static_assert(FQ_WAVES * PER_WAVE + ((TBL_ALIASED || AMAX_IN) ? 0 : FQ_WAVES * 64 * 4) <= 160 * 1024, "staging does not fit the LDS");
    static_assert(!AMAX_IN || (ROWS <= 16 && EPI == EPI_NONE), "row maxima are handed to plain projections of up to 16 rows per workgroup");
    constexpr int ROLE_ROUNDS = (NT * MB + FQ_WAVES - 1) / FQ_WAVES;
    constexpr int AL = AMAX_IN ? (ROWS + 7) / 8 : 0;  // loads of handed-over maxima per lane: 8 rows x 8 lanes x 16 bytes each
    constexpr int YOUNGER = KPW * NT * 2;             // weight requests issued behind the row loads
    auto rows_in_block = [](int mb) constexpr { return ROWS - 16 * mb < 16 ? ROWS - 16 * mb : 16; };

    __shared__ __attribute__((aligned(1024))) uint8_t smem[FQ_WAVES * PER_WAVE];
    __shared__ uint32_t amax_own[(TBL_ALIASED || AMAX_IN) ? 1 : FQ_WAVES * 64];
    constexpr bool MAKES_AMAX = EPI != EPI_NONE;      // AmaxOut exists for the epilogues an MLP's first projection has
    __shared__ uint32_t amax_made[MAKES_AMAX ? 64 : 1];   // AmaxOut: maxima of this workgroup's outputs per token row
    uint32_t* amax_tbl = TBL_ALIASED ? reinterpret_cast<uint32_t*>(smem + WB) : amax_own;   // [wavefront][TBL_ROWS]
    auto red = [&](int w, int nt, int mb, int l) -> v4f& {
        return reinterpret_cast<v4f*>(smem + w * PER_WAVE)[(nt * MB + mb) * kWave + l];
    };

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int l16 = lane & 15, q = lane >> 4;
    const int M = a_M, N = a_N, K = a_K;
    PHYAI_STAMP_BEGIN
    const int half_n = N / 2;
    const int n_out_total = GATED ? half_n : N;
    const int col0 = blockIdx.x * (COLS_PER_TILE * NT);
    const int total_steps = K >> 7;
    const int m_base = blockIdx.y * ROWS;

    // ---- 1a. this wavefront's K steps of the activation rows, bf16, straight into registers --------
    // (with AMAX_IN, in front of them, the maxima the producer left for this workgroup's rows: lane i
    // takes 8 slots of row i / 8)
    // instruction i of block mb covers rows 4i .. 4i+3 of the block: 16 lanes per row, 16 bytes
    // (8 elements) per lane, 256 bytes = one K step per row.  Rows past M repeat row M - 1.
    const int xr = lane >> 4, xc = lane & 15;
    v4i am[AL > 0 ? AL : 1];
    if constexpr (AMAX_IN) {
#pragma unroll
        for (int a = 0; a < AL; ++a) {
            int r = m_base + a * 8 + (lane >> 3);
            r = r < M ? r : M - 1;
            am[a] = fq_load16_async(a_amax_in, (uint32_t)r * (kAmaxSlots * 2) + (lane & 7) * 16);
        }
    }
    v4i xv[KPW][MB][4];
#pragma unroll
    for (int j = 0; j < KPW; ++j) {
        const int s = __builtin_amdgcn_readfirstlane(j * FQ_WAVES + wave);
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                // The load is unconditional at run time (a K step past the end re-reads the last one:
                // the same rows, so the row maxima are unchanged, and its codes are never multiplied):
                // a value that arrives behind the compiler's back must not pass through a conditional
                // copy before fq_landed() has waited for it.
                if (4 * i < rows_in_block(mb)) {
                    int r = m_base + mb * 16 + 4 * i + xr;
                    r = r < M ? r : M - 1;
                    const int s_safe = s < total_steps ? s : total_steps - 1;
                    xv[j][mb][i] = fq_load16_async(a_x + ((size_t)s_safe << 8), (uint32_t)r * (uint32_t)a_ldx_bytes + xc * 16);
                } else {
                    xv[j][mb][i] = v4i{0, 0, 0, 0};
                }
            }
    }
    // Every wavefront's row loads go out before any wavefront's weight requests: the CU's memory pipeline
    // serves requests in order, and a wavefront that starts late would otherwise queue its few row loads
    // behind the 16 KB of weights of each earlier one - the rows, not the weights, are what the workgroup
    // waits for first.  (A bare barrier: nothing is awaited, only the order of issue is fixed.)  Measured:
    // o 2048 -> 1024 at M = 50 4.54 -> 4.32 us; with one K step per wavefront (K = 1024) the later start
    // of the weight requests costs as much as the rows gain when the weights are staged through LDS (gate_up
    // 6.33 -> 6.41 us), so only K > 1024 there; with weights straight into registers it is level or 0.05 us
    // ahead at K = 1024 too (qkv 3.62 -> 3.57 us, gate_up 5.71 -> 5.65 us).
    if constexpr (KPW >= 2 || DIRECT) __builtin_amdgcn_s_barrier();
    // ---- 1b. the weights of the same K steps: into registers, or global -> LDS (as in gemm_skinny.hip) --
    const uint32_t lds_wave = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)smem + wave * PER_WAVE);
    uint8_t* my_stage = smem + wave * PER_WAVE;
    v4i wlo[DIRECT ? KPW : 1][DIRECT ? NT : 1], whi[DIRECT ? KPW : 1][DIRECT ? NT : 1];
    if constexpr (DIRECT) {
        const uint32_t w_units = (uint32_t)N >> 4;
#pragma unroll
        for (int j = 0; j < KPW; ++j) {
            const int s = __builtin_amdgcn_readfirstlane(j * FQ_WAVES + wave);
            const uint32_t s_safe = s < total_steps ? s : total_steps - 1;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                const uint32_t wu = blockIdx.x * NT + nt, unit = wu < w_units ? wu : w_units - 1;
                // unit (unit, s_safe) of the matrix: 2 KB, lane i wants chunks i and 64 + i of it
                const v4i* src = reinterpret_cast<const v4i*>(a_w + ((size_t)unit * (uint32_t)total_steps + s_safe) * kOperandStepBytes) + lane;
                if constexpr (STREAM) {
                    wlo[j][nt] = __builtin_nontemporal_load(src);
                    whi[j][nt] = __builtin_nontemporal_load(src + 64);
                } else {
                    wlo[j][nt] = src[0];
                    whi[j][nt] = src[64];
                }
            }
        }
    } else {
        const int c_row = lane >> 3, c_slot = lane & 7;
        uint32_t woff[NT][2];
#pragma unroll
        for (int hf = 0; hf < 2; ++hf) {
            const int r16 = hf * 8 + c_row;
            const uint32_t chunk = (uint32_t)((c_slot ^ ((r16 >> 1) & 7)) << 4);
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                int wr;
                if constexpr (GATED) {
                    // rows 4p .. 4p+3 of a gated tile: gate columns 2p, 2p+1, then up columns 2p, 2p+1, so
                    // that an MFMA lane (which owns four consecutive tile rows) holds both halves of two
                    // output columns and all 64 lanes take part in the epilogue
                    const int g = col0 + nt * 8 + 2 * (r16 >> 2) + (r16 & 1);
                    wr = ((r16 & 2) ? half_n : 0) + (g < half_n ? g : half_n - 1);
                } else {
                    const int r = col0 + nt * 16 + r16;
                    wr = r < N ? r : N - 1;
                }
                woff[nt][hf] = __umul24((uint32_t)wr, (uint32_t)K) + chunk;
            }
        }
#pragma unroll
        for (int j = 0; j < KPW; ++j) {
            const int s = __builtin_amdgcn_readfirstlane(j * FQ_WAVES + wave);
            const int s_safe = s < total_steps ? s : total_steps - 1;
            const uint32_t dst = lds_wave + j * STEP_BYTES;
#pragma unroll
            for (int nt = 0; nt < NT; ++nt)
#pragma unroll
                for (int hf = 0; hf < 2; ++hf) {
                    if constexpr (STREAM) copy16_to_lds_nt(a_w + ((size_t)s_safe << 7), woff[nt][hf], dst + (nt * 2 + hf) * 1024);
                    else copy16_to_lds(a_w + ((size_t)s_safe << 7), woff[nt][hf], dst + (nt * 2 + hf) * 1024);
                }
        }
    }

    // ---- epilogue roles: index arithmetic in the shadow of the row loads (no memory operation and no
    // branch here, see above) ---------------------------------------------------------------------------
    int e_mb[ROLE_ROUNDS], e_nt[ROLE_ROUNDS], e_m[ROLE_ROUNDS], e_n[ROLE_ROUNDS], e_n_safe[ROLE_ROUNDS];
    bool e_role[ROLE_ROUNDS], e_live[ROLE_ROUNDS];
#pragma unroll
    for (int rr = 0; rr < ROLE_ROUNDS; ++rr) {
        const int role = rr * FQ_WAVES + wave;
        e_mb[rr] = role % MB;
        e_nt[rr] = role / MB;
        e_role[rr] = e_nt[rr] < NT;
        const int r_in = e_mb[rr] * 16 + l16;                 // token row within the workgroup
        e_m[rr] = m_base + r_in;
        e_n[rr] = col0 + (e_nt[rr] < NT ? e_nt[rr] : 0) * COLS_PER_TILE + (GATED ? 2 : 4) * q;
        e_live[rr] = e_role[rr] && r_in < ROWS && e_m[rr] < M && e_n[rr] < n_out_total;
        e_n_safe[rr] = e_live[rr] ? e_n[rr] : 0;
    }
    // which of a lane's 8 handed-over slots exist (slot index < parts), as masks over its four words
    uint32_t am_mask[4] = {0, 0, 0, 0};
    if constexpr (AMAX_IN) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const int e0 = 8 * (lane & 7) + 2 * i;
            am_mask[i] = (e0 < a_amax_parts ? 0x7FFFu : 0u) | (e0 + 1 < a_amax_parts ? 0x7FFF0000u : 0u);
        }
    }

    // ---- 1c. the row loads have landed (the weight requests stay in flight) ----------------------------
    // exactly YOUNGER requests are younger than the row loads
    if constexpr (AMAX_IN) {
#pragma unroll
        for (int a = 0; a < AL; ++a) fq_landed<YOUNGER>(am[a]);
    }
#pragma unroll
    for (int j = 0; j < KPW; ++j)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (4 * i < rows_in_block(mb)) fq_landed<YOUNGER>(xv[j][mb][i]);

    PHYAI_STAMP(1)
    // ---- row scales: lane l holds the scale of "its" row and the reciprocal ----------------------------
    // own maxima: lane l <-> row l, every wavefront derives all scales from the table; handed-over maxima:
    // lanes 8 r .. 8 r + 7 of register set a <-> row 8 a + r
    constexpr int SETS = AMAX_IN ? AL : 1;
    float s_row[SETS], r_row[SETS];
    bool slow_row = false;
    if constexpr (AMAX_IN) {
#pragma unroll
        for (int a = 0; a < AL; ++a) {
            const uint4 w4 = fq_as_uint4(am[a]);
            uint32_t m2 = 0;
            m2 = absmax8_pk(make_uint4(w4.x & am_mask[0], w4.y & am_mask[1], w4.z & am_mask[2], w4.w & am_mask[3]), m2);
            uint32_t v = absmax_finish(m2), o;
            o = dpp_move_u32<0xB1>(v);  v = o > v ? o : v;      // the 8 lanes of a row
            o = dpp_move_u32<0x4E>(v);  v = o > v ? o : v;
            o = dpp_move_u32<0x141>(v); v = o > v ? o : v;
            s_row[a] = scale_from_amax_bits<QUANT_ACT_DYNAMIC>(v);
            r_row[a] = biased_reciprocal(s_row[a]);
            slow_row = slow_row || (__float_as_uint(s_row[a]) & 0x7FFFFFFFu) >= 0x7F800000u;
        }
    } else {
        // the maxima of this wavefront's K steps, one word per row into the table
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (4 * i >= rows_in_block(mb)) continue;
                uint32_t m2 = 0;
#pragma unroll
                for (int j = 0; j < KPW; ++j) m2 = absmax8_pk(fq_as_uint4(xv[j][mb][i]), m2);
                uint32_t v = absmax_finish(m2), o;
                o = dpp_move_u32<0xB1>(v);  v = o > v ? o : v;      // the 16 lanes of a row
                o = dpp_move_u32<0x4E>(v);  v = o > v ? o : v;
                o = dpp_move_u32<0x141>(v); v = o > v ? o : v;
                o = dpp_move_u32<0x140>(v); v = o > v ? o : v;
                if (xc == 0) amax_tbl[wave * TBL_ROWS + mb * 16 + 4 * i + xr] = v;
            }
        __syncthreads();
    }
    if constexpr (MAKES_AMAX) {
        // AmaxOut: the table the epilogue folds its outputs into starts at zero (ordered before the
        // epilogue by the barrier in front of the reduction)
        if (a_amax_out.table != nullptr && tid < 64) amax_made[tid] = 0u;
    }
    // ---- the column operands of the epilogue: requested here, off the path from the row loads to the
    // row maxima, and hidden behind the conversions ------------------------------------------------------
    v4f sw4[ROLE_ROUNDS], su4[ROLE_ROUNDS];
    uint2 bw2[ROLE_ROUNDS], bu2[ROLE_ROUNDS];
#pragma unroll
    for (int rr = 0; rr < ROLE_ROUNDS; ++rr) {
        su4[rr] = v4f{0.f, 0.f, 0.f, 0.f};
        bw2[rr] = make_uint2(0, 0); bu2[rr] = make_uint2(0, 0);
        if constexpr (GATED) {   // two output columns per lane: two scales and two bias values of each half
            const float2 sg = *reinterpret_cast<const float2*>(a_w_scale + e_n_safe[rr]);
            const float2 su = *reinterpret_cast<const float2*>(a_w_scale + half_n + e_n_safe[rr]);
            sw4[rr] = v4f{sg.x, sg.y, 0.f, 0.f};
            su4[rr] = v4f{su.x, su.y, 0.f, 0.f};
            if (a_bias) {
                bw2[rr].x = *reinterpret_cast<const uint32_t*>(a_bias + e_n_safe[rr]);
                bu2[rr].x = *reinterpret_cast<const uint32_t*>(a_bias + half_n + e_n_safe[rr]);
            }
        } else {
            sw4[rr] = *reinterpret_cast<const v4f*>(a_w_scale + e_n_safe[rr]);
            if (a_bias) bw2[rr] = *reinterpret_cast<const uint2*>(a_bias + e_n_safe[rr]);
        }
    }

    if constexpr (!AMAX_IN) {
        s_row[0] = 1.0f; r_row[0] = 1.0f;
        if (lane < ROWS) {
            uint32_t a = amax_tbl[lane];
#pragma unroll
            for (int w = 1; w < FQ_WAVES; ++w) a = amax_tbl[w * TBL_ROWS + lane] > a ? amax_tbl[w * TBL_ROWS + lane] : a;
            s_row[0] = scale_from_amax_bits<QUANT_ACT_DYNAMIC>(a);
            r_row[0] = biased_reciprocal(s_row[0]);
            slow_row = (__float_as_uint(s_row[0]) & 0x7FFFFFFFu) >= 0x7F800000u;   // an Inf or NaN in the row
        }
    }
    const bool any_slow = __builtin_amdgcn_ballot_w64(slow_row) != 0;       // wavefront-uniform
    if constexpr (TBL_ALIASED) __syncthreads();   // the table lies where codes go next: everyone has read it
    // value of `v` (s_row or r_row) for row R of the workgroup, R's register set known at compile time
    auto of_row = [&](const float* v, int set, int r_in_set) -> float {
        if constexpr (AMAX_IN) return fq_bpermute(v[set], 8 * r_in_set);
        else return fq_bpermute(v[0], set * 8 + r_in_set);
    };
    float sa[ROLE_ROUNDS];
#pragma unroll
    for (int rr = 0; rr < ROLE_ROUNDS; ++rr) {
        if constexpr (AMAX_IN) {   // one 16-row block: rows 0 .. 7 in set 0, 8 .. 15 in set 1 (an 8-row block repeats itself)
            const float lo = of_row(s_row, 0, l16 & 7);
            sa[rr] = lo;
            if constexpr (AL > 1) {
                const float hi = of_row(s_row, 1, l16 & 7);
                sa[rr] = (l16 & 8) ? hi : lo;
            }
        } else {
            sa[rr] = fq_bpermute(s_row[0], (e_mb[rr] * 16 + l16) & 63);
        }
    }

    // gated residual: requested now, behind the row loads whose wait counted instructions
    uint2 res2[ROLE_ROUNDS], gate2[ROLE_ROUNDS];
#pragma unroll
    for (int rr = 0; rr < ROLE_ROUNDS; ++rr) { res2[rr] = make_uint2(0, 0); gate2[rr] = make_uint2(0, 0); }
    if constexpr (EPI == EPI_NONE) {
#pragma unroll
        for (int rr = 0; rr < ROLE_ROUNDS; ++rr) {
            if (a_res.residual != nullptr && e_live[rr]) {
                res2[rr] = *reinterpret_cast<const uint2*>(a_res.residual + (int64_t)e_m[rr] * a_res.ld_res + e_n[rr]);
                gate2[rr] = *reinterpret_cast<const uint2*>(
                    a_res.gate + (int64_t)gate_row_of(e_m[rr], a_res.gate_group) * a_res.ld_gate + e_n[rr]);
            }
        }
    }

    PHYAI_STAMP(2)
    // ---- 1d. codes into the staging slice, in the layout the copies would have produced -----------
    // (all reciprocals are fetched before the first conversion, and the choice between the two
    // division forms is made once for the workgroup's rows, not per block of four rows)
    float r_of[MB][4], s_of[MB][4];
#pragma unroll
    for (int mb = 0; mb < MB; ++mb)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            r_of[mb][i] = 1.0f; s_of[mb][i] = 1.0f;
            // row mb * 16 + 4 i + xr: set 2 mb + i / 2, row 4 (i % 2) + xr of the set
            if (4 * i < rows_in_block(mb)) r_of[mb][i] = of_row(r_row, 2 * mb + (i >> 1), 4 * (i & 1) + xr);
        }
    auto write_codes = [&](auto fast_tag) {
        constexpr bool FAST = decltype(fast_tag)::value;
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (4 * i >= rows_in_block(mb)) continue;
                const int r16 = 4 * i + xr;
                RowDivisor dv;
                dv.s = s_of[mb][i];
                dv.r = r_of[mb][i];
                dv.fast = FAST;
                const int at = r16 * 128 + (((xc >> 1) ^ ((r16 >> 1) & 7)) << 4) + (xc & 1) * 8;
#pragma unroll
                for (int j = 0; j < KPW; ++j)
                    *reinterpret_cast<uint2*>(my_stage + j * STEP_BYTES + WB + mb * XB + at) =
                        encode8<QUANT_ACT_DYNAMIC>(fq_as_uint4(xv[j][mb][i]), dv);
            }
    };
    if (!any_slow) {
        write_codes(std::true_type{});
    } else {
#pragma unroll
        for (int mb = 0; mb < MB; ++mb)
#pragma unroll
            for (int i = 0; i < 4; ++i)
                if (4 * i < rows_in_block(mb)) s_of[mb][i] = of_row(s_row, 2 * mb + (i >> 1), 4 * (i & 1) + xr);
        write_codes(std::false_type{});
    }
    PHYAI_STAMP(3)
    if constexpr (!DIRECT) wait_copies<0>();   // the weights (and everything else this wavefront asked for)

    // ---- 2. MFMA over this wavefront's K steps -------------------------------------------------------
    v4f acc[NT][MB];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) acc[nt][mb] = v4f{0.f, 0.f, 0.f, 0.f};
    const int swz = (l16 >> 1) & 7;
    const int rd_lo = l16 * 128 + ((q ^ swz) << 4), rd_hi = l16 * 128 + (((4 + q) ^ swz) << 4);
    // token-row operand: an 8-row block is read twice over (columns 8 .. 15 of the product are not stored)
    const int xl = ROWS < 16 ? (l16 & (ROWS - 1)) : l16, xswz = (xl >> 1) & 7;
    const int xrd_lo = xl * 128 + ((q ^ xswz) << 4), xrd_hi = xl * 128 + (((4 + q) ^ xswz) << 4);
#pragma unroll
    for (int j = 0; j < KPW; ++j) {
        const int s = __builtin_amdgcn_readfirstlane(j * FQ_WAVES + wave);
        if (s < total_steps) {
            const uint8_t* blk = my_stage + j * STEP_BYTES;
            v8i xb[MB];
#pragma unroll
            for (int mb = 0; mb < MB; ++mb)
                xb[mb] = fq_join(*reinterpret_cast<const v4i*>(blk + WB + mb * XB + xrd_lo),
                                 *reinterpret_cast<const v4i*>(blk + WB + mb * XB + xrd_hi));
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                v8i a;
                if constexpr (DIRECT) a = fq_join(wlo[j][nt], whi[j][nt]);
                else a = fq_join(*reinterpret_cast<const v4i*>(blk + nt * 2048 + rd_lo),
                                 *reinterpret_cast<const v4i*>(blk + nt * 2048 + rd_hi));
#pragma unroll
                for (int mb = 0; mb < MB; ++mb)
                    acc[nt][mb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, xb[mb], acc[nt][mb], 0, 0, 0, 0, 0, 0);
            }
        }
    }
    // the partial sums below overwrite this wavefront's own staging: its reads must be done
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    PHYAI_STAMP(4)

    // AmaxOut: |bf16| bit patterns order like the values.  The maximum of a lane's outputs (two packed
    // pairs), then over the four lane groups that share a token row, then over the workgroup's tiles in LDS.
    auto fold_amax = [&](uint32_t p0, uint32_t p1, int mb) {
        const u16x2_t m = __builtin_elementwise_max(__builtin_bit_cast(u16x2_t, p0), __builtin_bit_cast(u16x2_t, p1));
        uint32_t v = absmax_finish(__builtin_bit_cast(uint32_t, m));
        const auto h16 = __builtin_amdgcn_permlane16_swap(v, v, false, false);
        v = h16[0] > h16[1] ? h16[0] : h16[1];
        const auto h32 = __builtin_amdgcn_permlane32_swap(v, v, false, false);
        v = h32[0] > h32[1] ? h32[0] : h32[1];
        if (q == 0) atomicMax(&amax_made[mb * 16 + l16], v);
    };

    // ---- 3. add the eight wavefronts' partial sums, in wavefront order ---------------------------
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
        for (int mb = 0; mb < MB; ++mb) red(wave, nt, mb, lane) = acc[nt][mb];
    __syncthreads();
    PHYAI_STAMP(5)
#pragma unroll
    for (int rr = 0; rr < ROLE_ROUNDS; ++rr) {
        if (e_nt[rr] >= NT) continue;   // wavefront-uniform: no block for this wavefront in this round
        v4f g = red(0, e_nt[rr], e_mb[rr], lane);
#pragma unroll
        for (int w = 1; w < FQ_WAVES; ++w) g += red(w, e_nt[rr], e_mb[rr], lane);
        if (!e_role[rr]) continue;

        // ---- 4. epilogue (the arithmetic of gemm_skinny.hip, operation for operation) --------------
        const float bwf[4] = {bf16_bits_to_f32(bw2[rr].x & 0xFFFFu), bf16_bits_to_f32(bw2[rr].x >> 16),
                              bf16_bits_to_f32(bw2[rr].y & 0xFFFFu), bf16_bits_to_f32(bw2[rr].y >> 16)};
        if constexpr (GATED) {
            // g[0], g[1]: gate sums of this lane's two columns; g[2], g[3]: their up sums
            const float buf[2] = {bf16_bits_to_f32(bu2[rr].x & 0xFFFFu), bf16_bits_to_f32(bu2[rr].x >> 16)};
            float vf[2];
#pragma unroll
            for (int r = 0; r < 2; ++r) {
                float v = __builtin_fmaf(g[r], sa[rr] * sw4[rr][r], bwf[r]);
                float up = __builtin_fmaf(g[2 + r], sa[rr] * su4[rr][r], buf[r]);
                round_bf16_pair(v, up);
                vf[r] = apply_act<EPI>(v) * up;
            }
            const uint32_t packed = pack_bf16x2(vf[0], vf[1]);
            if (e_live[rr]) *reinterpret_cast<uint32_t*>(a_out + (int64_t)e_m[rr] * a_ldo + e_n[rr]) = packed;
            if (a_amax_out.table != nullptr)   // wavefront-uniform
                fold_amax(e_live[rr] ? (packed & 0x7FFF7FFFu) : 0u, 0u, e_mb[rr]);
        } else {
            float vf[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                float v = __builtin_fmaf(g[r], sa[rr] * sw4[rr][r], bwf[r]);
                if constexpr (EPI != EPI_NONE) v = apply_act<EPI>(round_bf16(v));
                vf[r] = v;
            }
            if constexpr (EPI == EPI_NONE) {
                if (a_res.residual != nullptr) addcmul4(vf, res2[rr], gate2[rr]);
            }
            const uint2 packed = make_uint2(pack_bf16x2(vf[0], vf[1]), pack_bf16x2(vf[2], vf[3]));
            if (e_live[rr]) *reinterpret_cast<uint2*>(a_out + (int64_t)e_m[rr] * a_ldo + e_n[rr]) = packed;
            if constexpr (MAKES_AMAX) {
                if (a_amax_out.table != nullptr)
                    fold_amax(e_live[rr] ? (packed.x & 0x7FFF7FFFu) : 0u, e_live[rr] ? (packed.y & 0x7FFF7FFFu) : 0u, e_mb[rr]);
            }
        }
    }
    PHYAI_STAMP(6)
    if constexpr (MAKES_AMAX) {
        if (a_amax_out.table != nullptr) {
            __syncthreads();
            if (tid < ROWS && m_base + tid < M)
                a_amax_out.table[(size_t)(m_base + tid) * kAmaxSlots + blockIdx.x] = (uint16_t)amax_made[tid];
        }
    }
    PHYAI_STAMP_END(g_fq_stamps, ((size_t)blockIdx.x + (size_t)gridDim.x * blockIdx.y) * FQ_WAVES + wave, lane)
}

// ---- host side -------------------------------------------------------------------------------------

static int fq_ceil_div(int a, int b) { return (a + b - 1) / b; }

// LDS of a workgroup shape, as the kernel lays it out (the table of row maxima has its own 2 KB unless
// only the staging fits, see the kernel; none with handed-over maxima; weights that go straight to
// registers are not staged).
static constexpr bool fq_fits(int rows, int nt, int kpw, bool direct, bool amax_in, bool act_epilogue) {
    const int mb = (rows + 15) / 16;
    const int xb = rows < 16 ? rows * 128 : 2048;
    const int stage = kpw * ((direct ? 0 : nt * 2048) + mb * xb), redb = nt * mb * 1024;
    const int waves = FQ_WAVES * (stage > redb ? stage : redb) + (act_epilogue ? 256 : 0);   // + the table of AmaxOut
    if (amax_in) return rows <= 16 && waves <= 160 * 1024;
    if (waves + FQ_WAVES * 64 * 4 <= 160 * 1024) return true;
    return waves <= 160 * 1024 && FQ_WAVES * (rows < 64 ? rows : 64) * 4 <= xb;
}
// Registers: weights in registers are kpw * nt * 8 per lane beside kpw * (rows / 4) * 4 for the rows
// (256 per lane with two wavefronts per SIMD).
static constexpr bool fq_regs_ok(int rows, int nt, int kpw, bool direct) {
    return !direct || kpw * nt * 8 + kpw * ((rows + 3) / 4) * 4 <= 160;
}

// Shapes that exist as kernels: (rows, nt) below, with kpw = 1, 2 or 4 as K asks (K <= 4096).
// Up to 128 token rows the kernel is level with or ahead of quantizer + GEMM as long as a workgroup
// converts 16 rows or fewer (measured at M = 64 ... 256 on the expert shapes: 32-row workgroups lose).
static const int kFusedMaxM = 128;
static const int kFusedShapes[][2] = {{8, 2}, {8, 4}, {8, 5}, {8, 8}, {16, 1}, {16, 2}, {16, 4}, {16, 8}, {32, 2}, {32, 4}};
// with handed-over maxima (plain epilogue)
static constexpr bool fq_amax_in_shape(int rows, int nt) {
    return (rows == 8 && (nt == 2 || nt == 4)) || (rows == 16 && (nt == 1 || nt == 2));
}

FusedPlan fused_plan(int M, int N, int K, int epilogue, int64_t ldo, int weight_layout, bool amax_in) {
    FusedPlan pl = {0, 0, 0, 0, 0};
    if (const char* e = tuning_env("PHYAI_FP8_FUSED")) { if (atoi(e) == 0) return pl; }
    if (M < 1 || M > kFusedMaxM || K % 128 != 0 || K > 4096 || ldo % 4 != 0) return pl;
    if (amax_in && epilogue != EPI_NONE) return pl;
    const bool gated = epi_is_gated(epilogue);
    const bool direct = weight_layout != W_ROW_MAJOR;
    const int cols = gated ? N / 2 : N;
    if (cols % 8 != 0) return pl;
    const int per_wave = fq_ceil_div(K / 128, FQ_WAVES);
    const int kpw = per_wave > 2 ? 4 : (per_wave > 1 ? 2 : 1);
    const int per_tile = gated ? 8 : 16;
    // A workgroup's time: the conversions it repeats (rows x K elements on its 512 lanes) beside the
    // operand blocks it pulls through its vector cache.  Only grids that fit the 256 CUs at once are
    // taken: with a second round of workgroups the repeated conversions cost more than the quantizer's
    // launch (measured at 12288 x 2048 and 32768 x 2048: up to 3 x slower at M = 50), and the ranking
    // below agrees with the measured order of the shapes at 50 x {1024, 2560, 4096, 8192} x 1024, 16 x 2560 x 1024
    // and 50 x 1024 x 2048.
    double best = 1e30;
    int forced_rows = 0, forced_nt = 0;
    if (const char* e = tuning_env(amax_in ? "PHYAI_FP8_FUSED_PLAN_AMAX" : "PHYAI_FP8_FUSED_PLAN")) sscanf(e, "%d,%d", &forced_rows, &forced_nt);
    // Beyond K = 2048 (four K steps per wavefront) a kernel that finds its own row maxima is taken only in the
    // 8 rows x 2 tiles shape.  Measured on whole linears against quantizer + GEMM over M = 1 ... 128,
    // N = 256 ... 2048, K = 2560 / 3072 / 4096: that shape is 4 - 16 % ahead with weights in operand order
    // (50 x 1024 x 4096: 6.8 -> 6.1 us) and 0 - 13 % ahead row-major; 8 rows x 4 tiles is level (0.96 - 1.05).
    const bool long_k_alone = K > 2048 && !amax_in && !forced_rows;
    for (const auto& sh : kFusedShapes) {
        const int rows = sh[0], nt = sh[1];
        if (!fq_fits(rows, nt, kpw, direct, amax_in, epilogue != EPI_NONE) || !fq_regs_ok(rows, nt, kpw, direct)) continue;
        if (amax_in && !fq_amax_in_shape(rows, nt)) continue;
        if (long_k_alone && (rows != 8 || nt != 2)) continue;
        if (forced_rows && (rows != forced_rows || nt != forced_nt)) continue;
        const int tiles = fq_ceil_div(cols, per_tile * nt), msplit = fq_ceil_div(M, rows);
        if (!forced_rows) {
            if (rows > 16 && (rows >= 2 * M || M > 64)) continue;              // blocks that do not exist; see kFusedMaxM
            if ((int64_t)tiles * msplit > 256) continue;
        }
        const double conv = (double)rows * K * 5.5 / 64.0;                      // cycles of VALU per workgroup
        const double pull = (double)(nt * 16 + rows * 2) * K / 50.0;           // bytes through the vector cache
        // workgroups that share a weight tile sit on one XCD (and fetch the tile from HBM once) only when
        // the tile count is a multiple of 8: 27 tiles instead of 32 made qkv 1.6 x slower
        const double spread = (msplit > 1 && tiles % 8 != 0) ? 1.6 : 1.0;
        const double cost = (conv + pull) * spread;
        if (cost < best) { best = cost; pl.rows = rows; pl.nt = nt; pl.tiles = tiles; pl.msplit = msplit; }
    }
    pl.kpw = pl.rows ? kpw : 0;
    return pl;
}

template <int ROWS, int NT, int KPW, int EPI, bool DIRECT, bool AMAX_IN>
static int fq_launch_one(const GemmProblem& g, const FusedPlan& pl, hipStream_t st) {
    if constexpr (!fq_fits(ROWS, NT, KPW, DIRECT, AMAX_IN, EPI != EPI_NONE) || !fq_regs_ok(ROWS, NT, KPW, DIRECT) ||
                  (AMAX_IN && (EPI != EPI_NONE || !fq_amax_in_shape(ROWS, NT)))) {
        return -2;
    } else {
        const AmaxOut made = {EPI != EPI_NONE ? g.amax_out : nullptr};
        const int m_flags = g.M;   // (weights in operand order take the DIRECT kernels)
#define PHYAI_FQ_ARGS g.w, reinterpret_cast<const uint8_t*>(g.x_bf16), g.K, g.N, m_flags, (int)(g.ldx * 2),                     \
                      reinterpret_cast<const uint8_t*>(g.amax_in), g.amax_parts, g.w_scale, g.bias, g.out, g.ldo, residual_of(g), made
        if (g.stream_weights)
            hipLaunchKernelGGL((gemm_fp8_fusedq_kernel<ROWS, NT, KPW, EPI, true, DIRECT, AMAX_IN>), dim3(pl.tiles, pl.msplit),
                               dim3(FQ_THREADS), 0, st, PHYAI_FQ_ARGS);
        else
            hipLaunchKernelGGL((gemm_fp8_fusedq_kernel<ROWS, NT, KPW, EPI, false, DIRECT, AMAX_IN>), dim3(pl.tiles, pl.msplit),
                               dim3(FQ_THREADS), 0, st, PHYAI_FQ_ARGS);
#undef PHYAI_FQ_ARGS
        return 0;
    }
}

template <int ROWS, int NT, int KPW, int EPI>
static int fq_launch_variant(const GemmProblem& g, const FusedPlan& pl, hipStream_t st) {
    const bool direct = g.weight_layout != W_ROW_MAJOR;
    if (g.amax_in != nullptr) {
        if constexpr (EPI == EPI_NONE) {
            return direct ? fq_launch_one<ROWS, NT, KPW, EPI, true, true>(g, pl, st)
                          : fq_launch_one<ROWS, NT, KPW, EPI, false, true>(g, pl, st);
        } else {
            return -2;
        }
    }
    return direct ? fq_launch_one<ROWS, NT, KPW, EPI, true, false>(g, pl, st)
                  : fq_launch_one<ROWS, NT, KPW, EPI, false, false>(g, pl, st);
}

template <int ROWS, int NT, int EPI>
static int fq_launch_kpw(const GemmProblem& g, const FusedPlan& pl, hipStream_t st) {
    switch (pl.kpw) {
    case 1: return fq_launch_variant<ROWS, NT, 1, EPI>(g, pl, st);
    case 2: return fq_launch_variant<ROWS, NT, 2, EPI>(g, pl, st);
    case 4: return fq_launch_variant<ROWS, NT, 4, EPI>(g, pl, st);
    default: return -2;
    }
}

template <int EPI>
static int fq_launch_epi(const GemmProblem& g, const FusedPlan& pl, hipStream_t st) {
    switch (pl.rows * 100 + pl.nt) {
    case 802: return fq_launch_kpw<8, 2, EPI>(g, pl, st);
    case 804: return fq_launch_kpw<8, 4, EPI>(g, pl, st);
    case 805: return fq_launch_kpw<8, 5, EPI>(g, pl, st);
    case 808: return fq_launch_kpw<8, 8, EPI>(g, pl, st);
    case 1601: return fq_launch_kpw<16, 1, EPI>(g, pl, st);
    case 1602: return fq_launch_kpw<16, 2, EPI>(g, pl, st);
    case 1604: return fq_launch_kpw<16, 4, EPI>(g, pl, st);
    case 1608: return fq_launch_kpw<16, 8, EPI>(g, pl, st);
    case 3202: return fq_launch_kpw<32, 2, EPI>(g, pl, st);
    case 3204: return fq_launch_kpw<32, 4, EPI>(g, pl, st);
    default: return -2;
    }
}

int launch_set_stamp_sink_fused(unsigned long long* buf, unsigned int records) {
#ifdef PHYAI_FP8_STAMPS
    const StampSink s = {buf, records};
    return hipMemcpyToSymbol(HIP_SYMBOL(g_fq_stamps), &s, sizeof(s)) == hipSuccess ? 0 : -4;
#else
    (void)buf; (void)records;
    return -2;
#endif
}

int launch_gemm_fused(const GemmProblem& g, const FusedPlan& pl, hipStream_t st) {
    if (g.amax_out != nullptr && pl.tiles > kAmaxSlots) return -2;   // one slot per workgroup column
    if (g.amax_in != nullptr && (g.amax_parts < 1 || g.amax_parts > kAmaxSlots)) return -2;
    switch (g.epilogue) {
    case EPI_NONE: return fq_launch_epi<EPI_NONE>(g, pl, st);
    case EPI_GEGLU_TANH: return fq_launch_epi<EPI_GEGLU_TANH>(g, pl, st);
    case EPI_GEGLU_ERF: return fq_launch_epi<EPI_GEGLU_ERF>(g, pl, st);
    case EPI_SWIGLU: return fq_launch_epi<EPI_SWIGLU>(g, pl, st);
    case EPI_GELU_TANH: return fq_launch_epi<EPI_GELU_TANH>(g, pl, st);
    case EPI_GELU_ERF: return fq_launch_epi<EPI_GELU_ERF>(g, pl, st);
    default: return -2;
    }
}

}  // namespace phyai
