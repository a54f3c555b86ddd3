// LDS-staged fp8 x fp8 MFMA GEMM (NT: A = xq [M,K], B = w [N,K], both K-contiguous)
// with the dequant-scale-bias-activation epilogue fused, bf16 out.
//
// Workgroup = 256 threads = 4 wavefronts arranged WAVES_M x WAVES_N over a
// BM x BN output tile; K is consumed in 128-byte slabs, double-buffered in LDS.
// Global -> LDS: each thread moves 16 bytes per pass, 8 threads cover one
// 128-byte row slab (one cache line), 32 rows per pass.  LDS rows are 128 bytes;
// the 16-byte chunk index is XOR-ed with (row & 7) so that both the 128-bit
// stores and the MFMA operand reads (32 rows x the same logical chunk) spread
// over all banks.
// MFMA: v_mfma_f32_32x32x64_f8f6f4 (fp8 e4m3 x fp8 e4m3, fp32 accumulate).  Lane l
// supplies row (l % 32) of the 32x64 operand block and 32 consecutive K bytes
// starting at 32 * (l / 32); A and B use the same K split, so the dot products
// line up.  Accumulator register r of lane l is C[8*(r/4) + 4*(l/32) + r%4][l%32].
//
// Gated epilogues pair column n (gate) with column n + N/2 (up).  The B tile of
// a gated kernel is therefore gathered from two row ranges of w: within each
// wavefront's WN columns the first WN/2 are gate columns and the second WN/2 the
// matching up columns, so the pair sits in the same lane of two accumulators.
//
// Split-K (grid.z > 1): each split stores its fp32 accumulators to the
// workspace in fragment order; the last split to arrive at the tile's counter
// (device-scope atomic) sums all partials in split order - a fixed order, so
// results are reproducible - and runs the epilogue.  It then resets the
// counter, which keeps the workspace header zero between calls.
#include "fp8_device.h"
#include "launch.h"
#include "tuning.h"
#include "splitk.h"
#include "weight_layout.h"
#include <stdio.h>
#include <stdlib.h>

namespace phyai {

constexpr int BK = 128;  // bytes (= fp8 elements) of K per LDS slab

struct TileArgs {
    const uint8_t* __restrict__ a;   // xq
    const uint8_t* __restrict__ b;   // w
    const float* __restrict__ a_scale;
    const float* __restrict__ b_scale;
    const uint16_t* __restrict__ bias;
    uint16_t* __restrict__ out;
    float* __restrict__ partials;
    int* __restrict__ counters;
    int64_t ldo;
    int M, N, K;
    int a_scale_scalar;
    int k_tiles_per_split;  // in BK slabs
    int operand_w;          // weights in MFMA operand order (weight_layout.h; needs K % 128 == 0)
    ResidualArgs res;
};

__device__ __forceinline__ v8i lds_frag(const uint8_t* buf, int row, int ks, int h) {
    const int c0 = ks * 4 + h * 2;
    const int sw = row & 7;
    const uint8_t* r = buf + row * BK;
    const v4i lo = *reinterpret_cast<const v4i*>(r + ((c0 ^ sw) << 4));
    const v4i hi = *reinterpret_cast<const v4i*>(r + (((c0 + 1) ^ sw) << 4));
    v8i f;
    f[0] = lo[0]; f[1] = lo[1]; f[2] = lo[2]; f[3] = lo[3];
    f[4] = hi[0]; f[5] = hi[1]; f[6] = hi[2]; f[7] = hi[3];
    return f;
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI, bool SPLITK>
__global__ __launch_bounds__(256) void gemm_fp8_tile_kernel(const TileArgs p) {
    static_assert(WAVES_M * WAVES_N == 4, "4 wavefronts per workgroup");
    constexpr bool GATED = epi_is_gated(EPI);
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int TM = WM / 32, TN = WN / 32;
    static_assert(TM >= 1 && TN >= 1, "wave tile must hold a 32x32 block");
    static_assert(!GATED || (TN % 2 == 0), "gated epilogue needs gate/up block pairs per wave");
    constexpr int PA = BM / 32, PB = BN / 32;  // loader passes
    constexpr int TILE_BYTES = (BM + BN) * BK;

    __shared__ __attribute__((aligned(16))) uint8_t lds[2 * TILE_BYTES];
    __shared__ int s_last;

    const int tid = threadIdx.x;
    const int lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int l32 = lane & 31, h = lane >> 5;

    const int m0 = blockIdx.y * BM;
    // Gated: a tile spans BN/2 gate columns and the BN/2 up columns that pair with them.
    const int half_n = p.N / 2;
    const int n0 = GATED ? blockIdx.x * (BN / 2) : blockIdx.x * BN;

    // ---- loader geometry: thread -> (row within pass, 16-byte chunk) ----------
    const int lrow = tid >> 3, lchunk = tid & 7;
    int a_off[PA], b_off[PB];
#pragma unroll
    for (int i = 0; i < PA; ++i) {
        int r = m0 + i * 32 + lrow;
        r = r < p.M ? r : p.M - 1;
        a_off[i] = r * p.K;
    }
#pragma unroll
    for (int i = 0; i < PB; ++i) {
        const int jj = i * 32 + lrow;  // column within the tile
        int r;
        if constexpr (GATED) {
            const int w_ = jj / WN, j = jj % WN;
            const int up = j / (WN / 2);
            int g = n0 + w_ * (WN / 2) + j % (WN / 2);
            g = g < half_n ? g : half_n - 1;
            r = up * half_n + g;
            if (p.operand_w) { b_off[i] = (int)operand_offset_gated((uint32_t)g, (uint32_t)up, (uint32_t)p.K); continue; }
        } else {
            r = n0 + jj;
            r = r < p.N ? r : p.N - 1;
            if (p.operand_w) { b_off[i] = (int)operand_offset_plain((uint32_t)r, (uint32_t)p.K); continue; }
        }
        b_off[i] = r * p.K;
    }

    const int k_begin = SPLITK ? blockIdx.z * p.k_tiles_per_split * BK : 0;
    int k_end = SPLITK ? k_begin + p.k_tiles_per_split * BK : p.K;
    k_end = k_end < p.K ? k_end : p.K;
    const int n_slabs = (k_end - k_begin + BK - 1) / BK;

    uint4 ra[PA], rb[PB];
    auto load_global = [&](int slab) {
        const int k = k_begin + slab * BK + lchunk * 16;
        const bool ok = k < k_end;
        // operand order: the K step is 2 KB away and the chunk 256 bytes (K is a multiple of 128 then)
        const uint32_t kb = p.operand_w ? ((uint32_t)(k >> 7) << 11) + (uint32_t)lchunk * kOperandChunkBytes : (uint32_t)k;
#pragma unroll
        for (int i = 0; i < PA; ++i)
            ra[i] = ok ? *reinterpret_cast<const uint4*>(p.a + a_off[i] + k) : make_uint4(0, 0, 0, 0);
#pragma unroll
        for (int i = 0; i < PB; ++i)
            rb[i] = ok ? *reinterpret_cast<const uint4*>(p.b + (uint32_t)b_off[i] + kb) : make_uint4(0, 0, 0, 0);
    };
    auto store_lds = [&](int buf) {
        uint8_t* base = lds + buf * TILE_BYTES;
        const int sw = (lchunk ^ (lrow & 7)) << 4;
#pragma unroll
        for (int i = 0; i < PA; ++i)
            *reinterpret_cast<uint4*>(base + (i * 32 + lrow) * BK + sw) = ra[i];
#pragma unroll
        for (int i = 0; i < PB; ++i)
            *reinterpret_cast<uint4*>(base + BM * BK + (i * 32 + lrow) * BK + sw) = rb[i];
    };

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    if (n_slabs > 0) {
        load_global(0);
        store_lds(0);
    }
    __syncthreads();

    for (int s = 0; s < n_slabs; ++s) {
        const int cur = s & 1;
        if (s + 1 < n_slabs) load_global(s + 1);
        const uint8_t* abuf = lds + cur * TILE_BYTES;
        const uint8_t* bbuf = abuf + BM * BK;
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
            v8i fa[TM], fb[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[i] = lds_frag(abuf, wm * WM + i * 32 + l32, ks, h);
#pragma unroll
            for (int j = 0; j < TN; ++j) fb[j] = lds_frag(bbuf, wn * WN + j * 32 + l32, ks, h);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(
                        fa[i], fb[j], acc[i][j], 0, 0, 0, 0, 0, 0);
        }
        if (s + 1 < n_slabs) store_lds(cur ^ 1);
        __syncthreads();
    }

    // ---- split-K: publish partials, last arriver reduces -----------------------
    if constexpr (SPLITK) {
        const int S = gridDim.z;
        const int tile = blockIdx.y * gridDim.x + blockIdx.x;
        constexpr int FRAG = TM * TN * 16;  // floats per thread
        float frag[FRAG];
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) frag[(i * TN + j) * 16 + r] = acc[i][j][r];
        splitk_publish<FRAG, 256>(p.partials, tile, S, blockIdx.z, frag);
        if (!splitk_arrive(p.counters, tile, S, &s_last)) return;
        splitk_gather<FRAG, 256>(p.partials, p.counters, tile, S, frag);
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[i][j][r] = frag[(i * TN + j) * 16 + r];
    }

    // ---- epilogue ------------------------------------------------------------
    constexpr int TNO = GATED ? TN / 2 : TN;  // output column blocks per wave
    float sa[TM][16];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int m = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * h + (r % 4);
            sa[i][r] = p.a_scale[(p.a_scale_scalar || m >= p.M) ? 0 : m];
        }
#pragma unroll
    for (int j = 0; j < TNO; ++j) {
        const int n_out = n0 + (GATED ? wn * (WN / 2) : wn * WN) + j * 32 + l32;
        const int n_lim = GATED ? half_n : p.N;
        const bool n_ok = n_out < n_lim;
        const int n_safe = n_ok ? n_out : 0;
        const float sg = p.b_scale[n_safe];
        const float bg = p.bias ? bf16_bits_to_f32(p.bias[n_safe]) : 0.f;
        float su = 0.f, bu = 0.f;
        if constexpr (GATED) {
            su = p.b_scale[half_n + n_safe];
            bu = p.bias ? bf16_bits_to_f32(p.bias[half_n + n_safe]) : 0.f;
        }
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int m = m0 + wm * WM + i * 32 + 8 * (r / 4) + 4 * h + (r % 4);
                float v = __builtin_fmaf(acc[i][j][r], sa[i][r] * sg, bg);   // one rounding, like the other kernels
                if constexpr (GATED) {
                    const float u = __builtin_fmaf(acc[i][j + TN / 2][r], sa[i][r] * su, bu);
                    v = apply_act<EPI>(round_bf16(v)) * round_bf16(u);
                } else if constexpr (EPI != EPI_NONE) {
                    v = apply_act<EPI>(round_bf16(v));
                }
                if (m < p.M && n_ok) {
                    if constexpr (EPI == EPI_NONE) {
                        if (p.res.residual != nullptr)
                            v = bf16_bits_to_f32(p.res.residual[(int64_t)m * p.res.ld_res + n_out]) +
                                round_bf16(v) *
                                    bf16_bits_to_f32(p.res.gate[(int64_t)(m / p.res.gate_group) * p.res.ld_gate + n_out]);
                    }
                    p.out[(int64_t)m * p.ldo + n_out] = (uint16_t)(pack_bf16x2(v, 0.0f) & 0xFFFFu);
                }
            }
        }
    }
}

// ---- host side ---------------------------------------------------------------

constexpr size_t kHeaderBytes = kGemmHeaderBytes;

struct TileConfig {
    int bm, bn;
    int splits;
};

static int ceil_div(int a, int b) { return (a + b - 1) / b; }

// Tile shape and split count.  Small M is weight-streaming bound: use the
// smallest M tile and split K until there are enough workgroups to keep every
// CU pulling weight bytes.  Large M is MFMA bound: big square tiles, no split.
static TileConfig pick_config(int M, int N, int K, int epilogue) {
    const bool gated = epi_is_gated(epilogue);
    TileConfig c;
    if (M <= 64) {
        c.bm = 64;
        c.bn = gated ? 128 : 64;
    } else {
        c.bm = 128;
        c.bn = 128;
    }
    int forced_splits = 0;
    if (const char* e = tuning_env("PHYAI_FP8_TILE")) {  // "bm,bn,splits" tuning override
        int bm = 0, bn = 0, sp = 0;
        if (sscanf(e, "%d,%d,%d", &bm, &bn, &sp) == 3 && (bm == 64 || bm == 128 || bm == 256) &&
            (bn == 64 || bn == 128 || bn == 256) && !(bm == 64 && bn == 256) && !(bm == 256 && bn == 64) &&
            !(gated && bn == 64)) {
            c.bm = bm; c.bn = bn; forced_splits = sp;
        }
    }
    const int n_eff = gated ? N / 2 : N;
    const int bn_eff = gated ? c.bn / 2 : c.bn;
    const int tiles = ceil_div(M, c.bm) * ceil_div(n_eff, bn_eff);
    const int slabs = ceil_div(K, BK);
    int s = 1;
    if (tiles < 256) {
        s = ceil_div(512, tiles);
        const int max_s = slabs / 2 > 0 ? slabs / 2 : 1;  // at least 2 slabs per split
        if (s > max_s) s = max_s;
        if (s > 32) s = 32;
    }
    if (forced_splits > 0) s = forced_splits < slabs ? forced_splits : slabs;
    if (tiles > (int)(kGemmHeaderBytes / sizeof(int))) s = 1;   // one arrival counter per tile in the header
    // every split must own at least one slab
    const int per = ceil_div(slabs, s);
    s = ceil_div(slabs, per);
    c.splits = s;
    return c;
}

static size_t partial_bytes(const TileConfig& c, int M, int N, int epilogue) {
    if (c.splits <= 1) return 0;
    const bool gated = epi_is_gated(epilogue);
    const int n_eff = gated ? N / 2 : N;
    const int bn_eff = gated ? c.bn / 2 : c.bn;
    const size_t tiles = (size_t)ceil_div(M, c.bm) * ceil_div(n_eff, bn_eff);
    return tiles * c.splits * (size_t)c.bm * c.bn * sizeof(float);
}

size_t gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int epilogue, int64_t ldo) {
    if (M <= 0 || N <= 0 || K <= 0) return kHeaderBytes;
    if (M <= 64 && skinny_applicable((int)M, (int)N, (int)K, epilogue, ldo)) return kHeaderBytes;
    size_t big = 0;
    {
        for (int operand_w = 0; operand_w < 2; ++operand_w) {   // (the plan may depend on the weight layout)
            const BigPlan bp = big_plan((int)M, (int)N, (int)K, epilogue, operand_w != 0);
            const size_t b = bp.tile ? big_partial_bytes((int)M, (int)N, epilogue, bp) : 0;
            big = b > big ? b : big;
        }
    }
    const TileConfig c = pick_config((int)M, (int)N, (int)K, epilogue);
    const size_t own = partial_bytes(c, (int)M, (int)N, epilogue);
    return kHeaderBytes + (own > big ? own : big);  // either kernel may end up serving the call
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int EPI>
static void launch_one(const TileArgs& a, dim3 grid, bool split, hipStream_t st) {
    if (split)
        hipLaunchKernelGGL((gemm_fp8_tile_kernel<BM, BN, WAVES_M, WAVES_N, EPI, true>), grid, dim3(256), 0, st, a);
    else
        hipLaunchKernelGGL((gemm_fp8_tile_kernel<BM, BN, WAVES_M, WAVES_N, EPI, false>), grid, dim3(256), 0, st, a);
}

template <int EPI>
static int launch_epi(const TileArgs& a, const TileConfig& c, dim3 grid, hipStream_t st) {
    constexpr bool GATED = epi_is_gated(EPI);
    const bool split = c.splits > 1;
    const int key = c.bm * 1000 + c.bn;
    switch (key) {
    case 64064: if constexpr (!GATED) { launch_one<64, 64, 2, 2, EPI>(a, grid, split, st); return 0; } return -2;
    case 64128: launch_one<64, 128, 2, 2, EPI>(a, grid, split, st); return 0;
    case 128064: if constexpr (!GATED) { launch_one<128, 64, 2, 2, EPI>(a, grid, split, st); return 0; } return -2;
    case 128128: launch_one<128, 128, 2, 2, EPI>(a, grid, split, st); return 0;
    case 128256: launch_one<128, 256, 2, 2, EPI>(a, grid, split, st); return 0;
    case 256128: launch_one<256, 128, 2, 2, EPI>(a, grid, split, st); return 0;
    case 256256: launch_one<256, 256, 2, 2, EPI>(a, grid, split, st); return 0;
    default: return -2;
    }
}

// launch_gemm's choice of kernel for one problem, and the scratch that choice needs.
struct GemmChoice {
    enum Kind { SKINNY, BIG, GENERIC, FUSED } kind;
    FusedPlan fq;
    SkinnyPlan sk;
    BigPlan big;
    TileConfig tc;
    size_t need;   // workspace bytes (header + split-K partial sums), 0 if the kernel uses none
    bool takes_amax;   // FUSED: the plan is the one for handed-over row maxima
};

// Kernel choice (measured on the expert and prefill shapes, M = 50 .. 13056):
//   M <= 64                      weight-streaming kernel, nothing else comes close;
//   pipelined tile kernel        when big_plan finds a tile shape that fills the chip, or more
//                                than 64 tiles of 128 x 128;
//   64 < M <= 1024 otherwise     weight-streaming kernel again (few output columns: at
//                                N = 1024 it wins up to M = 1000, at N = 2560 up to M = 300);
//   32 .. 64 small tiles         pipelined tile kernel after all (M > 1024);
//   the rest                     generic LDS tile kernel (any K, any alignment).
// vec_ok: scales, bias and output are aligned for the weight-streaming kernel's 128- and 64-bit
// accesses; out16: the output is 16-byte addressable (pointer and row stride), which the pipelined
// tile kernel's epilogue needs.
// have_x: the bf16 activations are at hand (whole-linear entry points), so a kernel that quantizes
// its own rows may serve the call.
static GemmChoice choose_gemm(int M, int N, int K, int epilogue, int64_t ldo, bool vec_ok, bool out16, bool have_x,
                              int layout = W_ROW_MAJOR, bool amax_in = false) {
    GemmChoice c = {};
    if (have_x && vec_ok) {
        if (amax_in) {
            c.fq = fused_plan(M, N, K, epilogue, ldo, layout, true);
            if (c.fq.rows) { c.kind = GemmChoice::FUSED; c.need = 0; c.takes_amax = true; return c; }
        }
        c.fq = fused_plan(M, N, K, epilogue, ldo, layout, false);
        if (c.fq.rows) { c.kind = GemmChoice::FUSED; c.need = 0; return c; }
    }
    const bool skinny_ok = vec_ok && skinny_applicable(M, N, K, epilogue, ldo);
    auto small = [&]() {
        c.kind = GemmChoice::SKINNY;
        c.sk = skinny_plan(M, N, K, epilogue);
        c.need = 0;
        return c;
    };
    if (skinny_ok && M <= 64) return small();
    if (!tuning_env("PHYAI_FP8_TILE")) {
        const BigPlan bp = big_plan(M, N, K, epilogue, layout != W_ROW_MAJOR);
        const bool few_small_tiles = bp.tile == 128 && bp.cols == 128 && bp.tiles <= 64 && !tuning_env("PHYAI_FP8_BIG");
        if (bp.tile && out16 && !(few_small_tiles && skinny_ok)) {
            c.kind = GemmChoice::BIG;
            c.big = bp;
            c.need = bp.splits > 1 ? kHeaderBytes + big_partial_bytes(M, N, epilogue, bp) : 0;
            return c;
        }
        if (skinny_ok) return small();
    }
    c.kind = GemmChoice::GENERIC;
    c.tc = pick_config(M, N, K, epilogue);
    c.need = c.tc.splits > 1 ? kHeaderBytes + partial_bytes(c.tc, M, N, epilogue) : 0;
    return c;
}

static GemmChoice choose_gemm(const GemmProblem& g) {
    const bool vec_ok = (reinterpret_cast<uintptr_t>(g.w_scale) % 16 == 0) &&
                        (reinterpret_cast<uintptr_t>(g.bias) % 8 == 0) &&
                        (reinterpret_cast<uintptr_t>(g.out) % 8 == 0);
    const bool out16 = g.ldo % 8 == 0 && (reinterpret_cast<uintptr_t>(g.out) & 15) == 0;
    const bool have_x = g.x_bf16 != nullptr && (reinterpret_cast<uintptr_t>(g.x_bf16) & 15) == 0 && g.ldx % 8 == 0 &&
                        (int64_t)g.M * g.ldx * 2 < ((int64_t)1 << 32) && (int64_t)g.N * g.K < ((int64_t)1 << 32) &&
                        g.K < (1 << 24) && g.N < (1 << 24) && !g.x_scale_is_scalar;
    return choose_gemm(g.M, g.N, g.K, g.epilogue, g.ldo, vec_ok, out16, have_x, g.weight_layout,
                       g.amax_in != nullptr && g.amax_parts >= 1 && g.amax_parts <= kRowAmaxSlots &&
                           (reinterpret_cast<uintptr_t>(g.amax_in) & 15) == 0);
}

int gemm_row_maxima_slots(const GemmProblem& g) {
    if (g.M == 0 || g.N == 0 || g.epilogue == EPI_NONE) return 0;
    const GemmChoice c = choose_gemm(g);
    return (c.kind == GemmChoice::FUSED && c.fq.tiles <= kRowAmaxSlots) ? c.fq.tiles : 0;
}

bool gemm_takes_row_maxima(const GemmProblem& g) {
    if (g.M == 0 || g.N == 0) return false;
    const GemmChoice c = choose_gemm(g);
    return c.kind == GemmChoice::FUSED && c.takes_amax;
}

bool gemm_quantizes_itself(const GemmProblem& g) {
    if (g.M == 0 || g.N == 0) return false;
    return choose_gemm(g).kind == GemmChoice::FUSED;
}

size_t gemm_scratch_need(const GemmProblem& g) {
    if (g.M == 0 || g.N == 0) return 0;
    return choose_gemm(g).need;
}

int describe_gemm_plan(int M, int N, int K, int epilogue, char* buf, size_t n, int weight_layout) {
    // operands that satisfy every alignment requirement, dense output
    const int64_t ldo = epi_is_gated(epilogue) ? N / 2 : N;
    const GemmChoice c = choose_gemm(M, N, K, epilogue, ldo, true, ldo % 8 == 0, false, weight_layout);
    switch (c.kind) {
    case GemmChoice::SKINNY:
        return snprintf(buf, n, "small-m nt=%d mb=%d kpw=%d rounds=%d", c.sk.nt, c.sk.mb, c.sk.kpw, c.sk.rounds);
    case GemmChoice::BIG:
        if (c.big.regs)
            return snprintf(buf, n, "tile %dx%d depth=%d splits=%d tiles=%d weights in registers, ring of %d", c.big.tile,
                            c.big.cols, c.big.depth, c.big.splits, c.big.tiles, c.big.regs);
        return snprintf(buf, n, "tile %dx%d depth=%d splits=%d tiles=%d", c.big.tile, c.big.cols,
                        c.big.depth, c.big.splits, c.big.tiles);
    default:
        return snprintf(buf, n, "generic %dx%d splits=%d", c.tc.bm, c.tc.bn, c.tc.splits);
    }
}

int describe_linear_plan(int M, int N, int K, int epilogue, char* buf, size_t n, int weight_layout) {
    const int64_t ldo = epi_is_gated(epilogue) ? N / 2 : N;
    const GemmChoice c = choose_gemm(M, N, K, epilogue, ldo, true, ldo % 8 == 0, true, weight_layout);
    if (c.kind == GemmChoice::FUSED)
        return snprintf(buf, n, "one launch: small-m rows=%d nt=%d kpw=%d grid=%dx%d", c.fq.rows, c.fq.nt, c.fq.kpw, c.fq.tiles, c.fq.msplit);
    const int len = snprintf(buf, n, "quantizer + ");
    if (len < 0 || (size_t)len >= n) return len;
    return len + describe_gemm_plan(M, N, K, epilogue, buf + len, n - len, weight_layout);
}

int describe_mlp_plan(int M, int H, int I, int O, int epilogue, char* buf, size_t n, bool operand_order) {
    const int n1 = epi_is_gated(epilogue) ? 2 * I : I;
    const int lay1 = !operand_order ? W_ROW_MAJOR : (epi_is_gated(epilogue) ? W_OPERAND_GATED : W_OPERAND_PLAIN);
    const int lay2 = operand_order ? W_OPERAND_PLAIN : W_ROW_MAJOR;
    const GemmChoice a = choose_gemm(M, n1, H, epilogue, I, true, I % 8 == 0, true, lay1);
    bool handed = false;
    if (a.kind == GemmChoice::FUSED && a.fq.tiles <= kRowAmaxSlots) {
        const GemmChoice b = choose_gemm(M, O, I, EPI_NONE, O, true, O % 8 == 0, true, lay2, true);
        handed = b.kind == GemmChoice::FUSED && b.takes_amax;
    }
    int len = handed ? snprintf(buf, n, "row maxima handed over: ") : 0;
    if (len < 0 || (size_t)len >= n) return len;
    len += describe_linear_plan(M, n1, H, epilogue, buf + len, n - len, lay1);
    if ((size_t)len >= n) return len;
    len += snprintf(buf + len, n - len, " | ");
    if ((size_t)len >= n) return len;
    if (handed) {
        const GemmChoice b = choose_gemm(M, O, I, EPI_NONE, O, true, O % 8 == 0, true, lay2, true);
        return len + snprintf(buf + len, n - len, "one launch: small-m rows=%d nt=%d kpw=%d grid=%dx%d", b.fq.rows, b.fq.nt,
                              b.fq.kpw, b.fq.tiles, b.fq.msplit);
    }
    return len + describe_linear_plan(M, O, I, EPI_NONE, buf + len, n - len, lay2);
}

int launch_gemm(const GemmProblem& g, hipStream_t st) {
    if (g.M == 0 || g.N == 0) return 0;
    const GemmChoice ch = choose_gemm(g);
    if (ch.need > 0 && (g.workspace == nullptr || g.workspace_bytes < ch.need)) return -3;
    if (ch.kind == GemmChoice::FUSED) {
        if (g.amax_in != nullptr && !ch.takes_amax) {   // the plan finds the row maxima itself
            GemmProblem own = g;
            own.amax_in = nullptr;
            return launch_gemm_fused(own, ch.fq, st);
        }
        return launch_gemm_fused(g, ch.fq, st);
    }
    if (ch.kind == GemmChoice::SKINNY) return launch_gemm_skinny(g, ch.sk, st);
    if (ch.kind == GemmChoice::BIG) return launch_gemm_big(g, ch.big, st);
    const TileConfig& c = ch.tc;
    const bool gated = epi_is_gated(g.epilogue);
    const int n_eff = gated ? g.N / 2 : g.N;
    const int bn_eff = gated ? c.bn / 2 : c.bn;

    TileArgs a;
    a.a = g.xq; a.b = g.w; a.a_scale = g.x_scale; a.b_scale = g.w_scale; a.bias = g.bias;
    a.out = g.out; a.ldo = g.ldo; a.M = g.M; a.N = g.N; a.K = g.K;
    a.a_scale_scalar = g.x_scale_is_scalar;
    a.res = residual_of(g);
    a.operand_w = g.weight_layout != W_ROW_MAJOR;
    a.counters = static_cast<int*>(g.workspace);
    a.partials = g.workspace ? reinterpret_cast<float*>(static_cast<uint8_t*>(g.workspace) + kHeaderBytes) : nullptr;
    const int slabs = ceil_div(g.K, BK);
    a.k_tiles_per_split = ceil_div(slabs, c.splits);
    const dim3 grid(ceil_div(n_eff, bn_eff), ceil_div(g.M, c.bm), c.splits);

    switch (g.epilogue) {
    case EPI_NONE: return launch_epi<EPI_NONE>(a, c, grid, st);
    case EPI_GEGLU_TANH: return launch_epi<EPI_GEGLU_TANH>(a, c, grid, st);
    case EPI_GEGLU_ERF: return launch_epi<EPI_GEGLU_ERF>(a, c, grid, st);
    case EPI_SWIGLU: return launch_epi<EPI_SWIGLU>(a, c, grid, st);
    case EPI_GELU_TANH: return launch_epi<EPI_GELU_TANH>(a, c, grid, st);
    case EPI_GELU_ERF: return launch_epi<EPI_GELU_ERF>(a, c, grid, st);
    default: return -2;
    }
}

}  // namespace phyai
