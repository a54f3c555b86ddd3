// MFMA-bound fp8 GEMM for large M (prefix prefill, batched serving).
// Workgroup = 4 wavefronts (2 x 2); a wavefront owns TM x TN blocks of 32 x 32, so the
// workgroup tile is 64*TM x 64*TN: 256 x 256 (TM = TN = 4, one workgroup per CU) for long K,
// 192 x 128 (TM = 3, TN = 2, two workgroups per CU) when there are plenty of tiles and K is short,
// 128 x 128 (TM = TN = 2; ring of four stages, or of two with two workgroups per CU) for
// mid-sized problems, 128 x 64 (TM = 2, TN = 1) when even those leave half of the CUs idle.
//
// Why 4 x 4 blocks per wavefront for the large tile.  One v_mfma_f32_32x32x64_f8f6f4 takes 64
// cycles and consumes two 2 KB operand blocks.  A wavefront with TM x TN blocks reads (TM + TN)
// blocks from LDS per TM*TN MFMAs; LDS delivers 128 bytes per clock to the whole CU, so four
// wavefronts with 4 x 4 blocks ask for 64 bytes per clock, 2 x 2 blocks for 128.  The same ratio
// governs the bytes that must come from L2: (BM + BN) * K per tile, and L2 -> CU delivery
// (measured: 10-13 TB/s over all CUs inside these kernels) bounds the small tiles.  4 x 4 blocks
// of 16 accumulators are 256 registers: they live in AGPRs, one wavefront per SIMD, and latency
// is hidden inside the wavefront:
//
//  * global -> LDS copies bypass the register file (global_load_lds_dwordx4): lane i of a
//    wavefront fetches one 16-byte chunk and the hardware deposits chunk i at LDS base + 16*i.
//    An LDS row is 128 bytes of K - one L2 line per row per request; the XOR swizzle that keeps
//    the 128-bit operand reads conflict-free is therefore applied on the global side: lane i
//    (row i/8 of an 8-row group, slot i%8 of the row) fetches chunk (i%8) ^ swizzle(row).
//  * K is consumed in 128-byte stage-loads through a ring of DEPTH LDS stages: the copies of
//    load d+DEPTH are requested while loads d and d+1 are being multiplied, one or two copy
//    instructions per MFMA, so the wavefront never waits on the memory pipeline's issue queue
//    with its MFMA pipe empty.  One barrier per stage-load, placed in its second K half: it
//    publishes the next stage and tells everyone that the stage about to be refilled is no
//    longer read.  All wavefronts reach it at about the same time, with MFMAs queued.
//    Where the weights are in MFMA operand order and a wavefront owns its column blocks
//    (wavefronts 1 x 4: the 224 x 256 tile, and 128 x 128 tiles as 4 x 1 blocks per wavefront)
//    they do not go through LDS at all - each wavefront loads its own weight blocks straight into
//    a ring of register sets - and the barrier gives way to a hand-over through one progress word
//    per wavefront in LDS, which lets a wavefront run a stage or two ahead of the slowest
//    (see `hand_over` in the kernel).
//  * the operand blocks that open the next K half are read from LDS during the later row groups
//    of the current one into a second register set, and inside a half the A blocks of the later
//    row groups are read before the first group's MFMAs are issued, so ds_read latency overlaps
//    MFMA time.
//  * epilogue: the weight block is the MFMA's first operand, which gives a lane runs of four
//    consecutive output columns of one token row; each wavefront stages its bf16 tile in its own
//    slice of the (now idle) LDS and writes it out row-wise, 16 bytes per lane, whole row
//    segments per instruction.
//
// The smaller tiles (192 x 128, and 128 x 128 with a ring of two) keep within the register and
// LDS budget of two workgroups per CU, so that one workgroup's prologue and epilogue run under
// the other's MFMAs.
//
// Gated epilogues: within a wavefront's 32*TN columns the first half are gate columns and the
// second half the matching up columns, so the pair sits in the same lane of two accumulators.
// Requires K % 128 == 0 and K >= 512 per split (stage-loads are never partial and must fill the
// ring).
#include "fp8_device.h"
#include "launch.h"
#include "tuning.h"
#include "splitk.h"
#include "stamps.h"
#include "weight_layout.h"
#include <stdlib.h>
#include <type_traits>

namespace phyai {

constexpr int BIG_BK = 128;   // bytes of K per LDS row: one L2 cache line
// Measurement only (make stamps ABLATE=n builds the time-stamp library with it; results are WRONG by design): parts
// of the main loop left out, to see from the time stamps what each costs.  Bit 1: no copies / weight loads inside
// the loop (the operands of the prologue are multiplied over and over); bit 2: the activation blocks of a K half
// are not re-read from LDS; bit 4: no barrier / no hand-over between the wavefronts in the loop; bit 8 (weights in
// registers): only the weight loads of the loop are left out; bit 16 (either variant): only the activation copies.
#ifndef PHYAI_FP8_ABLATE
#define PHYAI_FP8_ABLATE 0
#endif
#if PHYAI_FP8_ABLATE && !defined(PHYAI_FP8_STAMPS)
#error "PHYAI_FP8_ABLATE is for the time-stamp build only"
#endif
// (debug build only: where the kernels below leave their time stamps - 1 first stage published, 2 main loop done,
// 3 split-K sums gathered, 4 epilogue arithmetic done and tile staged, 5 stores issued)
PHYAI_STAMP_SINK(g_big_stamps)

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
    // split-K (grid.z > 1): each split covers k_per_split bytes of K; see splitk.h
    int k_per_split;
    float* __restrict__ partials;
    int* __restrict__ counters;
    int m_tiles, n_tiles;            // tile grid; the launch is 1-D over it (see big_tile_of)
    int band;                        // tile rows per band of that order
    int by_rows;                     // the order with the roles of tile rows and columns exchanged
    int operand_w;                   // weights in MFMA operand order (weight_layout.h)
    ResidualArgs res;
};

// Workgroup id -> tile.  Workgroups go to the 8 XCDs round-robin (id % 8) and each XCD has its own
// L2, so ids are laid out for the tiles that share an XCD at a time to share operands: the tile
// grid is cut into bands of 4 tile rows; inside a band, 8 consecutive ids are 8 neighbouring
// tile columns (one per XCD), and the next 8 ids the same columns one tile row further down.  An
// XCD thus works on all (up to 4) tile rows of one tile column together - the weight rows come
// from HBM once per band - while the activation rows of the band stay in its L2.
// Tile columns beyond the last multiple of 8 would leave some XCDs a whole column more than
// others (20 columns: three for XCDs 0-3, two for the rest, and the launch lasts as long as the
// busiest XCD).  The tiles of those last columns are therefore taken in column-major order and
// cut into 8 runs of equal length (within one), one per XCD: still whole or half columns per
// XCD, and every XCD gets the same number of tiles.  Ids past an XCD's run have no tile.
struct BigTile { int m, n; };
__device__ __forceinline__ BigTile big_tile_of(int id, int m_tiles, int n_tiles, int band_rows) {
    const int full = n_tiles >> 3, rest = n_tiles & 7;   // whole groups of 8 tile columns; columns after them
    const int per_band = 8 * (band_rows * full + ((rest * band_rows + 7) >> 3));
    const int band = id / per_band;
    const int local = id - band * per_band;
    const int bm = m_tiles - band_rows * band < band_rows ? m_tiles - band_rows * band : band_rows;
    BigTile t;
    if (local < 8 * bm * full) {
        t.n = (local / (8 * bm)) * 8 + (local & 7);
        t.m = band_rows * band + (local >> 3) % bm;
    } else {
        const int j = local - 8 * bm * full, x = j & 7, total = rest * bm;
        const int e = ((x * total) >> 3) + (j >> 3);                  // (j / 8)-th tile of XCD x's run
        t.n = e < (((x + 1) * total) >> 3) ? 8 * full + e / bm : n_tiles;   // n_tiles: no tile
        t.m = band_rows * band + e % bm;
    }
    return t;
}
// Tiles of the busiest XCD under that order (host side; the same arithmetic, band by band).
static int big_max_tiles_per_xcd(int m_tiles, int n_tiles, int band_rows) {
    const int full = n_tiles >> 3, rest = n_tiles & 7;
    int per_xcd[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    for (int m = 0; m < m_tiles; m += band_rows) {
        const int bm = m_tiles - m < band_rows ? m_tiles - m : band_rows;
        for (int x = 0; x < 8; ++x) per_xcd[x] += bm * full + ((((x + 1) * rest * bm) >> 3) - ((x * rest * bm) >> 3));
    }
    int mx = 0;
    for (int x = 0; x < 8; ++x) mx = per_xcd[x] > mx ? per_xcd[x] : mx;
    return mx;
}
// Ids that order needs (host side).
static int big_grid_ids(int m_tiles, int n_tiles, int band_rows) {
    const int full = n_tiles >> 3, rest = n_tiles & 7;
    const int bands = m_tiles / band_rows, last = m_tiles % band_rows;
    return bands * 8 * (band_rows * full + ((rest * band_rows + 7) >> 3)) +
           (last ? 8 * (last * full + ((rest * last + 7) >> 3)) : 0);
}

// Swizzle of the eight 16-byte chunks of a 128-byte row.  LDS has 64 banks of 4 bytes, so one
// pass over the banks spans two rows and a 128-bit read is served 16 lanes at a time: the eight
// rows of equal parity among 16 consecutive ones must land in different chunk columns.
__device__ __forceinline__ int big_swizzle(int row) { return (row >> 1) & 7; }

// Operand block of v_mfma_f32_32x32x64 for K half kh (bytes [64 kh, 64 kh + 64) of the row): lane
// (l32, h) supplies 32 of the 64 K-bytes.  Which 32 is free as long as A and B agree; chunks h
// and 2+h of the half are taken so that the two halves of a wavefront never meet in a chunk
// column either.
__device__ __forceinline__ v8i big_frag(const uint8_t* buf, int row, int h, int kh) {
    const int sw = big_swizzle(row);
    const uint8_t* r = buf + row * BIG_BK;
    const v4i lo = *reinterpret_cast<const v4i*>(r + (((4 * kh + h) ^ sw) << 4));
    const v4i hi = *reinterpret_cast<const v4i*>(r + (((4 * kh + 2 + h) ^ sw) << 4));
    v8i f;
    f[0] = lo[0]; f[1] = lo[1]; f[2] = lo[2]; f[3] = lo[3];
    f[4] = hi[0]; f[5] = hi[1]; f[6] = hi[2]; f[7] = hi[3];
    return f;
}

__device__ __forceinline__ v8i big_join(v4i lo, v4i hi) {
    v8i f;
    f[0] = lo[0]; f[1] = lo[1]; f[2] = lo[2]; f[3] = lo[3];
    f[4] = hi[0]; f[5] = hi[1]; f[6] = hi[2]; f[7] = hi[3];
    return f;
}
// The same block out of weights staged in operand order (WMODE 1): `row` is the block's first row plus l32;
// chunk c of it lies at unit * 2 KB + c * 256 + (row % 16) * 16.  Sixteen consecutive lanes read 256 bytes in a
// row: no bank conflicts.
__device__ __forceinline__ v8i big_frag_operand(const uint8_t* buf, int row, int h, int kh) {
    const uint8_t* r = buf + (row >> 4) * 2048 + (row & 15) * 16;
    return big_join(*reinterpret_cast<const v4i*>(r + (4 * kh + h) * 256), *reinterpret_cast<const v4i*>(r + (4 * kh + 2 + h) * 256));
}

// Variants held to the register and LDS budget of two workgroups per CU (two wavefronts per SIMD).
__host__ __device__ constexpr bool big_two_per_cu(int tm, int tn, int depth, int wmode) {
    // (... and the 128 x 128 tile as 4 x 1 blocks per wavefront with weights in registers and a ring of four: 64 KB of
    // LDS, 64 accumulators)
    return (depth == 2 && tm < 4) || (wmode == 2 && tm == 4 && tn == 1 && depth == 4);
}

// DEPTH: stages of the LDS ring, each holding BIG_BK bytes of K for the whole tile.
// Variants whose ring leaves room for two workgroups per CU are held to the register budget of
// two wavefronts per SIMD: while one workgroup is in its prologue or epilogue the other one
// keeps the MFMA pipe busy.
//
// WGM x WGN: how the four wavefronts tile the workgroup's output (2 x 2, or 1 x 4 for the
// 224 x 256 tile: every wavefront then walks all the tile's token rows and a quarter of its columns).
//
// WMODE: how the weights are laid out and reach the MFMA.  0: row-major [N, K] (or operand order, gathered
// row by row into the same LDS layout: the slow way, kept for shapes without a dedicated variant), staged
// through LDS in 128-byte rows.  1: MFMA operand order (weight_layout.h), staged through LDS as they lie:
// a copy instruction moves 1 KB in a row, and lane (l32, h) finds chunk c of its row at
// unit * 2 KB + c * 256 + (l32 % 16) * 16.  2: operand order and WGM == 1, so that a wavefront's weight
// blocks are its own: they go global -> registers, DEPTH stage-loads ahead through a ring of register
// sets, and LDS carries the activations only.
template <int TM, int TN, int DEPTH, int EPI, bool SPLIT, int WGM = 2, int WGN = 2, int WMODE = 0>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(big_two_per_cu(TM, TN, DEPTH, WMODE) ? 2 : 1)))
void gemm_fp8_big_kernel(
    const uint8_t* __restrict__ a_a, const uint8_t* __restrict__ a_b, int a_K, int a_M, int a_N, int a_m_tiles,
    int a_n_tiles, int a_band, int a_by_rows, int a_k_per_split, const float* __restrict__ a_a_scale,
    const float* __restrict__ a_b_scale, const uint16_t* __restrict__ a_bias, uint16_t* __restrict__ a_out,
    int64_t a_ldo, int a_a_scale_scalar, float* __restrict__ a_partials, int* __restrict__ a_counters,
    const ResidualArgs a_res) {
    // scalar arguments, what the prologue needs first (the first 16 dwords are preloaded into SGPRs)
    BigArgs p;
    p.a = a_a; p.b = a_b; p.a_scale = a_a_scale; p.b_scale = a_b_scale; p.bias = a_bias; p.out = a_out;
    p.ldo = a_ldo; p.M = a_M; p.N = a_N; p.K = a_K; p.a_scale_scalar = a_a_scale_scalar;
    p.k_per_split = a_k_per_split; p.partials = a_partials; p.counters = a_counters;
    // a_by_rows = tile order | weights in operand order << 4
    p.m_tiles = a_m_tiles; p.n_tiles = a_n_tiles; p.band = a_band; p.by_rows = a_by_rows & 15; p.res = a_res;
    p.operand_w = __builtin_amdgcn_readfirstlane(a_by_rows >> 4);
    PHYAI_STAMP_BEGIN
    constexpr bool GATED = epi_is_gated(EPI);
    constexpr bool OPW = WMODE != 0, BDIRECT = WMODE == 2;
    static_assert(WGM * WGN == 4, "four wavefronts per workgroup");
    static_assert(!BDIRECT || (WGM == 1 && (DEPTH == 4 || DEPTH == 8)), "weights go straight to registers only where a wavefront owns them");
    constexpr int BM = WGM * 32 * TM, BN = WGN * 32 * TN;   // workgroup tile
    constexpr int WM = 32 * TM, WN = 32 * TN;        // wavefront tile
    constexpr int STAGE_BYTES = (BM + (BDIRECT ? 0 : BN)) * BIG_BK;  // one stage: A rows, then B rows (if staged)
    constexpr int CA = BM / 32, CB = BDIRECT ? 0 : BN / 32;   // copy instructions (8 rows each) per wavefront per stage
    constexpr int BL = BDIRECT ? TN * 4 : 0;         // 16-byte weight loads per lane per stage: TN blocks x 2 K halves x 2
    constexpr int COPIES = CA + CB + BL;             // vector-memory instructions per wavefront per stage-load
    constexpr int SLOTS_PER_STAGE = 2 * TM * TN;     // MFMAs of a wavefront per stage
    // Requests of a stage-load are numbered; request n goes out behind MFMA n / CPS counted from the barrier of
    // the stage that frees its target: CPS per MFMA, so that they are out by mid-stage.
    // LEAD: the barrier of stage d frees the target of stage-load d + LEAD.  Staged operands: LEAD = DEPTH - the
    // barrier waits for this wavefront's LDS reads of stage d, whose stage is then refilled.  Weights in registers:
    // LEAD = DEPTH - 1 - the targets (LDS stage and register set of stage d - 1) were last read by MFMAs that
    // every wavefront has issued before it reaches the barrier of stage d, so the barrier need not wait for the
    // LDS reads in flight (the activation blocks of the second K half, requested just before it), and no register
    // set is written while MFMAs of its stage are still to come.
    // Weights in registers, ring of eight (one column block per wavefront, stages of 8 MFMAs or fewer): LEAD = 6, so
    // that a wavefront may run two stages ahead of the slowest (see the hand-over below) with its weight loads six
    // stages and its activation copies three stages old when they are needed.
    constexpr int CPS = BDIRECT ? (COPIES + (TM - 1) * TN - 1) / ((TM - 1) * TN) : (COPIES * 2 + SLOTS_PER_STAGE - 1) / SLOTS_PER_STAGE;
    constexpr int LEAD = BDIRECT ? (DEPTH == 8 ? 6 : DEPTH - 1) : DEPTH;
    // (weights in registers) progress word d of a wavefront vouches for its activation copies up to stage-load
    // d + CLAIM; SLACK: how many stages a wavefront may be ahead of the slowest one
    constexpr int CLAIM = DEPTH == 8 ? 3 : 2;
    constexpr int SLACK = CLAIM - 1 < DEPTH - LEAD ? CLAIM - 1 : DEPTH - LEAD;
    constexpr int LATE = (TM - 1) * TN * CPS;        // first request number that falls into the next stage
    constexpr int IDX_END = COPIES;
    static_assert(!BDIRECT || COPIES <= LATE, "with weights in registers every request goes out behind the barrier");
    static_assert((TM == TN && TM % 2 == 0) || (TM == 3 && TN == 2) || (TM == 7 && TN == 2) || (TM == 2 && TN == 1 && !GATED) ||
                  (TM == 3 && TN == 1 && !GATED) || (TM == 4 && TN == 1 && !GATED && BDIRECT), "supported wavefront tiles");
    static_assert(BM % 32 == 0 && BN % 32 == 0, "every wavefront copies whole groups of 8 rows");
    static_assert(DEPTH == 2 || DEPTH == 4 || (DEPTH == 8 && BDIRECT), "ring depth");
    // (the epilogue stages the bf16 tile in the same LDS; where the ring is smaller than that, the ring grows)
    constexpr int EPI_STAGING = 4 * WM * ((GATED ? TN / 2 : TN) * 64);
    constexpr int LDS_BYTES = DEPTH * STAGE_BYTES > EPI_STAGING ? DEPTH * STAGE_BYTES : EPI_STAGING;
    // (weights in registers: 16 more bytes for the four wavefronts' progress words, see the main loop)
    __shared__ __attribute__((aligned(1024))) uint8_t lds[LDS_BYTES + (BDIRECT ? 16 : 0)];

    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int wm = wave / WGN, wn = wave % WGN;
    const int l32 = lane & 31, h = lane >> 5;
    (void)wm;
    const int half_n = p.N / 2;
    BigTile tile_id;
    int split_z = SPLIT ? (int)blockIdx.z : 0, n_splits = SPLIT ? (int)gridDim.z : 1;
    if (SPLIT && p.by_rows == 2) {
        // Split-K with an XCD per K range: XCD x (= id % 8) works on K range x % S of the tile
        // columns of group x / S, all tile rows.  The workgroups of an XCD then march along the same
        // K range together: its L2 fetches that range of the activation rows once, not all of K.
        n_splits = p.band;   // the split count rides in `band`, which this order does not use
        const int x = blockIdx.x & 7, r = blockIdx.x >> 3, groups = 8 / n_splits;
        const int cols = (p.n_tiles + groups - 1) / groups;
        split_z = x % n_splits;
        tile_id.n = (x / n_splits) * cols + r % cols;
        tile_id.m = r / cols;
    } else if (p.by_rows) {   // an XCD takes tile rows: bands of tile columns, 8 neighbouring tile rows per 8 ids
        const BigTile t = big_tile_of(blockIdx.x, p.n_tiles, p.m_tiles, p.band);
        tile_id.m = t.n; tile_id.n = t.m;
    } else {
        tile_id = big_tile_of(blockIdx.x, p.m_tiles, p.n_tiles, p.band);
    }
    if (tile_id.n >= p.n_tiles || tile_id.m >= p.m_tiles) return;   // padding of the tile order
    const int m0 = tile_id.m * BM;
    const int n0 = GATED ? tile_id.n * (BN / 2) : tile_id.n * BN;

    v16f acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    // ---- copy geometry: wavefront w moves 8-row groups w*CA .. of A and w*CB .. of B; lane i
    // fills slot i%8 of row i/8 of its group with the chunk that the swizzle assigns to it ------
    uint32_t aoff[CA], boff[CB > 0 ? CB : 1];
#pragma unroll
    for (int i = 0; i < CA; ++i) {
        const int rt = (wave * CA + i) * 8 + (lane >> 3);         // row of the tile
        int r = m0 + rt;
        r = r < p.M ? r : p.M - 1;
        aoff[i] = (uint32_t)r * (uint32_t)p.K + (((lane & 7) ^ big_swizzle(rt)) << 4);
    }
    // first 16-row unit of the tile in an operand-order matrix (plain: 16 weight rows; gated: 8 gate
    // columns and the 8 up columns that pair with them), and the units the matrix has
    const uint32_t unit0 = GATED ? (uint32_t)n0 >> 3 : (uint32_t)n0 >> 4, units = (uint32_t)p.N >> 4;
#pragma unroll
    for (int i = 0; i < CB; ++i) {
        if constexpr (WMODE == 1) {
            // instruction i moves half a unit (1 KB) as it lies; units past the matrix repeat the last one
            const uint32_t hu = wave * CB + i, u = unit0 + (hu >> 1);
            boff[i] = (u < units ? u : units - 1) * ((uint32_t)p.K << 4) + (hu & 1) * 1024 + lane * 16;
            continue;
        }
        const int jj = (wave * CB + i) * 8 + (lane >> 3);         // column of the output tile
        int rb;
        uint32_t ob;   // the row's place in operand order
        if constexpr (GATED) {
            const int w_ = jj / WN, j = jj % WN;
            int g = n0 + w_ * (WN / 2) + (j % (WN / 2));
            g = g < half_n ? g : half_n - 1;
            rb = (j / (WN / 2)) * half_n + g;
            ob = operand_offset_gated((uint32_t)g, (uint32_t)(j / (WN / 2)), (uint32_t)p.K);
        } else {
            rb = n0 + jj;
            rb = rb < p.N ? rb : p.N - 1;
            ob = operand_offset_plain((uint32_t)rb, (uint32_t)p.K);
        }
        const uint32_t chunk = (uint32_t)((lane & 7) ^ big_swizzle(jj));
        boff[i] = p.operand_w ? ob + chunk * kOperandChunkBytes : (uint32_t)rb * (uint32_t)p.K + (chunk << 4);
    }
    const int k_begin = SPLIT ? split_z * p.k_per_split : 0;
    const int b_step_shift = (OPW || p.operand_w) ? 4 : 0;   // a K step of operand-order weights is 2 KB away, not 128 bytes
    // BDIRECT: this lane's 16 bytes of chunk h of row l32 of weight block j, K step 0; chunk c of the same row
    // is c * 256 further, the next K step 2 KB
    const uint8_t* bsrc[BDIRECT ? TN : 1];
    v4i bring[BDIRECT ? DEPTH : 1][BDIRECT ? TN : 1][2][2];   // [stage-load % DEPTH][block][K half][chunk pair]
    if constexpr (BDIRECT) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            const uint32_t u = unit0 + (uint32_t)(wn * (WN / 16) + 2 * j) + ((uint32_t)l32 >> 4);
            bsrc[j] = p.b + (size_t)(u < units ? u : units - 1) * ((size_t)p.K << 4) + ((size_t)k_begin << 4) + h * 256 + (l32 & 15) * 16;
        }
    }
    const uint32_t lds_base = (uint32_t)(uintptr_t)lds;
    const uint32_t wave_a = __builtin_amdgcn_readfirstlane(lds_base + wave * (CA * 1024));
    const uint32_t wave_b = __builtin_amdgcn_readfirstlane(lds_base + BM * BIG_BK + wave * (CB * 1024));
    // copy c (0 .. COPIES-1) of this wavefront's share of stage-load `d` (K bytes [128 d, 128 d + 128))
    // (slot: d % DEPTH as a compile-time value, needed where the target is a register set)
    auto issue = [&](int d, int c, auto slot) {
        const int k = k_begin + d * BIG_BK;
        const uint32_t stage_off = (d % DEPTH) * STAGE_BYTES;
        if (c < CA) {
            if (!(PHYAI_FP8_ABLATE & 16) || d < LEAD) copy16_to_lds(p.a + k, aoff[c], wave_a + stage_off + c * 1024);
        } else if constexpr (BDIRECT) {
            constexpr int S = decltype(slot)::value;
            if ((PHYAI_FP8_ABLATE & 8) && d >= LEAD) return;
            const int e = c - CA, j = e >> 2, kh = (e >> 1) & 1, pr = e & 1;   // chunk 4 kh + 2 pr + h of block j
            bring[S][j][kh][pr] = *reinterpret_cast<const v4i*>(bsrc[j] + ((size_t)d << 11) + (4 * kh + 2 * pr) * 256);
        } else {
            copy16_to_lds(p.b + ((size_t)k << b_step_shift), boff[c - CA], wave_b + stage_off + (c - CA) * 1024);
        }
    };
    using Slot0 = std::integral_constant<int, 0>;

    const int n_loads = (SPLIT ? p.k_per_split : p.K) / BIG_BK;   // stage-loads in all, >= DEPTH
    const int arow = wm * WM + l32, brow = wn * WN + l32;
    auto stage_ptr = [&](int d) -> const uint8_t* { return lds + (d % DEPTH) * STAGE_BYTES; };
    // weight block with first row `row` - l32 out of the staged B rows, K half kh
    auto read_b = [&](const uint8_t* bbuf, int row, int kh) -> v8i {
        if constexpr (WMODE == 1) return big_frag_operand(bbuf, row, h, kh);
        else return big_frag(bbuf, row, h, kh);
    };

    // Weights in registers: LDS carries the activations only, and the wavefronts hand its stages to each other
    // through one progress word each instead of meeting at a barrier.  Word w = d says: wavefront w has issued all its
    // LDS reads of stage-loads <= d, and its own copies of stage-loads <= d + CLAIM have landed.  At its hand-over
    // point of stage d a wavefront publishes d and goes on once every word is >= d - SLACK: then stage-load d + 1 is
    // complete in LDS (SLACK <= CLAIM - 1) and the stage that stage-load d + LEAD refills has been read by everyone
    // (it held stage-load d + LEAD - DEPTH <= d - SLACK).  A wavefront may so run up to SLACK stages ahead of the
    // slowest instead of waiting for it at every stage: each stalls now and then on its own memory requests, and a
    // barrier per stage makes all four pay for every such stall (224 x 256 main loop at K = 2048: 40.2 k cycles with
    // the barrier, 32.7 k with none at all and with this).  The slowest wavefront never waits, so the scheme cannot
    // lock up; the spin is bounded all the same (a wavefront that gave up would read a stage early: wrong numbers,
    // never a hang).
    // The words are read BEFORE the stage's last batch of operand reads and looked at behind the MFMAs that follow it
    // (LDS answers in order: read at the hand-over point they would queue behind that batch, several hundred cycles
    // with two MFMAs in the pipe); a value that old can only be too small, and then the words are read again.
    // (pointers that say "LDS": through a generic pointer the accesses would be flat ones, counted with the copies)
    typedef __attribute__((address_space(3))) int lds_int_t;
    typedef __attribute__((address_space(3))) v4i lds_v4i_t;
    volatile lds_int_t* const progress = (volatile lds_int_t*)(lds + LDS_BYTES);
    auto progress_words = [&]() -> v4i { return *(const volatile lds_v4i_t*)(lds + LDS_BYTES); };
    auto hand_over = [&](int d, v4i seen) {
        if (lane == 0) progress[wave] = d;
        auto behind = [&](const v4i& w) {
            return __builtin_amdgcn_readfirstlane(min(min(w[0], w[1]), min(w[2], w[3]))) < d - SLACK;
        };
        if (__builtin_expect(behind(seen), 0)) {   // (its own block: the wait for `seen` above stays a counted one)
#pragma nounroll
            for (int spin = 0; spin < (1 << 18); ++spin) {
                __builtin_amdgcn_s_sleep(1);
                const v4i now = progress_words();
                if (!behind(now)) break;
            }
        }
    };

    // Operand blocks read one K half ahead: those of the current half (cur) and of the next one
    // (nxt); the two sets swap roles every half.  All B blocks and the first A block - or all A
    // blocks when there are only two row groups, which are too short to hide an LDS read.
    constexpr bool A_AHEAD = TM == 2;
    constexpr int NA = A_AHEAD ? TM : 1;             // A blocks read a half ahead
    v8i fa_cur[TM], fa_nxt[TM], fb_cur[TN], fb_nxt[TN];

// One K half (64 bytes, TM*TN MFMAs per wavefront) of stage-load D.  KH: which half.  FA0/FB: its
// opening blocks (in registers); NFA0/NFB receive those of the half that follows (the other half
// of the same stage, or half 0 of stage-load D+1).  NEXT: that half exists.
//
// LDS reads are issued long before their MFMAs: a batch of 128-bit reads takes several hundred
// cycles to land, a row group of four MFMAs 256.  Row group 0 requests the remaining A blocks of
// this half, row groups 1.. the opening blocks of the next half (B0 and A0 first).
//
// One barrier per stage-load, in half 1 after row group 0: by then a wavefront has issued every
// LDS read of stage-load D, so the barrier both publishes stage-load D+1 (own copies awaited
// first: AHEAD later stage-loads may stay in flight) and releases D's stage, which load D+DEPTH
// then refills.  Its copies are requested one or two at a time between the MFMAs that follow - a
// wavefront that queues them all at once sits in the memory pipeline's issue queue while its
// MFMA pipe runs dry.  ISSUE: load D+DEPTH exists (requests after the barrier); ISSUE_P: load
// D-1+DEPTH exists (requests still being spread before the barrier).  All flags are literals, so
// the steady-state loop body is straight-line code.
#define PHYAI_RUN_HALF(D, SLOT, KH, NEXT, AHEAD, ISSUE_P, ISSUE, FA0, FB, NFA0, NFB)                           \
    {                                                                                                          \
        const int d_ = (D);                                                                                    \
        const uint8_t* abuf_ = stage_ptr(d_);                                                                  \
        const uint8_t* nbuf_ = (KH) == 0 ? abuf_ : stage_ptr(d_ + 1);                                          \
        v8i fa_[TM];                                                                                           \
        v4i seen_ = {0, 0, 0, 0};                                                                              \
        if constexpr (BDIRECT) if ((KH) == 1 && (NEXT)) seen_ = progress_words();                              \
        _Pragma("unroll") for (int i_ = 0; i_ < TM; ++i_) fa_[i_] = FA0[A_AHEAD ? i_ : 0];                     \
        _Pragma("unroll") for (int i_ = 0; i_ < TM; ++i_) {                                                    \
            if (!A_AHEAD && i_ == 0) {                                                                         \
                _Pragma("unroll") for (int a_ = 1; a_ < TM; ++a_)                                              \
                    fa_[a_] = (PHYAI_FP8_ABLATE & 2) ? fa_[0] : big_frag(abuf_, arow + a_ * 32, h, KH);        \
            }                                                                                                  \
            if (i_ >= 1 && (NEXT)) {                                                                           \
                /* item 0: B0; items 1..NA: the A blocks; then B1..: spread over row groups 1..TM-1 */         \
                _Pragma("unroll") for (int q_ = 0; q_ < TN + NA; ++q_) {                                       \
                    if (q_ * (TM - 1) / (TN + NA) != i_ - 1) continue;                                         \
                    if (q_ >= 1 && q_ <= NA) NFA0[q_ - 1] = big_frag(nbuf_, arow + (q_ - 1) * 32, h, 1 - (KH)); \
                    else if constexpr (!BDIRECT) {                                                             \
                        const int j_ = q_ == 0 ? 0 : q_ - NA;                                                  \
                        NFB[j_] = read_b(nbuf_ + BM * BIG_BK, brow + j_ * 32, 1 - (KH));                       \
                    }                                                                                          \
                }                                                                                              \
            }                                                                                                  \
            const bool after_ = (KH) == 1 && i_ >= 1;   /* past this stage-load's barrier */                   \
            const bool req_ = after_ ? (ISSUE) : (ISSUE_P);                                                    \
            const int load_ = after_ ? d_ + LEAD : d_ - 1 + LEAD;                                              \
            /* MFMAs since the last barrier */                                                                 \
            const int slot0_ = after_ ? (i_ - 1) * TN : (TM - 1) * TN + ((KH) * TM + i_) * TN;                 \
            _Pragma("unroll") for (int j_ = 0; j_ < TN; ++j_) {                                                \
                v8i fb_;                                                                                       \
                if constexpr (BDIRECT) fb_ = big_join(bring[SLOT][j_][KH][0], bring[SLOT][j_][KH][1]);         \
                else fb_ = FB[j_];                                                                             \
                acc[i_][j_] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fb_, fa_[i_], acc[i_][j_],       \
                                                                               0, 0, 0, 0, 0, 0);              \
                _Pragma("unroll") for (int c_ = 0; c_ < CPS; ++c_)                                             \
                    if (req_ && (slot0_ + j_) * CPS + c_ < IDX_END && !(PHYAI_FP8_ABLATE & 1)) {               \
                        /* (register set of the load: its number modulo DEPTH) */                              \
                        if (after_) issue(load_, (slot0_ + j_) * CPS + c_, std::integral_constant<int, ((SLOT) + LEAD) % DEPTH>{});     \
                        else issue(load_, (slot0_ + j_) * CPS + c_, std::integral_constant<int, ((SLOT) + LEAD - 1) % DEPTH>{}); \
                    }                                                                                          \
                __builtin_amdgcn_sched_barrier(0);                                                             \
            }                                                                                                  \
            if ((KH) == 1 && i_ == 0 && (NEXT)) {                                                              \
                if constexpr (BDIRECT) {                                                                       \
                    /* my activation copies of D+CLAIM have landed (AHEAD: the stage-loads from that one on  */ \
                    /* that have been requested: its weight loads, which follow its copies, and all of the   */ \
                    /* later ones may be in flight); published, and everybody's of D+1 awaited               */ \
                    wait_copies<(AHEAD) == 0 ? 0 : ((AHEAD) - 1) * COPIES + (COPIES - CA)>();                  \
                    if (!(PHYAI_FP8_ABLATE & 4)) hand_over(d_, seen_);                                                \
                    asm volatile("" ::: "memory");                                                             \
                } else {                                                                                       \
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); /* my reads of stage-load D have landed */ \
                    wait_copies<COPIES * (AHEAD)>();               /* ... my copies of D+1 too ... */          \
                    if (!(PHYAI_FP8_ABLATE & 4)) __syncthreads();  /* ... and so have everybody's */           \
                }                                                                                              \
            }                                                                                                  \
        }                                                                                                      \
    }
// a whole stage-load: half 0 with the cur register set, half 1 with the nxt set
#define PHYAI_RUN_STAGE(D, SLOT, NEXT, AHEAD, ISSUE_P, ISSUE)                                                  \
    PHYAI_RUN_HALF(D, SLOT, 0, 1, 0, ISSUE_P, 0, fa_cur, fb_cur, fa_nxt, fb_nxt)                               \
    PHYAI_RUN_HALF(D, SLOT, 1, NEXT, AHEAD, ISSUE_P, ISSUE, fa_nxt, fb_nxt, fa_cur, fb_cur)

    // prologue: stage-loads 0 .. DEPTH-2 and the copies of load DEPTH-1 that the row groups after
    // a barrier would have requested in flight (the rest of it is spread over stage-load 0 like
    // every later one), load 0 published, its opening blocks in registers.
    // (as request numbers up to LATE, and as the instructions they are)
    constexpr int HEAD_IDX = LATE < IDX_END ? LATE : IDX_END;
    constexpr int HEAD = BDIRECT ? 0 : HEAD_IDX;
    if constexpr (BDIRECT) {   // stage-loads 0 .. LEAD - 1; stage-load d fills register set d % DEPTH
        // First what the first stage waits for: the activations of the stage-loads that progress word -1 vouches
        // for (0 .. CLAIM - 1; they come from L2) and the weights of stage-load 0; then the other weights of those
        // stage-loads and the later stage-loads whole, in the order the waits of the main loop count on.
        auto part = [&](auto slot, int c0, int c1) {
#pragma unroll
            for (int c = c0; c < c1; ++c) issue(decltype(slot)::value, c, slot);
        };
        using S0 = std::integral_constant<int, 0>; using S1 = std::integral_constant<int, 1>;
        using S2 = std::integral_constant<int, 2>;
        part(S0{}, CA, IDX_END);   // (the weights of stage-load 0 come from HBM: out first)
        part(S0{}, 0, CA);
        part(S1{}, 0, CA);
        if constexpr (CLAIM == 3) part(S2{}, 0, CA);
        part(S1{}, CA, IDX_END);
        if constexpr (CLAIM == 3) part(S2{}, CA, IDX_END);
        if constexpr (CLAIM == 2) part(S2{}, 0, IDX_END);
        if constexpr (LEAD == 6) {
            part(std::integral_constant<int, 3>{}, 0, IDX_END);
            part(std::integral_constant<int, 4>{}, 0, IDX_END);
            part(std::integral_constant<int, 5>{}, 0, IDX_END);
        }
    } else {
#pragma unroll
        for (int d = 0; d < DEPTH - 1; ++d)
#pragma unroll
            for (int c = 0; c < COPIES; ++c) issue(d, c, Slot0{});
#pragma unroll
        for (int c = 0; c < HEAD_IDX; ++c) issue(DEPTH - 1, c, Slot0{});
    }
    // (the large tiles' 224 - 256 accumulators are zeroed here, under the first stage-load's latency: left to the
    // compiler they are zeroed behind the wait, 1 - 2 k cycles in which nothing else happens)
    if constexpr (TM * TN >= 14) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) asm volatile("" : "+a"(acc[i][j]));
    }
    if constexpr (BDIRECT) {
        // stage-load 0 and the activations up to stage-load CLAIM - 1 have landed (what progress word -1 stands for)
        wait_copies<(LEAD - CLAIM) * COPIES + (CLAIM - 1) * (COPIES - CA)>();
        if (lane == 0) progress[wave] = -1;
    } else {
        wait_copies<COPIES * (LEAD - 2) + HEAD>();   // stage-load 0 has landed
    }
    __syncthreads();
    PHYAI_STAMP(1)
#pragma unroll
    for (int j = 0; j < TN; ++j)
        if constexpr (!BDIRECT) fb_cur[j] = read_b(lds + BM * BIG_BK, brow + j * 32, 0);
#pragma unroll
    for (int i = 0; i < (A_AHEAD ? TM : 1); ++i) fa_cur[i] = big_frag(lds, arow + i * 32, h, 0);
    int d = 0;
    if constexpr (BDIRECT) {
        // the register sets are named at compile time: DEPTH stage-loads per trip (the launcher sees to it
        // that their number is a multiple of DEPTH)
        // ring of four: at the hand-over of stage d stage-load d + 2 may be in flight; behind it d + 3 is requested
        for (; d < n_loads - DEPTH; d += DEPTH) {
            if constexpr (DEPTH == 4) {
                PHYAI_RUN_STAGE(d, 0, 1, 1, 0, 1)
                PHYAI_RUN_STAGE(d + 1, 1, 1, 1, 0, 1)
                PHYAI_RUN_STAGE(d + 2, 2, 1, 1, 0, 1)
                PHYAI_RUN_STAGE(d + 3, 3, 1, 1, 0, 1)
            } else {   // at the hand-over of stage d stage-loads d + 3 .. d + 5 may be in flight; d + 6 is requested behind it
                PHYAI_RUN_STAGE(d, 0, 1, 3, 0, 1)
                PHYAI_RUN_STAGE(d + 1, 1, 1, 3, 0, 1)
                PHYAI_RUN_STAGE(d + 2, 2, 1, 3, 0, 1)
                PHYAI_RUN_STAGE(d + 3, 3, 1, 3, 0, 1)
                PHYAI_RUN_STAGE(d + 4, 4, 1, 3, 0, 1)
                PHYAI_RUN_STAGE(d + 5, 5, 1, 3, 0, 1)
                PHYAI_RUN_STAGE(d + 6, 6, 1, 3, 0, 1)
                PHYAI_RUN_STAGE(d + 7, 7, 1, 3, 0, 1)
            }
        }
    } else {
        for (; d < n_loads - DEPTH; ++d) { PHYAI_RUN_STAGE(d, 0, 1, DEPTH - 2, 1, 1) }
    }
    // d == n_loads - DEPTH: the last requests are still being spread, then the ring drains
    if constexpr (BDIRECT && DEPTH == 8) {   // the last request goes out behind the hand-over of stage n - 7
        PHYAI_RUN_STAGE(d, 0, 1, 3, 0, 1)
        PHYAI_RUN_STAGE(d + 1, 1, 1, 3, 0, 1)
        PHYAI_RUN_STAGE(d + 2, 2, 1, 3, 0, 0)
        PHYAI_RUN_STAGE(d + 3, 3, 1, 2, 0, 0)
        PHYAI_RUN_STAGE(d + 4, 4, 1, 1, 0, 0)
        PHYAI_RUN_STAGE(d + 5, 5, 1, 0, 0, 0)
        PHYAI_RUN_STAGE(d + 6, 6, 1, 0, 0, 0)
        PHYAI_RUN_STAGE(d + 7, 7, 0, 0, 0, 0)
    } else if constexpr (BDIRECT) {   // the last request goes out behind the hand-over of stage n - 4
        PHYAI_RUN_STAGE(d, 0, 1, 1, 0, 1)
        PHYAI_RUN_STAGE(d + 1, 1, 1, 1, 0, 0)
        PHYAI_RUN_STAGE(d + 2, 2, 1, 0, 0, 0)
        PHYAI_RUN_STAGE(d + 3, 3, 0, 0, 0, 0)
    } else if constexpr (DEPTH == 2) {
        PHYAI_RUN_STAGE(d, 0, 1, 0, 1, 0)
        PHYAI_RUN_STAGE(d + 1, 0, 0, 0, 0, 0)
    } else {
        PHYAI_RUN_STAGE(d, 0, 1, 2, 1, 0)
        PHYAI_RUN_STAGE(d + 1, 1, 1, 1, 0, 0)
        PHYAI_RUN_STAGE(d + 2, 2, 1, 0, 0, 0)
        PHYAI_RUN_STAGE(d + 3, 3, 0, 0, 0, 0)
    }
#undef PHYAI_RUN_STAGE
#undef PHYAI_RUN_HALF
    PHYAI_STAMP(2)

    // ---- split-K: publish partial sums; the last split to arrive adds them in split order --
    // Two blocks (32 floats per lane) at a time, so that the 4 x 4 variant never holds more than
    // that outside its accumulators.
    // (K split in two) this workgroup arrived second: the half that the first one wrote is added where the epilogue
    // reads the accumulators, block by block, the loads of the next block under the arithmetic of the current one
    bool add_other = false;
    const int sp_tile = tile_id.m * p.n_tiles + tile_id.n;
    if constexpr (SPLIT) {
        constexpr int FRAG = TM * TN * 16, CHUNK = 32;
        const int S = n_splits;
        const int tile = sp_tile;
        auto publish = [&]() {
#pragma unroll
            for (int c = 0; c < TM * TN / 2; ++c) {
                float frag[CHUNK];
#pragma unroll
                for (int r = 0; r < 32; ++r) frag[r] = acc[(2 * c) / TN][(2 * c) % TN + r / 16][r % 16];
                splitk_publish_part<FRAG, 256, CHUNK>(p.partials, tile, S, split_z, c * CHUNK, frag);
            }
            wait_own_stores();
        };
        // gather: as much of the fragment per round trip as the registers allow
        constexpr int GCH = FRAG <= 64 ? FRAG : 32;
        if (S == 2) {   // (uniform) two splits: the first to arrive writes its half, the second adds it to its own
            const int found = splitk_arrive_early(p.counters, tile, reinterpret_cast<int*>(lds));
            if (found == 0) {
                publish();
                splitk_published(p.counters, tile);
                return;
            }
            splitk_await_published(p.counters, tile, found);
            add_other = true;
        } else {
            publish();
            // splitk_arrive opens with a barrier, after which nobody reads operands any more: a word
            // of the ring serves as its flag
            if (!splitk_arrive(p.counters, tile, S, reinterpret_cast<int*>(lds))) return;
#pragma unroll
            for (int c = 0; c < FRAG / GCH; ++c) {
                float frag[GCH];
                splitk_gather_part<FRAG, 256, GCH>(p.partials, tile, S, c * GCH, frag);
#pragma unroll
                for (int r = 0; r < GCH; ++r) {
                    const int blk = (c * GCH + r) / 16;
                    acc[blk / TN][blk % TN][r % 16] = frag[r];
                }
            }
        }
        splitk_reset(p.counters, tile);
    }

    PHYAI_STAMP(3)
    // ---- epilogue ------------------------------------------------------------------------
    // The weight block is the MFMA's first operand, so accumulator r of lane (l32, h) of block
    // (i, j) is the output at token row i*32 + l32, column j*32 + 8*(r/4) + 4*h + r%4: a lane
    // owns runs of four consecutive columns of one row.  A run becomes four bf16 with two packed
    // converts and goes to the wavefront's slice of the (now idle) LDS as one 8-byte write; the
    // staged tile leaves row-wise, 16 bytes per lane, whole row segments per instruction.  The
    // 16-byte slots of a staged row are XOR-swizzled with the row so that the 32 rows written by
    // one instruction spread over the banks.
    constexpr int TNO = GATED ? TN / 2 : TN;             // output column blocks per wavefront
    constexpr int ROWB = TNO * 64;                       // staged row length in bytes
    constexpr int SLOTS = ROWB / 16;
    constexpr int ROWS_PER_PASS = 16 / SLOTS > 0 ? 16 / SLOTS : 1;   // rows per 256 bytes of banks
    constexpr int STG_BYTES = WM * ROWB;                 // per wavefront
    static_assert(4 * STG_BYTES <= LDS_BYTES, "staging fits in the operand LDS");
    const int n_lim = GATED ? half_n : p.N;
    const int nbase = n0 + wn * (GATED ? WN / 2 : WN);
    // column constants are read 4 at a time when the arrays allow it (N is a multiple of 16, so
    // a run of four columns is valid or invalid as a whole)
    const bool vec_cols = (reinterpret_cast<uintptr_t>(p.b_scale) & 15) == 0 &&
                          (reinterpret_cast<uintptr_t>(p.bias) & 7) == 0;
    auto load_cols = [&](int n, v4f& sc, v4f& bi) {
        if (vec_cols) {
            sc = *reinterpret_cast<const v4f*>(p.b_scale + n);
            if (p.bias) {
                const uint2 b = *reinterpret_cast<const uint2*>(p.bias + n);
                bi[0] = bf16_bits_to_f32(b.x & 0xFFFFu); bi[1] = __uint_as_float(b.x & 0xFFFF0000u);
                bi[2] = bf16_bits_to_f32(b.y & 0xFFFFu); bi[3] = __uint_as_float(b.y & 0xFFFF0000u);
            } else {
                bi[0] = bi[1] = bi[2] = bi[3] = 0.f;
            }
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                sc[e] = p.b_scale[n + e];
                bi[e] = p.bias ? bf16_bits_to_f32(p.bias[n + e]) : 0.f;
            }
        }
    };
    float sa[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int m = m0 + wm * WM + i * 32 + l32;
        sa[i] = p.a_scale[p.a_scale_scalar ? 0 : (m < p.M ? m : p.M - 1)];
    }
    __syncthreads();  // every wavefront is done reading operands from LDS
    uint8_t* stg = lds + wave * STG_BYTES;
    // the other workgroup's 16 partial sums of block (i, j) (element (i TN + j) 16 + r of its fragment, splitk.h)
    auto other_half = [&](int i, int j, float* po) {
        if constexpr (SPLIT) {
            if (add_other) splitk_load_part<TM * TN * 16, 256, 16>(p.partials, sp_tile, 2, 1 - split_z, (i * TN + j) * 16, po);
        }
    };
    // accumulator r of a block, with the other half where there is one (a + b: the sum in split order either way)
    auto summed = [&](float a, const float* po, int r) { return SPLIT && add_other ? a + po[r] : a; };
    if constexpr (OPW && GATED) {
        // Weights in the gated operand order: rows 4p .. 4p+3 of a 16-row unit are gate columns 2p, 2p+1 and up
        // columns 2p, 2p+1.  Accumulator 4k + e of lane (l32, h) of block j is block row 8k + 4h + e, i.e. with
        // e = 2t + b: gate (t = 0) / up (t = 1) of output column 16 j + 4 k + 2 h + b of the wavefront - a lane
        // holds both halves of two neighbouring output columns per k.  Same arithmetic as below, operation for
        // operation.
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            float sgk[4][2], suk[4][2], bgk[4][2], buk[4][2];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const int n = nbase + 16 * j + 4 * k + 2 * h;
                const int n_safe = n < n_lim ? n : 0;
#pragma unroll
                for (int b = 0; b < 2; ++b) {
                    sgk[k][b] = p.b_scale[n_safe + b];
                    suk[k][b] = p.b_scale[half_n + n_safe + b];
                    bgk[k][b] = p.bias ? bf16_bits_to_f32(p.bias[n_safe + b]) : 0.f;
                    buk[k][b] = p.bias ? bf16_bits_to_f32(p.bias[half_n + n_safe + b]) : 0.f;
                }
            }
            float pn[16] = {};
            other_half(0, j, pn);
#pragma unroll
            for (int i = 0; i < TM; ++i) {
                const int row = i * 32 + l32;
                const int sw = (row / ROWS_PER_PASS) & (SLOTS - 1);
                float po[16];
#pragma unroll
                for (int r = 0; r < 16; ++r) po[r] = pn[r];
                if (i + 1 < TM) other_half(i + 1, j, pn);
#pragma unroll
                for (int k = 0; k < 4; ++k) {
                    const float g0 = __builtin_fmaf(summed(acc[i][j][4 * k + 0], po, 4 * k + 0), sa[i] * sgk[k][0], bgk[k][0]);
                    const float g1 = __builtin_fmaf(summed(acc[i][j][4 * k + 1], po, 4 * k + 1), sa[i] * sgk[k][1], bgk[k][1]);
                    const float u0 = __builtin_fmaf(summed(acc[i][j][4 * k + 2], po, 4 * k + 2), sa[i] * suk[k][0], buk[k][0]);
                    const float u1 = __builtin_fmaf(summed(acc[i][j][4 * k + 3], po, 4 * k + 3), sa[i] * suk[k][1], buk[k][1]);
                    // gate and up pass through bf16 first, as the two-launch form materialises them
                    const uint32_t g01 = pack_bf16x2(g0, g1), u01 = pack_bf16x2(u0, u1);
                    const float o0 = apply_act<EPI>(__uint_as_float(g01 << 16)) * __uint_as_float(u01 << 16);
                    const float o1 = apply_act<EPI>(__uint_as_float(g01 & 0xFFFF0000u)) * __uint_as_float(u01 & 0xFFFF0000u);
                    const int slot = (2 * j + (k >> 1)) ^ sw;
                    *reinterpret_cast<uint32_t*>(stg + row * ROWB + slot * 16 + 8 * (k & 1) + 4 * h) = pack_bf16x2(o0, o1);
                }
            }
        }
    } else {
#pragma unroll
    for (int j = 0; j < TNO; ++j) {
        v4f sg[4], bg[4], su[4], bu[4];
#pragma unroll
        for (int g = 0; g < 4; ++g) {
            const int n = nbase + j * 32 + 8 * g + 4 * h;
            const int n_safe = n < n_lim ? n : 0;
            load_cols(n_safe, sg[g], bg[g]);
            if constexpr (GATED) load_cols(half_n + n_safe, su[g], bu[g]);
        }
        float pn[16] = {}, un[16] = {};
        other_half(0, j, pn);
        if constexpr (GATED) other_half(0, j + TN / 2, un);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
            const int row = i * 32 + l32;
            const int sw = (row / ROWS_PER_PASS) & (SLOTS - 1);
            float po[16], pu[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) { po[r] = pn[r]; pu[r] = un[r]; }
            if (i + 1 < TM) {
                other_half(i + 1, j, pn);
                if constexpr (GATED) other_half(i + 1, j + TN / 2, un);
            }
#pragma unroll
            for (int g = 0; g < 4; ++g) {
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = __builtin_fmaf(summed(acc[i][j][4 * g + e], po, 4 * g + e), sa[i] * sg[g][e], bg[g][e]);
                if constexpr (GATED) {
                    float u[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) u[e] = __builtin_fmaf(summed(acc[i][j + TN / 2][4 * g + e], pu, 4 * g + e), sa[i] * su[g][e], bu[g][e]);
                    // gate and up pass through bf16 first, as the two-launch form materialises them
                    const uint32_t g01 = pack_bf16x2(o[0], o[1]), g23 = pack_bf16x2(o[2], o[3]);
                    const uint32_t u01 = pack_bf16x2(u[0], u[1]), u23 = pack_bf16x2(u[2], u[3]);
                    o[0] = apply_act<EPI>(__uint_as_float(g01 << 16)) * __uint_as_float(u01 << 16);
                    o[1] = apply_act<EPI>(__uint_as_float(g01 & 0xFFFF0000u)) * __uint_as_float(u01 & 0xFFFF0000u);
                    o[2] = apply_act<EPI>(__uint_as_float(g23 << 16)) * __uint_as_float(u23 << 16);
                    o[3] = apply_act<EPI>(__uint_as_float(g23 & 0xFFFF0000u)) * __uint_as_float(u23 & 0xFFFF0000u);
                } else if constexpr (EPI != EPI_NONE) {
                    const uint32_t g01 = pack_bf16x2(o[0], o[1]), g23 = pack_bf16x2(o[2], o[3]);
                    o[0] = apply_act<EPI>(__uint_as_float(g01 << 16));
                    o[1] = apply_act<EPI>(__uint_as_float(g01 & 0xFFFF0000u));
                    o[2] = apply_act<EPI>(__uint_as_float(g23 << 16));
                    o[3] = apply_act<EPI>(__uint_as_float(g23 & 0xFFFF0000u));
                } else {
                    if (p.res.residual != nullptr) {       // out = residual + bf16(linear) * gate
                        const int m = m0 + wm * WM + row;
                        const int n = nbase + j * 32 + 8 * g + 4 * h;
                        if (m < p.M && n < n_lim) {
                            const uint2 rs = *reinterpret_cast<const uint2*>(p.res.residual + (int64_t)m * p.res.ld_res + n);
                            const uint2 gt = *reinterpret_cast<const uint2*>(
                                p.res.gate + (int64_t)(m / p.res.gate_group) * p.res.ld_gate + n);
                            addcmul4(o, rs, gt);
                        }
                    }
                }
                uint2 w;
                w.x = pack_bf16x2(o[0], o[1]);
                w.y = pack_bf16x2(o[2], o[3]);
                const int slot = (j * 4 + g) ^ sw;
                *reinterpret_cast<uint2*>(stg + row * ROWB + slot * 16 + h * 8) = w;
            }
        }
    }
    }
    PHYAI_STAMP(4)
    // write the staged tile out: 1 KB (whole rows) per instruction.  The output is written once
    // and never read here: non-temporal stores keep it from evicting the operands that the
    // neighbouring tiles still want from L2 (4800 x 8192 x 2048 + GELU: 113 -> 95 us;
    // 13056 x 2560 x 2048: 76.6 -> 70.1 us; same box, alternating builds).
#pragma unroll 4
    for (int qd = 0; qd < STG_BYTES / 1024; ++qd) {
        const int byte = qd * 1024 + lane * 16;
        const int row = byte / ROWB, slot = (byte % ROWB) / 16;
        const int sw = (row / ROWS_PER_PASS) & (SLOTS - 1);
        const v4i v = *reinterpret_cast<const v4i*>(stg + row * ROWB + ((slot ^ sw) << 4));
        const int m = m0 + wm * WM + row;
        const int n = nbase + slot * 8;
        if (m < p.M && n < n_lim) __builtin_nontemporal_store(v, reinterpret_cast<v4i*>(p.out + (int64_t)m * p.ldo + n));
    }
    PHYAI_STAMP(5)
    PHYAI_STAMP_END(g_big_stamps, ((size_t)blockIdx.x + (size_t)gridDim.x * blockIdx.z) * 4 + wave, lane)
}

// ---- host side ---------------------------------------------------------------------------

static int big_ceil_div(int a, int b) { return (a + b - 1) / b; }

static int big_tiles(int M, int N, int epilogue, int bm, int bn) {
    const bool gated = epi_is_gated(epilogue);
    return big_ceil_div(M, bm) * big_ceil_div(gated ? N / 2 : N, gated ? bn / 2 : bn);
}

// Tile edge (256 or 128, 0 = this kernel does not apply) and K splits.  256 x 256 tiles once
// they fill the chip; 128 x 128 tiles for problems that are still MFMA-sized but have fewer
// tiles, and those are split along K when even the small tiles leave CUs idle: a CU can pull
// only about 45 GB/s from L2, so a mid-sized GEMM finishes sooner on more CUs even though the
// partial sums then make a round trip through memory.
static int big_tile_cols(int tile) { return (tile == 256 || tile == 224) ? 256 : 128; }

// Fraction of the tile slots that hold a tile, over all rounds of `slots` concurrent tiles.
static double big_fill(int tiles, int slots) {
    const int rounds = big_ceil_div(tiles, slots);
    return rounds > 0 ? (double)tiles / ((double)rounds * slots) : 1.0;
}

BigPlan big_plan(int M, int N, int K, int epilogue, bool operand_w) {
    BigPlan pl = {0, 0, 1, 0, 0, 0};
    if (K % 128 != 0 || K < 512) return pl;   // slabs come in pairs and must fill the ring
    int forced = -1;
    if (const char* e = tuning_env("PHYAI_FP8_BIG")) forced = atoi(e);   // "0": never; "256"/"192"/"128": force
    if (forced == 0) return pl;
    if (forced == 256 || forced == 224 || forced == 192 || forced == 128) pl.tile = forced;   // ("96": 96 x 128, below)
    else if (forced == 12864 && !epi_is_gated(epilogue)) { pl.tile = 128; pl.cols = 64; }   // "12864": 128 rows x 64 columns
    else if (forced == 96 && !epi_is_gated(epilogue)) { pl.tile = 96; pl.cols = 128; }
    else if (M < 128) return pl;
    // 256 x 256 tiles need the fewest bytes from L2 per flop but run one workgroup per CU, so a
    // tile's prologue and epilogue leave the MFMA pipe idle; 192 x 128 tiles fit twice and overlap
    // them.  The small tile wins once there are enough of them and while K is short enough for
    // prologue and epilogue to matter (measured: 4-18 % up to K = 8192), unless M pads worse or
    // its last round of 512 tiles would be much emptier than the large tile's last round of 256
    // (6528 x 2048 x 2048: 544 small tiles take 42 us, 208 large ones 37.5 us).
    else if (K <= 8192 && big_tiles(M, N, epilogue, 192, 128) >= 400 &&
             big_ceil_div(M, 192) * 192 <= big_ceil_div(M, 256) * 256 &&
             big_fill(big_tiles(M, N, epilogue, 192, 128), 512) >= big_fill(big_tiles(M, N, epilogue, 256, 256), 256) - 0.15)
        pl.tile = 192;
    // ... and also when it fits one round of two workgroups per CU while 128 x 128 tiles would just
    // spill into a second one (3264 x 2560 x 2048: 340 tiles of 192 x 128 take 27 us, 520 of
    // 128 x 128 take 33 us; with 416 of those, 3264 x 2048 x 2048, the smaller tile wins 20.6 to 25.3)
    else if (K <= 8192 && big_tiles(M, N, epilogue, 256, 256) < 200 && big_tiles(M, N, epilogue, 192, 128) > 256 &&
             big_tiles(M, N, epilogue, 192, 128) <= 512 && big_tiles(M, N, epilogue, 128, 128) > 512)
        pl.tile = 192;
    else if (big_tiles(M, N, epilogue, 256, 256) >= 200)
        // 224 x 256 tiles (every wavefront walks all 224 token rows) when they need no more tile
        // rows than 256 x 256: the same number of workgroups, fewer MFMAs on padding (816 rows:
        // 896 instead of 1024, gate_up 2048 -> 32768 at M = 816 67.4 -> 64.2 us).  The gain is
        // smaller than the saved MFMAs because each wavefront then reads all of the tile's
        // activation rows from LDS, which is the next limit (113 of 128 bytes per clock).
        pl.tile = big_ceil_div(M, 224) == big_ceil_div(M, 256) ? 224 : 256;
    else if (big_tiles(M, N, epilogue, 128, 128) >= 32) pl.tile = 128;   // fewer: the weight-streaming kernel wins
    else return pl;
    if (pl.cols == 0) pl.cols = big_tile_cols(pl.tile);
    int tiles = big_tiles(M, N, epilogue, pl.tile, pl.cols);
    // Few 128 x 128 tiles and a plain epilogue: 128 x 64 tiles (2 x 1 blocks per wavefront) put twice
    // as many CUs to work.  The kernel is bound by LDS bytes, and the narrow tile reads half as many
    // again per MFMA, so it pays only while the 128 x 128 grid leaves at least half of the CUs idle
    // (weights from HBM, 18 weight sets): 816 x 2048 x 2048 (112 -> 224 tiles) 11.4 -> 8.9 us,
    // 816 x 2048 x 4096 17.7 -> 13.8 us, 1100 x 1024 x 4096 16.6 -> 12.4 us; 816 x 2560 x 2048
    // (140 -> 280 tiles, a second round) 12.8 -> 15.1 us and stays; from K = 8192 on the 128 x 128
    // form with K split in two is level or ahead (27.9 against 28.7 us, K = 16384: 44 against 51).
    if (forced < 0 && pl.tile == 128 && !epi_is_gated(epilogue) && tiles > 64 && tiles <= 128 && K < 8192) {
        pl.cols = 64;
        tiles = big_tiles(M, N, epilogue, 128, 64);
    }
    // Between 129 and 255 tiles of 128 x 128 (and a plain epilogue) 96 x 128 tiles - wavefronts 1 x 4, three row
    // blocks each - put up to 256 CUs to work in one round where the 128-row grid leaves a fifth to a half of them
    // idle and 128 x 64 tiles would need a second round: 8 - 11 % faster on every shape measured (weights from HBM,
    // 12 - 18 weight sets): 816 x 2560 x 2048 (140 -> 180 tiles) 11.2 -> 9.95 us, 816 x 3072 x 2048 11.2 -> 10.1,
    // 700 x 4096 x 1024 8.4 -> 7.7, 1000 x 2304 x 2048 11.1 -> 10.1, 650 x 3584 x 4096 16.4 -> 14.9, 816 x 2560 x 4096
    // 16.1 -> 14.9, 560 x 4096 x 2048 10.9 -> 9.9.  Where the 128-row grid already fills the chip, or 128 x 64 tiles
    // fit one round, it loses (816 x 2048 x 2048: 9.6 against 8.2 us; 1632 x 2560 x 2048: 17.5 against 15.4).
    if (forced < 0 && pl.tile == 128 && pl.cols == 128 && !epi_is_gated(epilogue) && tiles > 128 && tiles < 256 && K < 8192) {
        const int t96 = big_tiles(M, N, epilogue, 96, 128);
        if (t96 > tiles && t96 <= 256) { pl.tile = 96; tiles = t96; }
    }
    pl.tiles = tiles;
    pl.depth = (pl.tile == 128 || pl.tile == 96) ? 4 : 2;
    bool to_224 = false;
    if (operand_w && forced < 0 && pl.tile != 224 && K >= 4096 && K % 512 == 0) {
        // Weights in operand order: the 224 x 256 tile loads them straight into registers and hands its activation
        // stages over without barriers - its main loop runs at 0.88 of the MFMA rate where the other shapes reach
        // 0.7 - 0.85 - and from K = 4096 on the prologue and epilogue that nothing overlaps in it weigh less than
        // that.  Taken when it has at least 160 tiles and fills its rounds of 256 workgroups with useful rows and
        // columns at least 0.8 times as well as the shape chosen above fills its own (weights from HBM, 4 - 6 weight
        // sets, us: 6528 x 2048 x 16384 185 -> 166, 13056 x 2048 x 16384 366 -> 317, 6528 x 2048 x 8192 96 -> 86,
        // 1632 x 8192 x 8192 96 -> 88, 4800 x 2048 x 8192 81 -> 74, 6528 x 4096 x 4096 106 -> 96, 13056 x 2048 x 4096
        // 107 -> 98, 3264 x 16384 x 4096 + GeGLU 202 -> 189; level: 4800 x 8192 x 4096, 3264 x 8192 x 4096; not taken,
        // and slower when forced: 2048 x 8192 x 8192 (320 tiles, two rounds: 150 against 103), 8000 x 1024 x 8192 (144
        // tiles: 74 against 69), 3264 x 2048 x 16384 (120 tiles: 129 against 125).  At K = 2048 the shapes that run
        // two workgroups per CU keep their lead.
        const int t224 = big_tiles(M, N, epilogue, 224, 256);
        const int slots = big_two_per_cu(pl.tile == 192 ? 3 : pl.tile == 256 ? 4 : 2, 2, pl.depth, 0) ? 512 : 256;
        const double area_now = (double)big_ceil_div(tiles * pl.splits, slots) * slots * pl.tile * pl.cols;
        const double area_224 = (double)big_ceil_div(t224, 256) * 256 * 224 * 256;
        if (t224 >= 160 && pl.splits == 1 && area_now >= 0.8 * area_224) to_224 = true;
    }
    if (to_224) {
        pl.tile = 224; pl.cols = 256; pl.depth = 2;
        pl.tiles = tiles = big_tiles(M, N, epilogue, 224, 256);
    }
    if ((pl.tile == 128 && pl.cols == 64) || pl.tile == 96) {
        // always one round of at most 256 workgroups here, or forced: deep ring, no split
    } else if (pl.tile == 128) {
        // Measured at M = 816: splitting pays for K = 16384 (67 -> 49 us with two splits) and
        // costs for K = 2048 (19 -> 25 us): the partial-sum round trip is worth about 6 us.
        if (tiles < 200 && K >= 8192 && K % 256 == 0) pl.splits = 2;
        // With more tiles than CUs a ring of two stages lets two workgroups share a CU instead of
        // queueing behind each other (800 x 8192 x 1024, 448 tiles: 17.5 -> 14.4 us; 1632 x 2560 x 2048,
        // 260 tiles: 23.3 -> 18.3 us); up to one tile per CU the deeper ring hides more latency
        // (1632 x 2048 x 2048, 208 tiles: 14.2 against 17.3 us).
        else if (tiles > 256) pl.depth = 2;
    }
    if (const char* e = tuning_env("PHYAI_FP8_BIG_SPLITS")) {
        const int s = atoi(e);
        if (pl.tile == 128 && pl.cols == 128 && s >= 1 && K % (s * 128) == 0 && K / s >= 512 && tiles * s <= 4096) pl.splits = s;
    }
    if (const char* e = tuning_env("PHYAI_FP8_BIG_DEPTH")) {
        const int d = atoi(e);
        if (pl.tile == 128 && pl.cols == 128 && pl.splits == 1 && (d == 2 || d == 4)) pl.depth = d;
    }
    // Weights in operand order and a whole number of trips round the ring per K range: the wavefronts load their own
    // weight blocks straight into registers (PHYAI_FP8_BIG_DIRECT=0: stage them like the rest).  224 x 256 tiles: ring
    // of four.  128 x 128 tiles with a ring of four LDS stages and a plain epilogue: wavefronts 1 x 4 with one column
    // block each and a ring of eight.  (Not the 96 x 128 tile: its main loop gains what its longer prologue - six
    // stage-loads requested up front, at what the CU's vector-memory path passes - loses: 816 x 2560 x 2048 10.0 ->
    // 10.1 us.)
    if (operand_w && !(tuning_env("PHYAI_FP8_BIG_DIRECT") && atoi(tuning_env("PHYAI_FP8_BIG_DIRECT")) == 0)) {
        if (pl.tile == 224 && pl.splits == 1 && K % 512 == 0) pl.regs = 4;
        else if (pl.tile == 128 && pl.cols == 128 && pl.depth == 4 && (K / pl.splits) % 1024 == 0 && !epi_is_gated(epilogue)) pl.regs = 8;
        // (more tiles than CUs: two workgroups per CU, each with a ring of four)
        else if (pl.tile == 128 && pl.cols == 128 && pl.depth == 2 && pl.splits == 1 && K % 512 == 0 && !epi_is_gated(epilogue)) pl.regs = 4;
    }
    return pl;
}

size_t big_partial_bytes(int M, int N, int epilogue, const BigPlan& pl) {
    if (pl.splits <= 1) return 0;
    const int bn = pl.cols;
    return (size_t)big_tiles(M, N, epilogue, pl.tile, bn) * pl.splits * pl.tile * bn * sizeof(float);
}

template <int TM, int TN, int DEPTH, int EPI, int WGM = 2, int WGN = 2, int WMODE = 0>
static void big_launch(BigArgs a, const GemmProblem& g, int splits, hipStream_t st) {
    const bool gated = epi_is_gated(EPI);
    constexpr int BM = WGM * 32 * TM, BN = WGN * 32 * TN;
    const int bn_eff = gated ? BN / 2 : BN;
    a.n_tiles = big_ceil_div(gated ? g.N / 2 : g.N, bn_eff);
    a.m_tiles = big_ceil_div(g.M, BM);
    // Which operand the XCDs share.  By default an XCD takes tile columns: its L2 then holds the
    // weight rows of those columns once, but every XCD streams all activation rows it meets.
    // With few tile columns and long rows of activations (816 x B tokens into a 16384 -> 2048
    // projection) that is eight copies of the larger operand; then the roles are exchanged.
    // Estimated bytes from HBM: the operand an XCD does not own is read once per XCD (up to 8
    // times), the other once per band.
    double chosen_bytes = 0.0;
    {
        const double a_bytes = (double)g.M * g.K, b_bytes = (double)g.N * g.K;
        const int band_c = 4, band_r = 4;
        const double by_cols = a_bytes * (a.n_tiles < 8 ? a.n_tiles : 8) + b_bytes * big_ceil_div(a.m_tiles, band_c);
        const double by_rows = b_bytes * (a.m_tiles < 8 ? a.m_tiles : 8) + a_bytes * big_ceil_div(a.n_tiles, band_r);
        a.by_rows = by_rows < 0.8 * by_cols;
        // ... unless the busiest XCD then needs one more round of tiles than in the other order
        // (13056 x 2560 x 2048 in 256 x 256 tiles: 510 tiles are 64 per XCD by tile columns, two
        // rounds on 32 CUs, but 65 on some XCDs by tile rows: 92 against 75.5 us)
        const int slots = 32 * (big_two_per_cu(TM, TN, DEPTH, WMODE) ? 2 : 1);
        const int rounds_c = big_ceil_div(big_max_tiles_per_xcd(a.m_tiles, a.n_tiles, 4), slots);
        const int rounds_r = big_ceil_div(big_max_tiles_per_xcd(a.n_tiles, a.m_tiles, 4), slots);
        if (rounds_c != rounds_r) a.by_rows = rounds_r < rounds_c;
        if (const char* e = tuning_env("PHYAI_FP8_BY_ROWS")) a.by_rows = atoi(e) != 0;
        chosen_bytes = a.by_rows ? by_rows : by_cols;
    }
    // bands of 4 tile rows; a grid of up to 8 tile rows whose activation rows still fit an XCD's
    // L2 beside the weight stream is one band, so that the weights come from HBM once
    a.band = 4;
    if (!a.by_rows && a.m_tiles <= 8 && (int64_t)a.m_tiles * BM * (g.K < 4096 ? g.K : 4096) <= (5 << 19)) a.band = a.m_tiles;
    if (const char* e = tuning_env("PHYAI_FP8_BAND")) { const int b = atoi(e); if (b >= 1 && b <= 16) a.band = b; }
    const int outer = a.by_rows ? a.n_tiles : a.m_tiles, inner = a.by_rows ? a.m_tiles : a.n_tiles;
    dim3 grid(big_grid_ids(outer, inner, a.band), 1, splits);
    // Split along K: an XCD per K range (see the kernel).  Every XCD then fetches 1 / splits of the
    // activation codes instead of all of them, and the weights of its tile columns once.  Taken when
    // that is the smaller estimate and the tile columns divide evenly among the 8 / splits groups
    // (816 x 2048 x 16384, K split in two: 155 -> 87 MB fetched; the time is the same to within 1 %,
    // the kernel being bound by its LDS traffic, so this saves HBM bandwidth, not microseconds).
    if (splits == 2 || splits == 4 || splits == 8) {
        const int groups = 8 / splits, cols = big_ceil_div(a.n_tiles, groups);
        const double by_k = (double)g.M * g.K * 8.0 / splits + (double)g.N * g.K;
        bool xcd_k = cols * groups == a.n_tiles && by_k < 0.8 * chosen_bytes;
        if (const char* e = tuning_env("PHYAI_FP8_XCD_SPLIT")) xcd_k = atoi(e) != 0;
        if (xcd_k) {
            a.by_rows = 2;
            a.band = splits;
            grid = dim3(8 * cols * a.m_tiles, 1, 1);
        }
    }
#define PHYAI_BIG_ARGS a.a, a.b, a.K, a.M, a.N, a.m_tiles, a.n_tiles, a.band, a.by_rows | (a.operand_w << 4), a.k_per_split, a.a_scale, \
                       a.b_scale, a.bias, a.out, a.ldo, a.a_scale_scalar, a.partials, a.counters, a.res
    if (splits > 1) {
        // (K splits: 128 x 128 tiles with a ring of four, staged or with weights in registers.  The 256 x 256 tile is
        // not built with them: its 256 accumulators leave the gather no registers, and a kernel that spills has
        // vector-memory instructions of the compiler's among the copies that the waits count by hand.)
        if constexpr ((TM == TN && TM == 2 && DEPTH == 4) || (WMODE == 2 && TN == 1 && !big_two_per_cu(TM, TN, DEPTH, WMODE)))
            hipLaunchKernelGGL((gemm_fp8_big_kernel<TM, TN, DEPTH, EPI, true, WGM, WGN, WMODE>), grid, dim3(256), 0, st, PHYAI_BIG_ARGS);
    } else {
        hipLaunchKernelGGL((gemm_fp8_big_kernel<TM, TN, DEPTH, EPI, false, WGM, WGN, WMODE>), grid, dim3(256), 0, st, PHYAI_BIG_ARGS);
    }
#undef PHYAI_BIG_ARGS
}

template <int TM, int TN, int DEPTH, int WGM = 2, int WGN = 2, int WMODE = 0>
static int big_launch_epi(const BigArgs& a, const GemmProblem& g, int splits, hipStream_t st) {
    switch (g.epilogue) {
    case EPI_NONE: big_launch<TM, TN, DEPTH, EPI_NONE, WGM, WGN, WMODE>(a, g, splits, st); return 0;
    case EPI_GEGLU_TANH: big_launch<TM, TN, DEPTH, EPI_GEGLU_TANH, WGM, WGN, WMODE>(a, g, splits, st); return 0;
    case EPI_GEGLU_ERF: big_launch<TM, TN, DEPTH, EPI_GEGLU_ERF, WGM, WGN, WMODE>(a, g, splits, st); return 0;
    case EPI_SWIGLU: big_launch<TM, TN, DEPTH, EPI_SWIGLU, WGM, WGN, WMODE>(a, g, splits, st); return 0;
    case EPI_GELU_TANH: big_launch<TM, TN, DEPTH, EPI_GELU_TANH, WGM, WGN, WMODE>(a, g, splits, st); return 0;
    case EPI_GELU_ERF: big_launch<TM, TN, DEPTH, EPI_GELU_ERF, WGM, WGN, WMODE>(a, g, splits, st); return 0;
    default: return -2;
    }
}

// (tiles with one column block per wavefront cannot hold a gate / up pair: plain epilogues only)
template <int TM, int TN, int DEPTH, int WGM = 2, int WGN = 2, int WMODE = 0>
static int big_launch_plain(const BigArgs& a, const GemmProblem& g, int splits, hipStream_t st) {
    switch (g.epilogue) {
    case EPI_NONE: big_launch<TM, TN, DEPTH, EPI_NONE, WGM, WGN, WMODE>(a, g, splits, st); return 0;
    case EPI_GELU_TANH: big_launch<TM, TN, DEPTH, EPI_GELU_TANH, WGM, WGN, WMODE>(a, g, splits, st); return 0;
    case EPI_GELU_ERF: big_launch<TM, TN, DEPTH, EPI_GELU_ERF, WGM, WGN, WMODE>(a, g, splits, st); return 0;
    default: return -2;
    }
}

// The same tile shape for row-major weights (or operand order gathered row by row) and for weights staged in
// operand order as they lie.
template <int TM, int TN, int DEPTH, int WGM = 2, int WGN = 2>
static int big_launch_layout(const BigArgs& a, const GemmProblem& g, int splits, hipStream_t st) {
    if (a.operand_w && !tuning_env("PHYAI_FP8_BIG_GATHER")) return big_launch_epi<TM, TN, DEPTH, WGM, WGN, 1>(a, g, splits, st);
    return big_launch_epi<TM, TN, DEPTH, WGM, WGN, 0>(a, g, splits, st);
}

int launch_set_stamp_sink_big(unsigned long long* buf, unsigned int records) {
#ifdef PHYAI_FP8_STAMPS
    const StampSink s = {buf, records};
    return hipMemcpyToSymbol(HIP_SYMBOL(g_big_stamps), &s, sizeof(s)) == hipSuccess ? 0 : -4;
#else
    (void)buf; (void)records;
    return -2;
#endif
}

int launch_gemm_big(const GemmProblem& g, const BigPlan& pl, hipStream_t st) {
    // the epilogue writes 16 bytes per lane (the caller chooses this kernel only for such outputs)
    if (g.ldo % 8 != 0 || (reinterpret_cast<uintptr_t>(g.out) & 15) != 0) return -2;
    BigArgs a;
    a.a = g.xq; a.b = g.w; a.a_scale = g.x_scale; a.b_scale = g.w_scale; a.bias = g.bias;
    a.out = g.out; a.ldo = g.ldo; a.M = g.M; a.N = g.N; a.K = g.K;
    a.a_scale_scalar = g.x_scale_is_scalar;
    a.res = residual_of(g);
    a.operand_w = g.weight_layout != W_ROW_MAJOR;
    a.k_per_split = g.K / pl.splits;
    a.counters = static_cast<int*>(g.workspace);
    a.partials = g.workspace ? reinterpret_cast<float*>(static_cast<uint8_t*>(g.workspace) + kGemmHeaderBytes) : nullptr;
    if (pl.splits > 1 && (g.workspace == nullptr ||
                          g.workspace_bytes < kGemmHeaderBytes + big_partial_bytes(g.M, g.N, g.epilogue, pl)))
        return -3;
    if (pl.tile == 256) return pl.splits == 1 ? big_launch_layout<4, 4, 2>(a, g, 1, st) : -2;
    if (pl.regs != 0 && !a.operand_w) return -2;
    if (pl.tile == 224) {
        if (pl.splits != 1) return -2;
        if (pl.regs == 4) return big_launch_epi<7, 2, 4, 1, 4, 2>(a, g, 1, st);
        return big_launch_layout<7, 2, 2, 1, 4>(a, g, 1, st);
    }
    if (pl.tile == 192 && pl.splits == 1) return big_launch_layout<3, 2, 2>(a, g, 1, st);
    if (pl.tile == 96) {   // 96 rows x 128 columns: wavefronts 1 x 4, three row blocks each; plain epilogues
        if (pl.splits != 1) return -2;
        return a.operand_w ? big_launch_plain<3, 1, 4, 1, 4, 1>(a, g, 1, st) : big_launch_plain<3, 1, 4, 1, 4, 0>(a, g, 1, st);
    }
    if (pl.tile == 128 && pl.cols == 64) {
        if (pl.splits != 1) return -2;
        return a.operand_w ? big_launch_plain<2, 1, 4, 2, 2, 1>(a, g, 1, st) : big_launch_plain<2, 1, 4, 2, 2, 0>(a, g, 1, st);
    }
    if (pl.tile == 128 && pl.depth == 4 && pl.regs == 8) return big_launch_plain<4, 1, 8, 1, 4, 2>(a, g, pl.splits, st);
    if (pl.tile == 128 && pl.depth == 2 && pl.regs == 4 && pl.splits == 1) return big_launch_plain<4, 1, 4, 1, 4, 2>(a, g, 1, st);
    if (pl.tile == 128 && pl.depth == 4) return big_launch_layout<2, 2, 4>(a, g, pl.splits, st);
    if (pl.tile == 128 && pl.splits == 1) return big_launch_layout<2, 2, 2>(a, g, 1, st);
    return -2;
}

}  // namespace phyai
