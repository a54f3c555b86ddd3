// Weight layouts the GEMM kernels read.
//
// ROW_MAJOR is what a checkpoint holds and what Fp8Spec.allocate registers: w[N, K], K contiguous.
// An MFMA lane wants 16 bytes of K of ONE weight row, and the lanes of a wavefront want the same
// 16 bytes of 16 (or 32) neighbouring rows: in row-major order those are K bytes apart, so a
// global -> VGPR load gives every row its own request, and the kernels stage weights through LDS.
//
// OPERAND order stores them the way the lanes ask for them.  The matrix is cut into units of 16
// rows x 128 bytes of K (one operand block of v_mfma_f32_16x16x128_f8f6f4, half a block of
// v_mfma_f32_32x32x64_f8f6f4 along the rows), K steps of a unit contiguous:
//     unit (u, s)      at  (u * K / 128 + s) * 2048
//     inside a unit    the 16-byte chunk c (0 .. 7) of row r (0 .. 15)  at  (c * 16 + r) * 16
// i.e. the 16 x 8 matrix of chunks transposed: sixteen lanes that read chunk c of rows 0 .. 15 read
// 256 contiguous bytes, and the whole unit is 2 KB in a row.
//
// Which weight row is row r of unit u:
//     OPERAND_PLAIN    16 u + r
//     OPERAND_GATED    for a fused gate | up matrix (gate = rows [0, N/2), up = rows [N/2, N)): unit u
//                      holds gate columns 8 u .. 8 u + 7 and the up columns that pair with them, in
//                      fours: r = 4 p + 2 t + b  ->  row t * N/2 + 8 u + 2 p + b.  An MFMA lane owns four
//                      consecutive operand rows, so it ends up with gate and up of two output columns.
// The gated order is the one the small-M kernels gather from a row-major matrix anyway; a matrix in
// OPERAND_GATED order can only be used with a gated epilogue and one in OPERAND_PLAIN order only
// without.  K must be a multiple of 128 and N of 16 (32 when gated).
#pragma once

#include <stdint.h>

namespace phyai {

enum WeightLayout : int { W_ROW_MAJOR = 0, W_OPERAND_PLAIN = 1, W_OPERAND_GATED = 2 };

// Byte offset of unit row (u, r), K step 0, chunk 0; add s * 2048 per K step and c * 256 per chunk.
__host__ __device__ __forceinline__ uint32_t operand_row_offset(uint32_t u, uint32_t r, uint32_t K) {
    return u * (K << 4) + (r << 4);
}
constexpr uint32_t kOperandStepBytes = 2048;   // one K step (128 bytes of K) of a unit
constexpr uint32_t kOperandChunkBytes = 256;   // one 16-byte chunk of K for the 16 rows of a unit

// (unit, row in unit) of weight row n of a plain matrix, of gate (t = 0) / up (t = 1) column g of a gated one.
__host__ __device__ __forceinline__ uint32_t operand_offset_plain(uint32_t n, uint32_t K) {
    return operand_row_offset(n >> 4, n & 15, K);
}
__host__ __device__ __forceinline__ uint32_t operand_offset_gated(uint32_t g, uint32_t t, uint32_t K) {
    return operand_row_offset(g >> 3, 4 * ((g & 7) >> 1) + 2 * t + (g & 1), K);
}

}  // namespace phyai
