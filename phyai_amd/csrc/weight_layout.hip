// Re-lays a row-major fp8 weight matrix into MFMA operand order (weight_layout.h), once per layer
// after loading.  One thread moves one 16-byte chunk; consecutive threads write consecutive chunks
// of the destination, so the writes are contiguous and the reads are 16-byte pieces of 16
// neighbouring rows.
#include <hip/hip_runtime.h>

#include "launch.h"
#include "weight_layout.h"

namespace phyai {

__global__ __launch_bounds__(256) void weight_to_operand_order_kernel(const uint4* __restrict__ w, uint4* __restrict__ out,
                                                                      uint32_t N, uint32_t K, int gated, uint64_t chunks) {
    const uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x;   // destination chunk
    if (i >= chunks) return;
    const uint32_t steps = K >> 7;
    const uint32_t r = (uint32_t)(i & 15), c = (uint32_t)((i >> 4) & 7);
    const uint64_t us = i >> 7;                                     // u * steps + s
    const uint32_t u = (uint32_t)(us / steps), s = (uint32_t)(us % steps);
    uint32_t row;
    if (gated) row = ((r >> 1) & 1) * (N >> 1) + 8 * u + 2 * (r >> 2) + (r & 1);
    else row = 16 * u + r;
    out[i] = w[((uint64_t)row * K + ((uint64_t)s << 7) + (c << 4)) >> 4];
}

int launch_weight_to_operand_order(const void* w, int64_t N, int64_t K, int gated, void* out, hipStream_t st) {
    const uint64_t chunks = (uint64_t)N * (uint64_t)K / 16;
    const uint64_t blocks = (chunks + 255) / 256;
    if (blocks > 0x7FFFFFFFull) return -2;
    hipLaunchKernelGGL(weight_to_operand_order_kernel, dim3((unsigned)blocks), dim3(256), 0, st,
                       static_cast<const uint4*>(w), static_cast<uint4*>(out), (uint32_t)N, (uint32_t)K, gated, chunks);
    return 0;
}

}  // namespace phyai
