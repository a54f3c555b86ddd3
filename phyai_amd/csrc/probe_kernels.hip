// Hardware probe: the rate at which the chip issues fp8 MFMAs when every CU does nothing else, and
// the shader clock it holds while doing so.  The vendor's dense fp8 figure assumes the peak engine
// clock; under a chip-wide MFMA load the clock settles lower, and that - not the data sheet - is
// the ceiling the tile kernels can be held to.
#include "fp8_device.h"
#include "launch.h"

namespace phyai {

// Four wavefronts per workgroup, 16 independent accumulators each (256 AGPRs, the register budget of
// the 256 x 256 tile kernel): `iters` rounds of 16 v_mfma_f32_32x32x64_f8f6f4, no memory traffic.
// Wavefront 0 of every workgroup records shader cycles (s_memtime) and 100 MHz ticks (s_memrealtime)
// over its loop: out[2 * workgroup] = cycles, out[2 * workgroup + 1] = ticks.
__global__ __launch_bounds__(256) void mfma_rate_kernel(int iters, unsigned long long* __restrict__ out, float* __restrict__ sink) {
    v16f acc[16];
#pragma unroll
    for (int i = 0; i < 16; ++i)
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;
    v8i a, b;
#pragma unroll
    for (int r = 0; r < 8; ++r) { a[r] = 0x38383838 + (int)threadIdx.x; b[r] = 0x30303030 + r; }
    const unsigned long long c0 = __builtin_readcyclecounter(), t0 = __builtin_amdgcn_s_memrealtime();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 16; ++i)
            acc[i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a, b, acc[i], 0, 0, 0, 0, 0, 0);
    }
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) s += acc[i][0];
    const unsigned long long c1 = __builtin_readcyclecounter(), t1 = __builtin_amdgcn_s_memrealtime();
    if (threadIdx.x == 0) {
        out[2 * blockIdx.x] = c1 - c0;
        out[2 * blockIdx.x + 1] = t1 - t0;
    }
    if (s == 12345.678f) sink[0] = s;   // keeps the MFMAs alive; never true for these operands
}

int launch_mfma_rate(int workgroups, int iters, unsigned long long* out, float* sink, hipStream_t st) {
    hipLaunchKernelGGL(mfma_rate_kernel, dim3(workgroups), dim3(256), 0, st, iters, out, sink);
    return 0;
}

}  // namespace phyai
