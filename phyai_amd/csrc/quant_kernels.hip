// Activation / weight quantizers for gfx950.
//
// One workgroup per row.  Each thread keeps its slice of the row in registers
// (CHUNKS x 8 bf16 = CHUNKS 128-bit loads), so the row is read from HBM once:
// pass 1 reduces |x| to the row maximum across the wavefront (cross-lane
// shuffles) and then across wavefronts through LDS; pass 2 divides, converts to
// e4m3fn and stores 8 codes per 64-bit store.
#include "fp8_device.h"
#include "launch.h"
#include "quant_device.h"

namespace phyai {

template <int THREADS>
__device__ __forceinline__ uint32_t block_max_u32(uint32_t v, uint32_t* smem) {
    v = wave_max_u32(v);
    if constexpr (THREADS > kWave) {
        constexpr int NW = THREADS / kWave;
        const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
        if (lane == 0) smem[wave] = v;
        __syncthreads();
        uint32_t r = smem[0];
#pragma unroll
        for (int i = 1; i < NW; ++i) r = smem[i] > r ? smem[i] : r;
        v = r;
    }
    return v;
}

// A tensor that is far larger than the caches and read once is loaded without keeping its lines
// in L2 (from 100 MB, long rows only: 13056 x 16384 119.9 -> 111.9 us; at 6528 x 2048 it would
// cost 10 %).  The codes are stored normally: streaming them out as well makes this kernel
// faster (816 x 16384: 12.0 -> 9.2 us) but the GEMM that reads them next slower by more.
// Same box, alternating builds.
__device__ __forceinline__ uint4 nt_load16(const uint16_t* p) {
    const v4i v = __builtin_nontemporal_load(reinterpret_cast<const v4i*>(p));
    return make_uint4((uint32_t)v[0], (uint32_t)v[1], (uint32_t)v[2], (uint32_t)v[3]);
}

template <int THREADS, int CHUNKS, int MODE, bool STREAM_IN>
__global__ __launch_bounds__(THREADS) void quant_rows_reg_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, int K, uint8_t* __restrict__ xq,
    float* __restrict__ scale) {
    __shared__ uint32_t smem[THREADS / kWave];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = x + row * ldx;
    uint4 v[CHUNKS];
    uint32_t m = 0;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int k = (c * THREADS + threadIdx.x) * 8;
        v[c] = make_uint4(0, 0, 0, 0);
        if (k < K) v[c] = STREAM_IN ? nt_load16(xr + k) : *reinterpret_cast<const uint4*>(xr + k);
        m = absmax8(v[c], m);
    }
    m = block_max_u32<THREADS>(m, smem);
    const float s = scale_from_amax_bits<MODE>(m);
    if (threadIdx.x == 0) scale[row] = s;
    const RowDivisor d = make_divisor(s);
    uint8_t* qr = xq + row * (int64_t)K;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int k = (c * THREADS + threadIdx.x) * 8;
        if (k < K) *reinterpret_cast<uint2*>(qr + k) = encode8<MODE>(v[c], d);
    }
}

// Rows too long for the register-resident form: two passes over global memory
// (the second one hits L2).
template <int MODE>
__global__ __launch_bounds__(256) void quant_rows_loop_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, int K, uint8_t* __restrict__ xq,
    float* __restrict__ scale) {
    __shared__ uint32_t smem[256 / kWave];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = x + row * ldx;
    uint32_t m = 0;
    for (int k = threadIdx.x * 8; k < K; k += 256 * 8)
        m = absmax8(*reinterpret_cast<const uint4*>(xr + k), m);
    m = block_max_u32<256>(m, smem);
    const float s = scale_from_amax_bits<MODE>(m);
    if (threadIdx.x == 0) scale[row] = s;
    const RowDivisor d = make_divisor(s);
    uint8_t* qr = xq + row * (int64_t)K;
    for (int k = threadIdx.x * 8; k < K; k += 256 * 8)
        *reinterpret_cast<uint2*>(qr + k) = encode8<MODE>(*reinterpret_cast<const uint4*>(xr + k), d);
}

// Static per-tensor quantizer: clamp(fp32(x)/s, +-448) -> e4m3fn.  torch.clamp
// lets NaN through, and so do fminf/fmaxf here only if ordered the other way,
// hence the explicit NaN test.
__global__ __launch_bounds__(256) void quant_static_kernel(
    const uint16_t* __restrict__ x, int64_t ldx, int64_t M, int K,
    const float* __restrict__ input_scale, uint8_t* __restrict__ xq) {
    const float s = *input_scale;
    const int64_t chunks_per_row = K / 8;
    const int64_t total = M * chunks_per_row;
    for (int64_t i = blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int64_t row = i / chunks_per_row;
        const int k = (int)(i % chunks_per_row) * 8;
        const uint4 q = *reinterpret_cast<const uint4*>(x + row * ldx + k);
        const uint32_t w[4] = {q.x, q.y, q.z, q.w};
        uint32_t c[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float a = bf16_bits_to_f32(w[j] & 0xFFFFu) / s;
            float b = bf16_bits_to_f32(w[j] >> 16) / s;
            a = (a != a) ? a : fminf(fmaxf(a, -kFp8Max), kFp8Max);
            b = (b != b) ? b : fminf(fmaxf(b, -kFp8Max), kFp8Max);
            c[j] = e4m3_pack2(a, b);
        }
        *reinterpret_cast<uint2*>(xq + row * (int64_t)K + k) =
            make_uint2(c[0] | (c[1] << 16), c[2] | (c[3] << 16));
    }
}

__global__ __launch_bounds__(256) void debug_cast_kernel(const float* __restrict__ v, int64_t n,
                                                         uint8_t* __restrict__ codes) {
    for (int64_t i = blockIdx.x * 256 + threadIdx.x; i < n; i += (int64_t)gridDim.x * 256)
        codes[i] = (uint8_t)(e4m3_pack2(v[i], 0.0f) & 0xFFu);
}

template <int MODE>
static int launch_quant_rows(const void* x, int64_t M, int64_t K, int64_t ld, void* xq,
                             float* scale, hipStream_t st) {
    if (M == 0) return 0;
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    uint8_t* qp = static_cast<uint8_t*>(xq);
    const dim3 grid((unsigned)M);
    const int k = (int)K;
    const bool stream_in = M * K * 2 >= ((int64_t)100 << 20);   // only long rows get that large in practice
#define PHYAI_QL(T, C)                                                                                             \
    do {                                                                                                           \
        if (C >= 4 && stream_in)                                                                                   \
            hipLaunchKernelGGL((quant_rows_reg_kernel<T, C, MODE, (C >= 4)>), grid, dim3(T), 0, st, xp, ld, k, qp, scale); \
        else                                                                                                       \
            hipLaunchKernelGGL((quant_rows_reg_kernel<T, C, MODE, false>), grid, dim3(T), 0, st, xp, ld, k, qp, scale);   \
    } while (0)
    if (K <= 512) PHYAI_QL(64, 1);
    else if (K <= 1024) PHYAI_QL(128, 1);
    else if (K <= 2048) PHYAI_QL(256, 1);
    else if (K <= 4096) PHYAI_QL(256, 2);
    else if (K <= 8192) PHYAI_QL(256, 4);
    else if (K <= 16384) PHYAI_QL(256, 8);
    else if (K <= 32768) PHYAI_QL(256, 16);
    else hipLaunchKernelGGL((quant_rows_loop_kernel<MODE>), grid, dim3(256), 0, st, xp, ld, k, qp, scale);
#undef PHYAI_QL
    return 0;
}

int launch_quant_rowwise(const void* x, int64_t M, int64_t K, int64_t ldx, void* xq, float* xs,
                         hipStream_t st) {
    return launch_quant_rows<QUANT_ACT_DYNAMIC>(x, M, K, ldx, xq, xs, st);
}
int launch_weight_quant(const void* w, int64_t N, int64_t K, int64_t ldw, void* wq, float* ws,
                        hipStream_t st) {
    return launch_quant_rows<QUANT_WEIGHT>(w, N, K, ldw, wq, ws, st);
}
// ---- RMSNorm / adaptive RMSNorm + quantizer ----------------------------------------------
template <int THREADS>
__device__ __forceinline__ float block_sum_f32(float v, float* smem) {
    v = wave_sum_f32(v);
    if constexpr (THREADS > kWave) {
        constexpr int NW = THREADS / kWave;
        const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
        if (lane == 0) smem[wave] = v;
        __syncthreads();
        float r = smem[0];
#pragma unroll
        for (int i = 1; i < NW; ++i) r += smem[i];
        v = r;
    }
    return v;
}

__device__ __forceinline__ void unpack8(uint4 q, float* f) {
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        f[2 * i] = bf16_bits_to_f32(w[i] & 0xFFFFu);
        f[2 * i + 1] = __uint_as_float(w[i] & 0xFFFF0000u);
    }
}

// One workgroup per row, the row in registers: sum of squares (fp32), normalise, affine, round to
// bf16 - the tensor the reference's norm kernel would have written - and, on those bf16 values,
// the per-token quantizer (row absmax, scale, codes) of quant_rows_reg_kernel.
template <int THREADS, int CHUNKS, bool ADAPTIVE>
__global__ __launch_bounds__(THREADS) void norm_quant_kernel(
    const uint16_t* __restrict__ a_x, int64_t a_ldx, int a_D, int a_group, const uint16_t* __restrict__ a_mod,
    int64_t a_ld_mod, const uint16_t* __restrict__ a_weight, float a_eps, int a_gemma, uint8_t* __restrict__ a_xq,
    float* __restrict__ a_scale, uint16_t* __restrict__ a_out, int64_t a_ldo, uint16_t* __restrict__ a_gate,
    int64_t a_ld_gate) {
    // scalar arguments in the order the kernel needs them (the first 16 dwords are preloaded)
    NormQuantArgs p;
    p.x = a_x; p.ldx = a_ldx; p.D = a_D; p.eps = a_eps; p.weight = a_weight; p.gemma = a_gemma; p.mod = a_mod;
    p.ld_mod = a_ld_mod; p.group = a_group; p.out = a_out; p.ldo = a_ldo; p.gate = a_gate; p.ld_gate = a_ld_gate;
    p.xq = a_xq; p.scale = a_scale;
    __shared__ float ssum[THREADS / kWave];
    __shared__ uint32_t smax[THREADS / kWave];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = p.x + row * p.ldx;
    float xf[CHUNKS][8];
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int k = (c * THREADS + threadIdx.x) * 8;
        uint4 v = make_uint4(0, 0, 0, 0);
        if (k < p.D) v = *reinterpret_cast<const uint4*>(xr + k);
        unpack8(v, xf[c]);
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += xf[c][e] * xf[c][e];
    }
    ss = block_sum_f32<THREADS>(ss, ssum);
    const float rstd = 1.0f / sqrtf(ss / (float)p.D + p.eps);

    const int64_t mrow = ADAPTIVE ? row / p.group : 0;
    const uint16_t* mr = ADAPTIVE ? p.mod + mrow * p.ld_mod : nullptr;
    uint4 ob[CHUNKS];
    uint32_t m = 0;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int k = (c * THREADS + threadIdx.x) * 8;
        ob[c] = make_uint4(0, 0, 0, 0);
        if (k < p.D) {
            float o[8];
            if constexpr (ADAPTIVE) {
                float sc[8], sh[8];
                unpack8(*reinterpret_cast<const uint4*>(mr + k), sc);
                unpack8(*reinterpret_cast<const uint4*>(mr + p.D + k), sh);
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = (xf[c][e] * rstd) * (1.0f + sc[e]) + sh[e];
                if (p.gate != nullptr && row % p.group == 0)
                    *reinterpret_cast<uint4*>(p.gate + mrow * p.ld_gate + k) =
                        *reinterpret_cast<const uint4*>(mr + 2 * p.D + k);
            } else {
                float w[8];
                unpack8(*reinterpret_cast<const uint4*>(p.weight + k), w);
#pragma unroll
                for (int e = 0; e < 8; ++e) o[e] = (xf[c][e] * rstd) * (p.gemma ? w[e] + 1.0f : w[e]);
            }
            ob[c].x = f32_to_bf16_bits(o[0]) | (f32_to_bf16_bits(o[1]) << 16);
            ob[c].y = f32_to_bf16_bits(o[2]) | (f32_to_bf16_bits(o[3]) << 16);
            ob[c].z = f32_to_bf16_bits(o[4]) | (f32_to_bf16_bits(o[5]) << 16);
            ob[c].w = f32_to_bf16_bits(o[6]) | (f32_to_bf16_bits(o[7]) << 16);
            if (p.out != nullptr) *reinterpret_cast<uint4*>(p.out + row * p.ldo + k) = ob[c];
        }
        m = absmax8(ob[c], m);
    }
    if (p.xq == nullptr) return;
    m = block_max_u32<THREADS>(m, smax);
    const float s = scale_from_amax_bits<QUANT_ACT_DYNAMIC>(m);
    if (threadIdx.x == 0) p.scale[row] = s;
    const RowDivisor d = make_divisor(s);
    uint8_t* qr = p.xq + row * (int64_t)p.D;
#pragma unroll
    for (int c = 0; c < CHUNKS; ++c) {
        const int k = (c * THREADS + threadIdx.x) * 8;
        if (k < p.D) *reinterpret_cast<uint2*>(qr + k) = encode8<QUANT_ACT_DYNAMIC>(ob[c], d);
    }
}

// Rows too long for registers (D > 8192, the reference's two-pass kernels): the row is read again
// for every pass - sum of squares, then the bf16 result and its absmax, then the codes.
template <bool ADAPTIVE>
__global__ __launch_bounds__(256) void norm_quant_loop_kernel(
    const uint16_t* __restrict__ a_x, int64_t a_ldx, int a_D, int a_group, const uint16_t* __restrict__ a_mod,
    int64_t a_ld_mod, const uint16_t* __restrict__ a_weight, float a_eps, int a_gemma, uint8_t* __restrict__ a_xq,
    float* __restrict__ a_scale, uint16_t* __restrict__ a_out, int64_t a_ldo, uint16_t* __restrict__ a_gate,
    int64_t a_ld_gate) {
    // scalar arguments in the order the kernel needs them (the first 16 dwords are preloaded)
    NormQuantArgs p;
    p.x = a_x; p.ldx = a_ldx; p.D = a_D; p.eps = a_eps; p.weight = a_weight; p.gemma = a_gemma; p.mod = a_mod;
    p.ld_mod = a_ld_mod; p.group = a_group; p.out = a_out; p.ldo = a_ldo; p.gate = a_gate; p.ld_gate = a_ld_gate;
    p.xq = a_xq; p.scale = a_scale;
    __shared__ float ssum[256 / kWave];
    __shared__ uint32_t smax[256 / kWave];
    const int64_t row = blockIdx.x;
    const uint16_t* xr = p.x + row * p.ldx;
    float ss = 0.f;
    for (int k = threadIdx.x * 8; k < p.D; k += 256 * 8) {
        float f[8];
        unpack8(*reinterpret_cast<const uint4*>(xr + k), f);
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += f[e] * f[e];
    }
    ss = block_sum_f32<256>(ss, ssum);
    const float rstd = 1.0f / sqrtf(ss / (float)p.D + p.eps);
    const int64_t mrow = ADAPTIVE ? row / p.group : 0;
    const uint16_t* mr = ADAPTIVE ? p.mod + mrow * p.ld_mod : nullptr;
    auto result8 = [&](int k) -> uint4 {
        float f[8], o[8];
        unpack8(*reinterpret_cast<const uint4*>(xr + k), f);
        if constexpr (ADAPTIVE) {
            float sc[8], sh[8];
            unpack8(*reinterpret_cast<const uint4*>(mr + k), sc);
            unpack8(*reinterpret_cast<const uint4*>(mr + p.D + k), sh);
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (f[e] * rstd) * (1.0f + sc[e]) + sh[e];
        } else {
            float w[8];
            unpack8(*reinterpret_cast<const uint4*>(p.weight + k), w);
#pragma unroll
            for (int e = 0; e < 8; ++e) o[e] = (f[e] * rstd) * (p.gemma ? w[e] + 1.0f : w[e]);
        }
        uint4 b;
        b.x = f32_to_bf16_bits(o[0]) | (f32_to_bf16_bits(o[1]) << 16);
        b.y = f32_to_bf16_bits(o[2]) | (f32_to_bf16_bits(o[3]) << 16);
        b.z = f32_to_bf16_bits(o[4]) | (f32_to_bf16_bits(o[5]) << 16);
        b.w = f32_to_bf16_bits(o[6]) | (f32_to_bf16_bits(o[7]) << 16);
        return b;
    };
    uint32_t m = 0;
    for (int k = threadIdx.x * 8; k < p.D; k += 256 * 8) {
        const uint4 b = result8(k);
        if (p.out != nullptr) *reinterpret_cast<uint4*>(p.out + row * p.ldo + k) = b;
        if constexpr (ADAPTIVE) {
            if (p.gate != nullptr && row % p.group == 0)
                *reinterpret_cast<uint4*>(p.gate + mrow * p.ld_gate + k) = *reinterpret_cast<const uint4*>(mr + 2 * p.D + k);
        }
        m = absmax8(b, m);
    }
    if (p.xq == nullptr) return;
    m = block_max_u32<256>(m, smax);
    const float s = scale_from_amax_bits<QUANT_ACT_DYNAMIC>(m);
    if (threadIdx.x == 0) p.scale[row] = s;
    const RowDivisor d = make_divisor(s);
    uint8_t* qr = p.xq + row * (int64_t)p.D;
    for (int k = threadIdx.x * 8; k < p.D; k += 256 * 8)
        *reinterpret_cast<uint2*>(qr + k) = encode8<QUANT_ACT_DYNAMIC>(result8(k), d);
}

template <bool ADAPTIVE>
static int launch_norm_quant_t(const NormQuantArgs& a, int64_t M, hipStream_t st) {
    const dim3 grid((unsigned)M);
#define PHYAI_NQ_ARGS a.x, a.ldx, a.D, a.group, a.mod, a.ld_mod, a.weight, a.eps, a.gemma, a.xq, a.scale, a.out, a.ldo, a.gate, a.ld_gate
#define PHYAI_NQ(T, C) hipLaunchKernelGGL((norm_quant_kernel<T, C, ADAPTIVE>), grid, dim3(T), 0, st, PHYAI_NQ_ARGS)
    if (a.D <= 512) PHYAI_NQ(64, 1);
    else if (a.D <= 1024) PHYAI_NQ(128, 1);
    else if (a.D <= 2048) PHYAI_NQ(256, 1);
    else if (a.D <= 4096) PHYAI_NQ(256, 2);
    else if (a.D <= 8192) PHYAI_NQ(256, 4);
    else hipLaunchKernelGGL((norm_quant_loop_kernel<ADAPTIVE>), grid, dim3(256), 0, st, PHYAI_NQ_ARGS);
#undef PHYAI_NQ
#undef PHYAI_NQ_ARGS
    return 0;
}

int launch_norm_quant(const NormQuantArgs& a, int64_t M, bool adaptive, hipStream_t st) {
    if (M == 0) return 0;
    return adaptive ? launch_norm_quant_t<true>(a, M, st) : launch_norm_quant_t<false>(a, M, st);
}

int launch_quant_static(const void* x, int64_t M, int64_t K, int64_t ldx, const float* input_scale,
                        void* xq, hipStream_t st) {
    if (M == 0) return 0;
    int64_t total = M * (K / 8);
    int blocks = (int)((total + 255) / 256);
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(quant_static_kernel, dim3(blocks), dim3(256), 0, st,
                       static_cast<const uint16_t*>(x), ldx, M, (int)K, input_scale,
                       static_cast<uint8_t*>(xq));
    return 0;
}
int launch_debug_cast(const float* v, int64_t n, void* codes, hipStream_t st) {
    if (n == 0) return 0;
    int blocks = (int)((n + 255) / 256);
    if (blocks > 8192) blocks = 8192;
    hipLaunchKernelGGL(debug_cast_kernel, dim3(blocks), dim3(256), 0, st, v, n,
                       static_cast<uint8_t*>(codes));
    return 0;
}

}  // namespace phyai
