// Device-side helpers shared by the gfx950 fp8 kernels: bf16 <-> fp32, the
// e4m3fn encoder, wavefront reductions and the epilogue activations.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace phyai {

constexpr int kWave = 64;          // CDNA wavefront width
constexpr float kFp8Max = 448.0f;  // largest finite e4m3fn
constexpr uint32_t kAmaxFloorBf16 = 0x2B8D;  // bf16(1e-12): clamp_min floor of the row absmax

typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t h) { return __uint_as_float(h << 16); }

// fp32 -> bf16 bits, round to nearest even, NaN -> 0x7FC0.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float f) {
    uint32_t u = __float_as_uint(f);
    uint32_t r = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
    return (f != f) ? 0x7FC0u : r;
}

// Two fp32 -> two bf16 (round to nearest even) packed as lo | hi << 16, one v_cvt_pk_bf16_f32.
typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    const f32x2_t v = {lo, hi};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

// Two fp32 -> two e4m3fn codes (OCP, round to nearest even) in the low 16 bits.
// The hardware convert is used for the in-range part; values at or beyond 480
// and NaN take the NaN code with the input's sign, which is what a software
// RNE cast without saturation gives.
__device__ __forceinline__ uint32_t e4m3_pack2(float a, float b) {
    uint32_t w = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a, b, 0, false);
    uint32_t ua = __float_as_uint(a), ub = __float_as_uint(b);
    if ((ua & 0x7FFFFFFFu) >= 0x43F00000u) w = (w & 0xFF00u) | ((ua >> 24) & 0x80u) | 0x7Fu;
    if ((ub & 0x7FFFFFFFu) >= 0x43F00000u) w = (w & 0x00FFu) | ((((ub >> 24) & 0x80u) | 0x7Fu) << 8);
    return w & 0xFFFFu;
}

// Cross-lane data movement inside a row of 16 lanes (DPP: a modifier of the VALU instruction
// itself, a few cycles) instead of a trip through the LDS crossbar (ds_bpermute: ~100 cycles each,
// six of them in a row for a 64-lane butterfly).  CTRL: 0xB1 = quad_perm [1,0,3,2], 0x4E =
// quad_perm [2,3,0,1], 0x141 = row_half_mirror, 0x140 = row_mirror; every lane has a source.
template <int CTRL>
__device__ __forceinline__ uint32_t dpp_move_u32(uint32_t v) {
    return (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, CTRL, 0xF, 0xF, true);
}

// Maximum over the wavefront, the same value in every lane: four DPP steps leave each row of 16
// lanes with its maximum, the four rows meet through scalar registers.
__device__ __forceinline__ uint32_t wave_max_u32(uint32_t v) {
    uint32_t o;
    o = dpp_move_u32<0xB1>(v);  v = o > v ? o : v;
    o = dpp_move_u32<0x4E>(v);  v = o > v ? o : v;
    o = dpp_move_u32<0x141>(v); v = o > v ? o : v;
    o = dpp_move_u32<0x140>(v); v = o > v ? o : v;
    const uint32_t r0 = (uint32_t)__builtin_amdgcn_readlane((int)v, 0), r1 = (uint32_t)__builtin_amdgcn_readlane((int)v, 16);
    const uint32_t r2 = (uint32_t)__builtin_amdgcn_readlane((int)v, 32), r3 = (uint32_t)__builtin_amdgcn_readlane((int)v, 48);
    const uint32_t a = r0 > r1 ? r0 : r1, b = r2 > r3 ? r2 : r3;
    return a > b ? a : b;
}

// Sum over the wavefront, the same value in every lane, in a fixed order (pairs, quads, halves of
// a row, rows of 16, then the four rows): reproducible from run to run.
__device__ __forceinline__ float wave_sum_f32(float v) {
    v += __uint_as_float(dpp_move_u32<0xB1>(__float_as_uint(v)));
    v += __uint_as_float(dpp_move_u32<0x4E>(__float_as_uint(v)));
    v += __uint_as_float(dpp_move_u32<0x141>(__float_as_uint(v)));
    v += __uint_as_float(dpp_move_u32<0x140>(__float_as_uint(v)));
    const float r0 = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 0));
    const float r1 = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 16));
    const float r2 = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 32));
    const float r3 = __uint_as_float((uint32_t)__builtin_amdgcn_readlane((int)__float_as_uint(v), 48));
    return (r0 + r1) + (r2 + r3);
}

// One 16-byte chunk per lane from global memory straight into LDS: lane i's chunk lands at
// lds_wave_base + 16*i.  Issued as inline assembly so that the compiler does not order its own
// LDS reads behind copies that are still in flight; the waits are placed by hand below.
__device__ __forceinline__ void copy16_to_lds(const uint8_t* base, uint32_t lane_offset, uint32_t lds_wave_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                 :: "v"(lane_offset), "s"(base), "s"(lds_wave_base) : "memory", "m0");
}

// The same copy for data that should not stay in the caches behind it (read once per pass over a
// working set that is larger than they are).
__device__ __forceinline__ void copy16_to_lds_nt(const uint8_t* base, uint32_t lane_offset, uint32_t lds_wave_base) {
    asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1 nt"
                 :: "v"(lane_offset), "s"(base), "s"(lds_wave_base) : "memory", "m0");
}

// s_waitcnt vmcnt(N) with a compile-time N: at most N of this wavefront's copies still in flight.
template <int N>
__device__ __forceinline__ void wait_copies() {
    static_assert(N >= 0 && N < 64, "vmcnt is a 6-bit counter");
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N) : "memory");
}

// ---- epilogue activations (fp32 math) ------------------------------------
// gelu_tanh(v) = 0.5 v (1 + tanh u), u = k0 (v + k1 v^3).  With tanh u = 1 - 2 / (exp(2u) + 1) this
// is v - v / (exp(2u) + 1): exact limits (v and 0) when the exponential overflows or underflows,
// no cancellation, and seven instructions: 2u log2(e) = v (a + b v^2) feeds v_exp_f32 directly.
__device__ __forceinline__ float gelu_tanh_f(float v) {
    constexpr float a = 2.0f * 0.7978845608028654f * 1.4426950408889634f;
    constexpr float b = a * 0.044715f;
    const float e = __builtin_amdgcn_exp2f(v * __builtin_fmaf(b, v * v, a));
    return __builtin_fmaf(-v, __builtin_amdgcn_rcpf(e + 1.0f), v);
}
// gelu(v) = 0.5 v (1 + erf(v / sqrt 2)) without branches.  For x >= 0, erfc(x) = t P(t) exp(-x^2)
// with t = 1 / (1 + 0.4 x) and P a degree-8 polynomial fitted to erfc(x) exp(x^2) with relative
// error 1.2e-7 on [0, 30] (the form of Abramowitz & Stegun 7.1.26, more terms).  1 + erf(v / sqrt 2)
// is erfc(|x|) for v < 0 - no cancellation in the negative tail - and 2 - erfc(x) otherwise.
// Relative error of the result below 1e-5, so it rounds to the same bf16 as the exact value
// except for about one input in 10^4.
__device__ __forceinline__ float gelu_erf_f(float v) {
    const float av = __builtin_fabsf(v);
    const float t = __builtin_amdgcn_rcpf(__builtin_fmaf(0.4f * 0.70710678118654752f, av, 1.0f));
    float q = __builtin_fmaf(t, 0.04973088949918747f, -0.18051011860370636f);
    q = __builtin_fmaf(t, q, 0.16458380222320557f);
    q = __builtin_fmaf(t, q, -0.0010123166721314192f);
    q = __builtin_fmaf(t, q, 0.13867421448230743f);
    q = __builtin_fmaf(t, q, 0.169526606798172f);
    q = __builtin_fmaf(t, q, 0.20764122903347015f);
    q = __builtin_fmaf(t, q, 0.2256908118724823f);
    q = __builtin_fmaf(t, q, 0.22567500174045563f);
    const float e = __builtin_amdgcn_exp2f((v * v) * (-0.5f * 1.4426950408889634f));
    const float erfc_abs = (q * t) * e;
    const float one_plus_erf = v < 0.0f ? erfc_abs : 2.0f - erfc_abs;
    return (0.5f * v) * one_plus_erf;
}
__device__ __forceinline__ float silu_f(float v) { return v * __builtin_amdgcn_rcpf(1.0f + __expf(-v)); }

enum Epilogue : int {
    EPI_NONE = 0,
    EPI_GEGLU_TANH = 1,
    EPI_GEGLU_ERF = 2,
    EPI_SWIGLU = 3,
    EPI_GELU_TANH = 4,
    EPI_GELU_ERF = 5,
};
__host__ __device__ constexpr bool epi_is_gated(int e) { return e >= EPI_GEGLU_TANH && e <= EPI_SWIGLU; }

template <int EPI>
__device__ __forceinline__ float apply_act(float v) {
    if constexpr (EPI == EPI_GEGLU_TANH || EPI == EPI_GELU_TANH) return gelu_tanh_f(v);
    else if constexpr (EPI == EPI_GEGLU_ERF || EPI == EPI_GELU_ERF) return gelu_erf_f(v);
    else if constexpr (EPI == EPI_SWIGLU) return silu_f(v);
    else return v;
}

// Round an fp32 value through bf16 (the reference materialises the GEMM output
// as a bf16 tensor before the activation kernel reads it).  The hardware convert rounds to nearest
// even like f32_to_bf16_bits; the two differ only in the bits of a NaN (the convert keeps sign and
// payload, the software form returns 0x7FC0).  All GEMM epilogues use the convert.
__device__ __forceinline__ float round_bf16(float v) { return __uint_as_float(pack_bf16x2(v, 0.0f) << 16); }
// Two values at once: three instructions instead of four.
__device__ __forceinline__ void round_bf16_pair(float& a, float& b) {
    const uint32_t p = pack_bf16x2(a, b);
    a = __uint_as_float(p << 16);
    b = __uint_as_float(p & 0xFFFF0000u);
}

// residual + y * gate on four consecutive columns; y is the linear's bf16 output.  The product of
// two bf16 values is exact in fp32, so this equals torch.addcmul's single rounding whether or
// not the multiply and the add are contracted.
__device__ __forceinline__ void addcmul4(float* y, uint2 res, uint2 gate) {
    const float r[4] = {bf16_bits_to_f32(res.x & 0xFFFFu), __uint_as_float(res.x & 0xFFFF0000u),
                        bf16_bits_to_f32(res.y & 0xFFFFu), __uint_as_float(res.y & 0xFFFF0000u)};
    const float g[4] = {bf16_bits_to_f32(gate.x & 0xFFFFu), __uint_as_float(gate.x & 0xFFFF0000u),
                        bf16_bits_to_f32(gate.y & 0xFFFFu), __uint_as_float(gate.y & 0xFFFF0000u)};
#pragma unroll
    for (int e = 0; e < 4; ++e) y[e] = r[e] + round_bf16(y[e]) * g[e];
}

}  // namespace phyai
