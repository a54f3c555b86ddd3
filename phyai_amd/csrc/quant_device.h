// Arithmetic of the row-wise activation / weight quantizers, shared by the stand-alone quantizer
// kernels and by the small-M GEMM that quantizes its own activation rows.
#pragma once

#include "fp8_device.h"

namespace phyai {

enum QuantMode : int {
    QUANT_ACT_DYNAMIC = 0,  // bf16 amax floored at bf16(1e-12); scale = fp32(bf16(amax/448)); no clamp
    QUANT_WEIGHT = 1,       // fp32 amax/448 floored at FLT_MIN; clamp to +-448
};

// Running maximum of |bf16| bit patterns, two per register (v_pk_max_u16): m2 holds the maxima of the
// even and of the odd elements seen so far; absmax_finish folds the two.
typedef unsigned short u16x2_t __attribute__((ext_vector_type(2)));
__device__ __forceinline__ uint32_t absmax8_pk(uint4 q, uint32_t m2) {
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const u16x2_t a = __builtin_bit_cast(u16x2_t, w[i] & 0x7FFF7FFFu), b = __builtin_bit_cast(u16x2_t, m2);
        m2 = __builtin_bit_cast(uint32_t, __builtin_elementwise_max(a, b));
    }
    return m2;
}
__device__ __forceinline__ uint32_t absmax_finish(uint32_t m2) {
    const uint32_t lo = m2 & 0xFFFFu, hi = m2 >> 16;
    return lo > hi ? lo : hi;
}
__device__ __forceinline__ uint32_t absmax8(uint4 q, uint32_t m) {
    const uint32_t r = absmax_finish(absmax8_pk(q, 0u));
    return r > m ? r : m;
}

// Divisor of one row.  The reference divides every element by the row scale with an IEEE fp32
// division and rounds the quotient to e4m3.  Both operands are bf16 values (8 significant bits), so
// the true quotient x / s is either exactly on an e4m3 rounding boundary - then it has at most 5
// significant bits - or at least 2^-13 (relative) away from every boundary.  Hence the same codes
// come from two instructions per element:
//     q = trunc16( x * r ),   r = rcp(s) * (1 + 2^-19),
// where rcp is the hardware reciprocal (1 ulp) and trunc16 clears the low 7 mantissa bits.  The
// product lies above the true quotient by a relative 2^-19 (+- 2^-21 for the rounding errors), so
// truncation returns a boundary value exactly and moves any other value by less than 2^-15, which
// cannot cross a boundary; signs of zeros survive both steps.  Checked on the CPU over every pair
// of mantissas and exponent distance with the reciprocal off by up to +-2 ulp, and exhaustively on
// the device over every finite bf16 value against every possible scale.  Rows with a non-finite
// scale (an Inf or NaN in the row) take the true division.
struct RowDivisor {
    float s, r;
    bool fast;
};
__device__ __forceinline__ float biased_reciprocal(float s) {
    return __builtin_amdgcn_rcpf(s) * 1.0000019073486328125f;   // 1 + 2^-19
}
__device__ __forceinline__ RowDivisor make_divisor(float s) {
    RowDivisor d;
    d.s = s;
    d.fast = (__float_as_uint(s) & 0x7FFFFFFFu) < 0x7F800000u;
    d.r = biased_reciprocal(s);
    return d;
}
__device__ __forceinline__ float div_exact(float x, const RowDivisor& d) {
    return __uint_as_float(__float_as_uint(x * d.r) & 0xFFFFFF80u);
}

template <int MODE>
__device__ __forceinline__ uint2 encode8(uint4 q, const RowDivisor& d) {
    const uint32_t w[4] = {q.x, q.y, q.z, q.w};
    uint32_t c[4];
    if (MODE == QUANT_ACT_DYNAMIC && d.fast) {
        // every |x| <= amax is finite, so |x / s| < 464: the hardware convert needs no guard.  The
        // convert writes two codes into the half of its destination that word_sel names and keeps
        // the other half: four codes per register without shifts or masks.
        uint32_t lo, hi;
        {
            const float a0 = div_exact(__uint_as_float(w[0] << 16), d), b0 = div_exact(__uint_as_float(w[0] & 0xFFFF0000u), d);
            const float a1 = div_exact(__uint_as_float(w[1] << 16), d), b1 = div_exact(__uint_as_float(w[1] & 0xFFFF0000u), d);
            lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a0, b0, 0, false);
            lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a1, b1, (int)lo, true);
        }
        {
            const float a0 = div_exact(__uint_as_float(w[2] << 16), d), b0 = div_exact(__uint_as_float(w[2] & 0xFFFF0000u), d);
            const float a1 = div_exact(__uint_as_float(w[3] << 16), d), b1 = div_exact(__uint_as_float(w[3] & 0xFFFF0000u), d);
            hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a0, b0, 0, false);
            hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(a1, b1, (int)hi, true);
        }
        return make_uint2(lo, hi);
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float a = bf16_bits_to_f32(w[i] & 0xFFFFu) / d.s;
            float b = bf16_bits_to_f32(w[i] >> 16) / d.s;
            if constexpr (MODE == QUANT_WEIGHT) {
                a = fminf(fmaxf(a, -kFp8Max), kFp8Max);
                b = fminf(fmaxf(b, -kFp8Max), kFp8Max);
            }
            c[i] = e4m3_pack2(a, b);
        }
    }
    return make_uint2(c[0] | (c[1] << 16), c[2] | (c[3] << 16));
}

// Row absmax as bf16 bits.  |bf16| bit patterns order like the values they
// encode, so an unsigned max over (bits & 0x7FFF) is the bf16 amax; a NaN in the
// row has the largest pattern and therefore wins, as torch.amax propagates it.
template <int MODE>
__device__ __forceinline__ float scale_from_amax_bits(uint32_t amax_bits) {
    if constexpr (MODE == QUANT_ACT_DYNAMIC) {
        amax_bits = amax_bits < kAmaxFloorBf16 ? kAmaxFloorBf16 : amax_bits;
        // amax / 448 rounded to bf16: the multiplication by fl(1 / 448) gives the same bf16 for every
        // finite amax (a quotient of an 8-bit mantissa by 7 is never within 2^-12 of a bf16 rounding
        // boundary unless it is exact; checked over all 32 639 values)
        // (an Inf or NaN amax gives the same Inf or NaN either way)
        return bf16_bits_to_f32(f32_to_bf16_bits(bf16_bits_to_f32(amax_bits) * (1.0f / kFp8Max)));
    } else {
        float s = bf16_bits_to_f32(amax_bits) / kFp8Max;
        return s >= 1.17549435e-38f ? s : 1.17549435e-38f;
    }
}

}  // namespace phyai
