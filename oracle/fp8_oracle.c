/*
 * CPU oracle for the W8A8 fp8 quantized-linear path.  TEST INFRASTRUCTURE ONLY.
 *
 * This file is the checker that the HIP kernels are compared against.  Nothing
 * in the shipped package may link, load or call it; only the tests, the smoke
 * check and the CPU-baseline leg of the benchmark do.
 *
 * Every function restates, in plain C, what the reference computes with torch
 * tensor ops, and names the reference lines it follows (paths are relative to
 * the reference checkout):
 *
 *   orc_quant_rowwise      phyai/src/phyai/layers/quant/fp8.py:150-155
 *   orc_quant_static       phyai/src/phyai/layers/quant/fp8.py:142-148
 *   orc_linear             phyai/src/phyai/layers/linear/backends/torch.py:155-176
 *                          (torch._scaled_mm row-wise semantics, restated as the
 *                          fp32 dequantize + matmul the benchmark baseline names)
 *   orc_act_* / epilogues  phyai/src/phyai/layers/mlp/dense_mlp.py:87-124,256-265
 *   orc_weight_quant       no reference function exists; the rule
 *                          "absmax/448 per output channel, RNE, saturate" is the
 *                          benchmark configuration's own definition.
 *
 * How each function is pinned (the tests that do it live in tests/test_oracle*.py):
 *   e4m3 encode/decode   all 256 codes against the OCP closed form; every fp32
 *                        midpoint between adjacent codes (tie -> even); a dense
 *                        sweep against torch's own .to(float8_e4m3fn) cast.
 *   bf16 RNE             exhaustive over the upper 16 bits x tie/above/below
 *                        tails against torch's .to(bfloat16).
 *   orc_quant_rowwise    torch CPU closed form of the three reference lines on
 *                        seeded inputs and on the committed golden fixtures;
 *                        invariants (argmax element encodes to 0x7E/0xFE).
 *   orc_linear           exact-integer cases (sums exact in fp32, so any order
 *                        gives the same bits) and torch fp32 matmul closed form.
 *   activations          torch.nn.functional.gelu (erf and tanh forms), silu.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_EXPORT __attribute__((visibility("default")))

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* ---- bf16 ------------------------------------------------------------- */

ORC_EXPORT float orc_bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* fp32 -> bf16, round to nearest, ties to even; NaN -> canonical quiet NaN. */
ORC_EXPORT uint16_t orc_f32_to_bf16(float f) {
    if (f != f) return 0x7FC0;
    uint32_t u = f32_bits(f);
    uint32_t keep = u >> 16;
    uint32_t tail = u & 0xFFFFu;
    if (tail > 0x8000u || (tail == 0x8000u && (keep & 1u))) keep += 1; /* carries into exp: ok */
    return (uint16_t)keep;
}

/* ---- OCP e4m3fn ------------------------------------------------------- */
/* 1 sign, 4 exponent (bias 7), 3 mantissa.  No infinities; S.1111.111 is NaN.
 * Largest finite 448 = 1.75 * 2^8.  Subnormal step 2^-9. */

ORC_EXPORT float orc_e4m3_to_f32(uint8_t c) {
    int s = c >> 7, e = (c >> 3) & 0xF, m = c & 7;
    float v;
    if (e == 0xF && m == 7) v = NAN;
    else if (e == 0) v = ldexpf((float)m, -9);
    else v = ldexpf((float)(8 + m), e - 10);
    return s ? -v : v;
}

/*
 * fp32 -> e4m3fn with round-to-nearest-even and the reference cast's overflow
 * rule: |v| >= 480 (the first value that would need mantissa 0b1000 at the top
 * exponent) and NaN/Inf become NaN (0x7F | sign).  Values in (448, 480) that
 * round down land on 448; [464, 480) rounds up to the NaN slot, matching
 * torch's .to(torch.float8_e4m3fn).  Written on integers: the value is put on
 * the grid of the target binade (or the subnormal grid) and rounded there.
 */
ORC_EXPORT uint8_t orc_f32_to_e4m3(float f) {
    uint32_t u = f32_bits(f);
    uint8_t sign = (uint8_t)((u >> 24) & 0x80u);
    uint32_t a = u & 0x7FFFFFFFu;
    if (a >= 0x43F00000u) return (uint8_t)(sign | 0x7F);       /* >= 480, Inf, NaN */
    int e = (int)(a >> 23) - 127;                               /* unbiased fp32 exponent */
    uint32_t man = (a & 0x7FFFFFu) | (a >= 0x00800000u ? 0x800000u : 0u);
    /* grid step: 2^(e-3) for normals (e >= -6), 2^-9 for everything below. */
    int step_exp = (e >= -6) ? (e - 3) : -9;
    /* value = man * 2^(e-23) (fp32 subnormals: e=-127 stands for 2^-126 scale,
     * far below the grid, they round to zero either way). */
    int shift = step_exp - (e - 23);                            /* bits to drop */
    uint32_t q;
    if (shift >= 32) q = 0;
    else {
        uint32_t lost = (shift == 0) ? 0 : (man & ((1u << shift) - 1u));
        uint32_t half = (shift == 0) ? 0 : (1u << (shift - 1));
        q = man >> shift;
        if (lost > half || (lost == half && half != 0 && (q & 1u))) q += 1;
    }
    /* q counts grid steps.  Normal binade: q in [8,16]; 16 rolls into the next binade. */
    uint32_t code;
    if (e >= -6) {
        int be = e + 7;                                         /* biased e4m3 exponent */
        if (q == 16) { be += 1; q = 8; }
        code = ((uint32_t)be << 3) | (q - 8);
    } else {
        code = q;                                               /* q in [0,8]; 8 == smallest normal */
    }
    if (code >= 0x7F) code = 0x7F;
    return (uint8_t)(sign | code);
}

/* ---- activation quantizer --------------------------------------------- */

#define ORC_FP8_MAX 448.0f

/*
 * Per-token dynamic quantization, fp8.py:150-155:
 *   x_amax  = x.abs().amax(-1, keepdim=True).clamp_min(1e-12)   (bf16 tensor ops;
 *             the python scalar 1e-12 is cast to bf16 first -> 0x2B8D)
 *   x_scale = (x_amax / 448.0).to(float32)        (fp32 divide, rounded to bf16,
 *             then widened)
 *   x_q     = (x / x_scale).to(float8_e4m3fn)     (bf16 / fp32 promotes to an
 *             fp32 IEEE divide; then the RNE cast above)
 * x is [M, K] bf16 bits with row stride ldx elements.
 */
ORC_EXPORT void orc_quant_rowwise(const uint16_t *x, int64_t M, int64_t K, int64_t ldx,
                                  uint8_t *xq, float *x_scale) {
    const uint16_t floor_bits = orc_f32_to_bf16(1e-12f);
#pragma omp parallel for schedule(static) if (M * K > 65536)
    for (int64_t m = 0; m < M; ++m) {
        const uint16_t *row = x + m * ldx;
        float amax = orc_bf16_to_f32(floor_bits);
        int saw_nan = 0;
        for (int64_t k = 0; k < K; ++k) {
            float v = fabsf(orc_bf16_to_f32(row[k]));
            if (v != v) saw_nan = 1;
            if (v > amax) amax = v;
        }
        if (saw_nan) amax = NAN;                   /* torch amax propagates NaN */
        float s = orc_bf16_to_f32(orc_f32_to_bf16(amax / ORC_FP8_MAX));
        x_scale[m] = s;
        for (int64_t k = 0; k < K; ++k)
            xq[m * K + k] = orc_f32_to_e4m3(orc_bf16_to_f32(row[k]) / s);
    }
}

/*
 * Static per-tensor quantization, fp8.py:142-148:
 *   x_q = (x.float() / input_scale).clamp(-448, 448).to(float8_e4m3fn)
 * torch.clamp propagates NaN.
 */
ORC_EXPORT void orc_quant_static(const uint16_t *x, int64_t M, int64_t K, int64_t ldx,
                                 float input_scale, uint8_t *xq) {
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < K; ++k) {
            float v = orc_bf16_to_f32(x[m * ldx + k]) / input_scale;
            if (v == v) v = v < -ORC_FP8_MAX ? -ORC_FP8_MAX : (v > ORC_FP8_MAX ? ORC_FP8_MAX : v);
            xq[m * K + k] = orc_f32_to_e4m3(v);
        }
}

/*
 * Offline per-output-channel weight quantization (harness-defined):
 *   s_w[n] = max_k |W[n,k]| (fp32) / 448, floored at 2^-126 so an all-zero row
 *   gets a finite positive scale; Wq = e4m3_rne(clamp(W/s_w, +-448)).
 */
ORC_EXPORT void orc_weight_quant(const uint16_t *w, int64_t N, int64_t K,
                                 uint8_t *wq, float *w_scale) {
#pragma omp parallel for schedule(static) if (N * K > 65536)
    for (int64_t n = 0; n < N; ++n) {
        float amax = 0.f;
        for (int64_t k = 0; k < K; ++k) {
            float v = fabsf(orc_bf16_to_f32(w[n * K + k]));
            if (v > amax) amax = v;
        }
        float s = amax / ORC_FP8_MAX;
        if (!(s >= 1.17549435e-38f)) s = 1.17549435e-38f;
        w_scale[n] = s;
        for (int64_t k = 0; k < K; ++k) {
            float v = orc_bf16_to_f32(w[n * K + k]) / s;
            v = v < -ORC_FP8_MAX ? -ORC_FP8_MAX : (v > ORC_FP8_MAX ? ORC_FP8_MAX : v);
            wq[n * K + k] = orc_f32_to_e4m3(v);
        }
    }
}

/* ---- activations (dense_mlp.py:87-124) -------------------------------- */

ORC_EXPORT float orc_gelu_tanh(float v) {
    const float k0 = 0.7978845608028654f, k1 = 0.044715f;
    return 0.5f * v * (1.0f + tanhf(k0 * (v + k1 * v * v * v)));
}
ORC_EXPORT float orc_gelu_erf(float v) { return 0.5f * v * (1.0f + erff(v * 0.70710678118654752f)); }
ORC_EXPORT float orc_silu(float v) { return v / (1.0f + expf(-v)); }

enum {
    ORC_EPI_NONE = 0,
    ORC_EPI_GEGLU_TANH = 1, /* gelu_tanh(gate) * up, gate = cols [0,I), up = [I,2I) */
    ORC_EPI_GEGLU_ERF = 2,
    ORC_EPI_SWIGLU = 3,
    ORC_EPI_GELU_TANH = 4,  /* plain fc1 -> act */
    ORC_EPI_GELU_ERF = 5,
};

static inline float act_of(int epi, float v) {
    switch (epi) {
    case ORC_EPI_GEGLU_TANH: case ORC_EPI_GELU_TANH: return orc_gelu_tanh(v);
    case ORC_EPI_GEGLU_ERF: case ORC_EPI_GELU_ERF: return orc_gelu_erf(v);
    case ORC_EPI_SWIGLU: return orc_silu(v);
    default: return v;
    }
}

/*
 * The W8A8 linear, torch.py:155-176:
 *   out = bf16( (xq.float()*x_scale) @ (wq.float()*w_scale[:,None]).T + bias )
 * accumulated in fp32 over k ascending, then the DenseMLP epilogue
 * (dense_mlp.py:256-265).  The reference runs GEMM and activation as two
 * launches with a bf16 tensor between them, so the GEMM result is rounded to
 * bf16 before the activation and the product is rounded once more; this
 * function keeps both roundings.  out_f32 (optional, [M, N]) receives the
 * pre-rounding, pre-activation fp32 GEMM+bias value that the parity tolerance
 * is stated against.
 * Shapes: xq [M,K], wq [N,K] (K contiguous), out [M, N] or [M, N/2] if gated.
 */
ORC_EXPORT int orc_linear(const uint8_t *xq, const float *x_scale,
                          const uint8_t *wq, const float *w_scale,
                          const uint16_t *bias, int64_t M, int64_t N, int64_t K,
                          int epilogue, uint16_t *out, float *out_f32) {
    int gated = epilogue >= ORC_EPI_GEGLU_TANH && epilogue <= ORC_EPI_SWIGLU;
    if (gated && (N & 1)) return -1;
    float lut[256];
    for (int c = 0; c < 256; ++c) lut[c] = orc_e4m3_to_f32((uint8_t)c);
    int64_t I = N / 2;
    float *full = (float *)malloc((size_t)M * (size_t)N * sizeof(float));
    float *adeq = (float *)malloc((size_t)M * (size_t)K * sizeof(float));
    if (!full || !adeq) { free(full); free(adeq); return -2; }
    for (int64_t m = 0; m < M; ++m)
        for (int64_t k = 0; k < K; ++k) adeq[m * K + k] = lut[xq[m * K + k]] * x_scale[m];
#pragma omp parallel
    {
        float *brow = (float *)malloc((size_t)K * sizeof(float));
#pragma omp for schedule(static)
        for (int64_t n = 0; n < N; ++n) {
            for (int64_t k = 0; k < K; ++k) brow[k] = lut[wq[n * K + k]] * w_scale[n];
            for (int64_t m = 0; m < M; ++m) {
                const float *arow = adeq + m * K;
                float acc = 0.f;
                for (int64_t k = 0; k < K; ++k) acc += arow[k] * brow[k];
                if (bias) acc += orc_bf16_to_f32(bias[n]);
                full[m * N + n] = acc;
            }
        }
        free(brow);
    }
    free(adeq);
    if (out_f32) memcpy(out_f32, full, (size_t)M * (size_t)N * sizeof(float));
    if (out) {
        for (int64_t m = 0; m < M; ++m) {
            if (gated) {
                for (int64_t i = 0; i < I; ++i) {
                    float g = orc_bf16_to_f32(orc_f32_to_bf16(full[m * N + i]));
                    float u = orc_bf16_to_f32(orc_f32_to_bf16(full[m * N + I + i]));
                    out[m * I + i] = orc_f32_to_bf16(act_of(epilogue, g) * u);
                }
            } else {
                for (int64_t n = 0; n < N; ++n) {
                    float v = full[m * N + n];
                    if (epilogue != ORC_EPI_NONE) v = act_of(epilogue, orc_bf16_to_f32(orc_f32_to_bf16(v)));
                    out[m * N + n] = orc_f32_to_bf16(v);
                }
            }
        }
    }
    free(full);
    return 0;
}

ORC_EXPORT int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* Array forms of the scalar casts, so tests can sweep millions of bit patterns. */
ORC_EXPORT void orc_f32_to_e4m3_array(const float *v, int64_t n, uint8_t *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_e4m3(v[i]);
}
ORC_EXPORT void orc_e4m3_to_f32_array(const uint8_t *c, int64_t n, float *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_e4m3_to_f32(c[i]);
}
ORC_EXPORT void orc_f32_to_bf16_array(const float *v, int64_t n, uint16_t *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = orc_f32_to_bf16(v[i]);
}
ORC_EXPORT void orc_act_array(int epilogue, const float *v, int64_t n, float *out) {
    for (int64_t i = 0; i < n; ++i) out[i] = act_of(epilogue, v[i]);
}
