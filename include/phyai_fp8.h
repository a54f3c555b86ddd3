/*
 * phyai_fp8.h - C ABI of the MI355X (gfx950) W8A8 fp8 quantized-linear library.
 *
 * Every entry point is `extern "C"`, takes raw device pointers, sizes and a HIP
 * stream (passed as `void*`, i.e. a `hipStream_t`), enqueues work on that stream
 * and returns without synchronising.  None of them allocates device memory;
 * scratch space is a caller-owned workspace sized by
 * phyai_fp8_linear_workspace_bytes().  Return value: 0 on success, a negative
 * PHYAI_FP8_E* code otherwise; phyai_fp8_last_error() gives the message of the
 * calling thread's last failure.
 *
 * The reference has no native fp8 code: on this path it runs torch tensor ops,
 * torch._scaled_mm and a flashinfer activation kernel.  Each declaration below
 * names the reference lines (paths relative to the reference checkout) whose
 * arithmetic it replaces.
 *
 * Layouts.  Activations x: [M, K] bf16, K contiguous, row stride ldx elements.
 * Codes xq: [M, K] e4m3fn bytes, dense.  Weights w: [N, K] e4m3fn bytes, dense,
 * K contiguous (the layout Fp8Spec.allocate registers, quant/fp8.py:74-79).
 * Scales: x_scale [M] fp32, w_scale [N] fp32.  bias: [N] bf16 or NULL.
 * out: bf16, row stride ldo elements, [M, N] (or [M, N/2] for gated epilogues,
 * where gate = columns [0, N/2) and up = columns [N/2, N), mlp/dense_mlp.py:11-15).
 */
#ifndef PHYAI_FP8_H
#define PHYAI_FP8_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PHYAI_FP8_ABI_VERSION 8

enum {
    PHYAI_FP8_OK = 0,
    PHYAI_FP8_EINVAL = -1,      /* bad pointer / size / alignment                 */
    PHYAI_FP8_EUNSUPPORTED = -2, /* shape outside what the kernels handle          */
    PHYAI_FP8_EWORKSPACE = -3,  /* workspace missing or too small                 */
    PHYAI_FP8_ELAUNCH = -4      /* HIP reported a launch error                    */
};

/* Epilogue applied to (acc * x_scale[m] * w_scale[n] + bias[n]).
 * mlp/dense_mlp.py:87-124 (activation table), :256-265 (where it is applied). */
enum {
    PHYAI_FP8_EPI_NONE = 0,
    PHYAI_FP8_EPI_GEGLU_TANH = 1, /* gelu_tanh(gate) * up  -> [M, N/2]             */
    PHYAI_FP8_EPI_GEGLU_ERF = 2,  /* gelu_erf(gate) * up   -> [M, N/2]             */
    PHYAI_FP8_EPI_SWIGLU = 3,     /* silu(gate) * up       -> [M, N/2]             */
    PHYAI_FP8_EPI_GELU_TANH = 4,  /* plain fc1 -> gelu_tanh -> [M, N]              */
    PHYAI_FP8_EPI_GELU_ERF = 5    /* plain fc1 -> gelu (erf) -> [M, N]             */
};

/*
 * Flags, OR-ed into the `epilogue` argument of phyai_fp8_gemm / phyai_fp8_linear (the epilogue
 * code is `epilogue & PHYAI_FP8_EPILOGUE_MASK`).
 *
 * STREAM_WEIGHTS: read this call's weight matrix with non-temporal loads, so that it does not
 * displace other data from the 256 MB Infinity Cache.  A model whose weights exceed that cache and
 * are re-read every step (the action expert: 311 MB per denoise step, ten steps per inference)
 * gets no cache hits at all when everything is cached alike; marking the largest matrices lets
 * the rest stay resident (phyai_amd/cache_plan.py picks them).  Honoured by the weight-streaming
 * kernel (what phyai_fp8_describe_plan reports as "small-m"), ignored by the tile kernels, whose
 * workgroups share weight rows through L2; results are bit-identical with and without it.  The
 * reference has no counterpart (its GEMM is a library call, linear/backends/torch.py:168-175).
 *
 * W_OPERAND_ORDER / W_OPERAND_GATED: `w` is not row-major [N, K] but in MFMA operand order, as
 * phyai_fp8_weight_to_operand_order() wrote it (plain form for the first flag, the fused gate | up
 * form for the second).  Every kernel accepts both layouts and gives bit-identical results; the
 * kernels whose weight blocks are private to a wavefront then load them straight into registers
 * instead of staging them through LDS.  A gated epilogue needs W_OPERAND_GATED, any other epilogue
 * W_OPERAND_ORDER; a mismatch is refused with PHYAI_FP8_EINVAL.  K must be a multiple of 128.
 */
#define PHYAI_FP8_EPILOGUE_MASK 0xFF
#define PHYAI_FP8_FLAG_STREAM_WEIGHTS 0x100
#define PHYAI_FP8_FLAG_W_OPERAND_ORDER 0x200
#define PHYAI_FP8_FLAG_W_OPERAND_GATED 0x600

int phyai_fp8_abi_version(void);
const char *phyai_fp8_last_error(void);

/*
 * Per-token dynamic activation quantizer.
 * Replaces Fp8Spec.quantize_activation, PER_CHANNEL/BLOCK branch
 * (layers/quant/fp8.py:150-155): bf16 absmax per row floored at bf16(1e-12),
 * scale = fp32(bf16(amax/448)), codes = e4m3fn_rne(fp32(x) / scale).
 * Bit-exact with that expression.  Requires K % 8 == 0 and 16-byte aligned rows.
 */
int phyai_fp8_quant_rowwise(const void *x, int64_t M, int64_t K, int64_t ldx,
                            void *xq, float *x_scale, void *stream);

/*
 * Static per-tensor activation quantizer.
 * Replaces Fp8Spec.quantize_activation, PER_TENSOR branch
 * (layers/quant/fp8.py:142-148): codes = e4m3fn(clamp(fp32(x)/input_scale[0], +-448)).
 * input_scale is a device pointer to one fp32.
 */
int phyai_fp8_quant_static(const void *x, int64_t M, int64_t K, int64_t ldx,
                           const float *input_scale, void *xq, void *stream);

/*
 * Offline per-output-channel weight quantizer: w_scale[n] = absmax_k(W[n,:])/448
 * in fp32 (floored at FLT_MIN), wq = e4m3fn(clamp(W/w_scale, +-448)).
 * The reference has no such function (TODO at layers/quant/fp8.py:80-83; its
 * model-optimizer package is empty); the rule is the benchmark's definition.
 */
int phyai_fp8_weight_quant_rowwise(const void *w, int64_t N, int64_t K, int64_t ldw,
                                   void *wq, float *w_scale, void *stream);

/*
 * Re-lays a row-major fp8 weight matrix w[N, K] into MFMA operand order, out of place (out: N * K
 * bytes, 16-byte aligned, must not overlap w).  Units of 16 rows x 128 bytes of K are stored
 * K step after K step, and inside a unit the 16-byte chunk c of row r sits at (c * 16 + r) * 16:
 * the sixteen lanes of a wavefront that want the same 16 bytes of K of sixteen neighbouring rows read
 * 256 contiguous bytes.  gated != 0: w is a fused gate | up matrix (gate = rows [0, N/2)); unit u
 * then holds gate columns 8 u .. 8 u + 7 and the up columns that pair with them, row 4 p + 2 t + b of
 * the unit being row t * N/2 + 8 u + 2 p + b of w, so that an MFMA lane ends up with gate and up of
 * the same output columns.  Needs K % 128 == 0 and N % 16 == 0 (N % 32 == 0 when gated).
 * This is the work the reference leaves to WeightSpec.process_after_loading
 * (layers/quant/base.py:55-70, layers/quant/fp8.py:127-135: "re-lay weights after loading");
 * pass the result to the GEMM entry points with PHYAI_FP8_FLAG_W_OPERAND_ORDER / _GATED.
 */
int phyai_fp8_weight_to_operand_order(const void *w, int64_t N, int64_t K, int gated, void *out,
                                      void *stream);

/*
 * Bytes of workspace phyai_fp8_linear / phyai_fp8_gemm need for this shape.
 * The workspace must be 256-byte aligned and its first
 * PHYAI_FP8_WORKSPACE_HEADER_BYTES must be zero before the first call that uses
 * it; every call leaves them zero again.  Two calls that may run concurrently
 * must not share a workspace.
 */
#define PHYAI_FP8_WORKSPACE_HEADER_BYTES 16384
size_t phyai_fp8_linear_workspace_bytes(int64_t M, int64_t N, int64_t K, int epilogue);

/*
 * fp8 x fp8 GEMM on already-quantized activations with fused
 * dequant-scale-bias-activation epilogue, bf16 out.
 * Replaces the torch._scaled_mm call of TorchKernel._fp8_per_channel
 * (layers/linear/backends/torch.py:166-175) and, for epilogue != NONE, the
 * following activation launch of DenseMLP.forward (mlp/dense_mlp.py:256-265).
 * Per-tensor layers (torch.py:123-153) pass x_scale_is_scalar = 1 and a pointer
 * to the single input scale.  Requires K % 16 == 0 and N % 16 == 0
 * (the same gate as TorchKernel.can_handle, torch.py:91).
 */
int phyai_fp8_gemm(const void *xq, const float *x_scale, int x_scale_is_scalar,
                   const void *w, const float *w_scale, const void *bias,
                   void *out, int64_t ldo, int64_t M, int64_t N, int64_t K,
                   int epilogue, void *workspace, size_t workspace_bytes, void *stream);

/*
 * The whole quantized linear: per-token quantization of bf16 x followed by the
 * GEMM above, as one call.  Replaces TorchKernel._fp8_per_channel
 * (layers/linear/backends/torch.py:155-176) end to end.
 *
 * Up to 128 token rows, K <= 4096 (a multiple of 128), with x and its row stride 16-byte
 * aligned and a workgroup shape whose grid fits the chip at once (beyond K = 2048: projections up to
 * about 2048 wide), this is ONE kernel: every workgroup
 * quantizes the token rows it multiplies (same codes, same scales, same output bits as
 * the two launches) and the workspace is not touched: such a call may pass workspace = NULL.
 * Otherwise the quantizer writes codes and scales into the workspace and a GEMM kernel follows
 * (PHYAI_FP8_EWORKSPACE without one).  phyai_fp8_describe_linear_plan tells which.
 */
int phyai_fp8_linear(const void *x, int64_t ldx, const void *w, const float *w_scale,
                     const void *bias, void *out, int64_t ldo, int64_t M, int64_t N,
                     int64_t K, int epilogue, void *workspace, size_t workspace_bytes,
                     void *stream);

/*
 * The same two with the gated residual of a decoder layer fused into the epilogue:
 *     out[m, n] = bf16( residual[m, n] + bf16(acc * x_scale[m] * w_scale[n] + bias[n]) * gate[m / g, n] )
 * computed in fp32 and rounded once, i.e. torch.addcmul(residual, linear(x), gate) on bf16
 * tensors (models/pi05/modeling_pi05.py:822-826,835: `h = torch.addcmul(residual, out, gate)`
 * after o_proj and after the MLP's down_proj).  residual: [M, N] bf16, row stride ld_res;
 * gate: [gate_rows, N] bf16, row stride ld_gate, M a multiple of gate_rows and g = M / gate_rows
 * (the gate of an adaptive norm has one row per modulation row).  No activation epilogue;
 * flags: PHYAI_FP8_FLAG_* bits (STREAM_WEIGHTS, W_OPERAND_ORDER) or 0.  out may alias residual.
 */
int phyai_fp8_gemm_addcmul(const void *xq, const float *x_scale, int x_scale_is_scalar,
                           const void *w, const float *w_scale, const void *bias,
                           const void *residual, int64_t ld_res, const void *gate, int64_t ld_gate,
                           int64_t gate_rows, void *out, int64_t ldo, int64_t M, int64_t N,
                           int64_t K, int flags, void *workspace, size_t workspace_bytes,
                           void *stream);
int phyai_fp8_linear_addcmul(const void *x, int64_t ldx, const void *w, const float *w_scale,
                             const void *bias, const void *residual, int64_t ld_res,
                             const void *gate, int64_t ld_gate, int64_t gate_rows, void *out,
                             int64_t ldo, int64_t M, int64_t N, int64_t K, int flags,
                             void *workspace, size_t workspace_bytes, void *stream);

/*
 * The two projections of an MLP as one call: out = W2 . act(W1 . x), both W8A8 with per-token
 * quantization of their input (x, then the activation's bf16 output h, which stays in the workspace).
 * Replaces DenseMLP.forward (layers/mlp/dense_mlp.py:256-265: gate_up_proj / fc1, the activation
 * launch, down_proj / fc2) for fp8 per-channel layers.  `epilogue` is the first projection's
 * activation (any PHYAI_FP8_EPI_* but NONE): w1 is [N1, H] with N1 = 2 I for the gated ones (gate | up
 * fused, dense_mlp.py:11-15) and N1 = I otherwise; w2 is [O, I].  flags1 / flags2: PHYAI_FP8_FLAG_* bits of
 * the two weight matrices (layout, streaming).  residual / gate (both or neither; residual [M, O], gate
 * [gate_rows, O]) put the decoder layer's addcmul behind the second projection as in
 * phyai_fp8_linear_addcmul.  Same bits as phyai_fp8_linear (epilogue) followed by
 * phyai_fp8_linear[_addcmul] on its output.
 *
 * What the one call buys: when both projections are served by the kernel that quantizes its own token
 * rows (M <= 128, H <= 2048, I <= 4096, see phyai_fp8_describe_mlp_plan), the first one also leaves the
 * |h| maximum of every token row per workgroup column in the workspace, and the second one starts its
 * conversions from those instead of first passing over its rows - which is what makes one launch pay
 * for a down projection with K = 4096.  Otherwise it is the two linears back to back.
 * Workspace: phyai_fp8_mlp_workspace_bytes(), same rules as for phyai_fp8_linear.
 */
size_t phyai_fp8_mlp_workspace_bytes(int64_t M, int64_t H, int64_t I, int64_t O, int epilogue);
int phyai_fp8_mlp(const void *x, int64_t ldx, const void *w1, const float *w1_scale, const void *bias1,
                  int flags1, const void *w2, const float *w2_scale, const void *bias2, int flags2,
                  const void *residual, int64_t ld_res, const void *gate, int64_t ld_gate,
                  int64_t gate_rows, void *out, int64_t ldo, int64_t M, int64_t H, int64_t I,
                  int64_t O, int epilogue, void *workspace, size_t workspace_bytes, void *stream);
/* "row maxima handed over: <first> | <second>" or "<first> | <second>", each part as
 * phyai_fp8_describe_linear_plan reports it.  Host only.  Row-major weights, or - with
 * PHYAI_FP8_FLAG_W_OPERAND_ORDER or-ed into `epilogue` - both matrices in operand order. */
int phyai_fp8_describe_mlp_plan(int64_t M, int64_t H, int64_t I, int64_t O, int epilogue, char *buf,
                                size_t n);

/*
 * phyai_fp8_linear for callers that cannot allocate device memory or hand over a workspace: code
 * under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  No counterpart
 * in the reference (its linear returns a tensor from torch's caching allocator,
 * layers/linear/backends/torch.py:168-176).  Same kernels and same results as phyai_fp8_linear;
 * the scratch (activation codes, per-token scales, split-K counters and partial sums) lives in a
 * device array of PHYAI_FP8_STATIC_SCRATCH_BYTES that is part of the library's code object: every
 * GPU the library runs on holds one until the process ends.  The call allocates nothing and frees
 * nothing.  A shape whose phyai_fp8_linear_workspace_bytes() exceeds the array is refused with
 * PHYAI_FP8_EWORKSPACE.  All calls on one GPU share that GPU's array: calls that may overlap there
 * (two streams, two threads) race; serialise them or use phyai_fp8_linear with one workspace
 * each.  The first call on a device looks the array's address up (hipGetSymbolAddress); make it
 * outside graph capture, e.g. in the warm-up runs.
 */
#define PHYAI_FP8_STATIC_SCRATCH_BYTES (32 * 1024 * 1024)
int phyai_fp8_linear_static(const void *x, int64_t ldx, const void *w, const float *w_scale,
                            const void *bias, void *out, int64_t ldo, int64_t M, int64_t N,
                            int64_t K, int epilogue, void *stream);

/*
 * RMSNorm whose output feeds the quantizer without a round trip through memory.
 * Replaces phyai_kernel.triton.rmsnorm / gemma_rmsnorm
 * (phyai-kernel/phyai_kernel/triton/rms_norm.py:42-75: fp32 reduction,
 * out = bf16(x * rsqrt(mean(x^2) + eps) * w), w + 1 for the Gemma form) followed
 * by Fp8Spec.quantize_activation (layers/quant/fp8.py:150-155) on that bf16
 * output.  x: [M, D] bf16, row stride ldx; weight: [D] bf16.  out ([M, D] bf16,
 * row stride ldo) may be NULL when only the codes are wanted; xq / x_scale may
 * both be NULL when only the normalised bf16 tensor is wanted.  D % 8 == 0; rows up
 * to 8192 elements stay in registers, longer ones are re-read per pass (the
 * reference's two-pass kernels, rms_norm.py:125-167).
 */
int phyai_fp8_rmsnorm_quant(const void *x, int64_t ldx, const void *weight, int gemma,
                            int64_t M, int64_t D, float eps, void *out, int64_t ldo,
                            void *xq, float *x_scale, void *stream);

/*
 * Adaptive RMSNorm (scale, shift, gate from a projected conditioning row) with the
 * same fused quantizer.  Replaces phyai_kernel.triton.adarmsnorm
 * (phyai-kernel/phyai_kernel/triton/ada_rms_norm.py:63-117:
 * out = bf16(x * rsqrt(mean(x^2) + eps) * (1 + scale) + shift), gate copied once per
 * modulation row) + the quantizer.  modulation: [mod_rows, 3 * D] bf16 = scale |
 * shift | gate, row stride ld_mod; M must be a multiple of mod_rows and row m uses
 * modulation row m / (M / mod_rows).  gate_out: [mod_rows, D] bf16 or NULL.
 */
int phyai_fp8_adarmsnorm_quant(const void *x, int64_t ldx, const void *modulation,
                               int64_t ld_mod, int64_t mod_rows, int64_t M, int64_t D,
                               float eps, void *out, int64_t ldo, void *gate_out,
                               int64_t ld_gate, void *xq, float *x_scale, void *stream);

/*
 * Which kernel phyai_fp8_gemm would launch for a problem with 16-byte aligned operands and a
 * dense output (ldo = output width): a short text such as
 *   "small-m nt=2 mb=4 kpw=1 rounds=1"      weight-streaming kernel
 *   "tile 192x128 depth=2 splits=1 tiles=2304"   pipelined tile kernel
 *   "tile 224x256 depth=2 splits=1 tiles=512 weights in registers, ring of 4"   the same with weights in
 *       operand order loaded straight into registers and no barrier in the main loop
 *   "generic 128x128 splits=2"               fallback tile kernel
 * written to buf (at most n bytes, always terminated).  Host only: nothing is launched, no GPU is
 * needed.  The layout flag of the weight matrix (PHYAI_FP8_FLAG_W_OPERAND_ORDER / _GATED) may be
 * OR-ed into `epilogue` as in the calls: the choice of tile can depend on it.  Returns the length
 * of the text, or a negative status for bad arguments.  The
 * reference has no counterpart (its dispatcher only picks between whole backends,
 * layers/linear/dispatch.py:28-95); this is for logs and for tests of the selection rules.
 */
int phyai_fp8_describe_plan(int64_t M, int64_t N, int64_t K, int epilogue, char *buf, size_t n);

/*
 * The same for phyai_fp8_linear (bf16 activations in, dense rows): either
 *   "one launch: small-m rows=8 nt=5 kpw=1 grid=32x7"      the kernel that quantizes its own token rows
 * or "quantizer + " followed by what phyai_fp8_describe_plan reports.  Host only.  The layout flag of
 * the weight matrix (PHYAI_FP8_FLAG_W_OPERAND_ORDER / _GATED) may be or-ed into `epilogue` as in the
 * calls: a few shapes are one launch only with weights in operand order (registers instead of LDS).
 */
int phyai_fp8_describe_linear_plan(int64_t M, int64_t N, int64_t K, int epilogue, char *buf, size_t n);

/*
 * Test hook: run the device fp32 -> e4m3fn cast used by the quantizers over n
 * values (device pointers), so that it can be compared exhaustively with the
 * CPU cast.  Not part of the reference surface.
 */
int phyai_fp8_debug_cast_e4m3(const float *v, int64_t n, void *codes, void *stream);

/*
 * Time stamps of the kernels' phases, for the debug build of the library only (`make stamps` in
 * phyai_amd/csrc builds lib/libphyai_fp8_stamps.so; the normal build returns PHYAI_FP8_EUNSUPPORTED).  From this
 * call on every wavefront of the pipelined tile kernel and of the one-launch small-M kernel writes one record of
 * PHYAI_FP8_STAMP_WORDS 64-bit words into `records` (device memory for n_records records, index = workgroup *
 * wavefronts per workgroup + wavefront; records past the end are dropped): shader-clock stamps of its phases in
 * words [0, 10), the 100 MHz counter at entry and at the end in the last two (csrc/stamps.h says what each
 * marks).  n_records = 0 switches the recording off.  Synchronises the device.  Not part of the reference surface:
 * this is how the cycle budgets of the kernels were measured.
 */
#define PHYAI_FP8_STAMP_WORDS 12
int phyai_fp8_debug_stamps(uint64_t *records, int64_t n_records);

/*
 * Hardware probe: `workgroups` workgroups of four wavefronts each issue iters x 16 independent
 * v_mfma_f32_32x32x64_f8f6f4 (32 x 32 x 64 x 2 flops each) and touch no memory.  counters (device,
 * 2 x workgroups 64-bit words) receives per workgroup the shader cycles and the 100 MHz ticks its
 * loop took; sink is one device float that is never written.  Gives the fp8 MFMA rate the chip
 * sustains and the clock it holds under that load - the method of the reference's roofline probe
 * (benchmark/pi05/hardware_probe.py:36-99) applied to the instruction this path is bound by.
 */
int phyai_fp8_debug_mfma_rate(int workgroups, int iters, uint64_t *counters, float *sink, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PHYAI_FP8_H */
