// extern "C" boundary of the fp8 linear library: argument validation, workspace
// carving and kernel selection.  No allocation, no synchronisation.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>

#include <mutex>

#include "../../include/phyai_fp8.h"
#include "fp8_device.h"
#include "launch.h"
#include "weight_layout.h"

// Scratch of phyai_fp8_linear_static: one array per GPU, part of the loaded code object (zero when
// the module is loaded), held until the process ends.  The name is only a handle on the host; the
// array's device address comes from hipGetSymbolAddress, per device (static_scratch_of below).
static __device__ __align__(256) uint8_t scratch[PHYAI_FP8_STATIC_SCRATCH_BYTES];

namespace {

thread_local char g_err[256] = "";

int fail(int code, const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int check_launch(const char* what) {
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(PHYAI_FP8_ELAUNCH, "%s: %s", what, hipGetErrorString(e));
    return PHYAI_FP8_OK;
}

bool aligned(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

size_t align_up(size_t v, size_t a) { return (v + a - 1) / a * a; }

constexpr int64_t kMaxElems = (int64_t)1 << 31;  // kernels index rows with 32-bit offsets

int check_epilogue(int epilogue, int64_t N) {
    if (epilogue < PHYAI_FP8_EPI_NONE || epilogue > PHYAI_FP8_EPI_GELU_ERF)
        return fail(PHYAI_FP8_EINVAL, "unknown epilogue %d", epilogue);
    if (phyai::epi_is_gated(epilogue) && (N % 32) != 0)
        return fail(PHYAI_FP8_EUNSUPPORTED, "gated epilogue needs N %% 32 == 0 (gate/up halves of 16-aligned width), got N=%lld", (long long)N);
    return 0;
}

// Workspace layout of phyai_fp8_linear: [GEMM region][xq codes][x_scale].
struct LinearCarve {
    size_t gemm_bytes, xq_off, xs_off, total;
};
LinearCarve carve(int64_t M, int64_t N, int64_t K, int epilogue) {
    LinearCarve c;
    {
        const int64_t n_out = phyai::epi_is_gated(epilogue) ? N / 2 : N;
        // worst case over output strides: the widest of the kernels that may be chosen
        size_t a = phyai::gemm_workspace_bytes(M, N, K, epilogue, n_out);
        size_t b = phyai::gemm_workspace_bytes(M, N, K, epilogue, 1);
        c.gemm_bytes = align_up(a > b ? a : b, 256);
    }
    c.xq_off = c.gemm_bytes;
    c.xs_off = c.xq_off + align_up((size_t)(M > 0 ? M : 0) * (size_t)(K > 0 ? K : 0), 256);
    c.total = c.xs_off + align_up((size_t)(M > 0 ? M : 0) * sizeof(float), 256);
    return c;
}

int check_quant_args(const char* fn, const void* x, int64_t M, int64_t K, int64_t ldx, const void* xq) {
    if (M < 0 || K <= 0) return fail(PHYAI_FP8_EINVAL, "%s: bad shape M=%lld K=%lld", fn, (long long)M, (long long)K);
    if (M == 0) return 0;
    if (!x || !xq) return fail(PHYAI_FP8_EINVAL, "%s: null pointer", fn);
    if (K % 8 != 0) return fail(PHYAI_FP8_EUNSUPPORTED, "%s: K=%lld must be a multiple of 8", fn, (long long)K);
    if (ldx < K || ldx % 8 != 0) return fail(PHYAI_FP8_EINVAL, "%s: row stride %lld must be >= K and a multiple of 8", fn, (long long)ldx);
    if (!aligned(x, 16) || !aligned(xq, 8)) return fail(PHYAI_FP8_EINVAL, "%s: x must be 16-byte and xq 8-byte aligned", fn);
    if (M * ldx >= kMaxElems * 4 || M >= kMaxElems) return fail(PHYAI_FP8_EUNSUPPORTED, "%s: tensor too large", fn);
    return 0;
}

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Device address of `scratch` on the current device: looked up once per device, with that device
// current, and kept (every GPU holds its own copy of the array at its own address).
int static_scratch_of(void** ptr) {
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return fail(PHYAI_FP8_ELAUNCH, "phyai_fp8_linear_static: hipGetDevice: %s", hipGetErrorString(e));
    if (dev < 0 || dev >= kMaxDevices) return fail(PHYAI_FP8_EUNSUPPORTED, "phyai_fp8_linear_static: device %d out of range", dev);
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (g_scratch_ptr[dev] == nullptr) {
        void* p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        if (e != hipSuccess || p == nullptr)
            return fail(PHYAI_FP8_ELAUNCH, "phyai_fp8_linear_static: hipGetSymbolAddress: %s", hipGetErrorString(e));
        g_scratch_ptr[dev] = p;
    }
    *ptr = g_scratch_ptr[dev];
    return 0;
}

// Zeroes the split-K arrival counters at the head of a workspace (a kernel, not a memset, so that it
// can be recorded into a graph).
__global__ __launch_bounds__(256) void zero_header_kernel(uint32_t* __restrict__ p, int n) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i < n) p[i] = 0u;
}

}  // namespace

extern "C" {

int phyai_fp8_abi_version(void) { return PHYAI_FP8_ABI_VERSION; }

const char* phyai_fp8_last_error(void) { return g_err; }

int phyai_fp8_quant_rowwise(const void* x, int64_t M, int64_t K, int64_t ldx, void* xq,
                            float* x_scale, void* stream) {
    if (int rc = check_quant_args("phyai_fp8_quant_rowwise", x, M, K, ldx, xq)) return rc;
    if (M == 0) return PHYAI_FP8_OK;
    if (!x_scale) return fail(PHYAI_FP8_EINVAL, "phyai_fp8_quant_rowwise: null x_scale");
    phyai::launch_quant_rowwise(x, M, K, ldx, xq, x_scale, static_cast<hipStream_t>(stream));
    return check_launch("phyai_fp8_quant_rowwise");
}

int phyai_fp8_quant_static(const void* x, int64_t M, int64_t K, int64_t ldx,
                           const float* input_scale, void* xq, void* stream) {
    if (int rc = check_quant_args("phyai_fp8_quant_static", x, M, K, ldx, xq)) return rc;
    if (M == 0) return PHYAI_FP8_OK;
    if (!input_scale) return fail(PHYAI_FP8_EINVAL, "phyai_fp8_quant_static: null input_scale");
    phyai::launch_quant_static(x, M, K, ldx, input_scale, xq, static_cast<hipStream_t>(stream));
    return check_launch("phyai_fp8_quant_static");
}

int phyai_fp8_weight_quant_rowwise(const void* w, int64_t N, int64_t K, int64_t ldw, void* wq,
                                   float* w_scale, void* stream) {
    if (int rc = check_quant_args("phyai_fp8_weight_quant_rowwise", w, N, K, ldw, wq)) return rc;
    if (N == 0) return PHYAI_FP8_OK;
    if (!w_scale) return fail(PHYAI_FP8_EINVAL, "phyai_fp8_weight_quant_rowwise: null w_scale");
    phyai::launch_weight_quant(w, N, K, ldw, wq, w_scale, static_cast<hipStream_t>(stream));
    return check_launch("phyai_fp8_weight_quant_rowwise");
}

int phyai_fp8_weight_to_operand_order(const void* w, int64_t N, int64_t K, int gated, void* out, void* stream) {
    const char* fn = "phyai_fp8_weight_to_operand_order";
    if (N < 0 || K <= 0) return fail(PHYAI_FP8_EINVAL, "%s: bad shape N=%lld K=%lld", fn, (long long)N, (long long)K);
    if (N == 0) return PHYAI_FP8_OK;
    if (!w || !out) return fail(PHYAI_FP8_EINVAL, "%s: null pointer", fn);
    if (K % 128 != 0 || N % (gated ? 32 : 16) != 0)
        return fail(PHYAI_FP8_EUNSUPPORTED, "%s: needs K %% 128 == 0 and N %% %d == 0, got N=%lld K=%lld", fn, gated ? 32 : 16,
                    (long long)N, (long long)K);
    if (!aligned(w, 16) || !aligned(out, 16)) return fail(PHYAI_FP8_EINVAL, "%s: w and out must be 16-byte aligned", fn);
    if (N * K >= kMaxElems) return fail(PHYAI_FP8_EUNSUPPORTED, "%s: matrix larger than 2^31 elements", fn);
    const uintptr_t a = reinterpret_cast<uintptr_t>(w), b = reinterpret_cast<uintptr_t>(out), n = (uintptr_t)(N * K);
    if (a < b + n && b < a + n) return fail(PHYAI_FP8_EINVAL, "%s: out overlaps w (the re-lay is not in place)", fn);
    if (phyai::launch_weight_to_operand_order(w, N, K, gated ? 1 : 0, out, static_cast<hipStream_t>(stream)) != 0)
        return fail(PHYAI_FP8_EUNSUPPORTED, "%s: matrix too large", fn);
    return check_launch(fn);
}

size_t phyai_fp8_linear_workspace_bytes(int64_t M, int64_t N, int64_t K, int epilogue) {
    return carve(M, N, K, epilogue & PHYAI_FP8_EPILOGUE_MASK).total;
}

namespace {
// Gated residual of phyai_fp8_gemm_addcmul / phyai_fp8_linear_addcmul; all null for the plain forms.
struct ResidualSpec {
    const void* residual;
    int64_t ld_res;
    const void* gate;
    int64_t ld_gate;
    int64_t gate_rows;
};

int check_residual(const char* fn, const ResidualSpec& r, int64_t M, int64_t N, int epilogue) {
    if (!r.residual && !r.gate) return 0;
    if (!r.residual || !r.gate) return fail(PHYAI_FP8_EINVAL, "%s: residual and gate go together", fn);
    if (epilogue != PHYAI_FP8_EPI_NONE) return fail(PHYAI_FP8_EINVAL, "%s: a gated residual excludes an activation epilogue", fn);
    if (!aligned(r.residual, 16) || !aligned(r.gate, 16) || r.ld_res < N || r.ld_gate < N || r.ld_res % 8 != 0 || r.ld_gate % 8 != 0)
        return fail(PHYAI_FP8_EINVAL, "%s: residual and gate must be 16-byte aligned with row strides >= N, multiples of 8", fn);
    if (r.gate_rows <= 0 || (M > 0 && M % r.gate_rows != 0))
        return fail(PHYAI_FP8_EINVAL, "%s: M=%lld must be a multiple of the gate rows (%lld)", fn, (long long)M, (long long)r.gate_rows);
    return 0;
}

// Validates a GEMM call and fills in the problem; nothing is launched.  `flagged_epilogue` may carry
// PHYAI_FP8_FLAG_* bits.  Returns 0, or a status after fail().
int prepare_gemm(const char* fn, const void* xq, const float* x_scale, int x_scale_is_scalar, const void* w,
                 const float* w_scale, const void* bias, const ResidualSpec& res, void* out, int64_t ldo, int64_t M,
                 int64_t N, int64_t K, int flagged_epilogue, void* workspace, size_t workspace_bytes,
                 phyai::GemmProblem* problem, const void* x_bf16 = nullptr, int64_t ldx = 0) {
    if (M < 0 || N <= 0 || K <= 0)
        return fail(PHYAI_FP8_EINVAL, "%s: bad shape M=%lld N=%lld K=%lld", fn, (long long)M, (long long)N, (long long)K);
    const int flags = flagged_epilogue & ~PHYAI_FP8_EPILOGUE_MASK;
    const int epilogue = flagged_epilogue & PHYAI_FP8_EPILOGUE_MASK;
    if (flags & ~(PHYAI_FP8_FLAG_STREAM_WEIGHTS | PHYAI_FP8_FLAG_W_OPERAND_GATED))
        return fail(PHYAI_FP8_EINVAL, "%s: unknown flag bits 0x%x", fn, flags);
    if (int rc = check_epilogue(epilogue, N)) return rc;
    int layout = phyai::W_ROW_MAJOR;
    if (flags & PHYAI_FP8_FLAG_W_OPERAND_GATED) {
        const bool gated_w = (flags & PHYAI_FP8_FLAG_W_OPERAND_GATED) == PHYAI_FP8_FLAG_W_OPERAND_GATED;
        if (!(flags & PHYAI_FP8_FLAG_W_OPERAND_ORDER))
            return fail(PHYAI_FP8_EINVAL, "%s: flag bits 0x%x name no weight layout", fn, flags);
        if (gated_w != phyai::epi_is_gated(epilogue))
            return fail(PHYAI_FP8_EINVAL, "%s: a gated epilogue needs weights in the gated operand order and any other "
                        "epilogue the plain one (epilogue %d, flags 0x%x)", fn, epilogue, flags);
        if (K % 128 != 0)
            return fail(PHYAI_FP8_EUNSUPPORTED, "%s: weights in operand order need K %% 128 == 0, got K=%lld", fn, (long long)K);
        layout = gated_w ? phyai::W_OPERAND_GATED : phyai::W_OPERAND_PLAIN;
    }
    if (K % 16 != 0 || N % 16 != 0)
        return fail(PHYAI_FP8_EUNSUPPORTED, "%s: K=%lld and N=%lld must be multiples of 16", fn, (long long)K, (long long)N);
    if (int rc = check_residual(fn, res, M, N, epilogue)) return rc;
    phyai::GemmProblem g = {};
    g.M = (int)M; g.N = (int)N; g.K = (int)K;
    *problem = g;
    if (M == 0) return PHYAI_FP8_OK;
    if (!xq || !x_scale || !w || !w_scale || !out) return fail(PHYAI_FP8_EINVAL, "%s: null pointer", fn);
    if (!aligned(xq, 16) || !aligned(w, 16)) return fail(PHYAI_FP8_EINVAL, "%s: xq and w must be 16-byte aligned", fn);
    const int64_t n_out = phyai::epi_is_gated(epilogue) ? N / 2 : N;
    if (ldo < n_out) return fail(PHYAI_FP8_EINVAL, "%s: ldo=%lld < output width %lld", fn, (long long)ldo, (long long)n_out);
    if (M * K >= kMaxElems || N * K >= kMaxElems || M * ldo >= kMaxElems * 2)
        return fail(PHYAI_FP8_EUNSUPPORTED, "%s: operand larger than 2^31 elements", fn);
    if (workspace && !aligned(workspace, 256)) return fail(PHYAI_FP8_EINVAL, "%s: workspace must be 256-byte aligned", fn);

    g.xq = static_cast<const uint8_t*>(xq);
    g.x_scale = x_scale;
    g.x_scale_is_scalar = x_scale_is_scalar ? 1 : 0;
    g.w = static_cast<const uint8_t*>(w);
    g.w_scale = w_scale;
    g.bias = static_cast<const uint16_t*>(bias);
    g.out = static_cast<uint16_t*>(out);
    g.ldo = ldo;
    g.epilogue = epilogue;
    g.stream_weights = (flags & PHYAI_FP8_FLAG_STREAM_WEIGHTS) ? 1 : 0;
    g.weight_layout = layout;
    g.workspace = workspace;
    g.workspace_bytes = workspace_bytes;
    g.gate_group = 1;
    g.x_bf16 = static_cast<const uint16_t*>(x_bf16);
    g.ldx = ldx;
    if (res.residual) {
        g.residual = static_cast<const uint16_t*>(res.residual);
        g.ld_res = res.ld_res;
        g.gate = static_cast<const uint16_t*>(res.gate);
        g.ld_gate = res.ld_gate;
        g.gate_group = (int)(M / res.gate_rows);
    }
    const size_t need = phyai::gemm_scratch_need(g);
    if (need > 0 && (workspace == nullptr || workspace_bytes < need))
        return fail(PHYAI_FP8_EWORKSPACE, "%s: workspace of %zu bytes is too small, need %zu", fn,
                    workspace ? workspace_bytes : (size_t)0, need);
    *problem = g;
    return PHYAI_FP8_OK;
}

int launch_prepared(const char* fn, const phyai::GemmProblem& g, void* stream) {
    if (g.M == 0) return PHYAI_FP8_OK;
    const int rc = phyai::launch_gemm(g, static_cast<hipStream_t>(stream));
    if (rc == -3) return fail(PHYAI_FP8_EWORKSPACE, "%s: workspace too small for the chosen kernel", fn);
    if (rc != 0) return fail(PHYAI_FP8_EUNSUPPORTED, "%s: no kernel for this problem (rc=%d)", fn, rc);
    return check_launch(fn);
}

int run_gemm(const char* fn, const void* xq, const float* x_scale, int x_scale_is_scalar, const void* w,
             const float* w_scale, const void* bias, const ResidualSpec& res, void* out, int64_t ldo, int64_t M,
             int64_t N, int64_t K, int epilogue, void* workspace, size_t workspace_bytes, void* stream) {
    phyai::GemmProblem g;
    if (int rc = prepare_gemm(fn, xq, x_scale, x_scale_is_scalar, w, w_scale, bias, res, out, ldo, M, N, K, epilogue,
                              workspace, workspace_bytes, &g))
        return rc;
    return launch_prepared(fn, g, stream);
}

// Quantizer + GEMM with the codes and scales staged at xq / xs and the GEMM's own scratch at
// gemm_ws.  Every argument of both launches is checked before the first one is enqueued.
int run_linear_at(const char* fn, const void* x, int64_t ldx, const void* w, const float* w_scale, const void* bias,
                  const ResidualSpec& res, void* out, int64_t ldo, int64_t M, int64_t N, int64_t K, int epilogue,
                  void* xq, float* xs, void* gemm_ws, size_t gemm_ws_bytes, void* stream) {
    if (int rc = check_quant_args(fn, x, M, K, ldx, xq)) return rc;
    phyai::GemmProblem g;
    if (int rc = prepare_gemm(fn, xq, xs, 0, w, w_scale, bias, res, out, ldo, M, N, K, epilogue, gemm_ws,
                              gemm_ws_bytes, &g, x, ldx))
        return rc;
    // small token counts: one kernel quantizes its rows and multiplies them; otherwise two launches
    if (!phyai::gemm_quantizes_itself(g)) {
        phyai::launch_quant_rowwise(x, M, K, ldx, xq, xs, static_cast<hipStream_t>(stream));
        if (int rc = check_launch(fn)) return rc;
    }
    return launch_prepared(fn, g, stream);
}

int run_linear(const char* fn, const void* x, int64_t ldx, const void* w, const float* w_scale, const void* bias,
               const ResidualSpec& res, void* out, int64_t ldo, int64_t M, int64_t N, int64_t K, int epilogue,
               void* workspace, size_t workspace_bytes, void* stream) {
    if (M < 0 || N <= 0 || K <= 0)
        return fail(PHYAI_FP8_EINVAL, "%s: bad shape M=%lld N=%lld K=%lld", fn, (long long)M, (long long)N, (long long)K);
    if (M == 0) return PHYAI_FP8_OK;
    const LinearCarve c = carve(M, N, K, epilogue & PHYAI_FP8_EPILOGUE_MASK);
    if (!workspace || workspace_bytes < c.total) {
        // The kernel that quantizes its own rows touches neither staged codes nor GEMM scratch: a call
        // that it serves needs no workspace at all (x stands in for the code and scale pointers, which
        // are never dereferenced then).
        phyai::GemmProblem g;
        if (x && check_quant_args(fn, x, M, K, ldx, x) == 0 &&
            prepare_gemm(fn, x, static_cast<const float*>(x), 0, w, w_scale, bias, res, out, ldo, M, N, K, epilogue, nullptr,
                         0, &g, x, ldx) == 0 &&
            phyai::gemm_quantizes_itself(g))
            return launch_prepared(fn, g, stream);
        return fail(PHYAI_FP8_EWORKSPACE, "%s: workspace of %zu bytes is too small, need %zu", fn,
                    workspace ? workspace_bytes : (size_t)0, c.total);
    }
    if (!aligned(workspace, 256)) return fail(PHYAI_FP8_EINVAL, "%s: workspace must be 256-byte aligned", fn);
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    return run_linear_at(fn, x, ldx, w, w_scale, bias, res, out, ldo, M, N, K, epilogue, ws + c.xq_off,
                         reinterpret_cast<float*>(ws + c.xs_off), workspace, c.gemm_bytes, stream);
}
}  // namespace

int phyai_fp8_gemm(const void* xq, const float* x_scale, int x_scale_is_scalar, const void* w,
                   const float* w_scale, const void* bias, void* out, int64_t ldo, int64_t M,
                   int64_t N, int64_t K, int epilogue, void* workspace, size_t workspace_bytes,
                   void* stream) {
    return run_gemm("phyai_fp8_gemm", xq, x_scale, x_scale_is_scalar, w, w_scale, bias, ResidualSpec{}, out, ldo,
                    M, N, K, epilogue, workspace, workspace_bytes, stream);
}

int phyai_fp8_gemm_addcmul(const void* xq, const float* x_scale, int x_scale_is_scalar, const void* w,
                           const float* w_scale, const void* bias, const void* residual, int64_t ld_res,
                           const void* gate, int64_t ld_gate, int64_t gate_rows, void* out, int64_t ldo,
                           int64_t M, int64_t N, int64_t K, int flags, void* workspace, size_t workspace_bytes,
                           void* stream) {
    if (!residual || !gate) return fail(PHYAI_FP8_EINVAL, "phyai_fp8_gemm_addcmul: null residual or gate");
    if (flags & PHYAI_FP8_EPILOGUE_MASK) return fail(PHYAI_FP8_EINVAL, "phyai_fp8_gemm_addcmul: flags 0x%x carry an epilogue", flags);
    const ResidualSpec r = {residual, ld_res, gate, ld_gate, gate_rows};
    return run_gemm("phyai_fp8_gemm_addcmul", xq, x_scale, x_scale_is_scalar, w, w_scale, bias, r, out, ldo, M, N,
                    K, PHYAI_FP8_EPI_NONE | flags, workspace, workspace_bytes, stream);
}

int phyai_fp8_linear(const void* x, int64_t ldx, const void* w, const float* w_scale,
                     const void* bias, void* out, int64_t ldo, int64_t M, int64_t N, int64_t K,
                     int epilogue, void* workspace, size_t workspace_bytes, void* stream) {
    return run_linear("phyai_fp8_linear", x, ldx, w, w_scale, bias, ResidualSpec{}, out, ldo, M, N, K, epilogue,
                      workspace, workspace_bytes, stream);
}

int phyai_fp8_linear_addcmul(const void* x, int64_t ldx, const void* w, const float* w_scale,
                             const void* bias, const void* residual, int64_t ld_res, const void* gate,
                             int64_t ld_gate, int64_t gate_rows, void* out, int64_t ldo, int64_t M,
                             int64_t N, int64_t K, int flags, void* workspace, size_t workspace_bytes, void* stream) {
    if (!residual || !gate) return fail(PHYAI_FP8_EINVAL, "phyai_fp8_linear_addcmul: null residual or gate");
    if (flags & PHYAI_FP8_EPILOGUE_MASK) return fail(PHYAI_FP8_EINVAL, "phyai_fp8_linear_addcmul: flags 0x%x carry an epilogue", flags);
    const ResidualSpec r = {residual, ld_res, gate, ld_gate, gate_rows};
    return run_linear("phyai_fp8_linear_addcmul", x, ldx, w, w_scale, bias, r, out, ldo, M, N, K,
                      PHYAI_FP8_EPI_NONE | flags, workspace, workspace_bytes, stream);
}

namespace {
// Workspace of phyai_fp8_mlp: [scratch of either linear][h: M x I bf16][row maxima: M x 64 x 16 bit].
struct MlpCarve {
    size_t linear_bytes, h_off, amax_off, total;
    LinearCarve first, second;
};
MlpCarve mlp_carve(int64_t M, int64_t H, int64_t I, int64_t O, int epilogue) {
    MlpCarve c;
    const int64_t n1 = phyai::epi_is_gated(epilogue) ? 2 * I : I;
    c.first = carve(M, n1, H, epilogue);
    c.second = carve(M, O, I, PHYAI_FP8_EPI_NONE);
    c.linear_bytes = c.first.total > c.second.total ? c.first.total : c.second.total;
    c.h_off = c.linear_bytes;
    c.amax_off = c.h_off + align_up((size_t)(M > 0 ? M : 0) * (size_t)(I > 0 ? I : 0) * 2, 256);
    c.total = c.amax_off + align_up((size_t)(M > 0 ? M : 0) * phyai::kRowAmaxSlots * 2, 256);
    return c;
}
}  // namespace

size_t phyai_fp8_mlp_workspace_bytes(int64_t M, int64_t H, int64_t I, int64_t O, int epilogue) {
    return mlp_carve(M, H, I, O, epilogue & PHYAI_FP8_EPILOGUE_MASK).total;
}

int phyai_fp8_mlp(const void* x, int64_t ldx, const void* w1, const float* w1_scale, const void* bias1, int flags1,
                  const void* w2, const float* w2_scale, const void* bias2, int flags2, const void* residual,
                  int64_t ld_res, const void* gate, int64_t ld_gate, int64_t gate_rows, void* out, int64_t ldo, int64_t M,
                  int64_t H, int64_t I, int64_t O, int epilogue, void* workspace, size_t workspace_bytes, void* stream) {
    const char* fn = "phyai_fp8_mlp";
    if (M < 0 || H <= 0 || I <= 0 || O <= 0)
        return fail(PHYAI_FP8_EINVAL, "%s: bad shape M=%lld H=%lld I=%lld O=%lld", fn, (long long)M, (long long)H, (long long)I, (long long)O);
    if ((epilogue & ~PHYAI_FP8_EPILOGUE_MASK) || epilogue <= PHYAI_FP8_EPI_NONE || epilogue > PHYAI_FP8_EPI_GELU_ERF)
        return fail(PHYAI_FP8_EINVAL, "%s: epilogue %d is not an activation", fn, epilogue);
    if ((flags1 | flags2) & PHYAI_FP8_EPILOGUE_MASK) return fail(PHYAI_FP8_EINVAL, "%s: flags carry an epilogue", fn);
    if ((residual == nullptr) != (gate == nullptr)) return fail(PHYAI_FP8_EINVAL, "%s: residual and gate go together", fn);
    if (M == 0) return PHYAI_FP8_OK;
    const MlpCarve c = mlp_carve(M, H, I, O, epilogue);
    if (!workspace || workspace_bytes < c.total)
        return fail(PHYAI_FP8_EWORKSPACE, "%s: workspace of %zu bytes is too small, need %zu", fn,
                    workspace ? workspace_bytes : (size_t)0, c.total);
    if (!aligned(workspace, 256)) return fail(PHYAI_FP8_EINVAL, "%s: workspace must be 256-byte aligned", fn);
    uint8_t* ws = static_cast<uint8_t*>(workspace);
    void* h = ws + c.h_off;
    uint16_t* table = reinterpret_cast<uint16_t*>(ws + c.amax_off);
    const int64_t n1 = phyai::epi_is_gated(epilogue) ? 2 * I : I;
    const ResidualSpec res = {residual, ld_res, gate, ld_gate, gate_rows};
    // both problems are validated before anything is enqueued
    phyai::GemmProblem g1, g2;
    if (int rc = check_quant_args(fn, x, M, H, ldx, ws + c.first.xq_off)) return rc;
    if (int rc = prepare_gemm(fn, ws + c.first.xq_off, reinterpret_cast<float*>(ws + c.first.xs_off), 0, w1, w1_scale, bias1,
                              ResidualSpec{}, h, I, M, n1, H, epilogue | flags1, workspace, c.first.gemm_bytes, &g1, x, ldx))
        return rc;
    if (int rc = prepare_gemm(fn, ws + c.second.xq_off, reinterpret_cast<float*>(ws + c.second.xs_off), 0, w2, w2_scale, bias2,
                              res, out, ldo, M, O, I, PHYAI_FP8_EPI_NONE | flags2, workspace, c.second.gemm_bytes, &g2, h, I))
        return rc;
    const int slots = phyai::gemm_row_maxima_slots(g1);
    if (slots > 0) {
        g2.amax_in = table;
        g2.amax_parts = slots;
        if (phyai::gemm_takes_row_maxima(g2)) g1.amax_out = table;
        else g2.amax_in = nullptr;
    }
    const hipStream_t st = static_cast<hipStream_t>(stream);
    if (!phyai::gemm_quantizes_itself(g1)) {
        phyai::launch_quant_rowwise(x, M, H, ldx, ws + c.first.xq_off, reinterpret_cast<float*>(ws + c.first.xs_off), st);
        if (int rc = check_launch(fn)) return rc;
    }
    if (int rc = launch_prepared(fn, g1, stream)) return rc;
    if (!phyai::gemm_quantizes_itself(g2)) {
        phyai::launch_quant_rowwise(h, M, I, I, ws + c.second.xq_off, reinterpret_cast<float*>(ws + c.second.xs_off), st);
        if (int rc = check_launch(fn)) return rc;
    }
    return launch_prepared(fn, g2, stream);
}

int phyai_fp8_linear_static(const void* x, int64_t ldx, const void* w, const float* w_scale, const void* bias,
                            void* out, int64_t ldo, int64_t M, int64_t N, int64_t K, int epilogue, void* stream) {
    const char* fn = "phyai_fp8_linear_static";
    constexpr size_t kScratch = PHYAI_FP8_STATIC_SCRATCH_BYTES;
    if (M < 0 || N <= 0 || K <= 0)
        return fail(PHYAI_FP8_EINVAL, "%s: bad shape M=%lld N=%lld K=%lld", fn, (long long)M, (long long)N, (long long)K);
    if (M == 0) return PHYAI_FP8_OK;
    // Layout of the array: [split-K counters | partial sums ...        ... codes | per-token scales].
    // The GEMM gets whatever the staging at the tail leaves; its need depends on the kernel that
    // serves exactly this call and is checked before anything is launched.
    if (M >= kMaxElems || K >= kMaxElems) return fail(PHYAI_FP8_EUNSUPPORTED, "%s: tensor too large", fn);
    const size_t xs_bytes = align_up((size_t)M * sizeof(float), 256), xq_bytes = align_up((size_t)M * (size_t)K, 256);
    if (xs_bytes + xq_bytes + PHYAI_FP8_WORKSPACE_HEADER_BYTES > kScratch)
        return fail(PHYAI_FP8_EWORKSPACE, "%s: the activation codes of this shape need %zu bytes, the static array holds %zu; "
                    "use phyai_fp8_linear with a caller-owned workspace", fn, xs_bytes + xq_bytes, kScratch);
    void* base = nullptr;
    if (int rc = static_scratch_of(&base)) return rc;
    uint8_t* ws = static_cast<uint8_t*>(base);
    const size_t xq_off = kScratch - xs_bytes - xq_bytes, gemm_bytes = xq_off;
    void* xq = ws + xq_off;
    float* xs = reinterpret_cast<float*>(ws + xq_off + xq_bytes);
    if (int rc = check_quant_args(fn, x, M, K, ldx, xq)) return rc;
    phyai::GemmProblem g;
    if (int rc = prepare_gemm(fn, xq, xs, 0, w, w_scale, bias, ResidualSpec{}, out, ldo, M, N, K, epilogue, ws,
                              gemm_bytes, &g, x, ldx)) {
        if (rc == PHYAI_FP8_EWORKSPACE)
            return fail(rc, "%s: this shape needs more scratch than the static array holds (%zu bytes, %zu of them for "
                        "activation codes); use phyai_fp8_linear with a caller-owned workspace", fn, kScratch, xs_bytes + xq_bytes);
        return rc;
    }
    const hipStream_t st = static_cast<hipStream_t>(stream);
    // The array keeps what the last call left.  Codes, scales and partial sums are written before
    // they are read; the split-K arrival counters must start at zero, and although the kernels put
    // them back to zero themselves, a call that uses them clears them first (with a kernel, not a
    // memset, so that the call can be recorded into a graph).
    if (phyai::gemm_scratch_need(g) > 0) {
        const int n = PHYAI_FP8_WORKSPACE_HEADER_BYTES / 4;
        hipLaunchKernelGGL(zero_header_kernel, dim3((n + 255) / 256), dim3(256), 0, st, reinterpret_cast<uint32_t*>(ws), n);
        if (int rc = check_launch(fn)) return rc;
    }
    if (!phyai::gemm_quantizes_itself(g)) {
        phyai::launch_quant_rowwise(x, M, K, ldx, xq, xs, st);
        if (int rc = check_launch(fn)) return rc;
    }
    return launch_prepared(fn, g, stream);
}

namespace {
int check_norm_args(const char* fn, const void* x, int64_t ldx, int64_t M, int64_t D, const void* out,
                    int64_t ldo, const void* xq, const float* x_scale) {
    if (M < 0 || D <= 0) return fail(PHYAI_FP8_EINVAL, "%s: bad shape M=%lld D=%lld", fn, (long long)M, (long long)D);
    if (M == 0) return 0;
    if (!x) return fail(PHYAI_FP8_EINVAL, "%s: null x", fn);
    if (!out && !xq) return fail(PHYAI_FP8_EINVAL, "%s: neither out nor xq given", fn);
    if ((xq == nullptr) != (x_scale == nullptr)) return fail(PHYAI_FP8_EINVAL, "%s: xq and x_scale go together", fn);
    if (D % 8 != 0) return fail(PHYAI_FP8_EUNSUPPORTED, "%s: D=%lld must be a multiple of 8", fn, (long long)D);
    if (D > (1 << 20)) return fail(PHYAI_FP8_EUNSUPPORTED, "%s: D=%lld exceeds 2^20", fn, (long long)D);
    if (ldx < D || ldx % 8 != 0 || (out && (ldo < D || ldo % 8 != 0)))
        return fail(PHYAI_FP8_EINVAL, "%s: row strides must be >= D and multiples of 8", fn);
    if (!aligned(x, 16) || (out && !aligned(out, 16)) || (xq && !aligned(xq, 8)))
        return fail(PHYAI_FP8_EINVAL, "%s: x and out must be 16-byte, xq 8-byte aligned", fn);
    if (M * ldx >= kMaxElems * 4 || M >= kMaxElems) return fail(PHYAI_FP8_EUNSUPPORTED, "%s: tensor too large", fn);
    return 0;
}
}  // namespace

int phyai_fp8_rmsnorm_quant(const void* x, int64_t ldx, const void* weight, int gemma, int64_t M,
                            int64_t D, float eps, void* out, int64_t ldo, void* xq, float* x_scale,
                            void* stream) {
    if (int rc = check_norm_args("phyai_fp8_rmsnorm_quant", x, ldx, M, D, out, ldo, xq, x_scale)) return rc;
    if (M == 0) return PHYAI_FP8_OK;
    if (!weight || !aligned(weight, 16)) return fail(PHYAI_FP8_EINVAL, "phyai_fp8_rmsnorm_quant: weight must be a 16-byte aligned pointer");
    phyai::NormQuantArgs a = {};
    a.x = static_cast<const uint16_t*>(x); a.ldx = ldx; a.D = (int)D; a.eps = eps;
    a.weight = static_cast<const uint16_t*>(weight); a.gemma = gemma ? 1 : 0;
    a.group = 1;
    a.out = static_cast<uint16_t*>(out); a.ldo = ldo;
    a.xq = static_cast<uint8_t*>(xq); a.scale = x_scale;
    if (phyai::launch_norm_quant(a, M, false, static_cast<hipStream_t>(stream)) != 0)
        return fail(PHYAI_FP8_EUNSUPPORTED, "phyai_fp8_rmsnorm_quant: no kernel for D=%lld", (long long)D);
    return check_launch("phyai_fp8_rmsnorm_quant");
}

int phyai_fp8_adarmsnorm_quant(const void* x, int64_t ldx, const void* modulation, int64_t ld_mod,
                               int64_t mod_rows, int64_t M, int64_t D, float eps, void* out,
                               int64_t ldo, void* gate_out, int64_t ld_gate, void* xq, float* x_scale,
                               void* stream) {
    if (int rc = check_norm_args("phyai_fp8_adarmsnorm_quant", x, ldx, M, D, out, ldo, xq, x_scale)) return rc;
    if (M == 0) return PHYAI_FP8_OK;
    if (!modulation || !aligned(modulation, 16) || ld_mod < 3 * D || ld_mod % 8 != 0)
        return fail(PHYAI_FP8_EINVAL, "phyai_fp8_adarmsnorm_quant: modulation must be 16-byte aligned with row stride >= 3*D, a multiple of 8");
    if (mod_rows <= 0 || M % mod_rows != 0)
        return fail(PHYAI_FP8_EINVAL, "phyai_fp8_adarmsnorm_quant: M=%lld must be a non-zero multiple of the modulation rows (%lld)", (long long)M, (long long)mod_rows);
    if (gate_out && (!aligned(gate_out, 16) || ld_gate < D || ld_gate % 8 != 0))
        return fail(PHYAI_FP8_EINVAL, "phyai_fp8_adarmsnorm_quant: gate_out must be 16-byte aligned with row stride >= D, a multiple of 8");
    phyai::NormQuantArgs a = {};
    a.x = static_cast<const uint16_t*>(x); a.ldx = ldx; a.D = (int)D; a.eps = eps;
    a.mod = static_cast<const uint16_t*>(modulation); a.ld_mod = ld_mod; a.group = (int)(M / mod_rows);
    a.out = static_cast<uint16_t*>(out); a.ldo = ldo;
    a.gate = static_cast<uint16_t*>(gate_out); a.ld_gate = ld_gate;
    a.xq = static_cast<uint8_t*>(xq); a.scale = x_scale;
    if (phyai::launch_norm_quant(a, M, true, static_cast<hipStream_t>(stream)) != 0)
        return fail(PHYAI_FP8_EUNSUPPORTED, "phyai_fp8_adarmsnorm_quant: no kernel for D=%lld", (long long)D);
    return check_launch("phyai_fp8_adarmsnorm_quant");
}

int phyai_fp8_describe_plan(int64_t M, int64_t N, int64_t K, int epilogue, char* buf, size_t n) {
    if (!buf || n == 0) return fail(PHYAI_FP8_EINVAL, "phyai_fp8_describe_plan: no buffer");
    buf[0] = 0;
    if (M < 0 || N <= 0 || K <= 0 || M >= kMaxElems || N >= kMaxElems || K >= kMaxElems)
        return fail(PHYAI_FP8_EINVAL, "phyai_fp8_describe_plan: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    const int layout_bits = epilogue & PHYAI_FP8_FLAG_W_OPERAND_GATED;
    epilogue &= PHYAI_FP8_EPILOGUE_MASK;   // of the flags only the layout of the weights bears on the choice of kernel
    if (int rc = check_epilogue(epilogue, N)) return rc;
    if (K % 16 != 0 || N % 16 != 0)
        return fail(PHYAI_FP8_EUNSUPPORTED, "phyai_fp8_describe_plan: K=%lld and N=%lld must be multiples of 16", (long long)K, (long long)N);
    int layout = phyai::W_ROW_MAJOR;
    if (layout_bits && K % 128 == 0 && N % (phyai::epi_is_gated(epilogue) ? 32 : 16) == 0)
        layout = phyai::epi_is_gated(epilogue) ? phyai::W_OPERAND_GATED : phyai::W_OPERAND_PLAIN;
    const int len = phyai::describe_gemm_plan((int)M, (int)N, (int)K, epilogue, buf, n, layout);
    buf[n - 1] = 0;
    return len;
}

int phyai_fp8_describe_linear_plan(int64_t M, int64_t N, int64_t K, int epilogue, char* buf, size_t n) {
    if (!buf || n == 0) return fail(PHYAI_FP8_EINVAL, "phyai_fp8_describe_linear_plan: no buffer");
    buf[0] = 0;
    if (M < 0 || N <= 0 || K <= 0 || M >= kMaxElems || N >= kMaxElems || K >= kMaxElems)
        return fail(PHYAI_FP8_EINVAL, "phyai_fp8_describe_linear_plan: bad shape M=%lld N=%lld K=%lld", (long long)M, (long long)N, (long long)K);
    const int layout_bits = epilogue & PHYAI_FP8_FLAG_W_OPERAND_GATED;
    epilogue &= PHYAI_FP8_EPILOGUE_MASK;
    if (int rc = check_epilogue(epilogue, N)) return rc;
    if (K % 16 != 0 || N % 16 != 0)
        return fail(PHYAI_FP8_EUNSUPPORTED, "phyai_fp8_describe_linear_plan: K=%lld and N=%lld must be multiples of 16", (long long)K, (long long)N);
    // (the layout flags of the weight matrix may ride in `epilogue` as in the calls; a layout that the calls would
    // refuse for this shape or epilogue is described as row-major)
    int layout = phyai::W_ROW_MAJOR;
    if (layout_bits && K % 128 == 0 && N % (phyai::epi_is_gated(epilogue) ? 32 : 16) == 0)
        layout = phyai::epi_is_gated(epilogue) ? phyai::W_OPERAND_GATED : phyai::W_OPERAND_PLAIN;
    const int len = phyai::describe_linear_plan((int)M, (int)N, (int)K, epilogue, buf, n, layout);
    buf[n - 1] = 0;
    return len;
}

int phyai_fp8_describe_mlp_plan(int64_t M, int64_t H, int64_t I, int64_t O, int epilogue, char* buf, size_t n) {
    const char* fn = "phyai_fp8_describe_mlp_plan";
    if (!buf || n == 0) return fail(PHYAI_FP8_EINVAL, "%s: no buffer", fn);
    buf[0] = 0;
    if (M < 0 || H <= 0 || I <= 0 || O <= 0 || M >= kMaxElems || H >= kMaxElems || I >= kMaxElems || O >= kMaxElems)
        return fail(PHYAI_FP8_EINVAL, "%s: bad shape", fn);
    const bool operand = (epilogue & PHYAI_FP8_FLAG_W_OPERAND_ORDER) != 0 && H % 128 == 0 && I % 128 == 0;
    epilogue &= ~PHYAI_FP8_FLAG_W_OPERAND_GATED;
    if (epilogue <= PHYAI_FP8_EPI_NONE || epilogue > PHYAI_FP8_EPI_GELU_ERF)
        return fail(PHYAI_FP8_EINVAL, "%s: epilogue %d is not an activation", fn, epilogue);
    const int64_t n1 = phyai::epi_is_gated(epilogue) ? 2 * I : I;
    if (int rc = check_epilogue(epilogue, n1)) return rc;
    if (H % 16 != 0 || I % 16 != 0 || O % 16 != 0)
        return fail(PHYAI_FP8_EUNSUPPORTED, "%s: H, I and O must be multiples of 16", fn);
    const int len = phyai::describe_mlp_plan((int)M, (int)H, (int)I, (int)O, epilogue, buf, n, operand);
    buf[n - 1] = 0;
    return len;
}

int phyai_fp8_debug_mfma_rate(int workgroups, int iters, uint64_t* counters, float* sink, void* stream) {
    if (workgroups <= 0 || workgroups > 65536 || iters <= 0 || iters > (1 << 20) || !counters || !sink)
        return fail(PHYAI_FP8_EINVAL, "phyai_fp8_debug_mfma_rate: bad arguments");
    phyai::launch_mfma_rate(workgroups, iters, reinterpret_cast<unsigned long long*>(counters), sink, static_cast<hipStream_t>(stream));
    return check_launch("phyai_fp8_debug_mfma_rate");
}

int phyai_fp8_debug_stamps(uint64_t* records, int64_t n_records) {
    if (n_records < 0 || n_records > 0x7FFFFFFF || (n_records > 0 && !records))
        return fail(PHYAI_FP8_EINVAL, "phyai_fp8_debug_stamps: bad arguments");
    const int a = phyai::launch_set_stamp_sink_big(reinterpret_cast<unsigned long long*>(records), (unsigned int)n_records);
    const int b = phyai::launch_set_stamp_sink_fused(reinterpret_cast<unsigned long long*>(records), (unsigned int)n_records);
    if (a == -2 || b == -2)
        return fail(PHYAI_FP8_EUNSUPPORTED, "phyai_fp8_debug_stamps: this library was built without time stamps "
                    "(make stamps builds lib/libphyai_fp8_stamps.so)");
    if (a != 0 || b != 0) return fail(PHYAI_FP8_ELAUNCH, "phyai_fp8_debug_stamps: hipMemcpyToSymbol failed");
    return PHYAI_FP8_OK;
}

int phyai_fp8_debug_cast_e4m3(const float* v, int64_t n, void* codes, void* stream) {
    if (n < 0 || (n > 0 && (!v || !codes))) return fail(PHYAI_FP8_EINVAL, "phyai_fp8_debug_cast_e4m3: bad arguments");
    phyai::launch_debug_cast(v, n, codes, static_cast<hipStream_t>(stream));
    return check_launch("phyai_fp8_debug_cast_e4m3");
}

}  // extern "C"
