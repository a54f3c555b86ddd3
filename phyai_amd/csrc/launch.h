// Host-side launch functions implemented by the kernel translation units and
// called from the C ABI layer.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace phyai {

int launch_quant_rowwise(const void* x, int64_t M, int64_t K, int64_t ldx, void* xq, float* xs,
                         hipStream_t st);
int launch_weight_quant(const void* w, int64_t N, int64_t K, int64_t ldw, void* wq, float* ws,
                        hipStream_t st);
int launch_quant_static(const void* x, int64_t M, int64_t K, int64_t ldx, const float* input_scale,
                        void* xq, hipStream_t st);
int launch_debug_cast(const float* v, int64_t n, void* codes, hipStream_t st);
// Row-major fp8 weights -> MFMA operand order (weight_layout.hip); gated: the fused gate | up form.
int launch_weight_to_operand_order(const void* w, int64_t N, int64_t K, int gated, void* out, hipStream_t st);
// fp8 MFMA issue-rate probe (probe_kernels.hip): out holds 2 x workgroups 64-bit counters.
int launch_mfma_rate(int workgroups, int iters, unsigned long long* out, float* sink, hipStream_t st);

// RMSNorm / adaptive RMSNorm with the activation quantizer fused behind it (quant_kernels.hip).
struct NormQuantArgs {
    const uint16_t* x;        // [M, D] bf16
    int64_t ldx;
    int D;
    float eps;
    const uint16_t* weight;   // RMSNorm: [D] bf16
    int gemma;                //          weight + 1
    const uint16_t* mod;      // adaptive: [M / group, 3 D] bf16 = scale | shift | gate
    int64_t ld_mod;
    int group;                //          rows of x per modulation row
    uint16_t* out;            // [M, D] bf16 or null
    int64_t ldo;
    uint16_t* gate;           // adaptive: [M / group, D] bf16 or null
    int64_t ld_gate;
    uint8_t* xq;              // [M, D] codes or null
    float* scale;             // [M]
};
int launch_norm_quant(const NormQuantArgs& a, int64_t M, bool adaptive, hipStream_t st);  // -2: D too large

struct GemmProblem {
    const uint8_t* xq;      // [M, K]
    const float* x_scale;   // [M] or [1]
    int x_scale_is_scalar;
    const uint8_t* w;       // [N, K]
    const float* w_scale;   // [N]
    const uint16_t* bias;   // [N] bf16 or null
    uint16_t* out;          // [M, N_out] bf16
    int64_t ldo;
    int M, N, K;
    int epilogue;
    void* workspace;        // header (counters) + split-K partials
    size_t workspace_bytes;
    // Gated residual (epilogue NONE only): out = residual + bf16(linear) * gate, in fp32, rounded
    // once.  gate row of token row m is m / gate_group.  Null residual: plain output.
    const uint16_t* residual;  // [M, N] bf16
    int64_t ld_res;
    const uint16_t* gate;      // [M / gate_group, N] bf16
    int64_t ld_gate;
    int gate_group;
    // Hint: read the weights with non-temporal loads (honoured by the weight-streaming kernel).
    int stream_weights;
    // Set by the whole-linear entry points: the bf16 activations behind xq / x_scale (row stride ldx
    // elements).  A kernel that quantizes its own rows reads these and ignores xq / x_scale, which are
    // then never written; null for the GEMM entry points.
    const uint16_t* x_bf16;
    int64_t ldx;
    // Layout of w (weight_layout.h): 0 row-major [N, K]; 1 MFMA operand order; 2 operand order of a fused
    // gate | up matrix (gated epilogues only).
    int weight_layout;
    // Row maxima handed from the producer of the activations to their consumer (the gate | up projection
    // of an MLP to its down projection; the one-launch small-M kernel only): amax_out, when set on a gated
    // launch, receives per token row and workgroup column the |bf16| maximum of the outputs
    // (table [M][64] of 16-bit patterns); amax_in / amax_parts give the consumer the table and the
    // number of slots per row that the producer wrote, and replace its own pass over the rows.
    uint16_t* amax_out;
    const uint16_t* amax_in;
    int amax_parts;
};

// What the kernels need of the above, by value.
struct ResidualArgs {
    const uint16_t* residual;
    const uint16_t* gate;
    int64_t ld_res, ld_gate;
    int gate_group;
};
inline ResidualArgs residual_of(const GemmProblem& g) {
    ResidualArgs r;
    r.residual = g.residual; r.gate = g.gate; r.ld_res = g.ld_res; r.ld_gate = g.ld_gate;
    r.gate_group = g.gate_group > 0 ? g.gate_group : 1;
    return r;
}

constexpr size_t kGemmHeaderBytes = 16384;  // split-K arrival counters (4096 ints) at the workspace start

size_t gemm_workspace_bytes(int64_t M, int64_t N, int64_t K, int epilogue, int64_t ldo);
// Workspace bytes the kernel chosen for exactly this problem (pointers and strides as given) needs:
// 0 when it uses none, else header + split-K partial sums.  launch_gemm returns -3 with less.
size_t gemm_scratch_need(const GemmProblem& p);
int launch_gemm(const GemmProblem& p, hipStream_t st);
// True when launch_gemm would serve this problem (x_bf16 set) with the kernel that quantizes its own
// rows: the caller then skips the quantizer launch.
bool gemm_quantizes_itself(const GemmProblem& p);
// Row maxima handed from one linear to the next (GemmProblem::amax_out / amax_in).  Slots per token row
// that launch_gemm would write for this producer (x_bf16 set, an activation epilogue), 0 when the kernel
// that serves it cannot; whether launch_gemm would serve this consumer (amax_in, amax_parts set) with
// the kernel that takes them.
int gemm_row_maxima_slots(const GemmProblem& p);
bool gemm_takes_row_maxima(const GemmProblem& p);
// Text form of the whole-linear choice for aligned operands and dense activations / output.
int describe_linear_plan(int M, int N, int K, int epilogue, char* buf, size_t n, int weight_layout = 0);

// Weight-streaming kernel for M <= 64 (gemm_skinny.hip).  It needs no workspace.
struct SkinnyPlan {
    int tiles;   // workgroups (each owns 16*nt weight rows over the whole K)
    int msplit;  // workgroups along M
    int mb;      // 16-row token blocks per workgroup
    int nt;      // weight tiles per workgroup
    int kpw;     // K steps per wavefront per round
    int rounds;
};
bool skinny_applicable(int M, int N, int K, int epilogue, int64_t ldo);
SkinnyPlan skinny_plan(int M, int N, int K, int epilogue);
int launch_gemm_skinny(const GemmProblem& p, const SkinnyPlan& pl, hipStream_t st);

// Small-M GEMM that quantizes its own activation rows (gemm_skinny_fused.hip): the whole linear in
// one launch.  rows == 0: does not apply.
struct FusedPlan {
    int rows;    // token rows per workgroup (8, 16, 32 or 64)
    int nt;      // 16-row weight tiles per workgroup
    int kpw;     // K steps per wavefront
    int tiles;   // workgroups along N
    int msplit;  // workgroups along M
};
FusedPlan fused_plan(int M, int N, int K, int epilogue, int64_t ldo, int weight_layout = 0, bool amax_in = false);
constexpr int kRowAmaxSlots = 64;   // slots per token row of a table of handed-over row maxima
int launch_gemm_fused(const GemmProblem& p, const FusedPlan& pl, hipStream_t st);

// Pipelined tile kernel for large M (gemm_big.hip), 256 x 256 or 128 x 128 tiles; the small
// tiles may be split along K (partials in the workspace, as for the generic tile kernel).
struct BigPlan {
    int tile;    // tile rows: 256 (x 256 columns), 224 (x 256), 192 (x 128), 128 (x 128 or x 64), 96 (x 128), or 0 if the kernel does not apply
    int cols;    // tile columns
    int splits;
    int tiles;   // output tiles of that size
    int depth;   // stages of the LDS ring
    int regs;    // weights in operand order loaded straight into a ring of this many register sets (4 or 8) by the
                 // wavefront that owns the columns, the activation stages handed over without barriers; 0: staged through LDS
};
BigPlan big_plan(int M, int N, int K, int epilogue, bool operand_w = false);
size_t big_partial_bytes(int M, int N, int epilogue, const BigPlan& pl);
int launch_gemm_big(const GemmProblem& p, const BigPlan& pl, hipStream_t st);

// Debug build (-DPHYAI_FP8_STAMPS) only: where the kernels of gemm_big.hip / gemm_skinny_fused.hip write their time
// stamps (stamps.h); -2 in the normal build.
int launch_set_stamp_sink_big(unsigned long long* buf, unsigned int records);
int launch_set_stamp_sink_fused(unsigned long long* buf, unsigned int records);
// Text form of what phyai_fp8_mlp launches for aligned, row-major operands.
int describe_mlp_plan(int M, int H, int I, int O, int epilogue, char* buf, size_t n, bool operand_order = false);
// Text form of launch_gemm's choice for aligned operands and a dense output; returns its length.
int describe_gemm_plan(int M, int N, int K, int epilogue, char* buf, size_t n, int weight_layout = 0);

}  // namespace phyai
