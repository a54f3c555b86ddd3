"""Reference arithmetic as torch CPU expressions.  TEST INFRASTRUCTURE ONLY.

Each function is the reference's own expression, restated with the same torch
ops on CPU tensors; the docstrings name the reference lines (paths relative to
the reference checkout).
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

FP8_MAX = 448.0

EPI_NONE = 0
EPI_GEGLU_TANH = 1
EPI_GEGLU_ERF = 2
EPI_SWIGLU = 3
EPI_GELU_TANH = 4
EPI_GELU_ERF = 5
GATED = (EPI_GEGLU_TANH, EPI_GEGLU_ERF, EPI_SWIGLU)


def quant_rowwise(x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-token dynamic fp8 quantization.

    phyai/src/phyai/layers/quant/fp8.py:150-155, PER_CHANNEL branch, verbatim
    op sequence: bf16 abs/amax/clamp_min, bf16 divide by 448, widen to fp32,
    promoted fp32 divide, cast to e4m3fn.  Returns ``(codes[..., K], scale[..., 1])``.
    """
    x_amax = x.abs().amax(dim=-1, keepdim=True).clamp_min(1e-12)
    x_scale = (x_amax / FP8_MAX).to(torch.float32)
    x_q = (x / x_scale).to(torch.float8_e4m3fn)
    return x_q, x_scale


def quant_static(x: torch.Tensor, input_scale: torch.Tensor) -> torch.Tensor:
    """Static per-tensor quantization, fp8.py:142-148."""
    return (x.float() / input_scale).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)


def weight_quant(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """Offline per-output-channel weight quantization.

    Not a reference function (the reference never quantizes fp8 weights); this
    is the rule the benchmark configuration states: ``s = absmax_k / 448`` in
    fp32, codes ``e4m3(clamp(W / s))``.  All-zero rows get the smallest normal
    fp32 as scale.
    """
    amax = w.float().abs().amax(dim=-1)
    s = (amax / FP8_MAX).clamp_min(torch.finfo(torch.float32).tiny)
    q = (w.float() / s[:, None]).clamp(-FP8_MAX, FP8_MAX).to(torch.float8_e4m3fn)
    return q, s


def gemm_f32(xq, x_scale, wq, w_scale, bias=None) -> torch.Tensor:
    """fp32 dequantize + matmul + bias: the closed form the parity tolerance is
    stated against (torch.py:155-176 computes the same product through
    ``torch._scaled_mm`` with ``scale_a=[M,1]``, ``scale_b=[1,N]``)."""
    K = xq.shape[-1]
    a = xq.reshape(-1, K).float() * x_scale.reshape(-1, 1).float()
    b = wq.float() * w_scale.float()[:, None]
    y = a @ b.t()
    if bias is not None:
        y = y + bias.float()
    return y


def _act(epi: int, v: torch.Tensor) -> torch.Tensor:
    if epi in (EPI_GEGLU_TANH, EPI_GELU_TANH):
        return F.gelu(v, approximate="tanh")
    if epi in (EPI_GEGLU_ERF, EPI_GELU_ERF):
        return F.gelu(v)
    if epi == EPI_SWIGLU:
        return F.silu(v)
    return v


def epilogue(y_f32: torch.Tensor, epi: int, out_dtype=torch.bfloat16) -> torch.Tensor:
    """DenseMLP activation on the GEMM output, dense_mlp.py:256-265.

    The reference rounds the GEMM result to bf16 (a separate tensor), applies
    the activation (fp32 math inside the kernel, bf16 in/out) and rounds again.
    gate = columns [0, I), up = columns [I, 2I) (dense_mlp.py:11-15).
    """
    y = y_f32.to(out_dtype)
    if epi == EPI_NONE:
        return y
    if epi in GATED:
        I = y.shape[-1] // 2
        g, u = y[..., :I].float(), y[..., I:].float()
        return (_act(epi, g) * u).to(out_dtype)
    return _act(epi, y.float()).to(out_dtype)


def linear(x, wq, w_scale, bias=None, epi: int = EPI_NONE) -> torch.Tensor:
    """Whole path: quantize activations, GEMM, bias, activation, bf16."""
    xq, xs = quant_rowwise(x)
    y = gemm_f32(xq, xs, wq, w_scale, bias)
    out = epilogue(y, epi, x.dtype)
    return out.reshape(*x.shape[:-1], out.shape[-1])


# ---- norms (phyai-kernel/phyai_kernel/triton/rms_norm.py:58-75, ada_rms_norm.py:83-117) --------

def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6, gemma: bool = False) -> torch.Tensor:
    """fp32 reduction, ``x_hat = x * rsqrt(var + eps)``, ``out = (x_hat * w).to(x.dtype)`` with
    ``w + 1`` for the Gemma form (rms_norm.py:58-73, the non-HF branch)."""
    xf = x.float()
    var = (xf * xf).sum(-1, keepdim=True) / x.shape[-1]
    x_hat = xf * torch.rsqrt(var + eps)
    w = weight.float()
    if gemma:
        w = w + 1.0
    return (x_hat * w).to(x.dtype)


def adarmsnorm(x: torch.Tensor, modulation: torch.Tensor, eps: float = 1e-6) -> tuple[torch.Tensor, torch.Tensor]:
    """``out = (x_hat * (1 + scale) + shift).to(x.dtype)``, ``gate = gate.to(x.dtype)``; modulation row
    ``r`` serves x rows ``[r * g, (r + 1) * g)`` (ada_rms_norm.py:77-117)."""
    D = x.shape[-1]
    x2 = x.reshape(-1, D).float()
    m2 = modulation.reshape(-1, 3 * D).float()
    g = x2.shape[0] // m2.shape[0]
    m_rows = m2.repeat_interleave(g, dim=0)
    scale, shift = m_rows[:, :D], m_rows[:, D:2 * D]
    var = (x2 * x2).sum(-1, keepdim=True) / D
    x_hat = x2 * torch.rsqrt(var + eps)
    out = (x_hat * (1.0 + scale) + shift).to(x.dtype).reshape(x.shape)
    gate = modulation[..., 2 * D:].to(x.dtype).contiguous()
    return out, gate


def addcmul(residual: torch.Tensor, y: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
    """``residual + y * gate`` on bf16 tensors, fp32 inside, one rounding - torch.addcmul as the
    decoder layer calls it (models/pi05/modeling_pi05.py:826,835); ``gate`` broadcasts over rows."""
    g = gate
    if g.shape != y.shape:
        g = g.reshape(-1, g.shape[-1]).repeat_interleave(y.reshape(-1, y.shape[-1]).shape[0] // g.reshape(-1, g.shape[-1]).shape[0], dim=0).reshape(y.shape)
    return (residual.float() + y.float() * g.float()).to(residual.dtype)
