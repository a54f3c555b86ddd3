"""Flat tensor ops over the HIP kernels, in the reference kernel package's style:
plain functions over device tensors with keyword-only optional pre-allocated
outputs, inputs flattened to 2-D, ``RuntimeError("phyai_amd.ops.<op>: ...")`` on
bad arguments, and an empty-input fast path (compare
``phyai-kernel/phyai_kernel/triton/ada_rms_norm.py:196-221,267-288`` and
``rms_norm.py:348-353`` in the reference).

The ops enqueue on the current torch stream and never synchronise, so they can
be recorded into a HIP graph once their workspace exists (see
:func:`reserve_workspace`).
"""

from __future__ import annotations

import contextlib
import contextvars

import torch

from phyai_amd import _lib

EPI_NONE = 0
EPI_GEGLU_TANH = 1
EPI_GEGLU_ERF = 2
EPI_SWIGLU = 3
EPI_GELU_TANH = 4
EPI_GELU_ERF = 5
_GATED = (EPI_GEGLU_TANH, EPI_GEGLU_ERF, EPI_SWIGLU)
EPILOGUES = {
    None: EPI_NONE, "none": EPI_NONE,
    "geglu_tanh": EPI_GEGLU_TANH, "geglu_erf": EPI_GEGLU_ERF, "swiglu": EPI_SWIGLU,
    "gelu_tanh": EPI_GELU_TANH, "gelu": EPI_GELU_ERF, "gelu_erf": EPI_GELU_ERF,
}

WORKSPACE_HEADER_BYTES = 16384
FLAG_STREAM_WEIGHTS = 0x100   # OR-ed into the epilogue argument of the C entry points
FLAG_W_OPERAND_ORDER = 0x200  # weight in MFMA operand order (fp8_weight_to_operand_order), plain form
FLAG_W_OPERAND_GATED = 0x600  # ... the form of a fused gate | up matrix (gated epilogues only)
WEIGHT_LAYOUTS = {None: 0, "row_major": 0, "operand": FLAG_W_OPERAND_ORDER, "operand_gated": FLAG_W_OPERAND_GATED}


def _err(op: str, msg: str) -> RuntimeError:
    return RuntimeError(f"phyai_amd.ops.{op}: {msg}")


def _stream_ptr() -> int:
    return torch.cuda.current_stream().cuda_stream


def _epi(op: str, epilogue) -> int:
    if isinstance(epilogue, int) and not isinstance(epilogue, bool):
        if epilogue not in range(6):
            raise _err(op, f"unknown epilogue {epilogue!r}")
        return epilogue
    try:
        return EPILOGUES[epilogue]
    except KeyError:
        raise _err(op, f"unknown epilogue {epilogue!r}; expected one of {sorted(k for k in EPILOGUES if k)}") from None


def _as_rows(op: str, x: torch.Tensor, name: str, dtype: torch.dtype) -> torch.Tensor:
    if not isinstance(x, torch.Tensor):
        raise _err(op, f"{name} must be a Tensor, got {type(x)!r}")
    if not x.is_cuda:
        raise _err(op, f"{name} must live on the GPU, got device={x.device}")
    if x.dtype != dtype:
        raise _err(op, f"{name} must be {dtype}, got {x.dtype}")
    if x.dim() < 1:
        raise _err(op, f"{name} must have at least one dim")
    x2 = x.reshape(-1, x.shape[-1])
    if x2.stride(-1) != 1 or (x2.shape[0] > 1 and x2.stride(0) % 8 != 0) or x2.data_ptr() % 16 != 0:
        x2 = x2.contiguous()
    return x2


# ---- workspace --------------------------------------------------------------
# Scratch of the GEMM (split-K counters and partial sums) and of the whole-linear entry points
# (activation codes and per-token scales): zero-initialised byte tensors whose header the kernels
# keep zero between calls.  Eager calls share one tensor per (device, stream).  A HIP graph bakes
# the addresses it was recorded with into its kernel nodes, so a graph owns its workspace
# (`WorkspaceOwner`, entered by `HipGraph.capture` around warm-up and recording): it lives as long
# as the graph and is shared with nobody - not with eager work that later runs on the pooled
# stream the graph was recorded on, not with other graphs.  A workspace that has to grow is
# replaced, never freed while anything may still hold its address: the old tensor stays with its
# owner (or, for the eager ones, in `_retired` until the process ends).
_workspaces: dict[tuple[int, int], torch.Tensor] = {}
_retired: list[torch.Tensor] = []


class WorkspaceOwner:
    """Scratch that lives as long as its owner (one captured graph): device index -> tensor."""

    def __init__(self) -> None:
        self.tensors: dict[int, torch.Tensor] = {}
        self.retired: list[torch.Tensor] = []


_owner: contextvars.ContextVar[WorkspaceOwner | None] = contextvars.ContextVar("phyai_amd_workspace_owner", default=None)


@contextlib.contextmanager
def workspace_owner(owner: WorkspaceOwner):
    """Calls inside the scope take their workspace from ``owner`` instead of the per-stream table."""
    token = _owner.set(owner)
    try:
        yield owner
    finally:
        _owner.reset(token)


def workspace_bytes(M: int, N: int, K: int, epilogue=EPI_NONE) -> int:
    return int(_lib.load().phyai_fp8_linear_workspace_bytes(M, N, K, _epi("workspace_bytes", epilogue)))


def describe_plan(M: int, N: int, K: int, epilogue=EPI_NONE, weight_layout: str | None = None) -> str:
    """Which kernel the GEMM entry point would launch for this problem and a weight in the given layout (host only,
    no GPU needed)."""
    import ctypes

    buf = ctypes.create_string_buffer(128)
    epi = _epi("describe_plan", epilogue)
    flag = _layout_flag("describe_plan", weight_layout, epi) if weight_layout else 0
    rc = _lib.load().phyai_fp8_describe_plan(M, N, K, epi | flag, buf, len(buf))
    if rc < 0:
        raise _err("describe_plan", _lib.load().phyai_fp8_last_error().decode())
    return buf.value.decode()


def describe_linear_plan(M: int, N: int, K: int, epilogue=EPI_NONE, weight_layout: str | None = None) -> str:
    """What the whole-linear entry point would launch (one kernel that quantizes its own rows, or the
    quantizer followed by a GEMM) for a weight in the given layout; host only."""
    import ctypes

    buf = ctypes.create_string_buffer(160)
    epi = _epi("describe_linear_plan", epilogue)
    flag = _layout_flag("describe_linear_plan", weight_layout, epi) if weight_layout else 0
    rc = _lib.load().phyai_fp8_describe_linear_plan(M, N, K, epi | flag, buf, len(buf))
    if rc < 0:
        raise _err("describe_linear_plan", _lib.load().phyai_fp8_last_error().decode())
    return buf.value.decode()


def reserve_workspace(nbytes: int, device: torch.device | None = None) -> torch.Tensor:
    """Make sure the workspace in scope on ``device`` (the enclosing graph's, else the current
    stream's) holds ``nbytes``."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    idx = dev.index if dev.index is not None else torch.cuda.current_device()
    owner = _owner.get()
    store, key, retired = (owner.tensors, idx, owner.retired) if owner is not None else (_workspaces, (idx, _stream_ptr()), _retired)
    ws = store.get(key)
    if ws is None or ws.numel() < nbytes:
        # Outside capture this is a one-off allocation.  Inside a capture (an op met for the first
        # time while recording) the tensor comes from the graph's memory pool and the zero fill is
        # recorded as a fill kernel - never a memset node - and replayed with the graph; warming
        # the op up before recording avoids that extra node.
        size = max(int(nbytes), 1 << 20, 2 * ws.numel() if ws is not None else 0)
        size = (size + 0xFFFFF) & ~0xFFFFF
        if ws is not None:
            retired.append(ws)     # recorded kernels or queued launches may still write through it
        ws = torch.zeros(size, dtype=torch.uint8, device=torch.device("cuda", idx))
        store[key] = ws
    return ws


def _workspace_for(M: int, N: int, K: int, epi: int, device: torch.device) -> torch.Tensor:
    return reserve_workspace(workspace_bytes(M, N, K, epi), device)


# ---- quantizers ---------------------------------------------------------------

def fp8_quant_rowwise(x: torch.Tensor, *, out: torch.Tensor | None = None,
                      scale_out: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """Per-token dynamic e4m3fn quantization of bf16 ``x[..., K]``.

    Returns ``(codes[..., K] float8_e4m3fn, scale[..., 1] float32)``, bit-exact
    with ``Fp8Spec.quantize_activation`` (reference ``layers/quant/fp8.py:150-155``).
    """
    op = "fp8_quant_rowwise"
    x2 = _as_rows(op, x, "x", torch.bfloat16)
    M, K = x2.shape
    if K % 8 != 0:
        raise _err(op, f"last dim {K} must be a multiple of 8")
    if out is None:
        out = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
    elif out.shape != x.shape or out.dtype != torch.float8_e4m3fn or not out.is_contiguous():
        raise _err(op, "out must be a contiguous float8_e4m3fn tensor shaped like x")
    sshape = (*x.shape[:-1], 1)
    if scale_out is None:
        scale_out = torch.empty(sshape, dtype=torch.float32, device=x.device)
    elif scale_out.shape != sshape or scale_out.dtype != torch.float32 or not scale_out.is_contiguous():
        raise _err(op, f"scale_out must be a contiguous float32 tensor of shape {sshape}")
    if M == 0:
        return out, scale_out
    rc = _lib.load().phyai_fp8_quant_rowwise(x2.data_ptr(), M, K, x2.stride(0) if M > 1 else K,
                                              out.data_ptr(), scale_out.data_ptr(), _stream_ptr())
    _lib.check(rc, op)
    return out, scale_out


# ---- norms with the quantizer fused behind them ------------------------------

def _norm_outputs(op: str, x: torch.Tensor, out, quantize: bool, want_out: bool):
    """Allocate / validate the bf16 output and the (codes, scale) pair of a fused norm."""
    if out is not None and (out.shape != x.shape or out.dtype != x.dtype or not out.is_contiguous()):
        raise _err(op, "`out` must be contiguous and match input shape and dtype")
    if out is None and want_out:
        out = torch.empty(x.shape, dtype=x.dtype, device=x.device)
    xq = xs = None
    if quantize:
        xq = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
        xs = torch.empty((*x.shape[:-1], 1), dtype=torch.float32, device=x.device)
    return out, xq, xs


def _rmsnorm(op: str, x, weight, eps, out, gemma: bool, quantize: bool, want_out: bool):
    x2 = _as_rows(op, x, "x", torch.bfloat16)
    M, D = x2.shape
    if not (isinstance(weight, torch.Tensor) and weight.is_cuda and weight.dtype == torch.bfloat16
            and weight.shape == (D,) and weight.is_contiguous()):
        raise _err(op, f"weight must be a contiguous bfloat16 GPU tensor of shape ({D},)")
    if D % 8 != 0:
        raise _err(op, f"last dim {D} must be a multiple of 8")
    out, xq, xs = _norm_outputs(op, x, out, quantize, want_out)
    if M == 0:
        return out, xq, xs
    ld = x2.stride(0) if M > 1 else D
    rc = _lib.load().phyai_fp8_rmsnorm_quant(
        x2.data_ptr(), ld, weight.data_ptr(), 1 if gemma else 0, M, D, float(eps),
        out.data_ptr() if out is not None else None, D,
        xq.data_ptr() if xq is not None else None, xs.data_ptr() if xs is not None else None, _stream_ptr())
    _lib.check(rc, op)
    return out, xq, xs


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6,
            out: torch.Tensor | None = None) -> torch.Tensor:
    """``(rsqrt(mean(x^2) + eps) * x * weight).to(x.dtype)``, fp32 inside - the reference's
    ``phyai_kernel.triton.rmsnorm`` (``phyai-kernel/phyai_kernel/triton/rms_norm.py:348-371``)."""
    return _rmsnorm("rmsnorm", x, weight, eps, out, False, False, True)[0]


def gemma_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6,
                  out: torch.Tensor | None = None) -> torch.Tensor:
    """RMSNorm with the Gemma ``(1 + weight)`` affine (``rms_norm.py:13,63-65``)."""
    return _rmsnorm("gemma_rmsnorm", x, weight, eps, out, True, False, True)[0]


def rmsnorm_fp8(x: torch.Tensor, weight: torch.Tensor, eps: float = 1e-6, *, gemma: bool = False,
                out: torch.Tensor | None = None, want_out: bool = False):
    """RMSNorm whose bf16 result goes straight into the per-token quantizer.

    Returns ``(codes, scale)`` - what ``Fp8Spec.quantize_activation`` gives on the norm's output -
    or ``(codes, scale, out)`` when the bf16 tensor is wanted too (``out=`` or ``want_out``)."""
    o, xq, xs = _rmsnorm("rmsnorm_fp8", x, weight, eps, out, gemma, True, want_out or out is not None)
    return (xq, xs) if o is None else (xq, xs, o)


def _adarmsnorm(op: str, x, modulation, eps, out, gate_out, quantize: bool, want_out: bool):
    if not (isinstance(modulation, torch.Tensor) and modulation.is_cuda):
        raise _err(op, "tensors must live on the GPU")
    if x.shape[-1] * 3 != modulation.shape[-1]:
        raise _err(op, f"modulation last dim ({modulation.shape[-1]}) must be 3x x last dim ({x.shape[-1]})")
    x2 = _as_rows(op, x, "x", torch.bfloat16)
    M, D = x2.shape
    mod2 = _as_rows(op, modulation, "modulation", torch.bfloat16)
    n_mod = mod2.shape[0]
    if D % 8 != 0:
        raise _err(op, f"last dim {D} must be a multiple of 8")
    out, xq, xs = _norm_outputs(op, x, out, quantize, want_out)
    gate_shape = (*modulation.shape[:-1], D)
    if gate_out is None:
        gate_out = torch.empty(gate_shape, dtype=x.dtype, device=x.device)
    elif tuple(gate_out.shape) != tuple(gate_shape) or gate_out.dtype != x.dtype or not gate_out.is_contiguous():
        raise _err(op, f"`gate_out` must be contiguous with shape {tuple(gate_shape)} and dtype {x.dtype}")
    if M == 0:
        return out, xq, xs, gate_out
    if n_mod == 0 or M % n_mod != 0:
        raise _err(op, f"x rows ({M}) must be a non-zero multiple of modulation rows ({n_mod})")
    rc = _lib.load().phyai_fp8_adarmsnorm_quant(
        x2.data_ptr(), x2.stride(0) if M > 1 else D, mod2.data_ptr(), mod2.stride(0) if n_mod > 1 else 3 * D,
        n_mod, M, D, float(eps), out.data_ptr() if out is not None else None, D, gate_out.data_ptr(), D,
        xq.data_ptr() if xq is not None else None, xs.data_ptr() if xs is not None else None, _stream_ptr())
    _lib.check(rc, op)
    return out, xq, xs, gate_out


def adarmsnorm(x: torch.Tensor, modulation: torch.Tensor, eps: float = 1e-6, *,
               out: torch.Tensor | None = None, gate_out: torch.Tensor | None = None):
    """Adaptive RMSNorm, ``(out, gate)`` - the reference's ``phyai_kernel.triton.adarmsnorm``
    (``phyai-kernel/phyai_kernel/triton/ada_rms_norm.py:214-221``): ``scale | shift | gate =
    modulation``; ``out = (x * rsqrt(mean(x^2) + eps) * (1 + scale) + shift).to(x.dtype)``; each
    modulation row serves ``rows(x) / rows(modulation)`` consecutive rows of ``x``."""
    o, _, _, g = _adarmsnorm("adarmsnorm", x, modulation, eps, out, gate_out, False, True)
    return o, g


def adarmsnorm_fp8(x: torch.Tensor, modulation: torch.Tensor, eps: float = 1e-6, *,
                   out: torch.Tensor | None = None, gate_out: torch.Tensor | None = None,
                   want_out: bool = False):
    """Adaptive RMSNorm feeding the per-token quantizer: ``(codes, scale, gate)`` or
    ``(codes, scale, gate, out)`` when the bf16 tensor is wanted too."""
    o, xq, xs, g = _adarmsnorm("adarmsnorm_fp8", x, modulation, eps, out, gate_out, True,
                               want_out or out is not None)
    return (xq, xs, g) if o is None else (xq, xs, g, o)


def fp8_quant_static(x: torch.Tensor, input_scale: torch.Tensor, *,
                     out: torch.Tensor | None = None) -> torch.Tensor:
    """Static per-tensor quantization (reference ``layers/quant/fp8.py:142-148``)."""
    op = "fp8_quant_static"
    x2 = _as_rows(op, x, "x", torch.bfloat16)
    M, K = x2.shape
    if K % 8 != 0:
        raise _err(op, f"last dim {K} must be a multiple of 8")
    if not (isinstance(input_scale, torch.Tensor) and input_scale.is_cuda and input_scale.dtype == torch.float32
            and input_scale.numel() == 1):
        raise _err(op, "input_scale must be a one-element float32 GPU tensor")
    if out is None:
        out = torch.empty(x.shape, dtype=torch.float8_e4m3fn, device=x.device)
    elif out.shape != x.shape or out.dtype != torch.float8_e4m3fn or not out.is_contiguous():
        raise _err(op, "out must be a contiguous float8_e4m3fn tensor shaped like x")
    if M == 0:
        return out
    rc = _lib.load().phyai_fp8_quant_static(x2.data_ptr(), M, K, x2.stride(0) if M > 1 else K,
                                             input_scale.data_ptr(), out.data_ptr(), _stream_ptr())
    _lib.check(rc, op)
    return out


def fp8_weight_quant(w: torch.Tensor, *, out: torch.Tensor | None = None,
                     scale_out: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
    """Offline per-output-channel weight quantization: ``(codes [N,K], scale [N])``."""
    op = "fp8_weight_quant"
    if w.dim() != 2:
        raise _err(op, f"w must be 2-D (N, K), got shape {tuple(w.shape)}")
    w2 = _as_rows(op, w, "w", torch.bfloat16)
    N, K = w2.shape
    if K % 8 != 0:
        raise _err(op, f"K={K} must be a multiple of 8")
    if out is None:
        out = torch.empty((N, K), dtype=torch.float8_e4m3fn, device=w.device)
    elif not (isinstance(out, torch.Tensor) and tuple(out.shape) == (N, K) and out.device == w.device
              and out.dtype in (torch.float8_e4m3fn, torch.uint8) and out.is_contiguous()):
        raise _err(op, f"out must be a contiguous float8_e4m3fn tensor of shape ({N}, {K}) on {w.device}")
    if scale_out is None:
        scale_out = torch.empty((N,), dtype=torch.float32, device=w.device)
    elif not (isinstance(scale_out, torch.Tensor) and tuple(scale_out.shape) == (N,) and scale_out.device == w.device
              and scale_out.dtype == torch.float32 and scale_out.is_contiguous()):
        raise _err(op, f"scale_out must be a contiguous float32 tensor of shape ({N},) on {w.device}")
    if N == 0:
        return out, scale_out
    rc = _lib.load().phyai_fp8_weight_quant_rowwise(w2.data_ptr(), N, K, w2.stride(0) if N > 1 else K,
                                                     out.data_ptr(), scale_out.data_ptr(), _stream_ptr())
    _lib.check(rc, op)
    return out, scale_out


def fp8_weight_to_operand_order(w: torch.Tensor, *, gated: bool = False, out: torch.Tensor | None = None) -> torch.Tensor:
    """Re-lay fp8 weights ``w[N, K]`` (row-major) into MFMA operand order: same shape and dtype, the
    bytes in the order the kernels' lanes read them (units of 16 rows x 128 bytes of K, the 16 x 8
    matrix of 16-byte chunks of a unit transposed).  ``gated``: ``w`` is a fused gate | up matrix and
    the result is for gated epilogues only.  Pass the result to :func:`fp8_gemm` / :func:`fp8_linear`
    with ``weight_layout="operand"`` (``"operand_gated"``).  Out of place.

    This is what ``Fp8Spec.process_after_loading`` runs once per layer (the reference's hook for
    "re-lay weights after loading", ``layers/quant/base.py:55-70``)."""
    op = "fp8_weight_to_operand_order"
    if not (isinstance(w, torch.Tensor) and w.is_cuda and w.dim() == 2 and w.is_contiguous()
            and w.dtype in (torch.float8_e4m3fn, torch.uint8)):
        raise _err(op, "w must be a contiguous 2-D float8_e4m3fn GPU tensor (N, K)")
    N, K = w.shape
    if K % 128 != 0 or N % (32 if gated else 16) != 0:
        raise _err(op, f"needs K % 128 == 0 and N % {32 if gated else 16} == 0, got N={N}, K={K}")
    if out is None:
        out = torch.empty_like(w)
    elif not (isinstance(out, torch.Tensor) and out.shape == w.shape and out.dtype == w.dtype and out.device == w.device
              and out.is_contiguous()):
        raise _err(op, "out must be a contiguous tensor shaped and typed like w")
    if N == 0:
        return out
    rc = _lib.load().phyai_fp8_weight_to_operand_order(w.data_ptr(), N, K, 1 if gated else 0, out.data_ptr(), _stream_ptr())
    _lib.check(rc, op)
    return out


def _layout_flag(op: str, weight_layout, epi: int) -> int:
    try:
        flag = WEIGHT_LAYOUTS[weight_layout]
    except (KeyError, TypeError):
        raise _err(op, f"unknown weight_layout {weight_layout!r}; expected one of {sorted(k for k in WEIGHT_LAYOUTS if k)}") from None
    if flag and (flag == FLAG_W_OPERAND_GATED) != (epi in _GATED):
        raise _err(op, f"weight_layout={weight_layout!r} does not go with epilogue {epi}: a gated epilogue needs "
                       "'operand_gated', any other epilogue 'operand'")
    return flag


# ---- GEMM / linear --------------------------------------------------------------

def _check_weight(op: str, weight: torch.Tensor, weight_scale: torch.Tensor, K: int) -> tuple[int, int]:
    if not (isinstance(weight, torch.Tensor) and weight.is_cuda and weight.dim() == 2):
        raise _err(op, "weight must be a 2-D GPU tensor (N, K)")
    if weight.dtype not in (torch.float8_e4m3fn, torch.uint8):
        raise _err(op, f"weight must be float8_e4m3fn, got {weight.dtype}")
    if not weight.is_contiguous():
        raise _err(op, "weight must be contiguous (N, K) with K innermost")
    N, Kw = weight.shape
    if Kw != K:
        raise _err(op, f"weight K={Kw} does not match activation K={K}")
    if K % 16 != 0 or N % 16 != 0:
        raise _err(op, f"K={K} and N={N} must be multiples of 16")
    if not (weight_scale.is_cuda and weight_scale.dtype == torch.float32 and weight_scale.numel() == N
            and weight_scale.is_contiguous()):
        raise _err(op, f"weight_scale must be a contiguous float32 GPU tensor with {N} elements")
    return N, K


def _check_bias(op: str, bias: torch.Tensor | None, N: int) -> int:
    if bias is None:
        return 0
    if not (bias.is_cuda and bias.dtype == torch.bfloat16 and bias.numel() == N and bias.is_contiguous()):
        raise _err(op, f"bias must be a contiguous bfloat16 GPU tensor with {N} elements")
    return bias.data_ptr()


def _out_for(op: str, lead: tuple[int, ...], n_out: int, out: torch.Tensor | None, device) -> torch.Tensor:
    shape = (*lead, n_out)
    if out is None:
        return torch.empty(shape, dtype=torch.bfloat16, device=device)
    if tuple(out.shape) != shape or out.dtype != torch.bfloat16 or not out.is_contiguous():
        raise _err(op, f"out must be a contiguous bfloat16 tensor of shape {shape}")
    return out


def _check_addcmul(op: str, residual, gate, lead: tuple[int, ...], M: int, N: int, epi: int, device):
    """Validate the gated-residual pair; returns ``(residual2d, gate2d)`` or ``(None, None)``."""
    if residual is None and gate is None:
        return None, None
    if residual is None or gate is None:
        raise _err(op, "residual and gate go together")
    if epi != EPI_NONE:
        raise _err(op, "a gated residual excludes an activation epilogue")
    for name, t in (("residual", residual), ("gate", gate)):
        if not (isinstance(t, torch.Tensor) and t.is_cuda and t.dtype == torch.bfloat16 and t.shape[-1] == N):
            raise _err(op, f"{name} must be a bfloat16 GPU tensor with last dim {N}")
    if tuple(residual.shape) != (*lead, N):
        raise _err(op, f"residual must have shape {(*lead, N)}, got {tuple(residual.shape)}")
    r2 = residual.reshape(-1, N)
    g2 = gate.reshape(-1, N)
    if not r2.is_contiguous():
        r2 = r2.contiguous()
    if not g2.is_contiguous():
        g2 = g2.contiguous()
    if g2.shape[0] == 0 or M % g2.shape[0] != 0:
        raise _err(op, f"rows ({M}) must be a non-zero multiple of gate rows ({g2.shape[0]})")
    return r2, g2


def fp8_gemm(xq: torch.Tensor, x_scale: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
             bias: torch.Tensor | None = None, *, epilogue=None, out: torch.Tensor | None = None,
             residual: torch.Tensor | None = None, gate: torch.Tensor | None = None,
             stream_weights: bool = False, weight_layout: str | None = None) -> torch.Tensor:
    """``bf16(act((xq @ weight.T) * x_scale * weight_scale + bias))`` on quantized inputs.

    ``weight_layout``: ``"operand"`` / ``"operand_gated"`` when ``weight`` went through
    :func:`fp8_weight_to_operand_order`; same result as with the row-major matrix.

    ``stream_weights``: read the weights past the caches (see :mod:`phyai_amd.cache_plan`);
    same result, honoured by the weight-streaming kernel (small M) without a gated residual.

    With ``residual`` and ``gate`` the result is ``torch.addcmul(residual, y, gate)`` of that
    linear output ``y`` (reference ``models/pi05/modeling_pi05.py:826,835``), in the same kernel;
    ``gate`` may have fewer rows than ``residual`` (one per modulation row).

    ``x_scale`` has one element per token row, or a single element (static
    per-tensor scale).  Replaces the ``torch._scaled_mm`` call at reference
    ``layers/linear/backends/torch.py:166-175`` (and ``:145-152``).
    """
    op = "fp8_gemm"
    epi = _epi(op, epilogue)
    if not (isinstance(xq, torch.Tensor) and xq.is_cuda and xq.dtype in (torch.float8_e4m3fn, torch.uint8)):
        raise _err(op, "xq must be a float8_e4m3fn GPU tensor")
    x2 = xq.reshape(-1, xq.shape[-1])
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    M, K = x2.shape
    N, _ = _check_weight(op, weight, weight_scale, K)
    if epi in _GATED and N % 32 != 0:
        raise _err(op, f"gated epilogue needs N % 32 == 0, got {N}")
    xs = x_scale.reshape(-1)
    if not (xs.is_cuda and xs.dtype == torch.float32 and xs.numel() in (1, M) and xs.is_contiguous()):
        raise _err(op, f"x_scale must be float32 with 1 or {M} elements")
    scalar = 1 if (xs.numel() == 1 and M != 1) else 0
    bias_ptr = _check_bias(op, bias, N)
    flags = _layout_flag(op, weight_layout, epi) | (FLAG_STREAM_WEIGHTS if stream_weights else 0)
    n_out = N // 2 if epi in _GATED else N
    r2, g2 = _check_addcmul(op, residual, gate, tuple(xq.shape[:-1]), M, N, epi, xq.device)
    out = _out_for(op, tuple(xq.shape[:-1]), n_out, out, xq.device)
    if M == 0:
        return out
    ws = _workspace_for(M, N, K, epi, xq.device)
    if r2 is not None:
        rc = _lib.load().phyai_fp8_gemm_addcmul(
            x2.data_ptr(), xs.data_ptr(), scalar, weight.data_ptr(), weight_scale.data_ptr(), bias_ptr,
            r2.data_ptr(), r2.stride(0) if M > 1 else N, g2.data_ptr(), g2.stride(0) if g2.shape[0] > 1 else N,
            g2.shape[0], out.data_ptr(), n_out, M, N, K, flags, ws.data_ptr(), ws.numel(), _stream_ptr())
    else:
        rc = _lib.load().phyai_fp8_gemm(x2.data_ptr(), xs.data_ptr(), scalar, weight.data_ptr(),
                                         weight_scale.data_ptr(), bias_ptr, out.data_ptr(), n_out, M, N, K,
                                         epi | flags, ws.data_ptr(), ws.numel(), _stream_ptr())
    _lib.check(rc, op)
    return out


def fp8_linear(x: torch.Tensor, weight: torch.Tensor, weight_scale: torch.Tensor,
               bias: torch.Tensor | None = None, *, epilogue=None, out: torch.Tensor | None = None,
               residual: torch.Tensor | None = None, gate: torch.Tensor | None = None,
               stream_weights: bool = False, weight_layout: str | None = None) -> torch.Tensor:
    """The whole W8A8 linear on bf16 ``x[..., K]``: per-token quantization, fp8 MFMA
    GEMM, per-channel dequantization, bias and optional activation, bf16 out.

    ``stream_weights``, ``weight_layout``: as for :func:`fp8_gemm`.

    Replaces ``TorchKernel._fp8_per_channel`` (reference
    ``layers/linear/backends/torch.py:155-176``) and, with a gated ``epilogue``,
    the activation launch that follows it in ``DenseMLP.forward``
    (``layers/mlp/dense_mlp.py:256-261``).
    """
    op = "fp8_linear"
    epi = _epi(op, epilogue)
    x2 = _as_rows(op, x, "x", torch.bfloat16)
    M, K = x2.shape
    N, _ = _check_weight(op, weight, weight_scale, K)
    if epi in _GATED and N % 32 != 0:
        raise _err(op, f"gated epilogue needs N % 32 == 0, got {N}")
    bias_ptr = _check_bias(op, bias, N)
    flags = _layout_flag(op, weight_layout, epi) | (FLAG_STREAM_WEIGHTS if stream_weights else 0)
    n_out = N // 2 if epi in _GATED else N
    r2, g2 = _check_addcmul(op, residual, gate, tuple(x.shape[:-1]), M, N, epi, x.device)
    out = _out_for(op, tuple(x.shape[:-1]), n_out, out, x.device)
    if M == 0:
        return out
    ws = _workspace_for(M, N, K, epi, x.device)
    if r2 is not None:
        rc = _lib.load().phyai_fp8_linear_addcmul(
            x2.data_ptr(), x2.stride(0) if M > 1 else K, weight.data_ptr(), weight_scale.data_ptr(), bias_ptr,
            r2.data_ptr(), r2.stride(0) if M > 1 else N, g2.data_ptr(), g2.stride(0) if g2.shape[0] > 1 else N,
            g2.shape[0], out.data_ptr(), n_out, M, N, K, flags, ws.data_ptr(), ws.numel(), _stream_ptr())
    else:
        rc = _lib.load().phyai_fp8_linear(x2.data_ptr(), x2.stride(0) if M > 1 else K, weight.data_ptr(),
                                           weight_scale.data_ptr(), bias_ptr, out.data_ptr(), n_out, M, N, K,
                                           epi | flags, ws.data_ptr(), ws.numel(), _stream_ptr())
    _lib.check(rc, op)
    return out


def describe_mlp_plan(M: int, H: int, I: int, O: int, epilogue, operand_order: bool = False) -> str:
    """What :func:`fp8_mlp` launches for this shape, with row-major weights or with both matrices in operand
    order; host only."""
    import ctypes

    buf = ctypes.create_string_buffer(256)
    epi = _epi("describe_mlp_plan", epilogue) | (FLAG_W_OPERAND_ORDER if operand_order else 0)
    rc = _lib.load().phyai_fp8_describe_mlp_plan(M, H, I, O, epi, buf, len(buf))
    if rc < 0:
        raise _err("describe_mlp_plan", _lib.load().phyai_fp8_last_error().decode())
    return buf.value.decode()


def fp8_mlp(x: torch.Tensor, weight1: torch.Tensor, weight1_scale: torch.Tensor, bias1: torch.Tensor | None,
            weight2: torch.Tensor, weight2_scale: torch.Tensor, bias2: torch.Tensor | None, *, epilogue,
            out: torch.Tensor | None = None, residual: torch.Tensor | None = None, gate: torch.Tensor | None = None,
            stream_weights1: bool = False, stream_weights2: bool = False, weight1_layout: str | None = None,
            weight2_layout: str | None = None) -> torch.Tensor:
    """Both projections of an MLP in one call: ``linear2(act(linear1(x)))`` with ``epilogue`` the
    activation of the first (gated: ``weight1`` is the fused gate | up matrix ``[2 I, H]``), optionally
    ``torch.addcmul(residual, ., gate)`` behind the second.  The bits of :func:`fp8_linear` with that
    epilogue followed by :func:`fp8_linear` on its output; the intermediate tensor lives in the workspace.
    For small token counts the first kernel hands the row maxima of its output to the second, which then
    quantizes those rows without first passing over them (see :func:`describe_mlp_plan`).

    Replaces ``DenseMLP.forward`` of the reference (``layers/mlp/dense_mlp.py:256-265``)."""
    op = "fp8_mlp"
    epi = _epi(op, epilogue)
    if epi == EPI_NONE:
        raise _err(op, "epilogue must be the first projection's activation")
    x2 = _as_rows(op, x, "x", torch.bfloat16)
    M, H = x2.shape
    N1, _ = _check_weight(op, weight1, weight1_scale, H)
    if epi in _GATED and N1 % 32 != 0:
        raise _err(op, f"gated epilogue needs N % 32 == 0, got {N1}")
    I = N1 // 2 if epi in _GATED else N1
    O, _ = _check_weight(op, weight2, weight2_scale, I)
    b1, b2 = _check_bias(op, bias1, N1), _check_bias(op, bias2, O)
    f1 = _layout_flag(op, weight1_layout, epi) | (FLAG_STREAM_WEIGHTS if stream_weights1 else 0)
    f2 = _layout_flag(op, weight2_layout, EPI_NONE) | (FLAG_STREAM_WEIGHTS if stream_weights2 else 0)
    r2, g2 = _check_addcmul(op, residual, gate, tuple(x.shape[:-1]), M, O, EPI_NONE, x.device)
    out = _out_for(op, tuple(x.shape[:-1]), O, out, x.device)
    if M == 0:
        return out
    lib = _lib.load()
    ws = reserve_workspace(int(lib.phyai_fp8_mlp_workspace_bytes(M, H, I, O, epi)), x.device)
    rc = lib.phyai_fp8_mlp(
        x2.data_ptr(), x2.stride(0) if M > 1 else H, weight1.data_ptr(), weight1_scale.data_ptr(), b1, f1,
        weight2.data_ptr(), weight2_scale.data_ptr(), b2, f2,
        r2.data_ptr() if r2 is not None else None, (r2.stride(0) if M > 1 else O) if r2 is not None else 0,
        g2.data_ptr() if g2 is not None else None, (g2.stride(0) if g2.shape[0] > 1 else O) if g2 is not None else 0,
        g2.shape[0] if g2 is not None else 0, out.data_ptr(), O, M, H, I, O, epi, ws.data_ptr(), ws.numel(), _stream_ptr())
    _lib.check(rc, op)
    return out


STAMP_WORDS = 12


def debug_stamps(n_records: int, device: torch.device | None = None) -> torch.Tensor | None:
    """Debug build only (``PHYAI_FP8_LIBRARY=stamps``): from now on every wavefront of the pipelined tile kernel and
    of the one-launch small-M kernel writes its time stamps into the returned ``[n_records, 12]`` int64 tensor (keep
    it alive while kernels run); ``n_records = 0`` switches the recording off and returns None.  Synchronises."""
    lib = _lib.load()
    if n_records <= 0:
        _lib.check(lib.phyai_fp8_debug_stamps(None, 0), "debug_stamps")
        return None
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    buf = torch.zeros(n_records, STAMP_WORDS, dtype=torch.int64, device=dev)
    torch.cuda.synchronize()
    _lib.check(lib.phyai_fp8_debug_stamps(buf.data_ptr(), n_records), "debug_stamps")
    return buf


def debug_cast_e4m3(v: torch.Tensor) -> torch.Tensor:
    """Device fp32 -> e4m3fn cast used by the quantizers, exposed for exhaustive tests."""
    if not (v.is_cuda and v.dtype == torch.float32 and v.is_contiguous()):
        raise _err("debug_cast_e4m3", "v must be a contiguous float32 GPU tensor")
    out = torch.empty(v.shape, dtype=torch.uint8, device=v.device)
    rc = _lib.load().phyai_fp8_debug_cast_e4m3(v.data_ptr(), v.numel(), out.data_ptr(), _stream_ptr())
    _lib.check(rc, "debug_cast_e4m3")
    return out


def mfma_rate_probe(workgroups: int = 1024, iters: int = 2000, device: torch.device | None = None) -> dict:
    """Chip-wide fp8 MFMA issue rate and the shader clock held under that load (a synchronising
    measurement, not an op): ``{"TFLOPs", "clock_GHz", "cycles_per_mfma"}``."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    counters = torch.zeros(2 * workgroups, dtype=torch.int64, device=dev)
    sink = torch.zeros(1, dtype=torch.float32, device=dev)
    lib = _lib.load()
    best = None
    for _ in range(3):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        _lib.check(lib.phyai_fp8_debug_mfma_rate(workgroups, iters, counters.data_ptr(), sink.data_ptr(), _stream_ptr()),
                   "mfma_rate_probe")
        b.record()
        torch.cuda.synchronize()
        ms = a.elapsed_time(b)
        best = ms if best is None or ms < best else best
    c = counters.cpu().reshape(workgroups, 2).double()
    cycles, ticks = c[:, 0].mean().item(), c[:, 1].mean().item()
    flops = workgroups * 4 * iters * 16 * (32 * 32 * 64 * 2)
    return {"TFLOPs": round(flops / (best * 1e-3) / 1e12, 1), "clock_GHz": round(cycles / (ticks / 100e6) / 1e9, 3),
            "cycles_per_mfma": round(cycles / (iters * 16), 2)}
