"""``Fp8Spec`` and ``Bf16Spec``.

``Fp8Spec`` keeps the reference's storage contract and activation-quantization
semantics (``phyai/layers/quant/fp8.py:46-157``) but runs the quantizer as one
HIP kernel instead of seven element-wise torch launches.
"""

from __future__ import annotations

import dataclasses

import torch
import torch.nn as nn

from phyai_amd.quant.types import ActivationView, AllocationRequest, Granularity


def _frozen(t: torch.Tensor) -> nn.Parameter:
    return nn.Parameter(t, requires_grad=False)


@dataclasses.dataclass
class Bf16Spec:
    """Unquantized weight in the layer's parameter dtype."""

    weight_dtype: torch.dtype = torch.bfloat16
    needs_act_quant: bool = False

    @property
    def spec_id(self) -> str:
        return "bf16"

    def allocate(self, layer: nn.Module, request: AllocationRequest) -> None:
        if len(request.weight_shape) != 2:
            raise ValueError(f"Bf16Spec.allocate expects a 2-D weight_shape (N, K), got {request.weight_shape!r}")
        layer.weight = _frozen(torch.empty(*request.weight_shape, dtype=request.params_dtype, device=request.device))
        layer.logical_widths = list(request.logical_widths)

    def process_after_loading(self, layer: nn.Module) -> None:
        return None


@dataclasses.dataclass
class Fp8Spec:
    """e4m3fn weight ``[N, K]`` plus scales at one of three granularities.

    * ``PER_TENSOR``: one fp32 scale per fused sub-matrix (fanned out to ``[N]``
      after loading) and one static activation scale.
    * ``PER_CHANNEL``: fp32 scale per output row; activations are quantized per
      token at run time.  This is the format the HIP kernels are built for.
    * ``BLOCK``: ``[N/bn, K/bk]`` weight scales (storage only here).
    """

    granularity: Granularity = Granularity.PER_CHANNEL
    block_shape: tuple[int, int] | None = None
    weight_dtype: torch.dtype = torch.float8_e4m3fn
    needs_act_quant: bool = True
    # Re-lay the weight into MFMA operand order after loading (``process_after_loading``): same
    # results, and the kernels whose weight blocks are private to a wavefront then load them straight
    # into registers.  Off by default: the row-major ``[N, K]`` tensor is what checkpoints hold and
    # what other code may read.
    operand_order: bool = False

    def __post_init__(self) -> None:
        if self.granularity is Granularity.BLOCK and self.block_shape is None:
            raise ValueError("Fp8Spec(granularity=BLOCK) requires block_shape")

    @property
    def spec_id(self) -> str:
        if self.granularity is Granularity.BLOCK:
            bn, bk = self.block_shape  # type: ignore[misc]
            return f"fp8_block_{bn}_{bk}"
        return f"fp8_{self.granularity.value}"

    # -- storage (reference fp8.py:65-126) ------------------------------------
    def allocate(self, layer: nn.Module, request: AllocationRequest) -> None:
        if len(request.weight_shape) != 2:
            raise ValueError(f"Fp8Spec.allocate expects a 2-D weight_shape (N, K), got {request.weight_shape!r}")
        n, k = request.weight_shape
        dev = request.device
        layer.weight = _frozen(torch.empty(n, k, dtype=self.weight_dtype, device=dev))
        if self.granularity is Granularity.PER_TENSOR:
            layer.weight_scale = _frozen(torch.ones(len(request.logical_widths), dtype=torch.float32, device=dev))
            layer.input_scale = _frozen(torch.ones(1, dtype=torch.float32, device=dev))
        elif self.granularity is Granularity.PER_CHANNEL:
            layer.weight_scale = _frozen(torch.ones(n, dtype=torch.float32, device=dev))
        else:
            bn, bk = self.block_shape  # type: ignore[misc]
            if n % bn:
                raise ValueError(f"Fp8Spec(BLOCK): out_per_rank={n} not divisible by block_n={bn}")
            if k % bk:
                raise ValueError(f"Fp8Spec(BLOCK): in_per_rank={k} not divisible by block_k={bk}")
            layer.weight_scale = _frozen(torch.ones(n // bn, k // bk, dtype=torch.float32, device=dev))
        layer.logical_widths = list(request.logical_widths)

    def process_after_loading(self, layer: nn.Module) -> None:
        """Per-tensor scales become one value per output row (reference fp8.py:128-135); with
        ``operand_order`` the weight is re-laid for the MFMA (the use the reference's protocol names
        for this hook, ``layers/quant/base.py:55-70``)."""
        if self.granularity is Granularity.PER_TENSOR and layer.weight_scale.numel() == len(layer.logical_widths) \
                and layer.weight_scale.numel() != layer.weight.shape[0]:
            widths = torch.tensor(layer.logical_widths, device=layer.weight_scale.device)
            layer.weight_scale = _frozen(torch.repeat_interleave(layer.weight_scale.detach(), widths).contiguous())
        if self.operand_order and self.granularity is not Granularity.BLOCK:
            self.to_operand_order_(layer)

    def to_operand_order_(self, layer: nn.Module) -> bool:
        """Re-lay ``layer.weight`` (row-major as loaded) in place; ``layer.weight_layout`` then says
        ``"operand"`` or, for a layer marked ``gated_pairs`` (the fused gate | up projection of an MLP
        whose activation runs in the GEMM epilogue), ``"operand_gated"``.  Returns False, leaving the
        layer as it is, when the shape does not allow it or the weight lives on the CPU.  A layer that
        already says so is left alone; whoever writes row-major bytes into the weight again (the
        checkpoint loader, ``quantize_weight_``) clears ``weight_layout`` first."""
        from phyai_amd import ops

        w = layer.weight
        if getattr(layer, "weight_layout", None):
            return True
        gated = bool(getattr(layer, "gated_pairs", False))
        n, k = w.shape
        if not w.is_cuda or k % 128 != 0 or n % (32 if gated else 16) != 0:
            return False
        w.data.copy_(ops.fp8_weight_to_operand_order(w.data, gated=gated))
        layer.weight_layout = "operand_gated" if gated else "operand"
        return True

    # -- activation quantization (reference fp8.py:137-157) ----------------------
    def quantize_activation(self, x: torch.Tensor, layer: nn.Module) -> ActivationView:
        from phyai_amd import ops

        if self.granularity is Granularity.PER_TENSOR:
            return ActivationView(ops.fp8_quant_static(x, layer.input_scale), layer.input_scale,
                                  Granularity.PER_TENSOR)
        if self.granularity in (Granularity.PER_CHANNEL, Granularity.BLOCK):
            x_q, x_scale = ops.fp8_quant_rowwise(x)
            return ActivationView(x_q, x_scale, self.granularity)
        raise RuntimeError(f"unhandled Fp8Spec granularity {self.granularity!r}")

    # -- offline weight quantization (no reference counterpart) ------------------
    def quantize_weight_(self, layer: nn.Module, w_bf16: torch.Tensor) -> None:
        """Fill ``layer.weight`` / ``layer.weight_scale`` from a bf16 ``[N, K]`` matrix with
        per-output-channel absmax/448 scales (PER_CHANNEL only)."""
        from phyai_amd import ops

        if self.granularity is not Granularity.PER_CHANNEL:
            raise RuntimeError("quantize_weight_ is defined for PER_CHANNEL only")
        if tuple(w_bf16.shape) != tuple(layer.weight.shape):
            raise ValueError(f"weight shape {tuple(w_bf16.shape)} != {tuple(layer.weight.shape)}")
        layer.weight_layout = None   # row-major again until process_after_loading re-lays it
        ops.fp8_weight_quant(w_bf16.to(device=layer.weight.device, dtype=torch.bfloat16).contiguous(),
                             out=layer.weight.data, scale_out=layer.weight_scale.data)


__all__ = ["Bf16Spec", "Fp8Spec"]
