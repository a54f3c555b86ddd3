"""The registered linear kernels.

``HipFp8Kernel`` ("hip_fp8") is the MI355X path: it takes every
``fp8_per_channel`` / ``fp8_per_tensor`` linear, in both regimes, eager or under
graph capture, and runs it as one C-ABI call (row-wise quantizer + fp8 MFMA GEMM
with the scale/bias epilogue).  It replaces ``TorchKernel._fp8_per_channel`` and
``_fp8_per_tensor`` of the reference (``layers/linear/backends/torch.py:123-176``).

``TorchBf16Kernel`` ("torch") only covers unquantized bf16 weights through
``F.linear``, as the reference's always-present fallback does for that spec
(``backends/torch.py:82-83,110-111``).  It never handles an fp8 spec: there is no
non-HIP fp8 path in this package.
"""

from __future__ import annotations

import torch
import torch.nn.functional as F

from phyai_amd.linear.backend import KernelProbe
from phyai_amd.linear.registry import register_linear_kernel
from phyai_amd.quant.types import ActivationView, Granularity

_FP8_SPECS = ("fp8_per_channel", "fp8_per_tensor")
_MIN_SM = 89   # same gate as the reference; gfx950 reports 95


@register_linear_kernel(prefer_for={(s, r) for s in _FP8_SPECS for r in ("prefill", "decode")})
class HipFp8Kernel:
    name = "hip_fp8"

    def supports_capture(self) -> bool:
        # No allocation beyond torch's caching allocator, no host sync, nothing compiled lazily.
        return True

    def can_handle(self, probe: KernelProbe) -> bool:
        if probe.spec_id not in _FP8_SPECS:
            return False
        if probe.sm < _MIN_SM:
            return False
        if probe.in_dtype != torch.bfloat16 or probe.out_dtype != torch.bfloat16:
            return False
        return probe.K % 16 == 0 and probe.N % 16 == 0

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, bias: torch.Tensor | None,
              *, epilogue=None, residual: torch.Tensor | None = None,
              gate: torch.Tensor | None = None) -> torch.Tensor:
        """``epilogue`` / ``residual`` + ``gate`` are extensions over the reference protocol:
        ``DenseMLP`` passes the gated activation here so that it runs inside the GEMM kernel, and a
        decoder layer its ``addcmul(residual, out, gate)`` (``forward_addcmul`` of the layers)."""
        from phyai_amd import ops

        # set by phyai_amd.cache_plan.plan_weight_streaming on the layers whose weights should
        # pass the Infinity Cache by
        stream = bool(getattr(layer, "stream_weights", False))
        # set by Fp8Spec.process_after_loading when it re-laid the weight in MFMA operand order
        layout = getattr(layer, "weight_layout", None)
        spec_id = layer.spec.spec_id
        if isinstance(x, ActivationView):
            # already quantized per token by the producer (a norm with the quantizer fused in)
            if spec_id != "fp8_per_channel" or x.granularity is not Granularity.PER_CHANNEL or x.x_scale is None:
                raise RuntimeError(f"HipFp8Kernel: pre-quantized activations need per-token scales and an "
                                   f"fp8_per_channel layer, got spec_id={spec_id!r}, granularity={x.granularity}")
            return ops.fp8_gemm(x.x, x.x_scale, layer.weight, layer.weight_scale, bias, epilogue=epilogue,
                                residual=residual, gate=gate, stream_weights=stream, weight_layout=layout)
        if spec_id == "fp8_per_channel":
            return ops.fp8_linear(x, layer.weight, layer.weight_scale, bias, epilogue=epilogue,
                                  residual=residual, gate=gate, stream_weights=stream, weight_layout=layout)
        if spec_id == "fp8_per_tensor":
            act = layer.spec.quantize_activation(x, layer)
            return ops.fp8_gemm(act.x, layer.input_scale, layer.weight, layer.weight_scale, bias,
                                epilogue=epilogue, residual=residual, gate=gate, stream_weights=stream,
                                weight_layout=layout)
        raise RuntimeError(f"HipFp8Kernel got unhandled spec_id={spec_id!r}")


@register_linear_kernel()
class TorchBf16Kernel:
    name = "torch"

    def supports_capture(self) -> bool:
        return True

    def can_handle(self, probe: KernelProbe) -> bool:
        return probe.spec_id == "bf16"

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, bias: torch.Tensor | None) -> torch.Tensor:
        if layer.spec.spec_id != "bf16":
            raise RuntimeError(f"TorchBf16Kernel got unhandled spec_id={layer.spec.spec_id!r}")
        return F.linear(x, layer.weight, bias)
