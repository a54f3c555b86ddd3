"""Weight-format vocabulary of the quantized-linear path.

Same names and meaning as the reference's ``phyai/layers/quant`` package for the
pieces on the fp8 path: ``Granularity`` (``granularity.py:12-17``),
``ActivationView`` / ``LinearActivationQuant`` (``linear.py:25-48``),
``AllocationRequest`` / ``WeightSpec`` (``base.py:24-70``), ``Fp8Spec``
(``fp8.py:46-157``) and ``Bf16Spec``.
"""

from phyai_amd.quant.types import (
    ActivationView,
    AllocationRequest,
    Granularity,
    LinearActivationQuant,
    WeightSpec,
)
from phyai_amd.quant.specs import Bf16Spec, Fp8Spec

__all__ = [
    "ActivationView",
    "AllocationRequest",
    "Bf16Spec",
    "Fp8Spec",
    "Granularity",
    "LinearActivationQuant",
    "WeightSpec",
]
