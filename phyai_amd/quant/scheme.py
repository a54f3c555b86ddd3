"""Semantic quantization IR and the rule table that maps layers to it.

Restates the reference's ``phyai/layers/quant/scheme.py:15-62`` (``QDType``, ``TensorQuant``,
``QuantScheme``), ``plan.py:13-40`` (``Matcher``, ``Rule``) and ``materialize.py:13-23``
(scheme -> physical spec).  Only the bf16 and fp8 e4m3 weight types lower to a spec here: the
other element types of the enum belong to formats this package has no kernels for.
"""

from __future__ import annotations

import fnmatch
import re
from dataclasses import dataclass
from enum import Enum
from typing import Literal

from phyai_amd.quant.specs import Bf16Spec, Fp8Spec
from phyai_amd.quant.types import Granularity


class QDType(Enum):
    """Quantized element type; ``BF16`` is the sentinel for 'not quantized'."""

    BF16 = "bf16"
    FP8_E4M3 = "fp8_e4m3"
    FP8_E5M2 = "fp8_e5m2"
    INT8 = "int8"
    INT4 = "int4"
    NVFP4 = "nvfp4"
    MXFP4 = "mxfp4"


@dataclass(frozen=True)
class TensorQuant:
    """How one tensor (weight or activation) is quantized (reference ``scheme.py:31-47``)."""

    dtype: QDType
    granularity: Granularity
    symmetric: bool = True
    dynamic: bool = False
    micro_scaled: bool = False
    block_shape: tuple[int, int] | None = None


@dataclass(frozen=True)
class QuantScheme:
    """The complete quantization decision for one layer; ``input=None`` means weight-only."""

    weight: TensorQuant
    input: TensorQuant | None = None
    online: bool = False

    @property
    def weight_only(self) -> bool:
        return self.input is None


MatchKind = Literal["name", "glob", "regex", "module_cls"]


@dataclass(frozen=True)
class Matcher:
    """Reference ``plan.py:13-28``: ``name`` matches the whole prefix or its last component,
    ``glob`` is fnmatch over the prefix, ``regex`` is ``re.match``, ``module_cls`` a substring of the
    layer class name."""

    kind: MatchKind
    pattern: str

    def matches(self, prefix: str, module_cls: type | None) -> bool:
        if self.kind == "name":
            return self.pattern == prefix or prefix.split(".")[-1] == self.pattern
        if self.kind == "glob":
            return fnmatch.fnmatch(prefix, self.pattern)
        if self.kind == "regex":
            return re.match(self.pattern, prefix) is not None
        if self.kind == "module_cls":
            return module_cls is not None and self.pattern in module_cls.__name__
        raise ValueError(f"unknown Matcher kind {self.kind!r}")


@dataclass(frozen=True)
class Rule:
    matcher: Matcher
    scheme: QuantScheme | None   # None = skip: the layer stays bf16


def materialize(scheme: QuantScheme) -> object:
    """Physical weight spec of ``scheme`` (reference ``materialize.py:13-23``)."""
    w = scheme.weight
    if w.dtype is QDType.BF16:
        return Bf16Spec()
    if w.dtype is QDType.FP8_E4M3:
        return Fp8Spec(granularity=w.granularity, block_shape=w.block_shape)
    raise NotImplementedError(f"materialize: no kernels for weight dtype {w.dtype!r} in this package")


FP8_PER_CHANNEL = QuantScheme(weight=TensorQuant(QDType.FP8_E4M3, Granularity.PER_CHANNEL),
                              input=TensorQuant(QDType.FP8_E4M3, Granularity.PER_CHANNEL, dynamic=True))

__all__ = ["QDType", "TensorQuant", "QuantScheme", "MatchKind", "Matcher", "Rule", "materialize", "FP8_PER_CHANNEL"]
