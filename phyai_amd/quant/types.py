"""Types shared by weight specs, layers and kernels."""

from __future__ import annotations

import dataclasses
import enum
from typing import Mapping, NamedTuple, Protocol, runtime_checkable

import torch
import torch.nn as nn


class Granularity(enum.Enum):
    """Layout of a scale tensor relative to its weight (reference ``quant/granularity.py:12-17``)."""

    PER_TENSOR = "per_tensor"
    PER_CHANNEL = "per_channel"
    BLOCK = "block"


class ActivationView(NamedTuple):
    """What ``quantize_activation`` hands to a kernel (reference ``quant/linear.py:25-30``)."""

    x: torch.Tensor
    x_scale: torch.Tensor | None
    granularity: Granularity


@runtime_checkable
class LinearActivationQuant(Protocol):
    """Spec mixin for formats that quantize activations before the matmul
    (reference ``quant/linear.py:33-48``)."""

    needs_act_quant: bool

    def quantize_activation(self, x: torch.Tensor, layer: nn.Module) -> ActivationView: ...


@dataclasses.dataclass(frozen=True)
class AllocationRequest:
    """Shape packet a layer gives its spec (reference ``quant/base.py:24-52``).

    ``weight_shape`` is the local ``(N, K)``; ``logical_widths`` lists the widths
    of the matrices fused along dim ``fused_dim`` (``[N]``, ``[gate, up]``,
    ``[q, k, v]``).
    """

    weight_shape: tuple[int, ...]
    logical_widths: list[int]
    fused_dim: int = 0
    params_dtype: torch.dtype = torch.bfloat16
    device: str | torch.device | None = None
    extras: Mapping[str, object] = dataclasses.field(default_factory=dict)


class WeightSpec(Protocol):
    """Storage format of a weight (reference ``quant/base.py:55-70``)."""

    spec_id: str
    weight_dtype: torch.dtype

    def allocate(self, layer: nn.Module, request: AllocationRequest) -> None: ...

    def process_after_loading(self, layer: nn.Module) -> None: ...
