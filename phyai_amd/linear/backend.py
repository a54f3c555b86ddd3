"""Kernel plug-in protocol of the linear layers.

Same surface as the reference's ``phyai/layers/linear/backend.py:25-62``: the
dispatcher describes a call with a ``KernelProbe`` and a kernel answers with
``can_handle``; ``apply(layer, x, bias)`` is the hot call.
"""

from __future__ import annotations

import dataclasses
from typing import Protocol, runtime_checkable

import torch

from phyai_amd.quant.types import Granularity  # noqa: F401  (historical import path)
from phyai_amd.state import Mode


@dataclasses.dataclass(frozen=True)
class KernelProbe:
    """Hashable description of one linear call; also the dispatcher's cache key."""

    spec_id: str
    M_bucket: int
    N: int
    K: int
    in_dtype: torch.dtype
    out_dtype: torch.dtype
    sm: int
    mode: Mode


@runtime_checkable
class LinearKernel(Protocol):
    name: str

    def can_handle(self, probe: KernelProbe) -> bool: ...

    def supports_capture(self) -> bool: ...

    def apply(self, layer: torch.nn.Module, x: torch.Tensor, bias: torch.Tensor | None) -> torch.Tensor: ...
