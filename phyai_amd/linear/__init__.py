"""phyai_amd.linear - linear layers with declarative kernel dispatch.

Mirrors the public names of the reference's ``phyai.layers.linear``
(``__init__.py:54-171``)::

    import phyai_amd.linear as L
    L.init()
    qkv = L.QKVParallelLinear(1024, 256, 8, 1, bias=False,
                              spec=L.Fp8Spec(granularity=L.Granularity.PER_CHANNEL))
    y, _ = qkv(x)
"""

from __future__ import annotations

from phyai_amd.linear.backend import Granularity, KernelProbe, LinearKernel
from phyai_amd.linear.dispatch import KernelDispatcher, _set_linear_dispatcher, get_linear_dispatcher
from phyai_amd.linear.kernels import HipFp8Kernel, TorchBf16Kernel
from phyai_amd.linear.layers import (
    ColumnParallelLinear,
    LinearBase,
    MergedColumnParallelLinear,
    QKVParallelLinear,
    ReplicatedLinear,
    RowParallelLinear,
)
from phyai_amd.linear.registry import (
    DefaultPolicy,
    ForcedPolicy,
    LinearKernelRegistry,
    Policy,
    list_registered_linear_kernels,
    register_linear_kernel,
)
from phyai_amd.quant import ActivationView, AllocationRequest, Bf16Spec, Fp8Spec, WeightSpec
from phyai_amd.utils import sm_arch


def supported_specs_for_sm(sm: int) -> list[str]:
    """Specs ``validate()`` must find a kernel for on this device: bf16 everywhere,
    per-tensor / per-channel fp8 where the device reports capability >= 89
    (reference ``__init__.py:54-79``; gfx950 reports 95)."""
    specs = ["bf16"]
    if sm >= 89:
        specs += ["fp8_per_tensor", "fp8_per_channel"]
    return specs


def init(*, validate: bool = True, sample_specs: list[str] | None = None,
         force: str | None = None) -> KernelDispatcher:
    """Build the process-wide dispatcher from the kernels declared so far."""
    reg = LinearKernelRegistry()
    for cls, prefer_for in list_registered_linear_kernels():
        reg.register(cls(), prefer_for=set(prefer_for) if prefer_for else None)
    if validate:
        sm = sm_arch()
        reg.validate(sample_specs=sample_specs if sample_specs is not None else supported_specs_for_sm(sm), sm=sm)
    d = KernelDispatcher(reg, force=force)
    _set_linear_dispatcher(d)
    return d


def _reset_for_test() -> None:
    _set_linear_dispatcher(None)


__all__ = [
    "init", "supported_specs_for_sm",
    "LinearBase", "ReplicatedLinear", "ColumnParallelLinear", "RowParallelLinear",
    "MergedColumnParallelLinear", "QKVParallelLinear",
    "Bf16Spec", "Fp8Spec", "ActivationView", "AllocationRequest", "WeightSpec", "Granularity",
    "KernelDispatcher", "get_linear_dispatcher", "LinearKernelRegistry", "DefaultPolicy", "ForcedPolicy",
    "Policy", "LinearKernel", "KernelProbe", "register_linear_kernel", "list_registered_linear_kernels",
    "HipFp8Kernel", "TorchBf16Kernel",
]
