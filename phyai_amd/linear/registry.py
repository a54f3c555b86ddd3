"""Kernel registry and selection policies.

Behaviour follows the reference's ``phyai/layers/linear/registry.py:34-205``:
classes announce themselves with ``@register_linear_kernel(prefer_for=...)`` at
import time, ``init()`` instantiates them into a ``LinearKernelRegistry``, and
``candidates(probe)`` lists kernels that accept the probe - those preferred for
the probe's ``(spec_id, regime)`` first, the rest in registration order - leaving
out kernels that cannot be captured while a graph is being recorded.
"""

from __future__ import annotations

from typing import Callable, Iterable, Protocol, runtime_checkable

import torch

from phyai_amd.linear.backend import KernelProbe, LinearKernel
from phyai_amd.state import Mode, NoBackendError

_DECLARED: list[tuple[type, frozenset[tuple[str, str]]]] = []


def register_linear_kernel(*, prefer_for: Iterable[tuple[str, str]] | None = None) -> Callable[[type], type]:
    """Class decorator: record a kernel class (not an instance) for ``init()``."""
    wins = frozenset(prefer_for or ())

    def remember(cls: type) -> type:
        _DECLARED.append((cls, wins))
        return cls

    return remember


def list_registered_linear_kernels() -> list[tuple[type, frozenset[tuple[str, str]]]]:
    return list(_DECLARED)


def _regime_of(M_bucket: int) -> str:
    """Buckets up to 3 (at most 7 rows) are "decode", everything longer "prefill"."""
    return "decode" if M_bucket <= 3 else "prefill"


class LinearKernelRegistry:
    def __init__(self) -> None:
        self._kernels: list[LinearKernel] = []
        self._prefer: dict[tuple[str, str], list[str]] = {}

    def register(self, kernel: LinearKernel, *, prefer_for: Iterable[tuple[str, str]] | None = None) -> None:
        self._kernels.append(kernel)
        for key in prefer_for or ():
            self._prefer.setdefault(key, []).append(kernel.name)

    def _usable(self, kernel: LinearKernel, probe: KernelProbe) -> bool:
        if probe.mode is Mode.GRAPH_CAPTURING and not kernel.supports_capture():
            return False
        return kernel.can_handle(probe)

    def candidates(self, probe: KernelProbe) -> list[LinearKernel]:
        preferred = self._prefer.get((probe.spec_id, _regime_of(probe.M_bucket)), [])
        by_name = {}
        for k in self._kernels:
            by_name.setdefault(k.name, k)
        first = [by_name[n] for n in preferred if n in by_name and self._usable(by_name[n], probe)]
        rest = [k for k in self._kernels if k.name not in preferred and self._usable(k, probe)]
        return first + rest

    def has(self, probe: KernelProbe) -> bool:
        return bool(self.candidates(probe))

    def all(self) -> list[LinearKernel]:
        return list(self._kernels)

    def validate(self, *, sample_specs: list[str], sm: int, N: int = 4096, K: int = 4096) -> None:
        """Start-up check: every preferred name exists, and each sampled spec has a
        kernel in both regimes (and under capture when any kernel claims capture)."""
        names = {k.name for k in self._kernels}
        for (spec_id, regime), prefs in self._prefer.items():
            for n in prefs:
                if n not in names:
                    raise NoBackendError(
                        f"prefer_for[({spec_id!r}, {regime!r})]={n!r} but no kernel with that name "
                        f"is registered (have: {sorted(names)})")
        modes = [Mode.EAGER]
        if any(k.supports_capture() for k in self._kernels):
            modes.append(Mode.GRAPH_CAPTURING)
        for spec_id in sample_specs:
            for bucket in (1, 10):
                for mode in modes:
                    probe = KernelProbe(spec_id=spec_id, M_bucket=bucket, N=N, K=K, in_dtype=torch.bfloat16,
                                        out_dtype=torch.bfloat16, sm=sm, mode=mode)
                    if not self.has(probe):
                        raise NoBackendError(
                            f"no LinearKernel for spec={spec_id!r} regime={_regime_of(bucket)} "
                            f"mode={mode.value} sm={sm}")


@runtime_checkable
class Policy(Protocol):
    def select(self, candidates: list[LinearKernel]) -> LinearKernel: ...


class DefaultPolicy:
    """First candidate wins; the registry has already ordered them."""

    def select(self, candidates: list[LinearKernel]) -> LinearKernel:
        if not candidates:
            raise NoBackendError("no LinearKernel candidate")
        return candidates[0]


class ForcedPolicy:
    """Pick the candidate called ``name`` if present, else defer to ``fallback``."""

    def __init__(self, name: str, fallback: Policy | None = None) -> None:
        self.name = name
        self.fallback = fallback or DefaultPolicy()

    def select(self, candidates: list[LinearKernel]) -> LinearKernel:
        return next((k for k in candidates if k.name == self.name), None) or self.fallback.select(candidates)
