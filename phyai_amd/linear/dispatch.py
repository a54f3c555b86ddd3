"""Cached kernel selection (reference ``phyai/layers/linear/dispatch.py:28-113``).

The key is ``(spec_id, M.bit_length(), N, K, in_dtype, out_dtype, sm, mode)``:
token counts are bucketed logarithmically and the eager / capturing mode is part
of the key, so a graph capture re-selects with the capture filter applied.
``PHYAI_FORCE_LINEAR_KERNEL=<name>`` forces a kernel by name when it is among
the candidates.
"""

from __future__ import annotations

import os
from typing import Any

import torch

from phyai_amd.linear.backend import KernelProbe, LinearKernel
from phyai_amd.linear.registry import DefaultPolicy, ForcedPolicy, LinearKernelRegistry, Policy
from phyai_amd.state import NoBackendError, current_mode
from phyai_amd.utils import sm_arch


def _M_bucket(M: int) -> int:
    return M.bit_length() if M > 0 else 0


class KernelDispatcher:
    def __init__(self, registry: LinearKernelRegistry, policy: Policy | None = None,
                 *, force: str | None = None) -> None:
        self.registry = registry
        forced = os.environ.get("PHYAI_FORCE_LINEAR_KERNEL") or force
        self.policy: Policy = policy if policy is not None else (ForcedPolicy(forced) if forced else DefaultPolicy())
        self._cache: dict[tuple[Any, ...], LinearKernel] = {}
        self._sm = sm_arch()

    def select(self, *, spec_id: str, M: int, N: int, K: int, in_dtype: torch.dtype,
               out_dtype: torch.dtype) -> LinearKernel:
        mode = current_mode()
        bucket = _M_bucket(M)
        key = (spec_id, bucket, N, K, in_dtype, out_dtype, self._sm, mode)
        hit = self._cache.get(key)
        if hit is not None:
            return hit
        probe = KernelProbe(spec_id=spec_id, M_bucket=bucket, N=N, K=K, in_dtype=in_dtype,
                            out_dtype=out_dtype, sm=self._sm, mode=mode)
        cands = self.registry.candidates(probe)
        if not cands:
            raise NoBackendError(
                f"no LinearKernel for spec={spec_id} M_bucket={bucket} N={N} K={K} in_dtype={in_dtype} "
                f"out_dtype={out_dtype} mode={mode.value} sm={self._sm}")
        chosen = self.policy.select(cands)
        self._cache[key] = chosen
        return chosen

    def clear_cache(self) -> None:
        self._cache.clear()


_dispatcher: KernelDispatcher | None = None


def get_linear_dispatcher() -> KernelDispatcher:
    if _dispatcher is None:
        raise RuntimeError("phyai_amd.linear.init(...) not called yet")
    return _dispatcher


def _set_linear_dispatcher(d: KernelDispatcher | None) -> None:
    global _dispatcher
    _dispatcher = d
