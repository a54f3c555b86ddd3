"""Which weight matrices should pass the Infinity Cache by.

An MI355X has 256 MB of memory-side cache behind its L2s.  A denoise loop re-reads the same weights
every step; when they exceed that cache (the Pi0.5 action expert: 311 MB of fp8 weights per step)
and everything is cached alike, each matrix is evicted before its next use and nothing ever hits.
Reading the largest matrices with non-temporal loads (``stream_weights``, flag
``PHYAI_FP8_FLAG_STREAM_WEIGHTS`` of the C ABI) leaves the rest resident from step to step: on the
expert set that is the 18 gate_up matrices (151 MB streamed, 160 MB resident) and 451 -> 426 us per
denoise step.  The reference has no counterpart; its matmul is a library call
(``layers/linear/backends/torch.py:168-175``).
"""
from __future__ import annotations

from typing import Iterable, Sequence

import torch

INFINITY_CACHE_BYTES = 256 << 20


def choose_streamed(sizes: Sequence[int], cache_bytes: int = INFINITY_CACHE_BYTES,
                    resident_fraction: float = 0.7) -> list[bool]:
    """For matrices of ``sizes`` bytes that are all read once per step: which to stream so that the
    others fit ``resident_fraction`` of the cache (the rest is left to activations, scales and
    whatever else the step touches).  Largest first: a streamed matrix costs its kernel a little
    latency, so as few launches as possible should pay it.  Nothing is streamed if all fit."""
    budget = int(cache_bytes * resident_fraction)
    total = sum(sizes)
    streamed = [False] * len(sizes)
    for i in sorted(range(len(sizes)), key=lambda i: (-sizes[i], i)):
        if total <= budget:
            break
        streamed[i] = True
        total -= sizes[i]
    return streamed


def plan_weight_streaming(layers: Iterable[torch.nn.Module], cache_bytes: int = INFINITY_CACHE_BYTES,
                          resident_fraction: float = 0.7) -> int:
    """Set ``layer.stream_weights`` on the quantized linear layers of one replayed step (every
    module with a ``weight`` tensor is counted).  Returns the number of bytes left resident."""
    mods = [m for m in layers if isinstance(getattr(m, "weight", None), torch.Tensor)]
    sizes = [m.weight.numel() * m.weight.element_size() for m in mods]
    flags = choose_streamed(sizes, cache_bytes, resident_fraction)
    for m, f in zip(mods, flags):
        m.stream_weights = bool(f)
    return sum(s for s, f in zip(sizes, flags) if not f)
