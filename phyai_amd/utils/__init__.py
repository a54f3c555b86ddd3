"""Small device helpers."""

from __future__ import annotations

import torch


def sm_arch(device=None) -> int:
    """``major * 10 + minor`` of the device's compute capability, 0 without a GPU.

    Same contract as the reference's ``phyai/utils/cuda.py:51-62``.  PyTorch-ROCm
    reports gfx950 as capability (9, 5), i.e. 95, which clears the reference's
    ``sm >= 89`` gate for fp8 (``layers/linear/backends/torch.py:86``).
    """
    if not torch.cuda.is_available():
        return 0
    try:
        major, minor = torch.cuda.get_device_capability(device)
    except (RuntimeError, AssertionError):
        return 0
    return major * 10 + minor


def gcn_arch(device=None) -> str:
    """Architecture name of the device (``"gfx950"`` on MI355X), ``""`` without a GPU."""
    if not torch.cuda.is_available():
        return ""
    name = getattr(torch.cuda.get_device_properties(device if device is not None else 0), "gcnArchName", "")
    return name.split(":")[0]


__all__ = ["sm_arch", "gcn_arch"]
