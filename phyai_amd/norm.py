"""RMSNorm modules whose output can go straight into an fp8 linear.

Mirrors the reference's ``RMSNorm`` / ``GemmaRMSNorm`` / ``AdaRMSNorm``
(``phyai/src/phyai/layers/layer_norm.py:64-220,409-590``): same constructor arguments,
same ``forward`` contracts, same parameter names and ``hf_keys``.  The extension is
``forward_fp8``: it returns the normalised activations already quantized per token, as the
``ActivationView`` the fp8 linear layers accept in place of a bf16 tensor, so that the bf16
tensor is never written and the separate quantizer launch disappears (the pre-attention and
pre-MLP norms of a decoder layer feed ``qkv_proj`` and ``gate_up_proj`` directly,
``models/pi05/modeling_pi05.py:814-835``).  Only the HIP backend exists here.
"""

from __future__ import annotations

import torch
from torch import nn

from phyai_amd.quant.types import ActivationView, Granularity


def _default_device() -> torch.device:
    return torch.device("cuda", torch.cuda.current_device()) if torch.cuda.is_available() else torch.device("cpu")


class RMSNorm(nn.Module):
    """``out = (x * rsqrt(mean(x^2) + eps) * weight).to(x.dtype)``; ``weight`` starts at one."""

    _gemma = False

    def __init__(self, hidden_size: int, eps: float = 1e-6, backend: str = "hip", *,
                 dtype: torch.dtype | None = None, device: torch.device | str | None = None,
                 prefix: str = "") -> None:
        super().__init__()
        if backend != "hip":
            raise ValueError(f"{type(self).__name__}: only the 'hip' backend exists in this package, got {backend!r}")
        self.backend = backend
        self.hidden_size = hidden_size
        self.variance_epsilon = eps
        self.prefix = prefix
        device = device if device is not None else _default_device()
        self.weight = nn.Parameter(self._initial_weight(hidden_size, dtype or torch.bfloat16, device),
                                   requires_grad=False)
        if prefix:
            self.weight.hf_keys = [(f"{prefix}.weight", None)]

    @staticmethod
    def _initial_weight(hidden_size: int, dtype, device) -> torch.Tensor:
        return torch.ones(hidden_size, dtype=dtype, device=device)

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        from phyai_amd import ops

        fn = ops.gemma_rmsnorm if self._gemma else ops.rmsnorm
        return fn(x, self.weight.data, self.variance_epsilon)

    def forward_fp8(self, x: torch.Tensor) -> ActivationView:
        from phyai_amd import ops

        xq, xs = ops.rmsnorm_fp8(x, self.weight.data, self.variance_epsilon, gemma=self._gemma)
        return ActivationView(xq, xs, Granularity.PER_CHANNEL)

    def extra_repr(self) -> str:
        return f"{self.hidden_size}, eps={self.variance_epsilon}, backend={self.backend!r}"


class GemmaRMSNorm(RMSNorm):
    """``(1 + weight)`` variant; ``weight`` starts at zero, so a fresh module is the plain norm."""

    _gemma = True

    @staticmethod
    def _initial_weight(hidden_size: int, dtype, device) -> torch.Tensor:
        return torch.zeros(hidden_size, dtype=dtype, device=device)


class AdaRMSNorm(nn.Module):
    """Adaptive RMSNorm: ``forward(x, cond) -> (out, gate)`` with ``scale | shift | gate =
    dense(cond)`` and ``out = (x * rsqrt(mean(x^2) + eps) * (1 + scale) + shift).to(x.dtype)``.
    ``dense`` is zero-initialised (a fresh module is the identity norm with a zero gate)."""

    def __init__(self, hidden_size: int, cond_dim: int, eps: float = 1e-6, backend: str = "hip", *,
                 dtype: torch.dtype | None = None, device: torch.device | str | None = None,
                 prefix: str = "") -> None:
        super().__init__()
        if hidden_size <= 0:
            raise ValueError(f"hidden_size must be positive, got {hidden_size}.")
        if cond_dim <= 0:
            raise ValueError(f"cond_dim must be positive, got {cond_dim}.")
        if backend != "hip":
            raise ValueError(f"AdaRMSNorm: only the 'hip' backend exists in this package, got {backend!r}")
        from phyai_amd.linear.layers import ReplicatedLinear

        self.backend = backend
        self.hidden_size = hidden_size
        self.cond_dim = cond_dim
        self.variance_epsilon = eps
        self.prefix = prefix
        self.dense = ReplicatedLinear(cond_dim, 3 * hidden_size, bias=True, params_dtype=dtype or torch.bfloat16,
                                      device=device if device is not None else _default_device(),
                                      prefix=f"{prefix}.dense" if prefix else "")
        nn.init.zeros_(self.dense.weight)
        nn.init.zeros_(self.dense.bias)

    def project_modulation(self, conds: torch.Tensor) -> torch.Tensor:
        """Project a fixed set of conditioning rows once; the caller feeds rows back through
        ``forward(x, modulation=row)`` (keeps ``dense`` out of a captured graph)."""
        if conds.shape[-1] != self.cond_dim:
            raise ValueError(f"AdaRMSNorm.project_modulation: conds last dim {conds.shape[-1]} "
                             f"does not match cond_dim={self.cond_dim}.")
        with torch.no_grad():
            return self.dense(conds)[0].contiguous()

    def _modulation(self, x, cond, modulation) -> torch.Tensor:
        if x.shape[-1] != self.hidden_size:
            raise ValueError(f"AdaRMSNorm: x last dim {x.shape[-1]} does not match hidden_size={self.hidden_size}.")
        if (cond is None) == (modulation is None):
            raise ValueError("AdaRMSNorm.forward: provide exactly one of `cond` or `modulation`.")
        if modulation is None:
            if cond.shape[-1] != self.cond_dim:
                raise ValueError(f"AdaRMSNorm: cond last dim {cond.shape[-1]} does not match cond_dim={self.cond_dim}.")
            modulation, _ = self.dense(cond)
        elif modulation.shape[-1] != 3 * self.hidden_size:
            raise ValueError(f"AdaRMSNorm: modulation last dim {modulation.shape[-1]} does not match "
                             f"3 * hidden_size={3 * self.hidden_size}.")
        if x.dim() == 3 and modulation.dim() == 2:
            modulation = modulation.unsqueeze(1)      # (B, 3D) serves every position of (B, S, D)
        return modulation

    def forward(self, x: torch.Tensor, cond: torch.Tensor | None = None, *,
                modulation: torch.Tensor | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        from phyai_amd import ops

        return ops.adarmsnorm(x, self._modulation(x, cond, modulation), self.variance_epsilon)

    def forward_fp8(self, x: torch.Tensor, cond: torch.Tensor | None = None, *,
                    modulation: torch.Tensor | None = None) -> tuple[ActivationView, torch.Tensor]:
        from phyai_amd import ops

        xq, xs, gate = ops.adarmsnorm_fp8(x, self._modulation(x, cond, modulation), self.variance_epsilon)
        return ActivationView(xq, xs, Granularity.PER_CHANNEL), gate

    def extra_repr(self) -> str:
        return f"{self.hidden_size}, cond_dim={self.cond_dim}, eps={self.variance_epsilon}, backend={self.backend!r}"
