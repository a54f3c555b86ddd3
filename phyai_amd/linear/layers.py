"""Linear layer classes of the reference, at tensor-parallel size 1.

Constructor signatures, attribute names and the ``(y, bias_or_None)`` return
convention follow ``phyai/layers/linear/layers.py:43-631`` of the reference, so
model code written against it can build these classes unchanged.  This build is
single-GPU: the ``axis`` / ``sp_axis`` / ``mesh`` arguments are accepted and
recorded, every layer holds its full weight (``tp_size == 1``, ``tp_rank == 0``)
and no collective is ever issued.  Sharding across GPUs would slot in exactly
where the reference has it: after ``kernel.apply`` in ``forward``.

Spec resolution order (reference ``layers.py:69-82``): explicit ``spec=``, else
the spec named by the active quantization plan for ``prefix`` (if a plan is
installed, see :mod:`phyai_amd.quant_plan`), else ``Bf16Spec``.
"""

from __future__ import annotations

from types import MappingProxyType
from typing import Mapping, Sequence

import torch
import torch.nn as nn

from phyai_amd.linear.dispatch import get_linear_dispatcher
from phyai_amd.quant import AllocationRequest, Bf16Spec
from phyai_amd.quant.types import ActivationView


def _M_of(x) -> int:
    if isinstance(x, ActivationView):
        x = x.x
    """Number of token rows: product of every dim but the last."""
    m = 1
    for s in x.shape[:-1]:
        m *= int(s)
    return m


def _max_of_legs(layer: nn.Module):
    """Loader of a scalar that every leg of a fused layer brings its own copy of: keep the largest
    of one load (``post_load`` forgets what was seen, so a reload starts afresh)."""

    def load(param: nn.Parameter, loaded: torch.Tensor, _shard_id=None) -> None:
        v = float(loaded.reshape(-1)[0])
        layer._fused_scalar_seen.append(v)
        param.data.fill_(max(layer._fused_scalar_seen))

    return load


def _default_device() -> torch.device:
    return torch.device("cuda", torch.cuda.current_device()) if torch.cuda.is_available() else torch.device("cpu")


class LinearBase(nn.Module):
    """State common to every variant; subclasses call :meth:`_allocate` once."""

    def __init__(self, in_features: int, out_features: int, *, bias: bool = True, skip_bias_add: bool = False,
                 params_dtype: torch.dtype | None = None, spec: object | None = None,
                 scheme: object | None = None, device: torch.device | str | None = None,
                 prefix: str = "") -> None:
        super().__init__()
        self.in_features = in_features
        self.out_features = out_features
        self.params_dtype = params_dtype or torch.get_default_dtype()
        self.skip_bias_add = skip_bias_add
        self.prefix = prefix
        self.device = device if device is not None else _default_device()
        self._bias_requested = bias
        if spec is not None:
            self.spec = spec
        else:
            from phyai_amd import quant_plan

            self.spec = quant_plan.resolve_spec(scheme=scheme, prefix=prefix, layer_cls=type(self)) or Bf16Spec()
        # single GPU
        self.tp_size = 1
        self.tp_rank = 0

    # -- construction helpers ------------------------------------------------------
    def _allocate(self, n: int, k: int, widths: list[int], bias: bool) -> None:
        self.spec.allocate(self, AllocationRequest(weight_shape=(n, k), logical_widths=widths, fused_dim=0,
                                                   params_dtype=self.params_dtype, device=self.device))
        self.input_size_per_partition = k
        self.output_size_per_partition = n
        self.input_size_global = k
        self.output_size_global = n
        if bias:
            self.bias = nn.Parameter(torch.zeros(n, dtype=self.params_dtype, device=self.device),
                                     requires_grad=False)
        else:
            self.register_parameter("bias", None)

    def _name_checkpoint_keys(self, legs: Sequence[tuple[str, object]] | None) -> None:
        """Record which checkpoint tensors feed which rows of the fused weight.

        ``legs`` is a list of ``(hf_module_path, shard_id)``; ``None`` means the
        layer's own prefix.  The scale parameters a spec allocated are marked
        optional, as checkpoints without quantization do not carry them.
        """
        if not self.prefix:
            return
        from phyai_amd import weights as W

        fused = legs is not None
        legs = list(legs) if fused else [(self.prefix, None)]
        # row range of every leg in the fused parameter
        offsets, off = {}, 0
        for (_, sid), width in zip(legs, getattr(self, "output_partition_sizes", [self.output_size_per_partition])):
            offsets[sid] = (off, width)
            off += width
        rows = W.fused_rows(offsets) if fused else W.replicated()
        self.weight.hf_keys = [(f"{base}.weight", sid) for base, sid in legs]
        self.weight.weight_loader = rows
        if self.bias is not None:
            self.bias.hf_keys = [(f"{base}.bias", sid) for base, sid in legs]
            self.bias.weight_loader = rows
        for name in ("weight_scale", "input_scale", "weight_global_scale"):
            p = getattr(self, name, None)
            if isinstance(p, nn.Parameter):
                p.hf_keys = [(f"{base}.{name}", sid) for base, sid in legs]
                p.optional = True
                if not fused:
                    p.weight_loader = W.replicated()
                elif p.shape[0] == self.output_size_per_partition:
                    p.weight_loader = rows                                    # one scale per output row
                elif p.shape[0] == len(legs):
                    p.weight_loader = W.leg_slots([sid for _, sid in legs])   # one scale per leg
                else:
                    # one value for the whole fused layer (a static activation scale): every leg
                    # of a checkpoint carries its own; the largest is the safe common choice
                    self._fused_scalar_seen = []
                    p.weight_loader = _max_of_legs(self)

    def post_load(self) -> None:
        if hasattr(self, "_fused_scalar_seen"):
            self._fused_scalar_seen = []
        hook = getattr(self.spec, "process_after_loading", None)
        if callable(hook):
            hook(self)

    # -- the hot call -----------------------------------------------------------------
    def _run(self, x, add_bias: bool = True, **kernel_kwargs) -> torch.Tensor:
        """``x`` is the bf16 activations or, for an fp8 layer, an ``ActivationView`` that a norm
        already quantized per token (``phyai_amd.norm``): then the layer's own quantizer is skipped."""
        quantized = isinstance(x, ActivationView)
        if quantized and not getattr(self.spec, "needs_act_quant", False):
            raise RuntimeError(f"{type(self).__name__}: got quantized activations but spec "
                               f"{self.spec.spec_id!r} does not quantize its input")
        kernel = get_linear_dispatcher().select(
            spec_id=self.spec.spec_id, M=_M_of(x), N=self.output_size_per_partition,
            K=self.input_size_per_partition, in_dtype=self.params_dtype if quantized else x.dtype,
            out_dtype=self.params_dtype)
        bias = self.bias if (add_bias and not self.skip_bias_add) else None
        return kernel.apply(self, x, bias, **kernel_kwargs)

    def forward(self, x: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor | None]:
        y = self._run(x)
        return y, (self.bias if self.skip_bias_add else None)

    def forward_fused(self, x: torch.Tensor, epilogue: str) -> torch.Tensor:
        """Run the linear with an activation fused into the GEMM epilogue.  Only kernels
        that advertise ``apply(..., epilogue=)`` can do this; callers check
        :func:`supports_fused_epilogue` first."""
        return self._run(x, epilogue=epilogue)

    def forward_addcmul(self, x, residual: torch.Tensor, gate: torch.Tensor) -> torch.Tensor:
        """``torch.addcmul(residual, self(x)[0], gate)`` with the multiply-add inside the GEMM epilogue
        (the gated residual after ``o_proj`` / ``down_proj``, reference
        ``models/pi05/modeling_pi05.py:826,835``).  Falls back to the separate op for kernels
        without the extension."""
        if self.supports_fused_epilogue(x):
            return self._run(x, residual=residual, gate=gate)
        y, _ = self.forward(x)
        return torch.addcmul(residual, y, gate)

    def supports_fused_epilogue(self, x) -> bool:
        kernel = get_linear_dispatcher().select(
            spec_id=self.spec.spec_id, M=_M_of(x), N=self.output_size_per_partition,
            K=self.input_size_per_partition,
            in_dtype=self.params_dtype if isinstance(x, ActivationView) else x.dtype, out_dtype=self.params_dtype)
        return getattr(kernel, "name", "") == "hip_fp8" and not self.skip_bias_add


class ReplicatedLinear(LinearBase):
    """Full weight on every rank (reference ``layers.py:126-198``)."""

    def __init__(self, in_features: int, out_features: int, *, bias: bool = True, skip_bias_add: bool = False,
                 params_dtype=None, spec=None, scheme=None, device=None, prefix: str = "") -> None:
        super().__init__(in_features, out_features, bias=bias, skip_bias_add=skip_bias_add,
                         params_dtype=params_dtype, spec=spec, scheme=scheme, device=device, prefix=prefix)
        self._allocate(out_features, in_features, [out_features], bias)
        self._name_checkpoint_keys(None)


class ColumnParallelLinear(LinearBase):
    """Output-dim sharded linear (reference ``layers.py:201-317``); unsharded here."""

    def __init__(self, in_features: int, out_features: int, *, axis: str = "tp", sp_axis: str | None = None,
                 gather_output: bool = False, bias: bool = True, skip_bias_add: bool = False,
                 params_dtype=None, spec=None, scheme=None, output_sizes: list[int] | None = None,
                 mesh: str = "model", device=None, prefix: str = "") -> None:
        super().__init__(in_features, out_features, bias=bias, skip_bias_add=skip_bias_add,
                         params_dtype=params_dtype, spec=spec, scheme=scheme, device=device, prefix=prefix)
        self.axis, self.sp_axis, self.gather_output, self.mesh_name = axis, sp_axis, gather_output, mesh
        sizes = list(output_sizes) if output_sizes is not None else [out_features]
        if sum(sizes) != out_features:
            raise ValueError(f"output_sizes sum ({sum(sizes)}) != out_features ({out_features})")
        self.output_partition_sizes = sizes
        self.output_sizes_global = list(sizes)
        self._allocate(out_features, in_features, sizes, bias)
        if len(sizes) == 1:
            self._name_checkpoint_keys(None)


class MergedColumnParallelLinear(ColumnParallelLinear):
    """Several projections fused along N, e.g. ``[gate, up]`` (reference ``layers.py:320-390``)."""

    DEFAULT_HF_LEGS: tuple[str, ...] = ("gate_proj", "up_proj")

    def __init__(self, in_features: int, output_sizes: list[int], *, axis: str = "tp",
                 sp_axis: str | None = None, gather_output: bool = False, bias: bool = True,
                 skip_bias_add: bool = False, params_dtype=None, spec=None, scheme=None,
                 hf_legs: Sequence[str] | None = None, mesh: str = "model", device=None,
                 prefix: str = "") -> None:
        super().__init__(in_features, sum(output_sizes), axis=axis, sp_axis=sp_axis, gather_output=gather_output,
                         bias=bias, skip_bias_add=skip_bias_add, params_dtype=params_dtype, spec=spec,
                         scheme=scheme, output_sizes=output_sizes, mesh=mesh, device=device, prefix=prefix)
        legs = tuple(hf_legs) if hf_legs is not None else self.DEFAULT_HF_LEGS
        if len(legs) != len(self.output_partition_sizes):
            raise ValueError(f"hf_legs length {len(legs)} != output_partition_sizes "
                             f"{len(self.output_partition_sizes)}")
        self.hf_legs = legs
        parent = prefix.rpartition(".")[0]
        self._name_checkpoint_keys([(f"{parent}.{leg}" if parent else leg, i) for i, leg in enumerate(legs)])


class QKVParallelLinear(ColumnParallelLinear):
    """q, k and v fused into one ``N = (heads + 2 * kv_heads) * head_dim`` GEMM
    (reference ``layers.py:393-521``)."""

    DEFAULT_HF_LEGS: Mapping[str, str] = MappingProxyType({"q": "q_proj", "k": "k_proj", "v": "v_proj"})

    def __init__(self, hidden_size: int, head_dim: int, num_heads: int, num_kv_heads: int | None = None, *,
                 axis: str = "tp", sp_axis: str | None = None, gather_output: bool = False, bias: bool = True,
                 skip_bias_add: bool = False, params_dtype=None, spec=None, scheme=None,
                 hf_legs: Mapping[str, str] | None = None, mesh: str = "model", device=None,
                 prefix: str = "") -> None:
        kv = num_heads if num_kv_heads is None else num_kv_heads
        q_size, kv_size = num_heads * head_dim, kv * head_dim
        super().__init__(hidden_size, q_size + 2 * kv_size, axis=axis, sp_axis=sp_axis,
                         gather_output=gather_output, bias=bias, skip_bias_add=skip_bias_add,
                         params_dtype=params_dtype, spec=spec, scheme=scheme,
                         output_sizes=[q_size, kv_size, kv_size], mesh=mesh, device=device, prefix=prefix)
        self.num_kv_replicas = 1
        self.head_dim, self.num_heads, self.num_kv_heads = head_dim, num_heads, kv
        legs = dict(hf_legs) if hf_legs is not None else dict(self.DEFAULT_HF_LEGS)
        for need in ("q", "k", "v"):
            if need not in legs:
                raise ValueError(f"hf_legs missing key {need!r}; got {legs!r}")
        self.hf_legs = legs
        parent = prefix.rpartition(".")[0]
        self._name_checkpoint_keys([(f"{parent}.{legs[k]}" if parent else legs[k], k) for k in ("q", "k", "v")])


class RowParallelLinear(LinearBase):
    """Input-dim sharded linear (reference ``layers.py:524-631``); unsharded here, so the
    exit all-reduce / reduce-scatter of the reference has nothing to do."""

    def __init__(self, in_features: int, out_features: int, *, axis: str = "tp", sp_axis: str | None = None,
                 input_is_parallel: bool = True, reduce_results: bool = True, bias: bool = True,
                 skip_bias_add: bool = False, params_dtype=None, spec=None, scheme=None,
                 mesh: str = "model", device=None, prefix: str = "") -> None:
        super().__init__(in_features, out_features, bias=bias, skip_bias_add=skip_bias_add,
                         params_dtype=params_dtype, spec=spec, scheme=scheme, device=device, prefix=prefix)
        self.axis, self.sp_axis, self.mesh_name = axis, sp_axis, mesh
        self.input_is_parallel, self.reduce_results = input_is_parallel, reduce_results
        self._allocate(out_features, in_features, [out_features], bias)
        self._name_checkpoint_keys(None)
