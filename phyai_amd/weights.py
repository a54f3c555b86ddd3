"""Checkpoint loading for the layers of this package (single GPU, local safetensors).

Restates the reference's loader contract (``phyai/src/phyai/weights/loader.py:174-330``,
``weights/shards.py:22-93``): every parameter that loads carries ``hf_keys`` - a list of
``(checkpoint key, shard_id)`` - and a ``weight_loader(param, tensor, shard_id)`` closure;
``load_pretrained`` streams the safetensors files, dispatches each tensor to its parameter, reports
missing / unexpected keys, and calls every module's ``post_load`` hook.  What the reference leaves
open and is wired here: the quantization scales of FUSED layers (q / k / v and gate / up come
from separate checkpoint modules, each with its own ``weight_scale``; the reference attaches a
whole-tensor copy to them, ``linear/layers.py:95-110``, which cannot assemble the fused ``[N]``).
"""

from __future__ import annotations

import dataclasses
from pathlib import Path
from typing import Callable, Iterable

import torch
from torch import nn

WeightLoader = Callable[[nn.Parameter, torch.Tensor, "int | str | None"], None]


def replicated() -> WeightLoader:
    """Full-tensor copy; a 0-D checkpoint scalar fills a one-element parameter (``shards.py:22-31``)."""

    def load(param: nn.Parameter, loaded: torch.Tensor, _shard_id=None) -> None:
        if loaded.dim() == 0 and param.numel() == 1:
            param.data.fill_(loaded.item())
            return
        if tuple(loaded.shape) != tuple(param.shape):
            raise ValueError(f"shape {tuple(loaded.shape)} does not fit parameter {tuple(param.shape)}")
        param.data.copy_(_as_param_dtype(loaded, param))

    return load


def _as_param_dtype(loaded: torch.Tensor, param: nn.Parameter) -> torch.Tensor:
    # fp8 <-> other dtypes: `copy_` would convert values; codes must be taken as stored
    if loaded.dtype == param.dtype:
        return loaded
    if param.dtype == torch.float8_e4m3fn and loaded.dtype == torch.uint8:
        return loaded.view(torch.float8_e4m3fn)
    if loaded.dtype in (torch.float8_e4m3fn, torch.float8_e5m2):
        # codes without their scale are not values: a quantized tensor for a module that was not
        # built as an fp8 linear (an embedding, a head) would silently load garbage
        raise ValueError(f"the checkpoint holds {loaded.dtype} codes for a {param.dtype} parameter; the module was not "
                         "built as an fp8 linear (is it missing from the checkpoint's ignored_layers?)")
    return loaded.to(param.dtype)


def fused_rows(legs: dict) -> WeightLoader:
    """Several checkpoint tensors into row ranges of one parameter (``shards.py:63-93`` at world size
    1): ``legs`` maps ``shard_id -> (row offset, rows)`` along dim 0.  Serves fused weights
    ``[N, K]``, biases ``[N]`` and per-channel scales ``[N]`` alike."""

    def load(param: nn.Parameter, loaded: torch.Tensor, shard_id) -> None:
        if shard_id not in legs:
            raise KeyError(f"fused parameter has no leg {shard_id!r} (legs: {sorted(map(str, legs))})")
        off, size = legs[shard_id]
        if loaded.dim() == 0:                       # a per-tensor scale of the leg serves all its rows
            param.data.narrow(0, off, size).fill_(loaded.item())
            return
        if loaded.shape[0] != size:
            raise ValueError(f"leg {shard_id!r}: {loaded.shape[0]} rows in the checkpoint, {size} in the layer")
        param.data.narrow(0, off, size).copy_(_as_param_dtype(loaded, param))

    return load


def leg_slots(order: list) -> WeightLoader:
    """One scalar per leg into a ``[legs]`` parameter (per-tensor fp8 scales of a fused layer, fanned
    out to rows by the spec's ``process_after_loading``, reference ``quant/fp8.py:36-43,128-135``)."""

    def load(param: nn.Parameter, loaded: torch.Tensor, shard_id) -> None:
        idx = order.index(shard_id) if shard_id in order else None
        if idx is None:
            raise KeyError(f"fused parameter has no leg {shard_id!r}")
        param.data[idx] = loaded.reshape(-1)[0].to(param.dtype)

    return load


@dataclasses.dataclass
class LoadReport:
    loaded: list = dataclasses.field(default_factory=list)
    missing: list = dataclasses.field(default_factory=list)
    optional_missing: list = dataclasses.field(default_factory=list)
    unexpected: list = dataclasses.field(default_factory=list)
    casts: list = dataclasses.field(default_factory=list)

    def summary(self) -> str:
        return (f"loaded={len(self.loaded)} missing={self.missing} optional_missing={len(self.optional_missing)} "
                f"unexpected={self.unexpected} casts={len(self.casts)}")


def _resolve_remap(remap):
    if remap is None:
        return lambda k: k
    if callable(remap):
        return remap
    if isinstance(remap, dict):
        rules = list(remap.items())

        def apply_rules(key: str):
            for src, dst in rules:
                if src in key:
                    key = key.replace(src, dst)
            return key

        return apply_rules
    raise TypeError(f"remap must be callable, dict, or None; got {type(remap).__name__}")


def _resolve_source(source) -> list[Path]:
    if isinstance(source, (str, Path)):
        p = Path(source)
        if p.is_dir():
            files = sorted(p.glob("*.safetensors"))
            if not files:
                raise FileNotFoundError(f"no .safetensors files in {p}")
            return files
        if p.is_file():
            return [p]
        raise FileNotFoundError(f"{p} is neither a local checkpoint folder nor a safetensors file "
                                f"(repository ids are not downloaded: there is no network)")
    return [Path(x) for x in source]


def load_pretrained(model: nn.Module, source: "str | Path | Iterable[str | Path]", *, remap=None,
                    strict: bool = True) -> LoadReport:
    """Load local safetensors checkpoints into ``model`` (``loader.py:174-330``)."""
    from safetensors import safe_open

    remap_fn = _resolve_remap(remap)
    index: dict[str, tuple] = {}
    optional: set[str] = set()
    for name, param in model.named_parameters():
        keys = getattr(param, "hf_keys", None)
        if keys is None:
            continue
        loader = getattr(param, "weight_loader", None) or replicated()
        for hf_key, shard_id in keys:
            if hf_key in index:
                raise RuntimeError(f"hf_key {hf_key!r} is claimed by two params; second hit on {name!r}.")
            index[hf_key] = (param, shard_id, loader)
            if getattr(param, "optional", False):
                optional.add(hf_key)

    report = LoadReport()
    seen: set[str] = set()
    for path in _resolve_source(source):
        with safe_open(str(path), framework="pt", device="cpu") as f:
            for raw in f.keys():
                hf = remap_fn(raw)
                if hf is None:
                    continue
                hit = index.get(hf)
                if hit is None:
                    report.unexpected.append(hf)
                    continue
                param, shard_id, loader = hit
                tensor = f.get_tensor(raw)
                if tensor.dtype != param.dtype:
                    report.casts.append((hf, tensor.dtype, param.dtype))
                loader(param, tensor, shard_id)
                seen.add(hf)
                report.loaded.append(hf)
    for hf_key in index:
        if hf_key not in seen:
            (report.optional_missing if hf_key in optional else report.missing).append(hf_key)
    if strict and (report.missing or report.unexpected):
        raise RuntimeError(f"load_pretrained strict failure: {report.summary()}")
    # A weight that an earlier post_load re-laid in MFMA operand order holds row-major bytes again
    # once every tensor that feeds it was loaded; a reload of only some of them would mix the two.
    for module in model.modules():
        if getattr(module, "weight_layout", None):
            keys = [k for k, _ in getattr(getattr(module, "weight", None), "hf_keys", None) or []]
            hits = [k in seen for k in keys]
            if keys and all(hits):
                module.weight_layout = None
            elif any(hits):
                raise RuntimeError(f"load_pretrained: {type(module).__name__} holds its weight in operand order and the "
                                   f"checkpoint reloads only part of it ({[k for k, h in zip(keys, hits) if h]})")
    for module in model.modules():
        post = getattr(module, "post_load", None)
        if callable(post):
            post()
    return report


__all__ = ["WeightLoader", "replicated", "fused_rows", "leg_slots", "LoadReport", "load_pretrained"]
