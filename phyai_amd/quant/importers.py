"""Config front-ends: a checkpoint's quantization config -> ``QuantPlan``.

Restates the reference's ``phyai/layers/quant/importers`` package: ``ConfigSources`` / the
``QuantImporter`` protocol (``base.py:11-26``), the HF flat fp8 importer (``fp8.py:11-36``), the
llm-compressor ``config_groups`` importer (``compressed_tensors.py:11-80``), the ModelOpt importer
(``modelopt.py:22-59``) and the ordered selection (``registry.py:20-42``).  Parsing is identical;
what cannot run here (nvfp4, int8/int4 weights) is parsed and then refused when the plan lowers a
layer's scheme to a spec.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Protocol, runtime_checkable

from phyai_amd.quant.scheme import Matcher, QDType, QuantScheme, Rule, TensorQuant
from phyai_amd.quant.types import Granularity
from phyai_amd.quant_plan import QuantPlan


@dataclass
class ConfigSources:
    """Every place a quant config may come from."""

    hf_quant_config: dict | None = None   # config.json's quantization_config
    standalone: dict | None = None        # standalone hf_quant_config.json (ModelOpt)
    torchao_cli: str | None = None


@runtime_checkable
class QuantImporter(Protocol):
    name: str

    def detect(self, src: ConfigSources) -> bool: ...

    def build_plan(self, src: ConfigSources) -> QuantPlan: ...


class Fp8Importer:
    name = "fp8"

    def detect(self, src: ConfigSources) -> bool:
        cfg = src.hf_quant_config
        return bool(cfg) and cfg.get("quant_method") == "fp8"

    def build_plan(self, src: ConfigSources) -> QuantPlan:
        cfg = src.hf_quant_config or {}
        block = cfg.get("weight_block_size")
        if block is not None:
            weight = TensorQuant(QDType.FP8_E4M3, Granularity.BLOCK, block_shape=(int(block[0]), int(block[1])))
        else:
            weight = TensorQuant(QDType.FP8_E4M3, Granularity.PER_CHANNEL)
        dynamic = cfg.get("activation_scheme", "dynamic") != "static"
        act = TensorQuant(QDType.FP8_E4M3, Granularity.PER_CHANNEL, dynamic=dynamic)
        ignored = cfg.get("ignored_layers") or cfg.get("modules_to_not_convert") or []
        return QuantPlan(rules=[Rule(Matcher("name", name), None) for name in ignored],
                         default=QuantScheme(weight=weight, input=act))


_STRATEGY_TO_GRAN = {
    "tensor": Granularity.PER_TENSOR,
    "channel": Granularity.PER_CHANNEL,
    "block": Granularity.BLOCK,
    "token": Granularity.PER_CHANNEL,   # per-token row-wise activation
    "group": Granularity.PER_CHANNEL,   # no group granularity in the enum
}


def _dtype_of(qtype: str, num_bits: int) -> QDType:
    if qtype == "float" and num_bits == 8:
        return QDType.FP8_E4M3
    if qtype == "int" and num_bits == 8:
        return QDType.INT8
    if qtype == "int" and num_bits == 4:
        return QDType.INT4
    raise NotImplementedError(f"compressed-tensors: unsupported type={qtype!r} num_bits={num_bits}")


def _to_tensorquant(args: dict) -> TensorQuant:
    strategy = args.get("strategy", "tensor")
    gran = _STRATEGY_TO_GRAN.get(strategy)
    if gran is None:
        raise NotImplementedError(f"compressed-tensors: unsupported strategy {strategy!r}")
    block = args.get("block_structure")
    block_shape = (int(block[0]), int(block[1])) if strategy == "block" and block else None
    return TensorQuant(dtype=_dtype_of(args.get("type", "int"), int(args.get("num_bits", 8))), granularity=gran,
                       symmetric=bool(args.get("symmetric", True)), dynamic=bool(args.get("dynamic", False)),
                       block_shape=block_shape)


def _target_matcher(target: str) -> Matcher:
    if target.startswith("re:"):
        return Matcher("regex", target[3:])
    if "." not in target and target[:1].isupper():   # a bare CamelCase token is a module class name
        return Matcher("module_cls", target)
    return Matcher("name", target)


class CompressedTensorsImporter:
    name = "compressed-tensors"

    def detect(self, src: ConfigSources) -> bool:
        cfg = src.hf_quant_config
        return bool(cfg) and cfg.get("quant_method") == "compressed-tensors"

    def build_plan(self, src: ConfigSources) -> QuantPlan:
        cfg = src.hf_quant_config or {}
        rules: list[Rule] = [Rule(_target_matcher(name), None) for name in cfg.get("ignore") or []]
        for group in (cfg.get("config_groups") or {}).values():
            weight = _to_tensorquant(group["weights"])
            input_args = group.get("input_activations")
            scheme = QuantScheme(weight=weight, input=_to_tensorquant(input_args) if input_args else None)
            rules.extend(Rule(_target_matcher(t), scheme) for t in group.get("targets") or [])
        return QuantPlan(rules=rules, default=None)


_MODELOPT_METHODS = {"modelopt", "modelopt_fp8", "modelopt_fp4"}


def _modelopt_block(src: ConfigSources) -> dict | None:
    if src.standalone and isinstance(src.standalone.get("quantization"), dict):
        return src.standalone["quantization"]
    cfg = src.hf_quant_config
    if cfg and cfg.get("quant_method") in _MODELOPT_METHODS:
        return cfg
    return None


def _scheme_for_algo(quant_algo: str) -> QuantScheme:
    algo = quant_algo.upper()
    if "FP4" in algo:
        return QuantScheme(weight=TensorQuant(QDType.NVFP4, Granularity.BLOCK, micro_scaled=True),
                           input=TensorQuant(QDType.NVFP4, Granularity.PER_CHANNEL, micro_scaled=True, dynamic=True))
    if "FP8" in algo:
        return QuantScheme(weight=TensorQuant(QDType.FP8_E4M3, Granularity.PER_CHANNEL),
                           input=TensorQuant(QDType.FP8_E4M3, Granularity.PER_CHANNEL, dynamic=True))
    raise NotImplementedError(f"modelopt: unsupported quant_algo {quant_algo!r}")


class ModelOptImporter:
    name = "modelopt"

    def detect(self, src: ConfigSources) -> bool:
        block = _modelopt_block(src)
        return block is not None and block.get("quant_algo") is not None

    def build_plan(self, src: ConfigSources) -> QuantPlan:
        block = _modelopt_block(src) or {}
        excluded = block.get("exclude_modules") or block.get("ignore") or []
        return QuantPlan(rules=[Rule(Matcher("name", name), None) for name in excluded],
                         default=_scheme_for_algo(block["quant_algo"]))


DEFAULT_IMPORTERS: tuple[QuantImporter, ...] = (Fp8Importer(), CompressedTensorsImporter(), ModelOptImporter())


def select_importer(src: ConfigSources, importers: tuple[QuantImporter, ...] = DEFAULT_IMPORTERS):
    """The first importer that recognises ``src``, else ``None``."""
    for importer in importers:
        if importer.detect(src):
            return importer
    return None


def build_quant_plan(src: ConfigSources, importers: tuple[QuantImporter, ...] = DEFAULT_IMPORTERS) -> QuantPlan | None:
    importer = select_importer(src, importers)
    return importer.build_plan(src) if importer is not None else None


def load_quant_plan(checkpoint_dir) -> QuantPlan | None:
    """The plan implied by a local checkpoint folder's ``config.json`` (``quantization_config`` or
    ``compression_config``) and / or ``hf_quant_config.json``; ``None`` for an unquantized one
    (reference ``active.py:36-92``; repo ids are not resolved here - there is no network)."""
    import json
    from pathlib import Path

    if checkpoint_dir is None:
        return None
    folder = Path(checkpoint_dir)
    if not folder.is_dir():
        raise FileNotFoundError(f"load_quant_plan: {folder} is not a local checkpoint folder")
    hf_quant_config = standalone = None
    config_path = folder / "config.json"
    if config_path.is_file():
        raw = json.loads(config_path.read_text(encoding="utf-8"))
        hf_quant_config = raw.get("quantization_config") or raw.get("compression_config")
    standalone_path = folder / "hf_quant_config.json"
    if standalone_path.is_file():
        standalone = json.loads(standalone_path.read_text(encoding="utf-8"))
    if not hf_quant_config and not standalone:
        return None
    return build_quant_plan(ConfigSources(hf_quant_config=hf_quant_config, standalone=standalone))


__all__ = ["ConfigSources", "QuantImporter", "Fp8Importer", "CompressedTensorsImporter", "ModelOptImporter",
           "DEFAULT_IMPORTERS", "select_importer", "build_quant_plan", "load_quant_plan"]
