"""Offline W8A8 fp8 weight quantizer: a bf16 safetensors checkpoint -> the HF flat fp8 layout.

The reference has no fp8 weight quantizer (``phyai/layers/quant/fp8.py:80-83`` leaves a TODO and its
``phyai-model-optimizer`` package is empty).  This tool writes what its loader and importers expect:
for every selected 2-D ``<module>.weight`` an e4m3fn tensor of the same name plus
``<module>.weight_scale`` ``[N]`` fp32 (per output channel, absmax / 448, computed by the library's
weight-quantizer kernel), every other tensor unchanged, and ``config.json`` with
``quantization_config = {"quant_method": "fp8", "activation_scheme": "dynamic", "ignored_layers":
[...]}`` - the form ``Fp8Importer`` reads (``quant/importers/fp8.py:14-36``).

Only matrices that the model builds as fp8 linears may be converted: an embedding table, the
``lm_head`` tied to it, position tables and norm weights are read by modules that have no
``weight_scale`` and would take the codes for values.  Modules whose name matches
``DEFAULT_KEEP`` are therefore left alone unless ``--only`` names them explicitly, and everything
left unquantized is listed in ``ignored_layers``.  A sharded checkpoint's
``model.safetensors.index.json`` is rewritten with the added ``weight_scale`` keys.

    python -m phyai_amd.quantize_checkpoint SRC_DIR DST_DIR [--ignore NAME ...] [--only GLOB ...]
"""

from __future__ import annotations

import argparse
import fnmatch
import json
from pathlib import Path

import torch


# Module-name patterns (matched against every dotted component) that are never fp8 linears.
DEFAULT_KEEP = ("*embed*", "lm_head", "*norm*", "*position*", "*pos_emb*", "wte", "wpe")


def _selected(module: str, only: list[str], ignore: list[str]) -> bool:
    if any(module == n or module.split(".")[-1] == n for n in ignore):
        return False
    if only:
        return any(fnmatch.fnmatch(module, g) for g in only)
    return not any(fnmatch.fnmatch(part, pat) for part in module.split(".") for pat in DEFAULT_KEEP)


_DTYPE_BYTES = {"F64": 8, "F32": 4, "F16": 2, "BF16": 2, "I64": 8, "I32": 4, "I16": 2, "I8": 1, "U8": 1, "BOOL": 1,
                "F8_E4M3": 1, "F8_E5M2": 1}


def quantize_state(tensors: dict, *, only: list[str] | None = None, ignore: list[str] | None = None,
                   device: torch.device | str = "cuda") -> tuple[dict, list[str]]:
    """``(new tensors, quantized module names)``.  A ``.weight`` is quantized when it is 2-D, bf16 /
    fp16 / fp32, has K % 16 == 0 and N % 16 == 0 (what the kernels accept) and its module is selected:
    named by ``only`` when that is given, otherwise not matching ``DEFAULT_KEEP``; never one in ``ignore``."""
    from phyai_amd import ops

    only, ignore = list(only or []), list(ignore or [])
    out, done = {}, []
    for key, t in tensors.items():
        module, _, leaf = key.rpartition(".")
        ok = (leaf == "weight" and t.dim() == 2 and t.dtype in (torch.bfloat16, torch.float16, torch.float32)
              and t.shape[0] % 16 == 0 and t.shape[1] % 16 == 0 and _selected(module, only, ignore))
        if not ok:
            out[key] = t
            continue
        wq, ws = ops.fp8_weight_quant(t.to(device=device, dtype=torch.bfloat16).contiguous())
        out[key] = wq.cpu()
        out[f"{module}.weight_scale"] = ws.cpu()
        done.append(module)
    return out, done


def quantize_checkpoint(src: str | Path, dst: str | Path, *, only: list[str] | None = None,
                        ignore: list[str] | None = None, device: torch.device | str = "cuda") -> list[str]:
    from safetensors import safe_open
    from safetensors.torch import save_file

    src, dst = Path(src), Path(dst)
    dst.mkdir(parents=True, exist_ok=True)
    done: list[str] = []
    skipped: list[str] = []
    for path in sorted(src.glob("*.safetensors")):
        with safe_open(str(path), framework="pt", device="cpu") as f:
            tensors = {k: f.get_tensor(k) for k in f.keys()}
        new, names = quantize_state(tensors, only=only, ignore=ignore, device=device)
        done += names
        skipped += [k.rpartition(".")[0] for k, t in new.items()
                    if k.endswith(".weight") and t.dim() == 2 and t.dtype != torch.float8_e4m3fn]
        save_file(new, str(dst / path.name))
    index_path = src / "model.safetensors.index.json"
    if index_path.is_file():
        index = json.loads(index_path.read_text(encoding="utf-8"))
        weight_map = dict(index.get("weight_map", {}))
        for module in done:
            shard = weight_map.get(f"{module}.weight")
            if shard is not None:
                weight_map[f"{module}.weight_scale"] = shard
        index["weight_map"] = dict(sorted(weight_map.items()))
        total = 0
        for path in sorted(dst.glob("*.safetensors")):
            with safe_open(str(path), framework="pt", device="cpu") as f:
                for k in f.keys():
                    sl = f.get_slice(k)
                    n = 1
                    for d in sl.get_shape():
                        n *= d
                    total += n * _DTYPE_BYTES.get(sl.get_dtype(), 0)
        index.setdefault("metadata", {})["total_size"] = total
        (dst / index_path.name).write_text(json.dumps(index, indent=2), encoding="utf-8")
    cfg_path = src / "config.json"
    cfg = json.loads(cfg_path.read_text(encoding="utf-8")) if cfg_path.is_file() else {}
    cfg["quantization_config"] = {"quant_method": "fp8", "activation_scheme": "dynamic",
                                  "ignored_layers": sorted(set(skipped))}
    (dst / "config.json").write_text(json.dumps(cfg, indent=2), encoding="utf-8")
    return done


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("src")
    ap.add_argument("dst")
    ap.add_argument("--only", nargs="*", default=[], help="globs over module names to quantize (default: all)")
    ap.add_argument("--ignore", nargs="*", default=[], help="module names (full or last component) to keep")
    args = ap.parse_args(argv)
    done = quantize_checkpoint(args.src, args.dst, only=args.only, ignore=args.ignore)
    print(f"quantized {len(done)} weight matrices into {args.dst}")
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
