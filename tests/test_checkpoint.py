"""Quant-config importers, the checkpoint loader for fused fp8 layers, and the offline quantizer."""

import json

import pytest
import torch
from torch import nn

from oracle import ref
from tests.conftest import seeded


# ---- importers (reference phyai/layers/quant/importers/*.py) -------------------------------------

def test_fp8_importer_flat_config():
    from phyai_amd.quant import Fp8Spec, Granularity
    from phyai_amd.quant.importers import ConfigSources, Fp8Importer, build_quant_plan, select_importer

    src = ConfigSources(hf_quant_config={"quant_method": "fp8", "activation_scheme": "dynamic",
                                         "ignored_layers": ["lm_head", "model.layers.3.mlp.down_proj"]})
    assert isinstance(select_importer(src), Fp8Importer)
    plan = build_quant_plan(src)
    spec = plan.resolve("model.layers.0.self_attn.qkv_proj")
    assert isinstance(spec, Fp8Spec) and spec.granularity is Granularity.PER_CHANNEL
    assert plan.resolve("lm_head") is None                                  # last component
    assert plan.resolve("model.layers.3.mlp.down_proj") is None             # whole prefix
    assert plan.resolve("model.layers.2.mlp.down_proj") is not None
    assert plan.default.input.dynamic is True
    static = build_quant_plan(ConfigSources(hf_quant_config={"quant_method": "fp8", "activation_scheme": "static",
                                                             "modules_to_not_convert": ["head"]}))
    assert static.default.input.dynamic is False and static.resolve("x.head") is None
    block = build_quant_plan(ConfigSources(hf_quant_config={"quant_method": "fp8", "weight_block_size": [128, 128]}))
    bs = block.resolve("a.b")
    assert bs.granularity is Granularity.BLOCK and bs.block_shape == (128, 128) and bs.spec_id == "fp8_block_128_128"


def test_compressed_tensors_importer():
    from phyai_amd.linear.layers import ColumnParallelLinear
    from phyai_amd.quant import Fp8Spec, Granularity
    from phyai_amd.quant.importers import CompressedTensorsImporter, ConfigSources, build_quant_plan, select_importer

    cfg = {"quant_method": "compressed-tensors", "ignore": ["lm_head", "re:.*vision.*"],
           "config_groups": {"group_0": {
               "targets": ["Linear"],
               "weights": {"type": "float", "num_bits": 8, "strategy": "channel", "symmetric": True},
               "input_activations": {"type": "float", "num_bits": 8, "strategy": "token", "dynamic": True}}}}
    src = ConfigSources(hf_quant_config=cfg)
    assert isinstance(select_importer(src), CompressedTensorsImporter)
    plan = build_quant_plan(src)
    spec = plan.resolve("model.layers.0.mlp.gate_up_proj", ColumnParallelLinear)    # class name contains "Linear"
    assert isinstance(spec, Fp8Spec) and spec.granularity is Granularity.PER_CHANNEL
    assert plan.resolve("lm_head", ColumnParallelLinear) is None
    assert plan.resolve("model.vision_tower.proj", ColumnParallelLinear) is None    # regex ignore comes first
    assert plan.resolve("model.layers.0.mlp.gate_up_proj", nn.Embedding) is None    # no rule, default None
    tensor = build_quant_plan(ConfigSources(hf_quant_config={
        "quant_method": "compressed-tensors",
        "config_groups": {"g": {"targets": ["q_proj"], "weights": {"type": "float", "num_bits": 8, "strategy": "tensor"}}}}))
    assert tensor.resolve("layers.0.q_proj").granularity is Granularity.PER_TENSOR
    with pytest.raises(NotImplementedError):
        build_quant_plan(ConfigSources(hf_quant_config={
            "quant_method": "compressed-tensors",
            "config_groups": {"g": {"targets": ["Linear"], "weights": {"type": "float", "num_bits": 4}}}}))


def test_modelopt_importer_and_unsupported_formats():
    from phyai_amd.quant import Fp8Spec
    from phyai_amd.quant.importers import ConfigSources, ModelOptImporter, build_quant_plan, select_importer

    standalone = ConfigSources(standalone={"quantization": {"quant_algo": "FP8", "exclude_modules": ["lm_head"]}})
    assert isinstance(select_importer(standalone), ModelOptImporter)
    plan = build_quant_plan(standalone)
    assert isinstance(plan.resolve("model.layers.0.mlp.down_proj"), Fp8Spec) and plan.resolve("lm_head") is None
    inline = build_quant_plan(ConfigSources(hf_quant_config={"quant_method": "modelopt_fp8", "quant_algo": "FP8"}))
    assert isinstance(inline.resolve("a"), Fp8Spec)
    fp4 = build_quant_plan(ConfigSources(hf_quant_config={"quant_method": "modelopt_fp4", "quant_algo": "NVFP4"}))
    with pytest.raises(NotImplementedError, match="no kernels"):
        fp4.resolve("a")                                 # parsed like the reference, refused when lowered
    assert build_quant_plan(ConfigSources()) is None
    assert build_quant_plan(ConfigSources(hf_quant_config={"quant_method": "awq"})) is None
    # the flat fp8 importer is asked first
    both = ConfigSources(hf_quant_config={"quant_method": "fp8"}, standalone={"quantization": {"quant_algo": "FP8"}})
    assert select_importer(both).name == "fp8"


def test_load_quant_plan_reads_the_checkpoint_folder(tmp_path):
    from phyai_amd.quant.importers import load_quant_plan

    assert load_quant_plan(None) is None
    (tmp_path / "config.json").write_text(json.dumps({"hidden_size": 8}))
    assert load_quant_plan(tmp_path) is None
    (tmp_path / "config.json").write_text(json.dumps({"compression_config": {"quant_method": "fp8"}}))
    assert load_quant_plan(tmp_path).resolve("a.b") is not None
    (tmp_path / "config.json").write_text(json.dumps({}))
    (tmp_path / "hf_quant_config.json").write_text(json.dumps({"quantization": {"quant_algo": "FP8"}}))
    assert load_quant_plan(tmp_path).resolve("a.b") is not None
    with pytest.raises(FileNotFoundError):
        load_quant_plan(tmp_path / "nope")


# ---- loader ----------------------------------------------------------------------------------------

class _Block(nn.Module):
    """qkv + o + gated MLP with the checkpoint names of a Gemma decoder layer."""

    def __init__(self, device, H=64, heads=2, kv=1, hd=32, inter=128, bias=False):
        super().__init__()
        from phyai_amd.linear.layers import MergedColumnParallelLinear, QKVParallelLinear, RowParallelLinear

        p = "model.layers.0"
        kw = dict(params_dtype=torch.bfloat16, device=device, bias=bias)
        self.qkv_proj = QKVParallelLinear(H, hd, heads, kv, prefix=f"{p}.self_attn.qkv_proj", **kw)
        self.o_proj = RowParallelLinear(heads * hd, H, prefix=f"{p}.self_attn.o_proj", **kw)
        self.gate_up_proj = MergedColumnParallelLinear(H, [inter, inter], prefix=f"{p}.mlp.gate_up_proj", **kw)
        self.down_proj = RowParallelLinear(inter, H, prefix=f"{p}.mlp.down_proj", **kw)


def _bf16_checkpoint(H=64, heads=2, kv=1, hd=32, inter=128, bias=False):
    p = "model.layers.0"
    shapes = {f"{p}.self_attn.q_proj": (heads * hd, H), f"{p}.self_attn.k_proj": (kv * hd, H),
              f"{p}.self_attn.v_proj": (kv * hd, H), f"{p}.self_attn.o_proj": (H, heads * hd),
              f"{p}.mlp.gate_proj": (inter, H), f"{p}.mlp.up_proj": (inter, H), f"{p}.mlp.down_proj": (H, inter)}
    t = {}
    for i, (name, shape) in enumerate(shapes.items()):
        t[f"{name}.weight"] = seeded(shape, seed=100 + i, scale=0.05)
        if bias:
            t[f"{name}.bias"] = seeded((shape[0],), seed=200 + i, scale=0.01)
    return t


def _oracle_fp8_checkpoint(bf16):
    out = {}
    for key, w in bf16.items():
        if key.endswith(".weight"):
            q, s = ref.weight_quant(w)
            out[key] = q
            out[key.replace(".weight", ".weight_scale")] = s
        else:
            out[key] = w
    return out


def test_loader_assembles_fused_fp8_layers_on_cpu(tmp_path):
    from safetensors.torch import save_file

    from phyai_amd.quant_plan import QuantPlan, use_quant_plan
    from phyai_amd.weights import load_pretrained

    bf16 = _bf16_checkpoint(bias=True)
    ck = _oracle_fp8_checkpoint(bf16)
    save_file(ck, str(tmp_path / "model.safetensors"))
    with use_quant_plan(QuantPlan.fp8_per_channel()):
        block = _Block("cpu", bias=True)
    rep = load_pretrained(block, tmp_path)
    assert not rep.missing and not rep.unexpected and len(rep.loaded) == len(ck)
    p = "model.layers.0"
    for layer, legs in ((block.qkv_proj, ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj")),
                        (block.gate_up_proj, ("mlp.gate_proj", "mlp.up_proj")),
                        (block.o_proj, ("self_attn.o_proj",)), (block.down_proj, ("mlp.down_proj",))):
        want_w = torch.cat([ck[f"{p}.{leg}.weight"].view(torch.uint8) for leg in legs])
        assert torch.equal(layer.weight.data.view(torch.uint8), want_w)
        assert torch.equal(layer.weight_scale.data, torch.cat([ck[f"{p}.{leg}.weight_scale"] for leg in legs]))
        assert torch.equal(layer.bias.data, torch.cat([ck[f"{p}.{leg}.bias"] for leg in legs]))
    # a checkpoint without scales: optional, reported, scales stay at one
    save_file({k: v for k, v in ck.items() if not k.endswith("weight_scale")}, str(tmp_path / "model.safetensors"))
    with use_quant_plan(QuantPlan.fp8_per_channel()):
        block2 = _Block("cpu", bias=True)
    rep2 = load_pretrained(block2, tmp_path)
    assert len(rep2.optional_missing) == 7 and bool((block2.qkv_proj.weight_scale == 1).all())
    # strictness and remapping
    save_file({**ck, "model.layers.0.extra.weight": torch.zeros(2)}, str(tmp_path / "model.safetensors"))
    with pytest.raises(RuntimeError, match="strict failure"):
        load_pretrained(block2, tmp_path)
    assert load_pretrained(block2, tmp_path, strict=False).unexpected == ["model.layers.0.extra.weight"]
    save_file({k.replace("model.", "paligemma."): v for k, v in ck.items()}, str(tmp_path / "model.safetensors"))
    assert not load_pretrained(block2, tmp_path, remap={"paligemma.": "model."}).missing
    save_file({k: v for k, v in ck.items() if "k_proj.weight" != k.rpartition("self_attn.")[2]},
              str(tmp_path / "model.safetensors"))
    with pytest.raises(RuntimeError, match="k_proj.weight"):
        load_pretrained(block2, tmp_path)


def test_per_tensor_scales_of_fused_legs(tmp_path):
    """One scale per checkpoint module: they land in the [legs] parameter and fan out to rows after
    loading (reference quant/fp8.py:36-43,128-135)."""
    from safetensors.torch import save_file

    from phyai_amd.quant import Fp8Spec, Granularity
    from phyai_amd.linear.layers import QKVParallelLinear
    from phyai_amd.weights import load_pretrained

    layer = QKVParallelLinear(64, 32, 2, 1, bias=False, params_dtype=torch.bfloat16, device="cpu",
                              spec=Fp8Spec(granularity=Granularity.PER_TENSOR), prefix="l.self_attn.qkv_proj")
    ck = {}
    for i, (leg, rows) in enumerate((("q_proj", 64), ("k_proj", 32), ("v_proj", 32))):
        ck[f"l.self_attn.{leg}.weight"] = torch.full((rows, 64), i + 1, dtype=torch.uint8).view(torch.float8_e4m3fn)
        ck[f"l.self_attn.{leg}.weight_scale"] = torch.tensor(0.5 * (i + 1))
        ck[f"l.self_attn.{leg}.input_scale"] = torch.tensor(0.1 * (3 - i))
    save_file(ck, str(tmp_path / "m.safetensors"))
    load_pretrained(layer, tmp_path / "m.safetensors")
    assert layer.weight_scale.shape == (128,)
    assert torch.equal(layer.weight_scale.data, torch.tensor([0.5] * 64 + [1.0] * 32 + [1.5] * 32))
    assert float(layer.input_scale) == pytest.approx(0.3)


def test_fp8_codes_for_an_unquantized_parameter_are_refused(tmp_path):
    """A quantized tensor for a module that was not built as an fp8 linear must not be cast into it."""
    from safetensors.torch import save_file

    from phyai_amd.linear.layers import ReplicatedLinear
    from phyai_amd.weights import load_pretrained

    layer = ReplicatedLinear(32, 16, bias=False, params_dtype=torch.bfloat16, device="cpu", prefix="head")
    assert layer.weight.dtype == torch.bfloat16
    save_file({"head.weight": torch.zeros(16, 32, dtype=torch.uint8).view(torch.float8_e4m3fn)}, str(tmp_path / "m.safetensors"))
    with pytest.raises(ValueError, match="not built as an fp8 linear"):
        load_pretrained(layer, tmp_path / "m.safetensors", strict=False)


def test_offline_quantizer_selects_linears_only():
    from phyai_amd.quantize_checkpoint import _selected

    for name in ("model.embed_tokens", "lm_head", "model.norm", "model.layers.0.input_layernorm",
                 "vision_tower.embeddings.position_embedding", "transformer.wte"):
        assert not _selected(name, [], [])
    for name in ("model.layers.0.self_attn.q_proj", "model.layers.3.mlp.down_proj", "vision_tower.encoder.layers.0.mlp.fc1"):
        assert _selected(name, [], [])
    assert not _selected("model.layers.0.self_attn.q_proj", [], ["q_proj"])
    assert _selected("lm_head", ["lm_*"], [])                      # an explicit allow-list wins over the defaults
    assert not _selected("model.layers.0.mlp.down_proj", ["lm_*"], [])


# ---- offline quantizer + end to end (GPU) ------------------------------------------------------------

@pytest.mark.gpu
def test_quantize_checkpoint_then_load_and_run(dev, tmp_path):
    from safetensors import safe_open
    from safetensors.torch import save_file

    import phyai_amd.linear as L
    from phyai_amd.quant.importers import load_quant_plan
    from phyai_amd.quant_plan import use_quant_plan
    from phyai_amd.quantize_checkpoint import quantize_checkpoint
    from phyai_amd.weights import load_pretrained

    src, dst = tmp_path / "bf16", tmp_path / "fp8"
    src.mkdir()
    bf16 = _bf16_checkpoint()
    bf16["model.norm.weight"] = seeded((64,), seed=1)                      # not a matrix: copied through
    bf16["lm_head.weight"] = seeded((96, 64), seed=2, scale=0.05)          # a head and an embedding table are
    bf16["model.embed_tokens.weight"] = seeded((96, 64), seed=3, scale=0.05)   # never fp8 linears: kept by default
    save_file(bf16, str(src / "model.safetensors"))
    (src / "config.json").write_text(json.dumps({"hidden_size": 64}))
    (src / "model.safetensors.index.json").write_text(json.dumps(
        {"metadata": {"total_size": 0}, "weight_map": {k: "model.safetensors" for k in bf16}}))
    done = quantize_checkpoint(src, dst)
    assert len(done) == 7
    cfg = json.loads((dst / "config.json").read_text())
    assert cfg["hidden_size"] == 64 and cfg["quantization_config"]["quant_method"] == "fp8"
    assert cfg["quantization_config"]["ignored_layers"] == ["lm_head", "model.embed_tokens"]
    index = json.loads((dst / "model.safetensors.index.json").read_text())
    assert all(index["weight_map"].get(f"{m}.weight_scale") == "model.safetensors" for m in done)
    assert index["metadata"]["total_size"] == sum(
        (v.numel() * (1 if k.rpartition(".")[0] in done and k.endswith(".weight") else v.element_size())
         for k, v in bf16.items())) + sum(4 * bf16[f"{m}.weight"].shape[0] for m in done)
    want = _oracle_fp8_checkpoint({k: v for k, v in bf16.items() if k.startswith("model.layers")})
    with safe_open(str(dst / "model.safetensors"), framework="pt", device="cpu") as f:
        got = {k: f.get_tensor(k) for k in f.keys()}
    assert got["model.embed_tokens.weight"].dtype == torch.bfloat16
    assert got["lm_head.weight"].dtype == torch.bfloat16 and torch.equal(got["model.norm.weight"], bf16["model.norm.weight"])
    for k, v in want.items():                                             # the kernel's codes and scales are the oracle's
        assert torch.equal(got[k].view(torch.uint8) if v.dtype == torch.float8_e4m3fn else got[k],
                           v.view(torch.uint8) if v.dtype == torch.float8_e4m3fn else v), k

    torch.cuda.set_device(dev)
    L.init()
    try:
        plan = load_quant_plan(dst)
        with use_quant_plan(plan):
            block = _Block(dev)
        assert block.qkv_proj.spec.spec_id == "fp8_per_channel"
        rep = load_pretrained(block, dst, strict=False)
        assert sorted(rep.unexpected) == ["lm_head.weight", "model.embed_tokens.weight", "model.norm.weight"] and not rep.missing
        x = seeded((50, 64), seed=9).to(dev)
        y, _ = block.qkv_proj(x)
        p = "model.layers.0.self_attn"
        wq = torch.cat([want[f"{p}.{leg}.weight"].view(torch.uint8) for leg in ("q_proj", "k_proj", "v_proj")]).view(torch.float8_e4m3fn)
        ws = torch.cat([want[f"{p}.{leg}.weight_scale"] for leg in ("q_proj", "k_proj", "v_proj")])
        xq, xs = ref.quant_rowwise(x.cpu())
        from tests.test_gpu_parity import assert_close_to_ref
        assert_close_to_ref(y, ref.gemm_f32(xq, xs, wq, ws), "loaded qkv_proj")
        h, _ = block.gate_up_proj(x)
        assert h.shape == (50, 256)
    finally:
        L._reset_for_test()
