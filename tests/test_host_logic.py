"""Host-side mirror of the reference's plug-in surface, on the CPU.

Modelled on the reference's own tests for this layer
(phyai/tests/layers/linear/test_dispatch.py, test_registry.py, test_spec.py,
test_layers.py, tests/layers/mlp/test_dense_mlp.py): fake kernels drive the
registry and the dispatcher; bf16 layers run through F.linear; fp8 specs are
checked for what they allocate.  Nothing here touches the GPU.
"""

from __future__ import annotations

import pytest
import torch
import torch.nn as nn
import torch.nn.functional as F

import phyai_amd.linear as L
from phyai_amd.linear.backend import KernelProbe
from phyai_amd.linear.dispatch import KernelDispatcher, _M_bucket, get_linear_dispatcher
from phyai_amd.linear.registry import (DefaultPolicy, ForcedPolicy, LinearKernelRegistry, _regime_of,
                                       list_registered_linear_kernels)
from phyai_amd.mlp import DenseMLP, _canonicalise_activation
from phyai_amd.quant import ActivationView, AllocationRequest, Bf16Spec, Fp8Spec, Granularity, LinearActivationQuant
from phyai_amd.quant_plan import QuantPlan, use_quant_plan
from phyai_amd.runtime import CudaGraph, HipGraph, HipGraphError, HipGraphRegistry
from phyai_amd.state import Mode, NoBackendError, current_mode, graph_capture


class FakeKernel:
    def __init__(self, name, *, specs, modes=(Mode.EAGER, Mode.GRAPH_CAPTURING), capture=True, min_sm=0):
        self.name, self._specs, self._modes, self._capture, self._min_sm = name, set(specs), set(modes), capture, min_sm

    def supports_capture(self):
        return self._capture

    def can_handle(self, probe):
        return probe.spec_id in self._specs and probe.mode in self._modes and probe.sm >= self._min_sm

    def apply(self, layer, x, bias):
        return torch.empty_like(x)


def probe(spec_id="bf16", M_bucket=1, N=512, K=512, mode=Mode.EAGER, sm=95):
    return KernelProbe(spec_id=spec_id, M_bucket=M_bucket, N=N, K=K, in_dtype=torch.bfloat16,
                       out_dtype=torch.bfloat16, sm=sm, mode=mode)


def reg_with(*kernels):
    r = LinearKernelRegistry()
    for k in kernels:
        r.register(k)
    return r


SEL = dict(N=512, K=512, in_dtype=torch.bfloat16, out_dtype=torch.bfloat16)


@pytest.fixture(autouse=True)
def _fresh_dispatcher(monkeypatch):
    monkeypatch.delenv("PHYAI_FORCE_LINEAR_KERNEL", raising=False)
    yield
    L._reset_for_test()


# ---- dispatcher / registry -----------------------------------------------------------

def test_M_bucket_and_regime():
    assert [_M_bucket(m) for m in (0, 1, 4, 7, 8, 50, 816, 1024)] == [0, 1, 3, 3, 4, 6, 10, 11]
    assert _regime_of(3) == "decode" and _regime_of(4) == "prefill"
    assert _regime_of(_M_bucket(50)) == "prefill" and _regime_of(_M_bucket(816)) == "prefill"


def test_dispatcher_first_candidate_cache_and_key():
    a, b = FakeKernel("a", specs={"bf16"}), FakeKernel("b", specs={"bf16"})
    r = reg_with(a, b)
    calls = []
    orig = r.candidates
    r.candidates = lambda p: (calls.append(p), orig(p))[1]
    d = KernelDispatcher(r)
    for _ in range(5):
        assert d.select(spec_id="bf16", M=8, **SEL).name == "a"
    assert len(calls) == 1
    d.select(spec_id="bf16", M=9, **SEL)            # same bucket (bit_length 4)
    assert len(calls) == 1
    d.select(spec_id="bf16", M=16, **SEL)           # next bucket
    d.select(spec_id="bf16", M=8, N=1024, K=512, in_dtype=torch.bfloat16, out_dtype=torch.bfloat16)
    d.select(spec_id="bf16", M=8, N=512, K=512, in_dtype=torch.float16, out_dtype=torch.bfloat16)
    assert len(calls) == 4
    d.clear_cache()
    assert not d._cache


def test_dispatcher_regimes_and_preference_order():
    dec, pre, other = (FakeKernel(n, specs={"bf16"}) for n in ("decode", "prefill", "other"))
    r = LinearKernelRegistry()
    r.register(other)
    r.register(dec, prefer_for={("bf16", "decode")})
    r.register(pre, prefer_for={("bf16", "prefill")})
    d = KernelDispatcher(r)
    assert d.select(spec_id="bf16", M=1, **SEL).name == "decode"
    assert d.select(spec_id="bf16", M=50, **SEL).name == "prefill"
    assert [k.name for k in r.candidates(probe(M_bucket=1))] == ["decode", "other", "prefill"]


def test_capture_mode_filters_and_is_part_of_the_key():
    eager_only = FakeKernel("eager_only", specs={"bf16"}, capture=False)
    safe = FakeKernel("safe", specs={"bf16"})
    d = KernelDispatcher(reg_with(eager_only, safe))
    assert d.select(spec_id="bf16", M=8, **SEL).name == "eager_only"
    assert current_mode() is Mode.EAGER
    with graph_capture():
        assert current_mode() is Mode.GRAPH_CAPTURING
        assert d.select(spec_id="bf16", M=8, **SEL).name == "safe"
    assert current_mode() is Mode.EAGER
    assert d.select(spec_id="bf16", M=8, **SEL).name == "eager_only"


def test_no_backend_and_uninitialised_errors():
    d = KernelDispatcher(reg_with(FakeKernel("a", specs={"bf16"})))
    with pytest.raises(NoBackendError, match="fp8_per_channel"):
        d.select(spec_id="fp8_per_channel", M=8, **SEL)
    L._reset_for_test()
    with pytest.raises(RuntimeError, match="init.*not called"):
        get_linear_dispatcher()
    with pytest.raises(NoBackendError):
        DefaultPolicy().select([])


def test_force_env_and_forced_policy(monkeypatch):
    a, b = FakeKernel("a", specs={"bf16"}), FakeKernel("b", specs={"bf16"})
    monkeypatch.setenv("PHYAI_FORCE_LINEAR_KERNEL", "b")
    assert KernelDispatcher(reg_with(a, b)).select(spec_id="bf16", M=8, **SEL).name == "b"
    monkeypatch.delenv("PHYAI_FORCE_LINEAR_KERNEL")
    assert KernelDispatcher(reg_with(a, b), force="b").select(spec_id="bf16", M=8, **SEL).name == "b"
    assert ForcedPolicy("zzz").select([a, b]) is a                     # absent name falls back


def test_validate_checks_preferences_and_coverage():
    r = LinearKernelRegistry()
    r.register(FakeKernel("a", specs={"bf16"}), prefer_for={("bf16", "decode")})
    r.validate(sample_specs=["bf16"], sm=95)
    with pytest.raises(NoBackendError, match="fp8_per_channel"):
        r.validate(sample_specs=["fp8_per_channel"], sm=95)
    r._prefer[("bf16", "prefill")] = ["ghost"]
    with pytest.raises(NoBackendError, match="ghost"):
        r.validate(sample_specs=["bf16"], sm=95)
    # a capture-capable kernel makes capture coverage mandatory
    r2 = reg_with(FakeKernel("cap", specs={"x"}), FakeKernel("eager", specs={"bf16"}, modes={Mode.EAGER}))
    with pytest.raises(NoBackendError, match="graph_capturing"):
        r2.validate(sample_specs=["bf16"], sm=95)


def test_registered_kernels_and_hip_kernel_capabilities():
    names = [cls.name for cls, _ in list_registered_linear_kernels()]
    assert names[:2] == ["hip_fp8", "torch"]
    k = L.HipFp8Kernel()
    assert k.supports_capture() is True
    assert k.can_handle(probe("fp8_per_channel", M_bucket=6, N=2560, K=1024))
    assert k.can_handle(probe("fp8_per_tensor", M_bucket=10, N=2048, K=2048, mode=Mode.GRAPH_CAPTURING))
    assert not k.can_handle(probe("fp8_per_channel", sm=80))           # same sm >= 89 gate as the reference
    assert not k.can_handle(probe("fp8_per_channel", sm=0))            # no GPU: no fp8 path at all
    assert not k.can_handle(probe("fp8_per_channel", N=16, K=15))
    assert k.can_handle(probe("fp8_per_channel", N=16, K=16))
    assert not k.can_handle(probe("bf16")) and not k.can_handle(probe("fp8_block_128_128"))
    t = L.TorchBf16Kernel()
    assert t.can_handle(probe("bf16", sm=0)) and not t.can_handle(probe("fp8_per_channel"))
    assert L.supported_specs_for_sm(0) == ["bf16"]
    assert L.supported_specs_for_sm(95) == ["bf16", "fp8_per_tensor", "fp8_per_channel"]


def test_init_prefers_hip_kernel_for_fp8(monkeypatch):
    d = L.init(validate=False)
    monkeypatch.setattr(d, "_sm", 95)
    for M in (1, 50, 816):
        assert d.select(spec_id="fp8_per_channel", M=M, N=2560, K=1024, in_dtype=torch.bfloat16,
                        out_dtype=torch.bfloat16).name == "hip_fp8"
    assert d.select(spec_id="bf16", M=4, **SEL).name == "torch"
    L.init()                                                            # validate passes on a CPU-only host


@pytest.mark.skipif(torch.cuda.is_available(), reason="describes a machine without a GPU")
def test_fp8_on_unsupported_device_raises_lazily():
    L.init()                                                            # sm == 0 here
    layer = L.ReplicatedLinear(32, 16, bias=False, params_dtype=torch.bfloat16,
                               spec=Fp8Spec(), device="cpu")
    with pytest.raises(NoBackendError, match="fp8_per_channel"):
        layer(torch.zeros(2, 32, dtype=torch.bfloat16))


# ---- specs -----------------------------------------------------------------------------

def _alloc(spec, N=8, K=32, widths=None):
    layer = nn.Module()
    layer.spec = spec
    spec.allocate(layer, AllocationRequest(weight_shape=(N, K), logical_widths=widths or [N], device="cpu"))
    return layer


def test_fp8_spec_allocation_per_granularity():
    pc = _alloc(Fp8Spec(granularity=Granularity.PER_CHANNEL))
    assert pc.weight.shape == (8, 32) and pc.weight.dtype == torch.float8_e4m3fn
    assert pc.weight_scale.shape == (8,) and pc.weight_scale.dtype == torch.float32
    assert torch.equal(pc.weight_scale, torch.ones(8)) and not hasattr(pc, "input_scale")
    assert not pc.weight.requires_grad and pc.logical_widths == [8]
    pt = _alloc(Fp8Spec(granularity=Granularity.PER_TENSOR), widths=[3, 5])
    assert pt.weight_scale.shape == (2,) and pt.input_scale.shape == (1,)
    pt.weight_scale.data = torch.tensor([2.0, 3.0])
    pt.spec.process_after_loading(pt)
    assert torch.equal(pt.weight_scale, torch.tensor([2.0] * 3 + [3.0] * 5))
    blk = _alloc(Fp8Spec(granularity=Granularity.BLOCK, block_shape=(4, 16)))
    assert blk.weight_scale.shape == (2, 2)
    with pytest.raises(ValueError):
        Fp8Spec(granularity=Granularity.BLOCK)
    with pytest.raises(ValueError, match="block_n"):
        _alloc(Fp8Spec(granularity=Granularity.BLOCK, block_shape=(3, 16)))
    with pytest.raises(ValueError, match="2-D"):
        Fp8Spec().allocate(nn.Module(), AllocationRequest(weight_shape=(8,), logical_widths=[8]))


def test_spec_ids_and_protocols():
    assert Fp8Spec().spec_id == "fp8_per_channel"
    assert Fp8Spec(granularity=Granularity.PER_TENSOR).spec_id == "fp8_per_tensor"
    assert Fp8Spec(granularity=Granularity.BLOCK, block_shape=(128, 128)).spec_id == "fp8_block_128_128"
    assert Bf16Spec().spec_id == "bf16"
    assert isinstance(Fp8Spec(), LinearActivationQuant) and Fp8Spec().needs_act_quant
    assert ActivationView._fields == ("x", "x_scale", "granularity")
    assert [g.value for g in Granularity] == ["per_tensor", "per_channel", "block"]


def test_quantize_activation_needs_the_gpu_library_path():
    """There is no CPU quantizer in the package: a CPU tensor is rejected, not silently handled."""
    with pytest.raises(RuntimeError, match="must live on the GPU"):
        Fp8Spec().quantize_activation(torch.zeros(2, 16, dtype=torch.bfloat16), nn.Module())


# ---- layers ------------------------------------------------------------------------------

def test_bf16_layers_match_F_linear_and_return_convention():
    L.init()
    torch.manual_seed(0)
    lin = L.ReplicatedLinear(32, 16, params_dtype=torch.bfloat16, device="cpu")
    nn.init.normal_(lin.weight, std=0.02)
    nn.init.normal_(lin.bias, std=0.02)
    x = torch.randn(2, 3, 32).bfloat16()
    y, b = lin(x)
    assert b is None and y.shape == (2, 3, 16)
    assert torch.equal(y, F.linear(x, lin.weight, lin.bias))
    skip = L.RowParallelLinear(32, 16, skip_bias_add=True, params_dtype=torch.bfloat16, device="cpu")
    nn.init.normal_(skip.weight, std=0.02)
    nn.init.ones_(skip.bias)
    y, b = skip(x)
    assert b is skip.bias and torch.equal(y, F.linear(x, skip.weight))


def test_fused_layer_shapes_and_checkpoint_keys():
    L.init()
    qkv = L.QKVParallelLinear(1024, 256, 8, 1, bias=False, params_dtype=torch.bfloat16, spec=Fp8Spec(),
                              device="cpu", prefix="model.layers.0.self_attn.qkv_proj")
    assert qkv.weight.shape == (2560, 1024) and qkv.output_partition_sizes == [2048, 256, 256]
    assert qkv.logical_widths == [2048, 256, 256] and qkv.bias is None and qkv.tp_size == 1
    assert qkv.weight.hf_keys == [("model.layers.0.self_attn.q_proj.weight", "q"),
                                  ("model.layers.0.self_attn.k_proj.weight", "k"),
                                  ("model.layers.0.self_attn.v_proj.weight", "v")]
    assert qkv.weight_scale.optional is True
    gu = L.MergedColumnParallelLinear(1024, [4096, 4096], bias=False, params_dtype=torch.bfloat16,
                                      spec=Fp8Spec(), device="cpu", prefix="m.mlp.gate_up_proj")
    assert gu.weight.shape == (8192, 1024)
    assert gu.weight.hf_keys == [("m.mlp.gate_proj.weight", 0), ("m.mlp.up_proj.weight", 1)]
    with pytest.raises(ValueError, match="output_sizes sum"):
        L.ColumnParallelLinear(8, 10, output_sizes=[4, 4], device="cpu")
    with pytest.raises(ValueError, match="hf_legs"):
        L.MergedColumnParallelLinear(8, [4, 4], hf_legs=("a",), device="cpu")
    with pytest.raises(ValueError, match="missing key"):
        L.QKVParallelLinear(8, 4, 2, hf_legs={"q": "q", "k": "k"}, device="cpu")


def test_quant_plan_resolution():
    L.init()
    plan = QuantPlan.fp8_per_channel(ignore=["*.lm_head"])
    with use_quant_plan(plan):
        a = L.ReplicatedLinear(32, 16, params_dtype=torch.bfloat16, device="cpu", prefix="m.layers.0.o_proj")
        b = L.ReplicatedLinear(32, 16, params_dtype=torch.bfloat16, device="cpu", prefix="m.lm_head")
        c = L.ReplicatedLinear(32, 16, params_dtype=torch.bfloat16, device="cpu")          # no prefix
        d = L.ReplicatedLinear(32, 16, params_dtype=torch.bfloat16, device="cpu", prefix="m.x", spec=Bf16Spec())
    assert a.spec.spec_id == "fp8_per_channel" and b.spec.spec_id == "bf16"
    assert c.spec.spec_id == "bf16" and d.spec.spec_id == "bf16"
    e = L.ReplicatedLinear(32, 16, params_dtype=torch.bfloat16, device="cpu", prefix="m.layers.0.o_proj")
    assert e.spec.spec_id == "bf16"                                                        # plan no longer active


# ---- DenseMLP ------------------------------------------------------------------------------

def test_dense_mlp_bf16_paths_match_torch():
    L.init()
    torch.manual_seed(1)
    x = torch.randn(5, 32).bfloat16()
    if torch.cuda.is_available():          # layers are created on the default device
        x = x.cuda()
    for act, ref_act in (("gelu_tanh", lambda t: F.gelu(t, approximate="tanh")), ("silu", F.silu), ("gelu", F.gelu)):
        mlp = DenseMLP(32, 64, activation=act, params_dtype=torch.bfloat16)
        for p in mlp.parameters():
            nn.init.normal_(p, std=0.05)
        fused, _ = mlp.gate_up_proj(x)
        want, _ = mlp.down_proj((ref_act(fused[..., :64].float()) * fused[..., 64:].float()).bfloat16())
        assert torch.equal(mlp(x), want)
    plain = DenseMLP(32, 64, activation="gelu", gated=False, bias=True, params_dtype=torch.bfloat16)
    for p in plain.parameters():
        nn.init.normal_(p, std=0.05)
    want, _ = plain.fc2(F.gelu(plain.fc1(x)[0]))
    assert torch.equal(plain(x), want)


def test_dense_mlp_activation_names():
    assert _canonicalise_activation("gelu_pytorch_tanh") == "gelu_tanh"
    assert _canonicalise_activation("GELU-new") == "gelu_tanh"
    L.init()
    with pytest.raises(ValueError, match="non-gated SiLU"):
        DenseMLP(8, 16, activation="silu", gated=False)
    with pytest.raises(ValueError, match="Unsupported gated activation"):
        DenseMLP(8, 16, activation="relu")
    m = DenseMLP(1024, 4096, activation="gelu_tanh", spec_in=Fp8Spec(), spec_out=Fp8Spec(),
                 params_dtype=torch.bfloat16, prefix="m.mlp")
    assert m.gate_up_proj.weight.shape == (8192, 1024) and m.down_proj.weight.shape == (1024, 4096)
    assert m._epilogue == "geglu_tanh"


# ---- graph wrapper ----------------------------------------------------------------------------

def test_graph_wrapper_error_paths_without_gpu():
    assert CudaGraph is HipGraph
    g = HipGraph()
    assert not g.is_captured
    with pytest.raises(HipGraphError, match="not been captured"):
        g.replay()
    with pytest.raises(HipGraphError, match="not been captured"):
        g.input_buffer("x")
    with pytest.raises(ValueError):
        HipGraph(num_warmup_iters=-1)
    if not torch.cuda.is_available():
        with pytest.raises(HipGraphError, match="requires a GPU"):
            g.capture(lambda: None, {})
    reg = HipGraphRegistry()
    with pytest.raises(HipGraphError, match="not been captured"):
        reg.register("k", g)
    with pytest.raises(HipGraphError, match="unknown key"):
        reg["k"]
    with pytest.raises(HipGraphError, match="unknown key"):
        reg.deregister("k")
    assert len(reg) == 0 and "k" not in reg and reg.get("k") is None


def test_ops_reject_bad_arguments_before_touching_the_gpu():
    from phyai_amd import ops

    x = torch.zeros(2, 16, dtype=torch.bfloat16)
    with pytest.raises(RuntimeError, match=r"phyai_amd\.ops\.fp8_quant_rowwise: x must live on the GPU"):
        ops.fp8_quant_rowwise(x)
    with pytest.raises(RuntimeError, match="must be a Tensor"):
        ops.fp8_linear([1, 2], None, None)
    with pytest.raises(RuntimeError, match="unknown epilogue"):
        ops.fp8_linear(x, None, None, epilogue="relu")
    assert ops.workspace_bytes(50, 2560, 1024) >= 16384 + 50 * 1024


def test_cache_plan_streams_the_largest_matrices_until_the_rest_fits():
    """phyai_amd.cache_plan: the action expert's 72 matrices (311 MB against a 256 MB cache): only
    gate_up matrices are streamed, as few as leave the rest within the resident share; a model
    that fits streams nothing; the module form marks the layers."""
    from phyai_amd.cache_plan import choose_streamed, plan_weight_streaming

    per_layer = [2560 * 1024, 1024 * 2048, 8192 * 1024, 1024 * 4096]
    sizes = per_layer * 18
    flags = choose_streamed(sizes)
    assert all(not f for s, f in zip(sizes, flags) if s != 8192 * 1024)        # only the largest kind
    resident = sum(s for s, f in zip(sizes, flags) if not f)
    assert resident <= 0.7 * (256 << 20) < resident + 8192 * 1024               # no more than needed
    assert sum(flags) == 15
    assert choose_streamed([10 << 20] * 10) == [False] * 10                     # 100 MB: fits
    assert choose_streamed([]) == []
    assert choose_streamed([300 << 20]) == [True]                               # one matrix larger than the cache

    class Lin(torch.nn.Module):
        def __init__(self, n, k):
            super().__init__()
            self.weight = torch.nn.Parameter(torch.empty(n, k, dtype=torch.uint8), requires_grad=False)

    mods = [Lin(n, k) for n, k in [(2560, 1024), (1024, 2048), (8192, 1024), (1024, 4096)] * 18] + [torch.nn.ReLU()]
    left = plan_weight_streaming(mods)
    assert left == resident
    assert [m.stream_weights for m in mods[:4]] == [False, False, True, False]
    assert not hasattr(mods[-1], "stream_weights")

