"""GPU tests of the host mirror: layers + dispatcher + HIP kernel, DenseMLP with the
activation fused into the GEMM epilogue, graph capture/replay, committed fixtures."""

from __future__ import annotations

import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import seeded
from oracle import ref
from test_gpu_parity import assert_close_to_ref

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp8_linear_golden.npz")


@pytest.fixture()
def L(dev):
    import phyai_amd.linear as L

    torch.cuda.set_device(dev)
    L.init()
    yield L
    L._reset_for_test()


def _load_fp8(layer, w_bf16):
    layer.spec.quantize_weight_(layer, w_bf16)
    return ref.weight_quant(w_bf16.cpu())


def test_sm_arch_reports_fp8_capable_device():
    from phyai_amd.utils import gcn_arch, sm_arch

    assert gcn_arch() == "gfx950"
    assert sm_arch() >= 89


def test_golden_fixture_on_device(dev):
    from phyai_amd import ops

    g = np.load(GOLDEN)

    def t16(a):
        return torch.from_numpy(a.copy()).view(torch.bfloat16).to(dev)

    for name in ("cfg1", "tiny", "edge"):
        q, s = ops.fp8_quant_rowwise(t16(g[f"{name}_x"]))
        np.testing.assert_array_equal(q.cpu().view(torch.uint8).numpy(), g[f"{name}_codes"])
        np.testing.assert_array_equal(s.cpu().numpy().reshape(-1).view(np.uint32), g[f"{name}_scale"].view(np.uint32))
    q = ops.fp8_quant_static(t16(g["static_x"]), torch.from_numpy(g["static_scale"]).to(dev))
    np.testing.assert_array_equal(q.cpu().view(torch.uint8).numpy(), g["static_codes"])
    for name in ("cfg1", "tiny"):
        wq, ws = ops.fp8_weight_quant(t16(g[f"{name}_w"]))
        np.testing.assert_array_equal(wq.cpu().view(torch.uint8).numpy(), g[f"{name}_wq"])
        np.testing.assert_array_equal(ws.cpu().numpy(), g[f"{name}_ws"])
        y = ops.fp8_linear(t16(g[f"{name}_x"]), wq, ws, t16(g[f"{name}_bias"]))
        assert_close_to_ref(y, torch.from_numpy(g[f"{name}_out_f32"]), f"golden {name}")
    epi_names = [None, "geglu_tanh", "geglu_erf", "swiglu", "gelu_tanh", "gelu"]
    wq = torch.from_numpy(g["tiny_wq"].copy()).view(torch.float8_e4m3fn).to(dev)
    ws = torch.from_numpy(g["tiny_ws"]).to(dev)
    for epi, nm in enumerate(epi_names):
        y = ops.fp8_linear(t16(g["tiny_x"]), wq, ws, t16(g["tiny_bias"]), epilogue=nm)
        want = torch.from_numpy(g[f"tiny_out_epi{epi}"].copy()).view(torch.bfloat16).float()
        assert_close_to_ref(y, want, f"golden tiny epi{epi}")


def test_layers_run_the_hip_kernel(L, dev):
    from phyai_amd.quant import Fp8Spec

    x = seeded((2, 25, 1024), 1).to(dev)
    qkv = L.QKVParallelLinear(1024, 256, 8, 1, bias=False, params_dtype=torch.bfloat16, spec=Fp8Spec())
    w = seeded((2560, 1024), 2, 0.02)
    wq, ws = _load_fp8(qkv, w.to(dev))
    assert torch.equal(qkv.weight.cpu().view(torch.uint8), wq.view(torch.uint8))
    y, b = qkv(x)
    assert b is None and y.shape == (2, 25, 2560) and y.dtype == torch.bfloat16
    xq, xs = ref.quant_rowwise(x.cpu())
    assert_close_to_ref(y, ref.gemm_f32(xq, xs, wq, ws), "qkv layer")
    d = L.get_linear_dispatcher()
    assert d.select(spec_id="fp8_per_channel", M=50, N=2560, K=1024, in_dtype=torch.bfloat16,
                    out_dtype=torch.bfloat16).name == "hip_fp8"

    row = L.RowParallelLinear(1024, 512, bias=True, skip_bias_add=True, params_dtype=torch.bfloat16, spec=Fp8Spec())
    w2 = seeded((512, 1024), 3, 0.02)
    wq2, ws2 = _load_fp8(row, w2.to(dev))
    row.bias.data = seeded((512,), 4, 0.5).to(dev)
    y2, b2 = row(x)
    assert b2 is row.bias
    assert_close_to_ref(y2, ref.gemm_f32(xq, xs, wq2, ws2), "skip_bias_add leaves the bias out")


def test_cache_plan_marks_layers_and_the_marked_layers_give_the_same_bits(L, dev):
    """plan_weight_streaming on a small stack of fp8 layers (cache size scaled down so that it has
    to choose): the largest layer is marked, HipFp8Kernel passes the hint on, outputs are equal."""
    from phyai_amd.cache_plan import plan_weight_streaming
    from phyai_amd.quant import Fp8Spec

    small = L.ReplicatedLinear(1024, 512, bias=False, params_dtype=torch.bfloat16, spec=Fp8Spec())
    large = L.MergedColumnParallelLinear(1024, [2048, 2048], bias=False, params_dtype=torch.bfloat16, spec=Fp8Spec())
    _load_fp8(small, seeded((512, 1024), 11, 0.02).to(dev))
    _load_fp8(large, seeded((4096, 1024), 12, 0.02).to(dev))
    x = seeded((50, 1024), 13).to(dev)
    before = [small(x)[0].clone(), large(x)[0].clone()]
    left = plan_weight_streaming([small, large], cache_bytes=2 << 20, resident_fraction=0.5)
    assert (small.stream_weights, large.stream_weights) == (False, True) and left == 512 * 1024
    after = [small(x)[0], large(x)[0]]
    torch.cuda.synchronize()
    for a, b in zip(before, after):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16))


def test_per_tensor_layer(L, dev):
    from phyai_amd.quant import Fp8Spec, Granularity

    lin = L.MergedColumnParallelLinear(256, [64, 64], bias=True, params_dtype=torch.bfloat16,
                                       spec=Fp8Spec(granularity=Granularity.PER_TENSOR))
    w = seeded((128, 256), 5, 0.1)
    lin.weight.data = w.to(torch.float8_e4m3fn).to(dev)
    lin.weight_scale.data = torch.tensor([0.5, 2.0], device=dev)
    lin.input_scale.data = torch.tensor([0.02], device=dev)
    lin.bias.data = seeded((128,), 6, 0.1).to(dev)
    lin.post_load()
    assert lin.weight_scale.shape == (128,)
    x = seeded((40, 256), 7)
    y, _ = lin(x.to(dev))
    xq = ref.quant_static(x, torch.tensor([0.02]))
    want = ref.gemm_f32(xq, torch.full((40, 1), 0.02), w.to(torch.float8_e4m3fn),
                        torch.cat([torch.full((64,), 0.5), torch.full((64,), 2.0)]), lin.bias.cpu())
    assert_close_to_ref(y, want, "per-tensor layer")


@pytest.mark.parametrize("M", [50, 816])
@pytest.mark.parametrize("act,epi", [("gelu_tanh", 1), ("silu", 3), ("gelu", 2)])
def test_dense_mlp_fused_matches_unfused_and_oracle(L, dev, M, act, epi):
    from phyai_amd.mlp import DenseMLP
    from phyai_amd.quant import Fp8Spec

    H, I = 256, 512
    mlp = DenseMLP(H, I, activation=act, params_dtype=torch.bfloat16, spec_in=Fp8Spec(), spec_out=Fp8Spec())
    wgu, wd = seeded((2 * I, H), 8, 0.05), seeded((H, I), 9, 0.05)
    gq, gs = _load_fp8(mlp.gate_up_proj, wgu.to(dev))
    dq, ds = _load_fp8(mlp.down_proj, wd.to(dev))
    x = seeded((M, H), 10)
    y_fused = mlp(x.to(dev))
    mlp.fuse_activation = False
    y_unfused = mlp(x.to(dev))
    # Stage by stage against the oracle, each stage on the inputs the device actually saw (the
    # stated tolerance is per linear; one bf16 ulp in h can flip an fp8 code of the next stage).
    h_dev = mlp.gate_up_proj.forward_fused(x.to(dev), mlp._epilogue)
    assert_close_to_ref(h_dev, ref.linear(x, gq, gs, None, epi).float(), "gate_up + activation")
    want = ref.gemm_f32(*ref.quant_rowwise(h_dev.cpu()), dq, ds)
    assert_close_to_ref(y_fused, want, "down on the fused activation")
    h_un, _ = mlp.gate_up_proj(x.to(dev))
    h_un = mlp._unfused_act(h_un)
    assert_close_to_ref(y_unfused, ref.gemm_f32(*ref.quant_rowwise(h_un.cpu()), dq, ds), "down, unfused")
    # end to end the two forms agree closely (the fused epilogue keeps the bf16 rounding of
    # gate and up that the two-launch form has)
    rel = (y_fused.float() - y_unfused.float()).norm() / y_unfused.float().norm()
    assert rel < 2e-2
    same = (h_dev == h_un).float().mean().item()
    assert same > 0.98, f"fused and unfused activations agree on only {same:.3f} of elements"


def test_plain_mlp_fused_gelu(L, dev):
    from phyai_amd.mlp import DenseMLP
    from phyai_amd.quant import Fp8Spec

    mlp = DenseMLP(256, 512, activation="gelu", gated=False, bias=True, params_dtype=torch.bfloat16,
                   spec_in=Fp8Spec(), spec_out=Fp8Spec())
    w1, w2 = seeded((512, 256), 11, 0.05), seeded((256, 512), 12, 0.05)
    q1, s1 = _load_fp8(mlp.fc1, w1.to(dev))
    q2, s2 = _load_fp8(mlp.fc2, w2.to(dev))
    mlp.fc1.bias.data = seeded((512,), 13, 0.1).to(dev)
    mlp.fc2.bias.data = seeded((256,), 14, 0.1).to(dev)
    x = seeded((70, 256), 15)
    y = mlp(x.to(dev))
    h_dev = mlp.fc1.forward_fused(x.to(dev), mlp._epilogue)
    assert_close_to_ref(h_dev, ref.linear(x, q1, s1, mlp.fc1.bias.cpu(), 5).float(), "fc1 + gelu")
    want = ref.gemm_f32(*ref.quant_rowwise(h_dev.cpu()), q2, s2, mlp.fc2.bias.cpu())
    assert_close_to_ref(y, want, "plain mlp")


def test_graph_replay_equals_eager_bit_for_bit(L, dev):
    """The per-step linear sequence recorded in one hipGraph: several replays with new inputs,
    eager work and synchronisation in between, every replay equal to the eager result."""
    from phyai_amd.mlp import DenseMLP
    from phyai_amd.quant import Fp8Spec
    from phyai_amd.runtime import HipGraph, HipGraphError

    H, I = 1024, 4096
    qkv = L.QKVParallelLinear(H, 256, 8, 1, bias=False, params_dtype=torch.bfloat16, spec=Fp8Spec())
    o = L.RowParallelLinear(2048, H, bias=False, params_dtype=torch.bfloat16, spec=Fp8Spec())
    mlp = DenseMLP(H, I, activation="gelu_tanh", params_dtype=torch.bfloat16, spec_in=Fp8Spec(), spec_out=Fp8Spec())
    for i, lay in enumerate((qkv, o, mlp.gate_up_proj, mlp.down_proj)):
        lay.spec.quantize_weight_(lay, seeded(tuple(lay.weight.shape), 20 + i, 0.02).to(dev))

    def step(x):
        for _ in range(3):                                   # a few "denoise steps"
            q, _ = qkv(x)
            a, _ = o(q[..., :2048].contiguous())
            x = x + mlp(a)
        return x

    x0 = seeded((50, H), 30).to(dev)
    g = HipGraph()
    g.capture(step, {"x": x0})
    assert g.is_captured and g.input_buffer("x").shape == (50, H)
    for seed in (31, 32, 33, 34):
        xi = seeded((50, H), seed).to(dev)
        out = g.replay({"x": xi}).clone()
        torch.cuda.synchronize()
        eager = step(xi)
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay with seed {seed} differs from eager"
    with pytest.raises(HipGraphError, match="shape"):
        g.replay({"x": torch.zeros(3, H, dtype=torch.bfloat16, device=dev)})
    with pytest.raises(HipGraphError, match="unknown input"):
        g.replay({"y": x0})
    with pytest.raises(HipGraphError, match="already captured"):
        g.capture(step, {"x": x0})


def test_capture_without_warmup_on_a_fresh_stream(L, dev):
    """Direct torch.cuda.graph use on a stream that never ran the op: the workspace is created
    inside the capture (zero fill recorded as a kernel) and replays stay correct."""
    from phyai_amd import ops

    x = seeded((130, 512), 40).to(dev)
    w = seeded((256, 512), 41, 0.02)
    wq, ws = ops.fp8_weight_quant(w.to(dev))
    eager = ops.fp8_linear(x, wq, ws)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = ops.fp8_linear(x, wq, ws)
    for _ in range(3):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)


def test_graph_replays_of_the_split_k_tile_kernel(L, dev):
    """The prefill down projection (816 x 2048 x 16384) runs the pipelined tile kernel with K split
    in two; its arrival counters must be back at zero after every replay, so replays - with eager
    calls of the same op in between - all equal the eager result."""
    from phyai_amd import ops

    assert ops.describe_plan(816, 2048, 16384) == "tile 128x128 depth=4 splits=2 tiles=112"
    x = seeded((816, 16384), 50).to(dev)
    wq, ws = ops.fp8_weight_quant(seeded((2048, 16384), 51, 0.02).to(dev))
    eager = ops.fp8_linear(x, wq, ws)
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        ops.fp8_linear(x, wq, ws)                           # creates that stream's workspace
        with torch.cuda.graph(graph, stream=side):
            out = ops.fp8_linear(x, wq, ws)
    for _ in range(4):
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)
        again = ops.fp8_linear(x, wq, ws)                   # eager work between the replays
        torch.cuda.synchronize()
        assert torch.equal(again, eager)



def test_a_graph_keeps_its_workspace_when_other_work_outgrows_it(L, dev):
    """A recorded graph holds the addresses of its scratch (activation codes, split-K counters and
    partial sums).  Larger problems that later run eagerly - on the pooled stream the graph was
    recorded on as well as on the current one - must neither free nor share that scratch: the
    replays stay bit-equal to the eager result while other tensors are allocated and overwritten."""
    from phyai_amd import ops
    from phyai_amd.runtime import HipGraph

    x = seeded((200, 1040), 60).to(dev)                      # generic kernel, K split: counters + partial sums
    wq, ws = ops.fp8_weight_quant(seeded((512, 1040), 61, 0.02).to(dev))
    assert ops.describe_plan(200, 512, 1040).startswith("generic 128x128 splits=")
    eager = ops.fp8_linear(x, wq, ws)
    g = HipGraph()
    g.capture(lambda x: ops.fp8_linear(x, wq, ws), {"x": x})
    owned = list(g._workspace.tensors.values())
    assert len(owned) == 1 and not g._workspace.retired
    # now outgrow every per-stream workspace in sight, on the graph's recording stream too
    xb = seeded((816, 16384), 62).to(dev)
    wqb, wsb = ops.fp8_weight_quant(seeded((2048, 16384), 63, 0.02).to(dev))
    big_eager = ops.fp8_linear(xb, wqb, wsb)
    g.capture_stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(g.capture_stream):
        big_side = ops.fp8_linear(xb, wqb, wsb)
    torch.cuda.current_stream().wait_stream(g.capture_stream)
    torch.cuda.synchronize()
    assert torch.equal(big_side, big_eager)
    assert list(g._workspace.tensors.values())[0] is owned[0]        # untouched by all that
    junk = [torch.full((1 << 20,), 0x7F, dtype=torch.uint8, device=dev) for _ in range(64)]   # reuse anything freed
    for seed in (64, 65, 66):
        xi = seeded((200, 1040), seed).to(dev)
        out = g.replay({"x": xi})
        for t in junk:
            t.add_(1)
        torch.cuda.synchronize()
        assert torch.equal(out, ops.fp8_linear(xi, wq, ws))
    # an eager workspace that grows is replaced, not freed: queued launches may still use it
    n_retired = len(ops._retired)
    ops.reserve_workspace(ops.reserve_workspace(1).numel() + 1)
    assert len(ops._retired) == n_retired + 1
