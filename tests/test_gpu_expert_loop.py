"""The action expert's denoise loop as a component (phyai_amd/runtime/expert_loop.py; reference
models/pi05/model_runner_pi05.py:689-738 and modeling_pi05.py:801-835) at the real shapes:
18 layers, hidden 1024, 8 x 256 query heads, one KV head, MLP 4096, 50 action tokens.

* the fused layer (8 kernels) equals the unfused one (12 kernels) bit for bit over 18 chained
  layers and 3 Euler steps - every intermediate hidden state, not only the result;
* a graph replay equals the eager loop bit for bit, for several inputs, with eager work between;
* layer by layer, on the hidden state the library's loop actually produced, each form is within
  the stated tolerance (max-abs <= 1e-2 max|ref|, cosine >= 0.9999) of the same layer computed
  with the reference's own arithmetic as torch library calls (torch._scaled_mm underneath).
"""

from __future__ import annotations

import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu

N_LAYERS, STEPS, CHUNK, ADIM, HIDDEN = 18, 3, 50, 32, 1024


@pytest.fixture(scope="module")
def rig(dev):
    import phyai_amd.linear as L
    from phyai_amd.runtime.expert_loop import ExpertDenoiseLoop, ExpertLayer, PrefixAttentionStandIn

    torch.cuda.set_device(dev)
    L.init()
    layers = []
    for i in range(N_LAYERS):
        lay = ExpertLayer(prefix=f"model.layers.{i}")
        for j, lin in enumerate((lay.qkv_proj, lay.o_proj, lay.mlp.gate_up_proj, lay.mlp.down_proj)):
            lin.spec.quantize_weight_(lin, seeded(tuple(lin.weight.shape), 1000 + 10 * i + j, 0.02).to(dev))
        for j, norm in enumerate((lay.input_layernorm, lay.post_attention_layernorm)):
            norm.dense.weight.data.copy_(seeded(tuple(norm.dense.weight.shape), 2000 + 10 * i + j, 0.01))
            norm.dense.bias.data.copy_(seeded(tuple(norm.dense.bias.shape), 3000 + 10 * i + j, 0.05))
        layers.append(lay)
    attend = PrefixAttentionStandIn(N_LAYERS, CHUNK, 816, device=dev)
    time_emb = seeded((STEPS, HIDDEN), 7, 1.0).to(dev)

    def loop(variant, use_graph):
        lp = ExpertDenoiseLoop(layers, attend, chunk_size=CHUNK, action_dim=ADIM, variant=variant, use_graph=use_graph)
        lp.embed_action.weight.data.copy_(seeded((HIDDEN, ADIM), 11, 0.3))
        lp.project_action.weight.data.copy_(seeded((ADIM, HIDDEN), 12, 0.03))
        lp.embed_action.bias.data.zero_()
        lp.project_action.bias.data.zero_()
        lp.final_norm.dense.weight.data.copy_(seeded((3 * HIDDEN, HIDDEN), 13, 0.01))
        lp.bind_euler_schedule(time_emb, -1.0 / STEPS, STEPS)
        lp.setup()
        return lp

    yield loop
    L._reset_for_test()


def test_fused_layers_equal_unfused_layers_bit_for_bit(rig, dev):
    fused, unfused = rig("fused", False), rig("unfused", False)
    noise = seeded((CHUNK, ADIM), 21).to(dev)
    tf, tu = [], []
    xf = fused._fwd_loop(noise=noise, trace=tf)
    xu = unfused._fwd_loop(noise=noise, trace=tu)
    torch.cuda.synchronize()
    assert len(tf) == len(tu) == STEPS * (N_LAYERS + 1)
    for i, (a, b) in enumerate(zip(tf, tu)):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16)), \
            f"hidden state {i} (step {i // (N_LAYERS + 1)}, before layer {i % (N_LAYERS + 1)}) differs"
    assert torch.equal(xf.view(torch.int16), xu.view(torch.int16))
    assert bool(torch.isfinite(xf.float()).all()) and float(xf.float().abs().max()) > 0


def test_graph_replay_equals_the_eager_loop(rig, dev):
    from phyai_amd import ops

    graphed, eager = rig("fused", True), rig("fused", False)
    assert graphed.graph is not None and graphed.graph.is_captured
    for seed in (31, 32, 33):
        noise = seeded((CHUNK, ADIM), seed).to(dev)
        want = eager.run(noise)
        got = graphed.run(noise)
        torch.cuda.synchronize()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"replay with seed {seed} differs"
        ops.fp8_quant_rowwise(seeded((64, 256), seed).to(dev))          # unrelated eager work between replays
    with pytest.raises(RuntimeError, match="bind_euler_schedule"):
        from phyai_amd.runtime.expert_loop import ExpertDenoiseLoop
        ExpertDenoiseLoop(graphed.layers, graphed.attend).setup()


@pytest.mark.parametrize("variant", ["fused", "unfused"])
def test_each_layer_is_within_tolerance_of_the_torch_path(rig, dev, variant):
    from phyai_amd.runtime.expert_loop import ExpertLayerModulation

    lib, ref_loop = rig(variant, False), rig("torch", False)
    noise = seeded((CHUNK, ADIM), 41).to(dev)
    trace = []
    lib._fwd_loop(noise=noise, trace=trace)
    torch.cuda.synchronize()
    try:
        ref_loop.layers[0](trace[0], ref_loop.attend, 0, ref_loop._mod_tables[0][0], "torch")
        torch.cuda.synchronize()
    except Exception as e:  # noqa: BLE001 - torch._scaled_mm may be unavailable on an image
        pytest.skip(f"torch._scaled_mm does not run here: {str(e)[:100]}")
    per = N_LAYERS + 1
    for step in range(STEPS):
        for i in range(N_LAYERS):
            h_in, h_out = trace[step * per + i], trace[step * per + i + 1]
            mod: ExpertLayerModulation = ref_loop._mod_tables[step][i]
            want = ref_loop.layers[i](h_in, ref_loop.attend, i, mod, "torch").float()
            got = h_out.float()
            err = (got - want).abs().max().item()
            cos = torch.nn.functional.cosine_similarity(got.reshape(-1), want.reshape(-1), dim=0).item()
            assert err <= 1e-2 * want.abs().max().item() and cos >= 0.9999, \
                f"step {step} layer {i}: max-abs {err:.4g} vs max|ref| {want.abs().max().item():.4g}, cosine {cos:.6f}"
