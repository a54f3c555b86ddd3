"""GPU parity of the norms with the quantizer fused behind them (through the C ABI)."""

import pytest
import torch

from oracle import ref
from tests.conftest import seeded
from tests.test_oracle import _bf16_ulp_diff

pytestmark = pytest.mark.gpu


def _ops():
    from phyai_amd import ops
    return ops


def _close_bf16(got: torch.Tensor, want: torch.Tensor, what: str, mag: torch.Tensor | None = None):
    """Within one bf16 step everywhere (the reduction order differs from the CPU's), nearly all equal,
    and inside the reference's own bf16 tolerance (phyai-kernel/tests/test_adarmsnorm.py:100-105).
    ``mag``: magnitude of the terms that were added; where they cancel, one bf16 step of THEM is the bar."""
    d = _bf16_ulp_diff(got.cpu(), want)
    if mag is None:
        assert int(d.max()) <= 1, f"{what}: off by {int(d.max())} bf16 steps"
    else:
        err = (got.cpu().float() - want.float()).abs()
        assert bool((err <= mag.float() * 2.0 ** -7 + 1e-30).all()), f"{what}: more than a bf16 step of the summands"
    assert float((d == 0).float().mean()) > 0.99, f"{what}: {float((d == 0).float().mean()):.4f} equal"
    torch.testing.assert_close(got.cpu().float(), want.float(), rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("gemma", [False, True])
@pytest.mark.parametrize("shape", [(17, 256), (50, 1024), (3, 11, 2048), (5, 3072), (2, 8192), (1, 8), (3, 12288)])
def test_rmsnorm_matches_oracle(dev, shape, gemma):
    ops = _ops()
    x = seeded(shape, seed=sum(shape), scale=0.5)
    w = seeded((shape[-1],), seed=shape[-1] + 7, scale=0.3)
    fn = ops.gemma_rmsnorm if gemma else ops.rmsnorm
    got = fn(x.to(dev), w.to(dev), 1e-6)
    assert got.shape == x.shape and got.dtype == torch.bfloat16
    _close_bf16(got, ref.rmsnorm(x, w, 1e-6, gemma), f"rmsnorm {shape}")


@pytest.mark.parametrize("gemma", [False, True])
@pytest.mark.parametrize("shape", [(50, 1024), (816, 2048), (7, 4096), (5, 12288)])
def test_rmsnorm_fp8_is_quantizer_of_its_own_output(dev, shape, gemma):
    """Codes and scales of the fused form are bit-equal to the quantizer applied to the bf16 tensor
    the same kernel writes - the norm adds nothing to the quantizer's arithmetic."""
    ops = _ops()
    x = seeded(shape, seed=3 + shape[0], scale=2.0)
    x[0, :8] = 0.0
    w = seeded((shape[-1],), seed=11, scale=0.3)
    xq, xs, out = ops.rmsnorm_fp8(x.to(dev), w.to(dev), 1e-6, gemma=gemma, want_out=True)
    _close_bf16(out, ref.rmsnorm(x, w, 1e-6, gemma), "fused norm output")
    q_ref, s_ref = ref.quant_rowwise(out.cpu())
    assert torch.equal(xs.cpu(), s_ref)
    assert torch.equal(xq.cpu().view(torch.uint8), q_ref.view(torch.uint8))
    # codes only: same codes, no bf16 tensor written
    xq2, xs2 = ops.rmsnorm_fp8(x.to(dev), w.to(dev), 1e-6, gemma=gemma)
    assert torch.equal(xq2.view(torch.uint8), xq.view(torch.uint8)) and torch.equal(xs2, xs)


@pytest.mark.parametrize("hidden", [256, 1024, 2048, 3072, 8192, 12288])
def test_adarmsnorm_per_token_and_broadcast(dev, hidden):
    """Shapes of the reference's tests (phyai-kernel/tests/test_adarmsnorm.py:133-200)."""
    ops = _ops()
    x = seeded((17, hidden), seed=hidden, scale=0.5)
    mod = seeded((17, 3 * hidden), seed=hidden + 1, scale=0.1)
    out, gate = ops.adarmsnorm(x.to(dev), mod.to(dev), 1e-6)
    want_out, want_gate = ref.adarmsnorm(x, mod, 1e-6)

    def summands(xx, mm):
        x64 = xx.double()
        xh = x64 / torch.sqrt((x64 * x64).mean(-1, keepdim=True) + 1e-6)
        return (xh * (1.0 + mm[..., :hidden].double())).abs() + mm[..., hidden:2 * hidden].double().abs()

    _close_bf16(out, want_out, f"adarmsnorm 2d {hidden}", summands(x, mod))
    assert torch.equal(gate.cpu(), want_gate)
    x3 = seeded((4, 13, hidden), seed=hidden + 2, scale=0.5)
    mod_b = seeded((4, 3 * hidden), seed=hidden + 3, scale=0.1)
    out3, gate3 = ops.adarmsnorm(x3.to(dev), mod_b.to(dev), 1e-6)
    want3, wgate3 = ref.adarmsnorm(x3, mod_b, 1e-6)
    assert gate3.shape == (4, hidden)
    _close_bf16(out3, want3, f"adarmsnorm broadcast {hidden}", summands(x3, mod_b[:, None, :]))
    assert torch.equal(gate3.cpu(), wgate3)


def test_adarmsnorm_fp8_feeds_the_gemm(dev):
    """adarmsnorm_fp8 -> fp8_gemm equals adarmsnorm -> fp8_linear bit for bit (same codes, same GEMM)."""
    ops = _ops()
    M, D, N = 50, 1024, 2560
    x = seeded((M, D), seed=21, scale=0.7).to(dev)
    mod = seeded((1, 3 * D), seed=22, scale=0.1).to(dev)
    w = seeded((N, D), seed=23, scale=0.02)
    wq, ws = ref.weight_quant(w)
    wq, ws = wq.to(dev), ws.to(dev)
    xq, xs, gate, n = ops.adarmsnorm_fp8(x, mod, 1e-6, want_out=True)
    assert gate.shape == (1, D)
    fused = ops.fp8_gemm(xq, xs, wq, ws, None)
    n2, gate2 = ops.adarmsnorm(x, mod, 1e-6)
    assert torch.equal(n, n2) and torch.equal(gate, gate2)
    two_step = ops.fp8_linear(n2, wq, ws, None)
    assert torch.equal(fused, two_step)
    q_ref, s_ref = ref.quant_rowwise(n.cpu())
    assert torch.equal(xq.cpu().view(torch.uint8), q_ref.view(torch.uint8)) and torch.equal(xs.cpu(), s_ref)


def test_norm_argument_errors(dev):
    ops = _ops()
    x = torch.zeros(4, 64, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="adarmsnorm"):
        ops.adarmsnorm(x, torch.zeros(4, 128, dtype=torch.bfloat16, device=dev))          # not 3 * D
    with pytest.raises(RuntimeError, match="multiple of modulation rows"):
        ops.adarmsnorm(x, torch.zeros(3, 192, dtype=torch.bfloat16, device=dev))
    with pytest.raises(RuntimeError, match="gate_out"):
        ops.adarmsnorm(x, torch.zeros(4, 192, dtype=torch.bfloat16, device=dev),
                       gate_out=torch.zeros(2, 64, dtype=torch.bfloat16, device=dev))
    with pytest.raises(RuntimeError, match="weight"):
        ops.rmsnorm(x, torch.zeros(32, dtype=torch.bfloat16, device=dev))
    with pytest.raises(RuntimeError, match="multiple of 8"):
        ops.rmsnorm(torch.zeros(2, 12, dtype=torch.bfloat16, device=dev), torch.zeros(12, dtype=torch.bfloat16, device=dev))
    empty, g = ops.adarmsnorm(x[:0], torch.zeros(0, 192, dtype=torch.bfloat16, device=dev))
    assert empty.shape == (0, 64) and g.shape == (0, 64)


def test_norm_modules_feed_fp8_layers(dev):
    """GemmaRMSNorm / AdaRMSNorm ``forward_fp8`` -> fp8 layer == bf16 norm -> same layer, bit for bit,
    and DenseMLP takes the quantized view through its fused gate_up epilogue."""
    import phyai_amd.linear as L
    from phyai_amd.linear.layers import ColumnParallelLinear
    from phyai_amd.mlp import DenseMLP
    from phyai_amd.norm import AdaRMSNorm, GemmaRMSNorm
    from phyai_amd.quant import Fp8Spec
    from phyai_amd.quant.types import ActivationView, Granularity

    torch.cuda.set_device(dev)
    L.init()
    try:
        _norm_modules_body(dev, GemmaRMSNorm, AdaRMSNorm, ColumnParallelLinear, DenseMLP, Fp8Spec,
                           ActivationView, Granularity)
    finally:
        L._reset_for_test()


def _norm_modules_body(dev, GemmaRMSNorm, AdaRMSNorm, ColumnParallelLinear, DenseMLP, Fp8Spec,
                       ActivationView, Granularity):
    D, N, M = 1024, 2560, 50
    torch.manual_seed(4)
    norm = GemmaRMSNorm(D, device=dev, prefix="layers.0.input_layernorm")
    norm.weight.data.copy_((torch.randn(D) * 0.1).to(torch.bfloat16))
    layer = ColumnParallelLinear(D, N, bias=False, params_dtype=torch.bfloat16, spec=Fp8Spec(), device=dev)
    layer.spec.quantize_weight_(layer, (torch.randn(N, D) * 0.02).to(torch.bfloat16).to(dev))
    x = (torch.randn(M, D) * 0.8).to(torch.bfloat16).to(dev)
    view = norm.forward_fp8(x)
    assert isinstance(view, ActivationView) and view.granularity is Granularity.PER_CHANNEL
    y_fused, _ = layer(view)
    y_plain, _ = layer(norm(x))
    assert torch.equal(y_fused, y_plain)

    ada = AdaRMSNorm(D, 1024, device=dev)
    ada.dense.weight.data.copy_((torch.randn(3 * D, 1024) * 0.01).to(torch.bfloat16))
    cond = torch.randn(1, 1024).to(torch.bfloat16).to(dev)
    table = ada.project_modulation(cond)
    v2, gate = ada.forward_fp8(x, modulation=table)
    n2, gate2 = ada(x, modulation=table)
    assert torch.equal(gate, gate2) and gate.shape == (1, D)
    assert torch.equal(layer(v2)[0], layer(n2)[0])
    # gated residual fused into the same layer's epilogue, gate of one modulation row
    res = (torch.randn(M, N) * 0.5).to(torch.bfloat16).to(dev)
    g_row = (torch.randn(1, N) * 0.3).to(torch.bfloat16).to(dev)
    assert torch.equal(layer.forward_addcmul(v2, res, g_row), torch.addcmul(res, layer(v2)[0], g_row))

    mlp = DenseMLP(D, 4096, activation="gelu_tanh", gated=True, bias=False, params_dtype=torch.bfloat16,
                   spec_in=Fp8Spec(), spec_out=Fp8Spec())
    for lin, shape in ((mlp.gate_up_proj, (8192, D)), (mlp.down_proj, (D, 4096))):
        lin.spec.quantize_weight_(lin, (torch.randn(*shape) * 0.02).to(torch.bfloat16).to(dev))
    assert torch.equal(mlp(v2), mlp(n2))
