"""Weights in MFMA operand order (phyai_fp8_weight_to_operand_order, phyai_amd/csrc/weight_layout.h).

The re-lay is what the reference leaves to WeightSpec.process_after_loading
(layers/quant/base.py:55-70, layers/quant/fp8.py:127-135).  It moves bytes and changes no arithmetic:
 * the re-laid matrix is checked byte for byte against index arithmetic on the CPU;
 * every kernel family must give the bits it gives with the row-major matrix, whose outputs are
   pinned against the oracle elsewhere (tests/test_gpu_parity.py, tests/test_gpu_configs.py).
"""

from __future__ import annotations

import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu

GATED = ("geglu_tanh", "geglu_erf", "swiglu")


def _ops():
    from phyai_amd import ops
    return ops


def _bits(t):
    return t.contiguous().view(torch.int16)


def _operand_order_on_cpu(w: torch.Tensor, gated: bool) -> torch.Tensor:
    """w: uint8 [N, K] on the CPU.  Unit u, K step s, chunk c, row r -> 16 bytes at
    ((u * steps + s) * 128 + c * 16 + r) * 16."""
    N, K = w.shape
    steps = K // 128
    u = torch.arange(N // 16).view(-1, 1, 1, 1)
    s = torch.arange(steps).view(1, -1, 1, 1)
    c = torch.arange(8).view(1, 1, -1, 1)
    r = torch.arange(16).view(1, 1, 1, -1)
    if gated:
        row = ((r >> 1) & 1) * (N // 2) + 8 * u + 2 * (r >> 2) + (r & 1)
    else:
        row = 16 * u + r
    chunks = w.view(N, K // 16, 16)                      # [row, chunk of K, 16 bytes]
    col = (s * 8 + c).expand(N // 16, steps, 8, 16)
    return chunks[row.expand_as(col), col].reshape(N, K)


@pytest.mark.parametrize("N,K,gated", [(16, 128, False), (32, 128, True), (1024, 4096, False), (8192, 1024, True),
                                       (2560, 2048, False), (96, 384, True), (48, 1152, False)])
def test_relay_matches_index_arithmetic(dev, N, K, gated):
    ops = _ops()
    g = torch.Generator().manual_seed(N + K)
    w = torch.randint(0, 256, (N, K), generator=g, dtype=torch.uint8)
    got = ops.fp8_weight_to_operand_order(w.to(dev).view(torch.float8_e4m3fn), gated=gated)
    assert got.dtype == torch.float8_e4m3fn and got.shape == (N, K)
    assert torch.equal(got.view(torch.uint8).cpu(), _operand_order_on_cpu(w, gated))


def test_relay_refuses_what_it_cannot_do(dev):
    ops = _ops()
    from phyai_amd import _lib

    w = torch.zeros(32, 192, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    with pytest.raises(RuntimeError, match="K % 128"):
        ops.fp8_weight_to_operand_order(w)
    w = torch.zeros(48, 128, dtype=torch.uint8, device=dev).view(torch.float8_e4m3fn)
    with pytest.raises(RuntimeError, match="N % 32"):
        ops.fp8_weight_to_operand_order(w, gated=True)
    lib = _lib.load()
    w = torch.zeros(32, 128, dtype=torch.uint8, device=dev)
    assert lib.phyai_fp8_weight_to_operand_order(w.data_ptr(), 32, 128, 0, w.data_ptr(), None) == -1   # in place
    assert b"overlaps" in lib.phyai_fp8_last_error()


def _problem(dev, M, N, K, seed):
    ops = _ops()
    x = seeded((M, K), seed=seed)
    w = seeded((N, K), seed=seed + 1, scale=0.02).to(dev)
    b = seeded((N,), seed=seed + 2, scale=0.01).to(dev)
    wq, ws = ops.fp8_weight_quant(w)
    return x.to(dev), wq, ws, b


def _both_layouts(dev, M, N, K, epi, seed, *, residual=False):
    """(row-major output, operand-order output) of fp8_linear and of fp8_gemm on the quantizer's codes."""
    ops = _ops()
    x, wq, ws, b = _problem(dev, M, N, K, seed)
    gated = epi in GATED
    wo = ops.fp8_weight_to_operand_order(wq, gated=gated)
    layout = "operand_gated" if gated else "operand"
    kw = {}
    if residual:
        kw = dict(residual=seeded((M, N), seed=seed + 3).to(dev), gate=seeded((1, N), seed=seed + 4, scale=0.5).to(dev))
    xq, xs = ops.fp8_quant_rowwise(x)
    out = []
    for w_, lay in ((wq, None), (wo, layout)):
        out.append((ops.fp8_linear(x, w_, ws, b, epilogue=epi, weight_layout=lay, **kw),
                    ops.fp8_gemm(xq, xs, w_, ws, b, epilogue=epi, weight_layout=lay, **kw)))
    torch.cuda.synchronize()
    return out


# the benchmark's layer sets and a few awkward widths: one-launch small-M kernel, weight-streaming
# kernel (on ready codes), every pipelined tile shape by automatic choice
SHAPES = [
    (4800, 2048, 8192, None), (1632, 8192, 8192, "gelu"), (3264, 2048, 4096, "geglu_tanh"),   # 224 x 256 by the layout-aware rule
    # more 128 x 128 tiles than CUs: 4 x 1 blocks per wavefront, weights in registers, ring of four, two workgroups per CU
    (1632, 2560, 2048, None), (3264, 2048, 1536, "gelu"), (2100, 2048, 512, None), (2305, 2064, 1024, "gelu_tanh"),
    (50, 2560, 1024, None), (50, 1024, 2048, None), (50, 8192, 1024, "geglu_tanh"), (50, 1024, 4096, None),
    (1, 256, 128, None), (7, 272, 512, "gelu"), (33, 528, 2048, "gelu_tanh"), (64, 2048, 4096, "geglu_erf"),
    (100, 2560, 1024, None), (200, 1024, 4096, None), (400, 8192, 1024, "geglu_tanh"), (800, 1024, 2048, None),
    (816, 2560, 2048, None), (816, 2048, 2048, None), (816, 4096, 2048, "geglu_tanh"), (816, 2048, 16384, None),
    (300, 544, 1280, "swiglu"), (1000, 272, 2048, None), (260, 288, 1024, "swiglu"),
]


@pytest.mark.parametrize("M,N,K,epi", SHAPES)
def test_operand_order_gives_the_row_major_bits(dev, M, N, K, epi):
    (lin_rm, gemm_rm), (lin_op, gemm_op) = _both_layouts(dev, M, N, K, epi, seed=M + N + K)
    assert torch.equal(_bits(lin_op), _bits(lin_rm)), "whole linear"
    assert torch.equal(_bits(gemm_op), _bits(gemm_rm)), "GEMM on ready codes"


@pytest.mark.parametrize("M,N,K", [(50, 1024, 2048), (50, 1024, 4096), (816, 2048, 2048), (300, 512, 1280)])
def test_operand_order_with_the_gated_residual(dev, M, N, K):
    (lin_rm, gemm_rm), (lin_op, gemm_op) = _both_layouts(dev, M, N, K, None, seed=M + N + K + 9, residual=True)
    assert torch.equal(_bits(lin_op), _bits(lin_rm)) and torch.equal(_bits(gemm_op), _bits(gemm_rm))


# how the pipelined tile kernel takes weights in operand order: staged through LDS as they lie (and, for the
# 224-row tile with K a multiple of 512, straight into registers); the same without the register path; gathered
# row by row into the row-major staging layout
@pytest.mark.parametrize("mode", ["", "PHYAI_FP8_BIG_DIRECT=0", "PHYAI_FP8_BIG_GATHER=1"])
@pytest.mark.parametrize("tile", ["256", "224", "192", "128", "128/2", "12864", "96"])
@pytest.mark.parametrize("M,N,K,epi", [(816, 768, 1024, None), (513, 400, 1536, "gelu"), (816, 1024, 1152, "geglu_tanh"),
                                       (260, 288, 1024, "swiglu"), (300, 544, 2048, "geglu_erf")])
def test_operand_order_in_every_pipelined_tile_shape(dev, monkeypatch, mode, tile, M, N, K, epi):
    t, _, depth = tile.partition("/")
    monkeypatch.setenv("PHYAI_FP8_BIG", t)
    if depth:
        monkeypatch.setenv("PHYAI_FP8_BIG_DEPTH", depth)
    if mode:
        monkeypatch.setenv(*mode.split("="))
    (lin_rm, _), (lin_op, _) = _both_layouts(dev, M, N, K, epi, seed=M + N + K + 1)
    assert torch.equal(_bits(lin_op), _bits(lin_rm))


# 128 x 128 tiles with weights in operand order, a plain epilogue and K (per split) a multiple of 1024:
# wavefronts 1 x 4, weights straight into registers through a ring of eight, activation stages handed over through
# progress words.  One trip round the ring (tail only), several, K split 2 and 4, ragged M and N.
@pytest.mark.parametrize("tile,splits,M,N,K,epi", [
    ("128", "1", 816, 768, 1024, None), ("128", "1", 816, 768, 2048, "gelu"), ("128", "2", 816, 768, 2048, None),
    ("128", "1", 513, 400, 3072, "gelu_tanh"), ("128", "1", 300, 272, 8192, None), ("128", "2", 300, 272, 8192, "gelu"),
    ("128", "4", 300, 272, 8192, None), ("128", "2", 130, 2048, 16384, None), ("128", "1", 129, 144, 5120, None),
    ("128", "1", 97, 144, 1024, "gelu_erf"), ("128", "1", 480, 1024, 7168, None),
])
def test_register_weights_ring_of_eight(dev, monkeypatch, tile, splits, M, N, K, epi):
    monkeypatch.setenv("PHYAI_FP8_BIG", tile)
    monkeypatch.setenv("PHYAI_FP8_BIG_SPLITS", splits)
    (lin_rm, gemm_rm), (lin_op, gemm_op) = _both_layouts(dev, M, N, K, epi, seed=M + N + K + 5)
    assert torch.equal(_bits(lin_op), _bits(lin_rm)) and torch.equal(_bits(gemm_op), _bits(gemm_rm))
    monkeypatch.setenv("PHYAI_FP8_BIG_DIRECT", "0")      # the same tiles with the weights staged through LDS
    (_, _), (lin_st, _) = _both_layouts(dev, M, N, K, epi, seed=M + N + K + 5)
    assert torch.equal(_bits(lin_st), _bits(lin_op))


def test_layout_and_epilogue_must_match(dev):
    ops = _ops()
    from phyai_amd import _lib

    x, wq, ws, b = _problem(dev, 16, 64, 128, seed=3)
    with pytest.raises(RuntimeError, match="does not go with"):
        ops.fp8_linear(x, wq, ws, b, epilogue="geglu_tanh", weight_layout="operand")
    with pytest.raises(RuntimeError, match="does not go with"):
        ops.fp8_linear(x, wq, ws, b, weight_layout="operand_gated")
    lib = _lib.load()
    out = torch.empty(16, 64, dtype=torch.bfloat16, device=dev)
    need = lib.phyai_fp8_linear_workspace_bytes(16, 64, 128, 0)
    wsp = torch.zeros(need, dtype=torch.uint8, device=dev)
    rc = lib.phyai_fp8_linear(x.data_ptr(), 128, wq.data_ptr(), ws.data_ptr(), None, out.data_ptr(), 64, 16, 64, 128,
                              0 | ops.FLAG_W_OPERAND_GATED, wsp.data_ptr(), need, None)
    assert rc == -1 and b"operand order" in lib.phyai_fp8_last_error()
    rc = lib.phyai_fp8_linear(x.data_ptr(), 128, wq.data_ptr(), ws.data_ptr(), None, out.data_ptr(), 64, 16, 64, 128,
                              0x400, wsp.data_ptr(), need, None)
    assert rc == -1


def test_spec_relays_after_loading_and_layers_give_the_same_bits(dev):
    """Fp8Spec(operand_order=True): post_load re-lays the weight once (a second call is a no-op), the layer
    and the MLP built on it give the bits of the row-major layers."""
    from phyai_amd import linear as L
    from phyai_amd.mlp import DenseMLP
    from phyai_amd.quant import Fp8Spec

    L.init()
    ops = _ops()
    H, I, M = 256, 512, 50
    wgu, wd = seeded((2 * I, H), 8, 0.05).to(dev), seeded((H, I), 9, 0.05).to(dev)
    x = seeded((M, H), 10).to(dev)
    outs = []
    for operand in (False, True):
        mlp = DenseMLP(H, I, activation="gelu_tanh", params_dtype=torch.bfloat16, spec_in=Fp8Spec(operand_order=operand),
                       spec_out=Fp8Spec(operand_order=operand))
        for lin, w in ((mlp.gate_up_proj, wgu), (mlp.down_proj, wd)):
            lin.spec.quantize_weight_(lin, w)
            before = lin.weight.detach().clone()
            lin.post_load()
            lin.post_load()
            if operand:
                gated = lin is mlp.gate_up_proj
                assert lin.weight_layout == ("operand_gated" if gated else "operand")
                assert torch.equal(lin.weight.view(torch.uint8), ops.fp8_weight_to_operand_order(before, gated=gated).view(torch.uint8))
            else:
                assert getattr(lin, "weight_layout", None) is None and torch.equal(lin.weight.view(torch.uint8), before.view(torch.uint8))
        outs.append((mlp(x), mlp.down_proj(x.new_ones(M, I))[0]))
        if operand:
            mlp.fuse_activation = False
            with pytest.raises(RuntimeError, match="gated operand order"):
                mlp(x)
            # a reload puts row-major bytes back; the next post_load re-lays them again
            mlp.down_proj.spec.quantize_weight_(mlp.down_proj, wd)
            mlp.down_proj.post_load()
            assert torch.equal(_bits(mlp.down_proj(x.new_ones(M, I))[0]), _bits(outs[-1][1]))
    assert torch.equal(_bits(outs[0][0]), _bits(outs[1][0])) and torch.equal(_bits(outs[0][1]), _bits(outs[1][1]))
