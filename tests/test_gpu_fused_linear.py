"""The one-launch small-M linear (phyai_amd/csrc/gemm_skinny_fused.hip): the kernel that quantizes its
own activation rows (reference quant/fp8.py:150-155) in front of the fp8 GEMM
(linear/backends/torch.py:155-176) must give the bits of quantizer launch + GEMM launch, whose
codes, scales and outputs are pinned against the oracle elsewhere.

Every workgroup shape the kernel exists in is forced in turn; the automatic choice is checked
against the oracle as well, since for M <= 128 it is what `fp8_linear` now runs.
"""

from __future__ import annotations

import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu

PLANS = ["", "8,2", "8,4", "8,5", "8,8", "16,1", "16,2", "16,4", "16,8", "32,2", "32,4"]
EPI_ID = {None: 0, "geglu_tanh": 1, "geglu_erf": 2, "swiglu": 3, "gelu_tanh": 4, "gelu": 5}


def _ops():
    from phyai_amd import ops
    return ops


def _bits(t):
    return t.contiguous().view(torch.int16)


def _awkward_rows(x):
    """zeros only, signed zeros, an outlier, tiny values, the largest bf16, an Inf, a NaN."""
    M = x.shape[0]
    x = x.clone()
    x[0] = 0
    if M > 1: x[1, ::2] = -0.0
    if M > 2: x[2, 5] = 300.0
    if M > 3: x[3] = x[3] * 1e-30
    if M > 5:
        x[4, 7] = torch.finfo(torch.bfloat16).max
        x[5, 3] = float("inf")
    if M > 6: x[6, 9] = float("nan")
    return x


def _same(a, b):
    """bit equality (rows with an Inf or a NaN included: both paths do the same arithmetic)"""
    return torch.equal(_bits(a), _bits(b))


CASES = [
    (50, 2560, 1024, None), (50, 1024, 2048, None), (50, 8192, 1024, "geglu_tanh"), (50, 1024, 4096, None),
    (1, 256, 128, None), (7, 272, 512, "gelu"), (16, 1024, 1024, "swiglu"), (33, 528, 2048, "gelu_tanh"),
    (64, 2048, 4096, "geglu_erf"), (50, 4096, 1024, None), (23, 144, 384, None), (9, 64, 3072, None),
    (64, 288, 256, "geglu_tanh"), (17, 48, 1152, None),
    (100, 2560, 1024, None), (128, 1024, 2048, None), (77, 528, 512, "gelu"), (90, 1056, 1024, "geglu_tanh"),
]


@pytest.mark.parametrize("M,N,K,epi", CASES)
def test_every_workgroup_shape_equals_two_launches_bit_for_bit(dev, monkeypatch, M, N, K, epi):
    ops = _ops()
    x = _awkward_rows(seeded((M, K), seed=M * 131 + N + K))
    wide = torch.zeros(M, K + 64, dtype=torch.bfloat16)
    wide[:, :K] = x
    xd = wide.to(dev)[:, :K]                                    # row stride K + 64
    w = seeded((N, K), seed=N + 7 * K, scale=0.02).to(dev)
    b = seeded((N,), seed=N, scale=0.01).to(dev)
    wq, ws = ops.fp8_weight_quant(w)
    # the same weights in MFMA operand order: the kernel then loads them straight into registers
    gated = epi in ("geglu_tanh", "geglu_erf", "swiglu")
    operand = K % 128 == 0 and N % (32 if gated else 16) == 0
    wo = ops.fp8_weight_to_operand_order(wq, gated=gated) if operand else None
    layout = "operand_gated" if gated else "operand"
    res = seeded((M, N), seed=5).to(dev)
    gate = seeded((1, N), seed=6, scale=0.5).to(dev)

    monkeypatch.setenv("PHYAI_FP8_FUSED", "0")
    assert ops.describe_linear_plan(M, N, K, epi).startswith("quantizer + ")
    want = {bias is None: ops.fp8_linear(xd, wq, ws, bias, epilogue=epi) for bias in (None, b)}
    want_res = ops.fp8_linear(xd, wq, ws, b, residual=res, gate=gate) if epi is None else None
    monkeypatch.setenv("PHYAI_FP8_FUSED", "1")
    ran = 0
    for plan in PLANS:
        if plan:
            monkeypatch.setenv("PHYAI_FP8_FUSED_PLAN", plan)
        else:
            monkeypatch.delenv("PHYAI_FP8_FUSED_PLAN", raising=False)
        desc = ops.describe_linear_plan(M, N, K, epi)
        if not desc.startswith("one launch"):
            continue
        ran += 1
        for bias in (None, b):
            for streamed in (False, True):
                got = ops.fp8_linear(xd, wq, ws, bias, epilogue=epi, stream_weights=streamed)
                torch.cuda.synchronize()
                assert _same(got, want[bias is None]), \
                    f"{desc}, bias={bias is not None}, streamed={streamed}: " \
                    f"{int((_bits(got) != _bits(want[bias is None])).sum())} outputs differ"
                if operand:
                    got = ops.fp8_linear(xd, wo, ws, bias, epilogue=epi, stream_weights=streamed, weight_layout=layout)
                    assert _same(got, want[bias is None]), f"{desc}, weights in operand order, bias={bias is not None}, streamed={streamed}"
        if want_res is not None:
            got = ops.fp8_linear(xd, wq, ws, b, residual=res, gate=gate)
            assert _same(got, want_res), f"{desc}: gated residual differs"
            if operand:
                got = ops.fp8_linear(xd, wo, ws, b, residual=res, gate=gate, weight_layout=layout)
                assert _same(got, want_res), f"{desc}: gated residual with weights in operand order differs"
            buf = res.clone()                                   # writing over the residual
            ops.fp8_linear(xd, wq, ws, b, residual=buf, gate=gate, out=buf)
            assert _same(buf, want_res), f"{desc}: gated residual written in place differs"
    assert ran >= 1, "no one-launch kernel exists for this case"


@pytest.mark.parametrize("M,N,K,epi", [(50, 4096, 1024, None), (50, 8192, 1024, "geglu_tanh"), (50, 1024, 2048, None),
                                       (1, 2560, 1024, None), (64, 1024, 1024, "gelu_tanh"), (100, 1024, 2048, None),
                                       # four K steps per wavefront: the kernel finds its own row maxima beyond K = 2048 too
                                       (50, 1024, 4096, None), (16, 2048, 3072, None), (128, 512, 4096, None),
                                       (100, 256, 2560, None)])
def test_automatic_choice_is_the_one_launch_kernel_and_matches_the_oracle(dev, M, N, K, epi):
    from oracle import ref
    ops = _ops()
    assert ops.describe_linear_plan(M, N, K, epi).startswith("one launch")
    x = seeded((M, K), seed=M + K)
    w = seeded((N, K), seed=N + K, scale=0.02)
    b = seeded((N,), seed=3, scale=0.01)
    wq, ws = ref.weight_quant(w)
    got = ops.fp8_linear(x.to(dev), wq.to(dev), ws.to(dev), b.to(dev), epilogue=epi)
    xq, xs = ref.quant_rowwise(x)
    want = ref.gemm_f32(xq, xs, wq, ws, b)
    want = ref.epilogue(want, EPI_ID[epi]).float() if epi else want
    err = (got.float().cpu() - want).abs().max().item()
    cos = torch.nn.functional.cosine_similarity(got.float().cpu().reshape(-1), want.reshape(-1), dim=0).item()
    assert err <= 1e-2 * want.abs().max().item() and cos >= 0.9999, (err, cos)


def test_gate_rows_per_group_and_batched_leading_dims(dev, monkeypatch):
    """one gate row per group of token rows (the reference's per-sample modulation), x as (B, T, K)"""
    ops = _ops()
    B, T, N, K = 4, 12, 1024, 1024
    x = seeded((B, T, K), seed=1).to(dev)
    w = seeded((N, K), seed=2, scale=0.02).to(dev)
    wq, ws = ops.fp8_weight_quant(w)
    res = seeded((B, T, N), seed=3).to(dev)
    gate = seeded((B, 1, N), seed=4, scale=0.5).to(dev)
    monkeypatch.setenv("PHYAI_FP8_FUSED", "0")
    want = ops.fp8_linear(x, wq, ws, None, residual=res, gate=gate)
    monkeypatch.setenv("PHYAI_FP8_FUSED", "1")
    assert ops.describe_linear_plan(B * T, N, K, None).startswith("one launch")
    got = ops.fp8_linear(x, wq, ws, None, residual=res, gate=gate)
    assert got.shape == (B, T, N) and _same(got, want)


def test_activations_the_kernel_cannot_read_fall_back_to_two_launches(dev):
    """a row stride that is not a multiple of 8 elements (rows not 16-byte aligned) still works:
    the quantizer copes with it and the result is the same"""
    ops = _ops()
    M, N, K = 20, 512, 1024
    x = seeded((M, K), seed=11)
    wide = torch.zeros(M, K + 4, dtype=torch.bfloat16)
    wide[:, :K] = x
    w = seeded((N, K), seed=12, scale=0.02).to(dev)
    wq, ws = ops.fp8_weight_quant(w)
    want = ops.fp8_linear(x.to(dev), wq, ws, None)
    got = ops.fp8_linear(wide.to(dev)[:, :K], wq, ws, None)
    assert _same(got, want)


def test_graph_replay_of_the_one_launch_kernel(dev):
    from phyai_amd.runtime import HipGraph
    ops = _ops()
    M, N, K = 50, 2560, 1024
    w = seeded((N, K), seed=21, scale=0.02).to(dev)
    wq, ws = ops.fp8_weight_quant(w)
    x_static = torch.zeros(M, K, dtype=torch.bfloat16, device=dev)
    out = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
    gr = HipGraph()
    gr.capture(lambda: ops.fp8_linear(x_static, wq, ws, None, out=out), {})
    for seed in (31, 32, 33):
        x = seeded((M, K), seed=seed).to(dev)
        want = ops.fp8_linear(x, wq, ws, None).clone()
        x_static.copy_(x)
        gr.replay()
        torch.cuda.synchronize()
        assert _same(out, want), f"replay with seed {seed}"


def test_random_shapes_equal_two_launches_bit_for_bit(dev, monkeypatch):
    """200 seeded random problems the automatic choice serves with the one-launch kernel (M up to 128, K up to 4096,
    every epilogue, with and without bias, streamed weights or not, tiny and outlier rows)."""
    import random

    ops = _ops()
    rnd = random.Random(7)
    epis = [None, "gelu", "gelu_tanh", "geglu_tanh", "geglu_erf", "swiglu"]
    ran = 0
    for it in range(200):
        M = rnd.choice([1, 2, 3, 5, 7, 8, 9, 15, 16, 17, 31, 33, 47, 50, 63, 64, 65, 77, 96, 100, 127, 128])
        K = 128 * rnd.randint(1, 32)
        epi = rnd.choice(epis)
        N = (32 if epi in ("geglu_tanh", "geglu_erf", "swiglu") else 16) * rnd.randint(1, 96)
        monkeypatch.setenv("PHYAI_FP8_FUSED", "1")
        desc = ops.describe_linear_plan(M, N, K, epi)
        if not desc.startswith("one launch"):
            continue
        ran += 1
        x = seeded((M, K), seed=it)
        if it % 5 == 0:
            x[M // 2] *= 1e-20
        if it % 7 == 0:
            x[0, K // 2] = 1000.0
        xd = x.to(dev)
        wq, ws = ops.fp8_weight_quant(seeded((N, K), seed=1000 + it, scale=0.02).to(dev))
        b = seeded((N,), seed=2000 + it, scale=0.01).to(dev) if it % 2 else None
        got = ops.fp8_linear(xd, wq, ws, b, epilogue=epi, stream_weights=it % 3 == 0)
        monkeypatch.setenv("PHYAI_FP8_FUSED", "0")
        want = ops.fp8_linear(xd, wq, ws, b, epilogue=epi)
        torch.cuda.synchronize()
        assert _same(got, want), f"case {it}: {M}x{N}x{K} {epi} ({desc}): {int((_bits(got) != _bits(want)).sum())} outputs differ"
    assert ran >= 100
