"""phyai_fp8_mlp: the two projections of an MLP as one call (reference DenseMLP.forward,
layers/mlp/dense_mlp.py:256-265), with the first kernel's output row maxima handed to the second.

The hand-over changes where the row maximum of the intermediate tensor is found (in the producer's
epilogue instead of a pass over the rows; reference quantizer layers/quant/fp8.py:150-155), not its
value: the result must be the bits of phyai_fp8_linear (activation epilogue) followed by
phyai_fp8_linear on its output, which are pinned against the oracle elsewhere.
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


def _mlp_problem(dev, M, H, I, O, epi, seed, bias):
    ops = _ops()
    n1 = 2 * I if epi in GATED else I
    x = seeded((M, H), seed=seed)
    w1 = seeded((n1, H), seed=seed + 1, scale=0.05).to(dev)
    w2 = seeded((O, I), seed=seed + 2, scale=0.05).to(dev)
    q1, s1 = ops.fp8_weight_quant(w1)
    q2, s2 = ops.fp8_weight_quant(w2)
    b1 = seeded((n1,), seed=seed + 3, scale=0.05).to(dev) if bias else None
    b2 = seeded((O,), seed=seed + 4, scale=0.05).to(dev) if bias else None
    return x.to(dev), q1, s1, b1, q2, s2, b2


def _two_linears(x, q1, s1, b1, q2, s2, b2, epi, **kw):
    ops = _ops()
    h = ops.fp8_linear(x, q1, s1, b1, epilogue=epi)
    return h, ops.fp8_linear(h, q2, s2, b2, **kw)


# (M, H, I, O, epilogue): the expert MLP, small and ragged shapes, plain GELU, and shapes whose second
# projection cannot take the hand-over (K of the second > 4096, M > 128, K not a multiple of 128)
CASES = [
    (50, 1024, 4096, 1024, "geglu_tanh"), (50, 256, 512, 256, "geglu_tanh"), (1, 128, 256, 64, "swiglu"),
    (7, 512, 1024, 272, "geglu_erf"), (16, 1024, 2048, 1024, "gelu_tanh"), (33, 256, 1536, 528, "gelu"),
    (64, 2048, 4096, 2048, "geglu_tanh"), (100, 1024, 4096, 1024, "geglu_tanh"), (128, 512, 2048, 512, "swiglu"),
    (50, 1024, 8192, 1024, "geglu_tanh"), (200, 1024, 4096, 1024, "geglu_tanh"), (50, 256, 528, 256, "gelu_tanh"),
    (816, 512, 1024, 512, "geglu_tanh"),
]


@pytest.mark.parametrize("M,H,I,O,epi", CASES)
@pytest.mark.parametrize("bias", [False, True])
def test_mlp_equals_two_linears_bit_for_bit(dev, M, H, I, O, epi, bias):
    ops = _ops()
    x, q1, s1, b1, q2, s2, b2 = _mlp_problem(dev, M, H, I, O, epi, seed=M + H + I + O, bias=bias)
    _, want = _two_linears(x, q1, s1, b1, q2, s2, b2, epi)
    got = ops.fp8_mlp(x, q1, s1, b1, q2, s2, b2, epilogue=epi)
    torch.cuda.synchronize()
    assert torch.equal(_bits(got), _bits(want)), ops.describe_mlp_plan(M, H, I, O, epi)
    # a second call on the workspace as the first left it, and a smaller one behind it
    again = ops.fp8_mlp(x, q1, s1, b1, q2, s2, b2, epilogue=epi)
    assert torch.equal(_bits(again), _bits(want))
    if M > 3:
        part = ops.fp8_mlp(x[: M // 2], q1, s1, b1, q2, s2, b2, epilogue=epi)
        assert torch.equal(_bits(part), _bits(want[: M // 2]))


def test_the_expert_mlp_hands_its_row_maxima_over():
    ops = _ops()
    plan = ops.describe_mlp_plan(50, 1024, 4096, 1024, "geglu_tanh")
    assert plan.startswith("row maxima handed over: one launch:") and " | one launch:" in plan, plan
    assert not ops.describe_mlp_plan(816, 2048, 16384, 2048, "geglu_tanh").startswith("row maxima")
    assert not ops.describe_mlp_plan(50, 1024, 8192, 1024, "geglu_tanh").startswith("row maxima")


@pytest.mark.parametrize("M,H,I,O,epi", [(50, 1024, 4096, 1024, "geglu_tanh"), (20, 256, 512, 256, "swiglu"),
                                         (50, 512, 2048, 512, "gelu_tanh")])
def test_mlp_with_awkward_rows_residual_and_layouts(dev, M, H, I, O, epi):
    """Rows of zeros, an Inf and a NaN in the input (they reach the intermediate tensor as zeros / NaN rows and
    take the slow division), the gated residual behind the second projection, and every combination of weight
    layouts - all against the two linears on row-major weights."""
    ops = _ops()
    x, q1, s1, b1, q2, s2, b2 = _mlp_problem(dev, M, H, I, O, epi, seed=3 * M + H, bias=True)
    x = x.clone()
    x[0] = 0
    x[1, 3] = float("inf")
    x[2, 5] = float("nan")
    x[3] = x[3] * 1e-30
    x[4, 7] = 3000.0
    res = seeded((M, O), seed=5).to(dev)
    gate = seeded((1, O), seed=6, scale=0.5).to(dev)
    h, want = _two_linears(x, q1, s1, b1, q2, s2, b2, epi)
    _, want_res = _two_linears(x, q1, s1, b1, q2, s2, b2, epi, residual=res, gate=gate)
    assert not torch.isfinite(h.float()).all() and bool((h[0] == h[0]).all())
    o1 = ops.fp8_weight_to_operand_order(q1, gated=epi in GATED)
    o2 = ops.fp8_weight_to_operand_order(q2)
    lay1 = "operand_gated" if epi in GATED else "operand"
    for w1, l1 in ((q1, None), (o1, lay1)):
        for w2, l2 in ((q2, None), (o2, "operand")):
            got = ops.fp8_mlp(x, w1, s1, b1, w2, s2, b2, epilogue=epi, weight1_layout=l1, weight2_layout=l2)
            assert torch.equal(_bits(got), _bits(want)), (l1, l2)
            got = ops.fp8_mlp(x, w1, s1, b1, w2, s2, b2, epilogue=epi, weight1_layout=l1, weight2_layout=l2,
                              residual=res, gate=gate)
            assert torch.equal(_bits(got), _bits(want_res)), (l1, l2, "residual")


@pytest.mark.parametrize("plan", ["8,2", "8,4", "16,1", "16,2"])
@pytest.mark.parametrize("I", [512, 2048, 4096])
def test_every_shape_of_the_consumer_kernel(dev, monkeypatch, plan, I):
    """The second projection's kernel with handed-over maxima exists in four workgroup shapes and with one, two
    or four K steps per wavefront; each is forced in turn (the first projection keeps its automatic shape),
    with row-major weights (staged through LDS) and weights in operand order (straight into registers)."""
    ops = _ops()
    M, H, O = 50, 256, 256
    x, q1, s1, b1, q2, s2, b2 = _mlp_problem(dev, M, H, I, O, "geglu_tanh", seed=I + 11, bias=True)
    _, want = _two_linears(x, q1, s1, b1, q2, s2, b2, "geglu_tanh")
    o2 = ops.fp8_weight_to_operand_order(q2)
    monkeypatch.setenv("PHYAI_FP8_FUSED_PLAN_AMAX", plan)
    rows, nt = plan.split(",")
    told = ops.describe_mlp_plan(M, H, I, O, "geglu_tanh")
    if told.startswith("row maxima handed over"):   # (a shape whose staging does not fit the LDS falls back)
        assert f"| one launch: small-m rows={rows} nt={nt} " in told, told
    else:
        assert (plan, I) in (("16,2", 4096), ("8,4", 4096)), told
    for w2, l2 in ((q2, None), (o2, "operand")):
        got = ops.fp8_mlp(x, q1, s1, b1, w2, s2, b2, epilogue="geglu_tanh", weight2_layout=l2)
        assert torch.equal(_bits(got), _bits(want)), (plan, I, l2)


def test_mlp_in_a_graph_replays_like_eager(dev):
    from phyai_amd.runtime import HipGraph

    ops = _ops()
    M, H, I, O = 50, 1024, 4096, 1024
    x, q1, s1, b1, q2, s2, b2 = _mlp_problem(dev, M, H, I, O, "geglu_tanh", seed=77, bias=False)
    want = ops.fp8_mlp(x, q1, s1, b1, q2, s2, b2, epilogue="geglu_tanh")
    out = torch.empty_like(want)
    static_x = x.clone()

    def fn():
        ops.fp8_mlp(static_x, q1, s1, b1, q2, s2, b2, epilogue="geglu_tanh", out=out)

    g = HipGraph()
    g.capture(fn, {})
    for i in range(3):
        out.zero_()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(_bits(out), _bits(want)), f"replay {i}"
        # eager work between the replays, on another input
        ops.fp8_mlp(x * 0.5, q1, s1, b1, q2, s2, b2, epilogue="geglu_tanh")


def test_dense_mlp_uses_the_one_call_path(dev):
    from phyai_amd import linear as L
    from phyai_amd.mlp import DenseMLP
    from phyai_amd.quant import Fp8Spec

    L.init()
    H, I, M = 256, 512, 50
    wgu, wd = seeded((2 * I, H), 8, 0.05).to(dev), seeded((H, I), 9, 0.05).to(dev)
    x = seeded((M, H), 10).to(dev)
    res, gate = seeded((M, H), 11).to(dev), seeded((1, H), 12, 0.3).to(dev)
    outs = []
    for operand in (False, True):
        mlp = DenseMLP(H, I, activation="gelu_tanh", params_dtype=torch.bfloat16, spec_in=Fp8Spec(operand_order=operand),
                       spec_out=Fp8Spec(operand_order=operand))
        for lin, w in ((mlp.gate_up_proj, wgu), (mlp.down_proj, wd)):
            lin.spec.quantize_weight_(lin, w)
            lin.post_load()
        assert mlp._one_call(mlp.gate_up_proj, mlp.down_proj, x)
        h = mlp.gate_up_proj.forward_fused(x, "geglu_tanh")
        want = mlp.down_proj(h)[0]
        outs.append(mlp(x))
        assert torch.equal(_bits(outs[-1]), _bits(want))
        assert torch.equal(_bits(mlp(x, residual=res, gate=gate)), _bits(mlp.down_proj.forward_addcmul(h, res, gate)))
    assert torch.equal(_bits(outs[0]), _bits(outs[1]))
