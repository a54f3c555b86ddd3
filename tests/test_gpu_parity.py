"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle.

Quantizer codes and scales must be bit-exact.  GEMM outputs must satisfy
max|out - ref| <= 1e-2 * max|ref| and cosine >= 0.9999 against the fp32
dequantized matmul (the tolerance the benchmark definition states); cases whose
sums are exact in fp32 must be bit-exact.
"""

from __future__ import annotations

import numpy as np
import pytest
import torch

from conftest import seeded
from oracle import cport, ref

pytestmark = pytest.mark.gpu

TOL_MAXABS = 1e-2
TOL_COS = 0.9999


def _ops():
    from phyai_amd import ops
    return ops


def _bits(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.uint16).numpy()


def _codes(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


def assert_close_to_ref(out: torch.Tensor, ref_f32: torch.Tensor, what=""):
    o = out.detach().float().cpu().reshape(-1).double()
    r = ref_f32.detach().float().cpu().reshape(-1).double()
    assert torch.isfinite(o).all(), f"{what}: non-finite output"
    scale = r.abs().max().item()
    err = (o - r).abs().max().item()
    cos = (o @ r / (o.norm() * r.norm()).clamp_min(1e-30)).item() if scale > 0 else 1.0
    assert err <= TOL_MAXABS * scale + 1e-30, f"{what}: max abs err {err:.4g} > 1e-2*{scale:.4g}"
    assert cos >= TOL_COS, f"{what}: cosine {cos:.6f} < {TOL_COS}"


# ---------------------------------------------------------------------------
# device cast
# ---------------------------------------------------------------------------

def test_device_cast_matches_oracle_dense_sweep(dev):
    """Every fp32 pattern on a 2^-12-relative grid below 512 (both signs, several
    sub-grid tails incl. exact ties) through the device cast vs the C oracle."""
    ops = _ops()
    hi = (np.arange(0, 0x44000000 >> 12, dtype=np.uint32) << 12)
    for tail in (0, 1, 0x7FF, 0x800, 0x801, 0xFFF):
        for sgn in (0, 0x80000000):
            b = (hi | np.uint32(tail) | np.uint32(sgn)).astype(np.uint32)
            v = b.view(np.float32)
            want = cport.f32_to_e4m3(v)
            got = ops.debug_cast_e4m3(torch.from_numpy(v.copy()).to(dev)).cpu().numpy()
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, (
                f"tail={tail:#x} sign={sgn:#x}: {bad.size} mismatches, first at bits "
                f"{b[bad[0]]:#010x} ({v[bad[0]]!r}): device {got[bad[0]]:#04x} oracle {want[bad[0]]:#04x}")


def test_device_cast_special_values(dev):
    ops = _ops()
    v = np.array([0.0, -0.0, 448.0, -448.0, 463.9, 464.0, 465.0, 479.9, 480.0, 1e9, -1e9,
                  np.inf, -np.inf, 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -10, 2.0 ** -6, 1e-30], np.float32)
    want = cport.f32_to_e4m3(v)
    got = ops.debug_cast_e4m3(torch.from_numpy(v).to(dev)).cpu().numpy()
    assert (got == want).all(), list(zip(v.tolist(), got.tolist(), want.tolist()))
    nan = ops.debug_cast_e4m3(torch.tensor([float("nan")], device=dev)).cpu().numpy()
    assert (nan & 0x7F) == 0x7F


# ---------------------------------------------------------------------------
# quantizer
# ---------------------------------------------------------------------------

QUANT_SHAPES = [(1, 16), (3, 8), (8, 64), (50, 1024), (50, 2048), (50, 4096), (7, 520), (33, 1000),
                (5, 8192), (3, 16384), (2, 32768), (2, 40000), (816, 2048)]


@pytest.mark.parametrize("M,K", QUANT_SHAPES)
def test_quant_rowwise_bit_exact(dev, M, K):
    ops = _ops()
    x = seeded((M, K), seed=100 + M + K)
    q, s = ops.fp8_quant_rowwise(x.to(dev))
    wq, ws = cport.quant_rowwise(_bits(x))
    assert q.shape == (M, K) and s.shape == (M, 1) and s.dtype == torch.float32
    np.testing.assert_array_equal(s.cpu().numpy().reshape(-1).view(np.uint32), ws.view(np.uint32))
    np.testing.assert_array_equal(_codes(q), wq)
    tq, ts = ref.quant_rowwise(x)
    np.testing.assert_array_equal(_codes(q), _codes(tq))
    assert torch.equal(s.cpu(), ts)


def test_quant_rowwise_edge_rows(dev):
    """All-zero row, +-0, subnormal bf16, power-of-two amax, bf16 max, an outlier row."""
    ops = _ops()
    K = 256
    x = seeded((8, K), seed=7)
    x[0] = 0
    x[1] = 0; x[1, 0] = -0.0; x[1, 5] = 1e-38
    x[2] = torch.full((K,), 9.2e-41).bfloat16(); x[2, 3] = -9.2e-41
    x[3, 17] = 64.0; x[3] = x[3].clamp(-64, 64)
    x[4, 0] = torch.finfo(torch.bfloat16).max
    x[5, 100] = 2000.0
    x[6] = x[6] * 1e-20
    x[7] = -x[7].abs()
    q, s = ops.fp8_quant_rowwise(x.to(dev))
    wq, ws = cport.quant_rowwise(_bits(x))
    np.testing.assert_array_equal(s.cpu().numpy().reshape(-1).view(np.uint32), ws.view(np.uint32))
    np.testing.assert_array_equal(_codes(q), wq)
    tq, ts = ref.quant_rowwise(x)
    np.testing.assert_array_equal(_codes(q), _codes(tq))


def test_quant_rowwise_all_bf16_values(dev):
    """Every finite bf16 bit pattern as x, against a sweep of row maxima."""
    ops = _ops()
    allbits = np.arange(0, 1 << 16, dtype=np.uint16)
    finite = allbits[(allbits & 0x7F80) != 0x7F80]
    K = 65536
    rows = []
    for amax in (1.0, 3.140625, 448.0, 0.0078125, 1e-20, 3e38, 17.5, 2.0 ** -100):
        row = np.zeros(K, np.uint16)
        vals = torch.from_numpy(finite.copy()).view(torch.bfloat16).float()
        keep = finite[(vals.abs() <= amax).numpy()]
        row[: keep.size] = keep
        row[-1] = torch.tensor([amax]).bfloat16().view(torch.uint16).item()
        rows.append(row)
    xb = np.stack(rows)
    x = torch.from_numpy(xb).view(torch.bfloat16)
    q, s = ops.fp8_quant_rowwise(x.to(dev))
    wq, ws = cport.quant_rowwise(xb)
    np.testing.assert_array_equal(s.cpu().numpy().reshape(-1).view(np.uint32), ws.view(np.uint32))
    np.testing.assert_array_equal(_codes(q), wq)


def test_quant_rowwise_strided_and_batched(dev):
    ops = _ops()
    x = seeded((4, 6, 128), seed=3).to(dev)
    q, s = ops.fp8_quant_rowwise(x)
    assert q.shape == (4, 6, 128) and s.shape == (4, 6, 1)
    tq, ts = ref.quant_rowwise(x.cpu())
    np.testing.assert_array_equal(_codes(q), _codes(tq))
    big = seeded((10, 512), seed=4).to(dev)
    view = big[:, 128:384]
    q2, s2 = ops.fp8_quant_rowwise(view)
    tq2, ts2 = ref.quant_rowwise(view.cpu())
    np.testing.assert_array_equal(_codes(q2), _codes(tq2))
    assert torch.equal(s2.cpu(), ts2)


def test_quant_rowwise_empty(dev):
    ops = _ops()
    q, s = ops.fp8_quant_rowwise(torch.empty((0, 64), dtype=torch.bfloat16, device=dev))
    assert q.shape == (0, 64) and s.shape == (0, 1)


def test_quant_static_bit_exact(dev):
    ops = _ops()
    x = seeded((33, 256), seed=11, scale=3.0)
    for sc in (1.0, 0.01, 0.37):
        scale = torch.tensor([sc], dtype=torch.float32)
        q = ops.fp8_quant_static(x.to(dev), scale.to(dev))
        np.testing.assert_array_equal(_codes(q), _codes(ref.quant_static(x, scale)))
        np.testing.assert_array_equal(_codes(q), cport.quant_static(_bits(x), sc))


@pytest.mark.parametrize("N,K", [(64, 128), (256, 1024), (100, 72)])
def test_weight_quant_bit_exact(dev, N, K):
    ops = _ops()
    w = seeded((N, K), seed=N + K, scale=0.02)
    w[1] = 0
    q, s = ops.fp8_weight_quant(w.to(dev))
    wq, ws = cport.weight_quant(_bits(w))
    np.testing.assert_array_equal(s.cpu().numpy().view(np.uint32), ws.view(np.uint32))
    np.testing.assert_array_equal(_codes(q), wq)
    tq, ts = ref.weight_quant(w)
    np.testing.assert_array_equal(_codes(q), _codes(tq))
    assert torch.equal(s.cpu(), ts)


# ---------------------------------------------------------------------------
# GEMM
# ---------------------------------------------------------------------------

def _problem(M, N, K, seed, bias=True):
    x = seeded((M, K), seed=seed)
    w = seeded((N, K), seed=seed + 1, scale=0.02)
    b = seeded((N,), seed=seed + 2, scale=0.01) if bias else None
    wq, ws = ref.weight_quant(w)
    return x, wq, ws, b


def test_gemm_exact_integer_layout(dev):
    """Small-integer codes and power-of-two scales: every product and partial sum
    is exact in fp32, so any accumulation order gives the same bits.  A wrong
    lane/row mapping, a dropped K slab or a transposed operand changes the result."""
    ops = _ops()
    g = torch.Generator().manual_seed(5)
    for (M, N, K) in [(64, 64, 128), (50, 96, 256), (128, 256, 384), (200, 144, 1040), (33, 2560, 1024)]:
        xi = torch.randint(-4, 5, (M, K), generator=g).float()
        wi = torch.randint(-4, 5, (N, K), generator=g).float()
        xq = xi.to(torch.float8_e4m3fn)
        wq = wi.to(torch.float8_e4m3fn)
        xs = torch.full((M, 1), 0.5)
        ws = torch.full((N,), 0.25)
        want = ((xi @ wi.t()) * 0.125).bfloat16()
        got = ops.fp8_gemm(xq.to(dev), xs.to(dev), wq.to(dev), ws.to(dev))
        assert torch.equal(got.cpu(), want), f"{(M, N, K)}: {(got.cpu().float() - want.float()).abs().max()}"


def test_gemm_row_col_identity(dev):
    """x = one-hot rows, w = distinct per-row values: out[m, n] must be w[n, k(m)]."""
    ops = _ops()
    M, N, K = 64, 128, 128
    xq = torch.zeros(M, K)
    for m in range(M):
        xq[m, (m * 7) % K] = 1.0
    w = ((torch.arange(N)[:, None] * 3 + torch.arange(K)[None, :]) % 15 - 7).float()
    got = ops.fp8_gemm(xq.to(torch.float8_e4m3fn).to(dev), torch.ones(M, 1, device=dev),
                       w.to(torch.float8_e4m3fn).to(dev), torch.ones(N, device=dev))
    want = (xq @ w.t()).bfloat16()
    assert torch.equal(got.cpu(), want)


GEMM_SHAPES = [
    (50, 4096, 1024),    # config 1
    (50, 2560, 1024), (50, 1024, 2048), (50, 1024, 4096),   # expert qkv / o / down
    (1, 256, 1024), (7, 48, 80), (64, 64, 128), (65, 80, 144), (130, 272, 528),
    (816, 2048, 2048), (300, 1024, 4096),
]


@pytest.mark.parametrize("M,N,K", GEMM_SHAPES)
def test_linear_matches_oracle(dev, M, N, K):
    ops = _ops()
    x, wq, ws, b = _problem(M, N, K, seed=M + N + K)
    got = ops.fp8_linear(x.to(dev), wq.to(dev), ws.to(dev), b.to(dev))
    xq, xs = ref.quant_rowwise(x)
    want_f32 = ref.gemm_f32(xq, xs, wq, ws, b)
    assert got.shape == (M, N) and got.dtype == torch.bfloat16
    assert_close_to_ref(got, want_f32, f"linear {M}x{N}x{K}")
    # much tighter than the stated tolerance: bf16 rounding noise only
    rel = (got.cpu().float() - want_f32).norm() / want_f32.norm()
    assert rel < 4e-3, f"relative Frobenius error {rel:.3g}"


@pytest.mark.parametrize("M,N,K", [(50, 512, 256), (9, 64, 128)])
def test_linear_matches_c_oracle_small(dev, M, N, K):
    ops = _ops()
    x, wq, ws, b = _problem(M, N, K, seed=1)
    got = ops.fp8_linear(x.to(dev), wq.to(dev), ws.to(dev), b.to(dev))
    q, s = cport.quant_rowwise(_bits(x))
    _, f32 = cport.linear(q, s, _codes(wq), ws.numpy(), _bits(b), 0, want_f32=True)
    assert_close_to_ref(got, torch.from_numpy(f32), "c-oracle")


@pytest.mark.parametrize("epi_name,epi", [("geglu_tanh", 1), ("geglu_erf", 2), ("swiglu", 3),
                                          ("gelu_tanh", 4), ("gelu", 5)])
@pytest.mark.parametrize("M,N,K", [(50, 8192, 1024), (70, 192, 272), (816, 1024, 512)])
def test_linear_epilogues(dev, epi_name, epi, M, N, K):
    ops = _ops()
    x, wq, ws, b = _problem(M, N, K, seed=epi * 1000 + M)
    got = ops.fp8_linear(x.to(dev), wq.to(dev), ws.to(dev), b.to(dev), epilogue=epi_name)
    xq, xs = ref.quant_rowwise(x)
    y = ref.gemm_f32(xq, xs, wq, ws, b)
    want = ref.epilogue(y, epi).float()
    n_out = N // 2 if epi in ref.GATED else N
    assert got.shape == (M, n_out)
    assert_close_to_ref(got, want, f"{epi_name} {M}x{N}x{K}")


@pytest.mark.parametrize("epi_name,epi", [("gelu_tanh", 4), ("gelu", 5), ("geglu_tanh", 1), ("geglu_erf", 2), ("swiglu", 3)])
@pytest.mark.parametrize("M,force_big", [(64, ""), (256, "256"), (256, "128"), (200, "192")])
def test_epilogue_activation_values(dev, monkeypatch, epi_name, epi, M, force_big):
    """One-hot weights hand chosen values to the epilogue: every e4m3 value times a per-row power of
    two reaches the activation exactly, so the device activation is compared with torch's value by
    value (within one bf16 step of the rounded result; most must agree exactly)."""
    ops = _ops()
    if force_big:
        monkeypatch.setenv("PHYAI_FP8_BIG", force_big)
    K = 1024                                                       # also the number of pass-through columns
    codes = torch.arange(K, dtype=torch.int32) % 256
    codes[(codes & 0x7F) == 0x7F] = 0                              # no NaN codes
    xq = codes.to(torch.uint8).repeat(M, 1).view(torch.float8_e4m3fn)
    xs = torch.tensor([2.0 ** ((m % 13) - 9) for m in range(M)], dtype=torch.float32).reshape(M, 1)
    gated = epi in ref.GATED
    N = 2 * K if gated else K
    w = torch.zeros(N, K)
    w[torch.arange(K), torch.arange(K)] = 1.0                      # gate / plain rows: column n passes code n
    if gated:
        w[K + torch.arange(K), 0x38] = 1.0                         # up rows: the column that holds 1.0
    wq = w.to(torch.float8_e4m3fn)
    ws = torch.ones(N)
    got = ops.fp8_gemm(xq.to(dev), xs.to(dev), wq.to(dev), ws.to(dev), None, epilogue=epi_name).float().cpu()
    y = ref.gemm_f32(xq, xs, wq, ws)
    want = ref.epilogue(y, epi).float()
    assert got.shape == want.shape == (M, K)
    step = torch.maximum(want.abs(), torch.full_like(want, 2.0 ** -126)) * 2.0 ** -7    # one bf16 step
    # negative tail: 1 + tanh / 1 + erf cancel in the textbook form, leaving an error of about one
    # fp32 epsilon of the argument; the device form does not cancel
    slack = 3e-7 * y[:, :K].abs() * (y[:, K:].abs() if gated else 1.0)
    bad = (got - want).abs() > step + slack
    assert not bool(bad.any()), (f"{epi_name}: off by more than one bf16 step at pre-activation values "
                                 f"{y[:, :K][bad][:8].tolist()}: got {got[bad][:8].tolist()} want {want[bad][:8].tolist()}")
    # exact agreement is asked only where the textbook form is itself accurate (no cancellation)
    clean = y[:, :K] > -2.0
    agree = float((got == want)[clean].float().mean())
    assert agree > 0.995, f"{epi_name}: only {agree:.4f} of the rounded results agree"


def test_linear_no_bias_and_batched(dev):
    ops = _ops()
    x = seeded((2, 25, 1024), seed=9)
    w = seeded((2560, 1024), seed=10, scale=0.02)
    wq, ws = ref.weight_quant(w)
    got = ops.fp8_linear(x.to(dev), wq.to(dev), ws.to(dev))
    assert got.shape == (2, 25, 2560)
    xq, xs = ref.quant_rowwise(x)
    assert_close_to_ref(got, ref.gemm_f32(xq, xs, wq, ws), "batched")


def test_linear_zero_weight_gives_bias(dev):
    """The reference's own exact case (tests/layers/linear/test_kernel_torch.py:199-215)."""
    ops = _ops()
    N, K = 32, 64
    wq = torch.zeros(N, K, dtype=torch.float8_e4m3fn, device=dev)
    ws = torch.ones(N, device=dev)
    bias = torch.ones(N, dtype=torch.bfloat16, device=dev)
    x = torch.zeros(4, K, dtype=torch.bfloat16, device=dev)
    y = ops.fp8_linear(x, wq, ws, bias)
    assert torch.equal(y, bias.expand(4, N))


def test_gemm_scalar_x_scale(dev):
    ops = _ops()
    x, wq, ws, b = _problem(40, 128, 256, seed=21)
    scale = torch.tensor([0.05])
    xq = ref.quant_static(x, scale)
    got = ops.fp8_gemm(xq.to(dev), scale.to(dev), wq.to(dev), ws.to(dev), b.to(dev))
    want = ref.gemm_f32(xq, scale.expand(40, 1), wq, ws, b)
    assert_close_to_ref(got, want, "per-tensor")


def test_linear_repeatable_and_workspace_stays_clean(dev):
    """Split-K path: same bits on every call (fixed reduction order) and the
    counters in the workspace header return to zero."""
    ops = _ops()
    x, wq, ws, b = _problem(50, 1024, 4096, seed=33)
    xd, wd, sd, bd = x.to(dev), wq.to(dev), ws.to(dev), b.to(dev)
    first = ops.fp8_linear(xd, wd, sd, bd).clone()
    for _ in range(5):
        assert torch.equal(ops.fp8_linear(xd, wd, sd, bd), first)
    torch.cuda.synchronize()
    for w in ops._workspaces.values():
        assert int(w[: ops.WORKSPACE_HEADER_BYTES].max().item()) == 0


# ---------------------------------------------------------------------------
# Pipelined tile kernel (large M), every variant forced on shapes small enough for the oracle
# ---------------------------------------------------------------------------

def _force_big(monkeypatch, spec):
    """spec = "rows" or "rows/ring depth": 256 (x 256 columns), 224 (x 256), 192 (x 128), 128 (x 128, ring of 4 or 2),
    12864 (128 x 64) and 96 (96 x 128): plain epilogues only, a gated one keeps the default choice."""
    tile, _, depth = spec.partition("/")
    monkeypatch.setenv("PHYAI_FP8_BIG", tile)
    if depth:
        monkeypatch.setenv("PHYAI_FP8_BIG_DEPTH", depth)


@pytest.mark.parametrize("M,N,K,epi_name,epi", [
    (256, 256, 1024, None, 0), (300, 512, 1280, None, 0), (816, 768, 1024, None, 0), (513, 400, 1536, "gelu", 5),
    (816, 1024, 1152, "geglu_tanh", 1), (260, 288, 1024, "swiglu", 3), (1000, 256, 2048, None, 0),
])
@pytest.mark.parametrize("tile", ["256", "224", "192", "128", "128/2", "12864", "96"])
def test_big_tile_kernel_forced(dev, monkeypatch, tile, M, N, K, epi_name, epi):
    ops = _ops()
    _force_big(monkeypatch, tile)
    x, wq, ws, b = _problem(M, N, K, seed=7 * M + N + K)
    got = ops.fp8_linear(x.to(dev), wq.to(dev), ws.to(dev), b.to(dev), epilogue=epi_name)
    torch.cuda.synchronize()
    xq, xs = ref.quant_rowwise(x)
    want = ref.epilogue(ref.gemm_f32(xq, xs, wq, ws, b), epi).float()
    assert_close_to_ref(got, want, f"big kernel {M}x{N}x{K} epi={epi_name}")


@pytest.mark.parametrize("tile", ["256", "224", "192", "128", "128/2", "12864", "96"])
def test_big_tile_kernel_exact_integer(dev, monkeypatch, tile):
    ops = _ops()
    _force_big(monkeypatch, tile)
    g = torch.Generator().manual_seed(11)
    for (M, N, K) in [(256, 256, 1024), (700, 528, 1280), (257, 784, 1152)]:
        xi = torch.randint(-4, 5, (M, K), generator=g).float()
        wi = torch.randint(-4, 5, (N, K), generator=g).float()
        got = ops.fp8_gemm(xi.to(torch.float8_e4m3fn).to(dev), torch.full((M, 1), 0.5, device=dev),
                           wi.to(torch.float8_e4m3fn).to(dev), torch.full((N,), 0.25, device=dev))
        want = ((xi @ wi.t()) * 0.125).bfloat16()
        assert torch.equal(got.cpu(), want), f"{(M, N, K)}"


def test_tile_variants_agree_bit_for_bit_on_random_shapes(dev, monkeypatch):
    """Every variant of the pipelined tile kernel, and the generic tile kernel, walks K in the same
    order with the same MFMA, so without split-K their outputs must be identical bit for bit
    whatever the tile shape: 30 seeded shapes with ragged M, N off the tile grid, K down to the
    smallest the ring accepts, all epilogues; one variant is also held to the oracle tolerance."""
    ops = _ops()
    rng = np.random.default_rng(20240607)
    epis = [(None, 0), ("geglu_tanh", 1), ("geglu_erf", 2), ("swiglu", 3), ("gelu_tanh", 4), ("gelu", 5)]
    for case in range(30):
        M = int(rng.integers(65, 700))
        N = 32 * int(rng.integers(1, 40))
        K = 128 * int(rng.integers(4, 14))
        epi_name, epi = epis[case % len(epis)]
        x, wq, ws, b = _problem(M, N, K, seed=1000 + case)
        xq, xs = ops.fp8_quant_rowwise(x.to(dev))
        wd, sd, bd = wq.to(dev), ws.to(dev), b.to(dev)
        outs = {}
        for spec in ("256", "224", "192", "128", "128/2", "12864", "96", "256/rows", "224/rows", "128/rows", "12864/rows", "96/rows", "generic"):
            monkeypatch.delenv("PHYAI_FP8_BIG", raising=False)
            monkeypatch.delenv("PHYAI_FP8_BIG_DEPTH", raising=False)
            monkeypatch.delenv("PHYAI_FP8_TILE", raising=False)
            monkeypatch.delenv("PHYAI_FP8_BY_ROWS", raising=False)
            if spec == "generic":
                monkeypatch.setenv("PHYAI_FP8_TILE", "128,128,1")     # generic kernel, no split-K
            elif spec.endswith("/rows"):                               # the tile order that gives an XCD tile rows
                _force_big(monkeypatch, spec.split("/")[0])
                monkeypatch.setenv("PHYAI_FP8_BY_ROWS", "1")
            else:
                _force_big(monkeypatch, spec)
                monkeypatch.setenv("PHYAI_FP8_BY_ROWS", "0")
            outs[spec] = ops.fp8_gemm(xq, xs, wd, sd, bd, epilogue=epi_name)
        torch.cuda.synchronize()
        monkeypatch.delenv("PHYAI_FP8_BY_ROWS", raising=False)
        for spec, o in outs.items():
            assert torch.equal(_as_bits(o), _as_bits(outs["256"])), \
                f"case {case} {(M, N, K, epi_name)}: {spec} differs from 256 in {int((_as_bits(o) != _as_bits(outs['256'])).sum())} outputs"
        want = ref.epilogue(ref.gemm_f32(*ref.quant_rowwise(x), wq, ws, b), epi).float()
        assert_close_to_ref(outs["192"], want, f"case {case} {(M, N, K, epi_name)}")


@pytest.mark.parametrize("M,N,K,epi_name", [
    (50, 2560, 1024, None), (50, 8192, 1024, "geglu_tanh"), (50, 1024, 4096, None), (1, 12288, 2048, None),
    (64, 4096, 1024, "gelu_tanh"), (33, 1024, 16384, None), (200, 1024, 4096, None), (816, 2048, 2048, None),
])
def test_streamed_weights_give_the_same_bits(dev, M, N, K, epi_name):
    """Weights read with non-temporal loads (the flag that keeps a matrix out of the Infinity
    Cache) change where the bytes are cached, never the result - in the kernel that honours the
    flag (small M, also over several rounds of K steps) and in those that ignore it."""
    ops = _ops()
    x, wq, ws, b = _problem(M, N, K, seed=11 * M + N + K)
    xd, wd, sd, bd = x.to(dev), wq.to(dev), ws.to(dev), b.to(dev)
    xq, xs = ops.fp8_quant_rowwise(xd)
    plain = ops.fp8_linear(xd, wd, sd, bd, epilogue=epi_name)
    streamed = ops.fp8_linear(xd, wd, sd, bd, epilogue=epi_name, stream_weights=True)
    streamed_gemm = ops.fp8_gemm(xq, xs, wd, sd, bd, epilogue=epi_name, stream_weights=True)
    torch.cuda.synchronize()
    assert torch.equal(_as_bits(streamed), _as_bits(plain))
    assert torch.equal(_as_bits(streamed_gemm), _as_bits(plain))


def test_weight_streaming_kernel_workgroup_shapes_agree_bit_for_bit(dev, monkeypatch):
    """The weight-streaming kernel above 64 token rows, in each of its workgroup shapes
    (1-2 weight tiles x 1-4 blocks of 16 token rows, 4 tiles x 3-4 blocks) and as the dispatcher picks it: a wavefront
    always walks its K steps in the same order and the eight partial sums are added in wavefront
    order, so the shape must not change a single bit.  Ragged M (last workgroup partly or wholly
    past M), N off the tile width, all epilogues, gated residual; one shape is held to the oracle."""
    ops = _ops()
    rng = np.random.default_rng(77)
    epis = [(None, 0), ("geglu_tanh", 1), ("gelu", 5), ("swiglu", 3)]
    monkeypatch.setenv("PHYAI_FP8_BIG", "0")              # keep the tile kernels out of the way
    monkeypatch.setenv("PHYAI_FP8_SKINNY_MAXM", "2048")
    for case in range(12):
        M = int(rng.integers(65, 900))
        N = 32 * int(rng.integers(1, 48))
        K = 128 * int(rng.integers(1, 34))
        epi_name, epi = epis[case % len(epis)]
        x, wq, ws, b = _problem(M, N, K, seed=3000 + case)
        xq, xs = ops.fp8_quant_rowwise(x.to(dev))
        wd, sd, bd = wq.to(dev), ws.to(dev), b.to(dev)
        res = gate = None
        if epi == 0 and case % 8 == 0:
            res = seeded((M, N), seed=4000 + case).to(dev)
            gate = seeded((1, N), seed=5000 + case).to(dev)
        outs = {}
        for plan in [None] + [f"{nt},{mb}" for nt in (1, 2) for mb in (1, 2, 3, 4)] + ["4,3", "4,4"]:
            if plan is None:
                monkeypatch.delenv("PHYAI_FP8_SKINNY_PLAN", raising=False)
            else:
                monkeypatch.setenv("PHYAI_FP8_SKINNY_PLAN", plan)
            assert ops.describe_plan(M, N, K, epi_name).startswith("small-m ")
            outs[plan] = ops.fp8_gemm(xq, xs, wd, sd, bd, epilogue=epi_name, residual=res, gate=gate)
        torch.cuda.synchronize()
        for plan, o in outs.items():
            assert torch.equal(_as_bits(o), _as_bits(outs[None])), \
                f"case {case} {(M, N, K, epi_name)}: shape {plan} differs in {int((_as_bits(o) != _as_bits(outs[None])).sum())} outputs"
        if res is None:
            want = ref.epilogue(ref.gemm_f32(*ref.quant_rowwise(x), wq, ws, b), epi).float()
            assert_close_to_ref(outs[None], want, f"case {case} {(M, N, K, epi_name)}")


@pytest.mark.parametrize("tile", ["128"])
def test_big_tile_kernel_split_k(dev, monkeypatch, tile):
    """The K range split over two and four workgroups (partials in the workspace)."""
    ops = _ops()
    monkeypatch.setenv("PHYAI_FP8_BIG", tile)
    x, wq, ws, b = _problem(300, 384, 4096, seed=77)
    xq, xs = ref.quant_rowwise(x)
    want = ref.gemm_f32(xq, xs, wq, ws, b)
    outs = []
    for splits in ("1", "2", "4"):
        monkeypatch.setenv("PHYAI_FP8_BIG_SPLITS", splits)
        got = ops.fp8_linear(x.to(dev), wq.to(dev), ws.to(dev), b.to(dev))
        torch.cuda.synchronize()
        assert_close_to_ref(got, want, f"split-K {splits}")
        again = ops.fp8_linear(x.to(dev), wq.to(dev), ws.to(dev), b.to(dev))
        assert torch.equal(got, again), "split-K result must not depend on arrival order"
        outs.append(got)
    for w in ops._workspaces.values():
        assert int(w[: ops.WORKSPACE_HEADER_BYTES].max().item()) == 0


@pytest.mark.parametrize("M,N,K,epi_name", [
    (50, 1024, 2048, None), (50, 1024, 4096, None), (16, 1024, 1024, None), (64, 512, 2048, None),
    (33, 1024, 4096, "gelu_tanh"), (50, 2048, 2048, "geglu_tanh"), (7, 256, 1024, "swiglu"), (48, 768, 4096, None),
])
def test_linear_equals_quantizer_then_gemm_bit_for_bit(dev, M, N, K, epi_name):
    """The linear entry point (bf16 in) against the GEMM entry point fed by the stand-alone quantizer
    (whose codes and scales are pinned bit-exactly elsewhere): the outputs must be equal bit for
    bit, whatever staging the library uses between its quantizer and its GEMM.  Rows with zeros
    only, a signed zero, an outlier, tiny values, the largest finite bf16 and an Inf are
    included, and the activations are also passed as a strided view."""
    ops = _ops()
    x, wq, ws, b = _problem(M, N, K, seed=3 * M + N + K)
    x = x.clone()
    x[0] = 0
    x[1, ::2] = -0.0
    x[2, 5] = 300.0
    x[3] = x[3] * 1e-30
    if M > 5:
        x[4, 7] = torch.finfo(torch.bfloat16).max
        x[5, 3] = float("inf")
    wide = torch.zeros(M, K + 64, dtype=torch.bfloat16)
    wide[:, :K] = x
    xd = wide.to(dev)[:, :K]                                   # row stride K + 64
    assert not xd.is_contiguous()
    wd, sd, bd = wq.to(dev), ws.to(dev), b.to(dev)
    xq, xs = ops.fp8_quant_rowwise(x.to(dev))
    want = ops.fp8_gemm(xq, xs, wd, sd, bd, epilogue=epi_name)
    for xin in (x.to(dev), xd):
        got = ops.fp8_linear(xin, wd, sd, bd, epilogue=epi_name)
        torch.cuda.synchronize()
        assert torch.equal(_as_bits(got), _as_bits(want)), f"{(M, N, K, epi_name)}: {int((_as_bits(got) != _as_bits(want)).sum())} outputs differ"
    if epi_name is None:
        res = seeded((M, N), seed=8)
        gate = seeded((1, N), seed=9, scale=0.5)
        want = ops.fp8_gemm(xq, xs, wd, sd, bd, residual=res.to(dev), gate=gate.to(dev))
        got = ops.fp8_linear(xd, wd, sd, bd, residual=res.to(dev), gate=gate.to(dev))
        assert torch.equal(_as_bits(got), _as_bits(want))


def _as_bits(t):
    return t.contiguous().view(torch.int16)


@pytest.mark.parametrize("force,shape", [(("PHYAI_FP8_BIG", "128"), (300, 384, 4096)), (("PHYAI_FP8_BIG", "128"), (816, 2048, 8192)),
                                         (("PHYAI_FP8_TILE", "128,128,4"), (200, 512, 1040))])
def test_split_k_many_runs_one_result(dev, monkeypatch, force, shape):
    """The split-K hand-over (write-through partial sums, own-store wait, barrier, arrival counter,
    write-through reads) orders nothing on paper; it rests on how gfx950 executes those accesses.
    200 back-to-back launches, no synchronisation in between, against the first result: stops at the
    first mismatch."""
    ops = _ops()
    monkeypatch.setenv(*force)
    if force[0] == "PHYAI_FP8_BIG":
        monkeypatch.setenv("PHYAI_FP8_BIG_SPLITS", "4")
    M, N, K = shape
    x, wq, ws, b = _problem(M, N, K, seed=1234)
    xd, wd, sd, bd = x.to(dev), wq.to(dev), ws.to(dev), b.to(dev)
    xq, xs = ops.fp8_quant_rowwise(xd)
    first = ops.fp8_gemm(xq, xs, wd, sd, bd)
    assert_close_to_ref(first, ref.gemm_f32(*ref.quant_rowwise(x), wq, ws, b), "split-K")
    outs = [ops.fp8_gemm(xq, xs, wd, sd, bd) for _ in range(200)]
    torch.cuda.synchronize()
    for i, o in enumerate(outs):
        assert torch.equal(_as_bits(o), _as_bits(first)), f"launch {i} differs from the first"


@pytest.mark.parametrize("M,N,K,tile,splits", [(816, 2048, 16384, "", ""), (816, 2048, 8192, "128", "2"), (300, 1024, 4096, "128", "4"),
                                               (300, 2048, 4096, "128", "8"), (520, 2048, 4096, "128", "2"), (300, 768, 4096, "128", "4")])
def test_split_k_with_an_xcd_per_k_range_gives_the_same_bits(dev, monkeypatch, M, N, K, tile, splits):
    """Split-K launches can hand every XCD one K range (its L2 then fetches that range of the activation
    codes once) instead of whole tile columns; the tiles, the K ranges and the order in which the partial
    sums are added are the same, so the output must be equal bit for bit.  Includes a tile-column count
    that does not divide among the groups (768 / 128 = 6 columns in 2 groups of 4 K ranges: padding ids)."""
    ops = _ops()
    if tile:
        monkeypatch.setenv("PHYAI_FP8_BIG", tile)
        monkeypatch.setenv("PHYAI_FP8_BIG_SPLITS", splits)
    x, wq, ws, b = _problem(M, N, K, seed=M + N)
    xq, xs = ops.fp8_quant_rowwise(x.to(dev))
    wd, sd, bd = wq.to(dev), ws.to(dev), b.to(dev)
    assert "splits=" in ops.describe_plan(M, N, K) and "splits=1" not in ops.describe_plan(M, N, K)
    outs = {}
    for order in ("0", "1"):
        monkeypatch.setenv("PHYAI_FP8_XCD_SPLIT", order)
        outs[order] = ops.fp8_gemm(xq, xs, wd, sd, bd)
        again = ops.fp8_gemm(xq, xs, wd, sd, bd)
        torch.cuda.synchronize()
        assert torch.equal(_as_bits(outs[order]), _as_bits(again))
    assert torch.equal(_as_bits(outs["0"]), _as_bits(outs["1"]))
    monkeypatch.delenv("PHYAI_FP8_XCD_SPLIT")
    assert torch.equal(_as_bits(ops.fp8_gemm(xq, xs, wd, sd, bd)), _as_bits(outs["0"]))   # the automatic choice
    assert_close_to_ref(outs["1"], ref.gemm_f32(*ref.quant_rowwise(x), wq, ws, b), "split-K, an XCD per K range")
    for w in ops._workspaces.values():
        assert int(w[: ops.WORKSPACE_HEADER_BYTES].max().item()) == 0


def test_two_streams_run_split_k_linears_concurrently(dev, monkeypatch):
    """Each (device, stream) pair has its own workspace (split-K counters and partials, code
    staging), so linears issued on two streams at once must give the serial results bit for bit."""
    ops = _ops()
    monkeypatch.setenv("PHYAI_FP8_BIG", "128")
    monkeypatch.setenv("PHYAI_FP8_BIG_SPLITS", "4")
    probs = []
    for i in range(2):
        x, wq, ws, b = _problem(300 + 20 * i, 384, 4096, seed=900 + i)
        probs.append((x.to(dev), wq.to(dev), ws.to(dev), b.to(dev)))
    serial = [ops.fp8_linear(*p) for p in probs]
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[], []]
    for rep in range(8):
        for i, st in enumerate(streams):
            st.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(st):
                outs[i].append(ops.fp8_linear(*probs[i]))
    torch.cuda.synchronize()
    for i in range(2):
        for o in outs[i]:
            assert torch.equal(_as_bits(o), _as_bits(serial[i]))
    keys = {k for k in ops._workspaces}
    assert len({s.cuda_stream for s in streams} & {k[1] for k in keys}) == 2, "one workspace per stream"


def test_quant_rowwise_exhaustive_all_values_all_scales(dev):
    """Every finite bf16 value against every possible row maximum (32 640 of them, hence every
    possible scale): 2.1e9 quotients.  The expected codes are the reference's own expression
    evaluated with torch on the device (IEEE fp32 division, torch's e4m3fn cast), which the
    sampled tests above tie to the CPU oracle."""
    ops = _ops()
    allbits = torch.arange(0, 1 << 16, dtype=torch.int32, device=dev)
    finite = allbits[(allbits & 0x7F80) != 0x7F80].to(torch.uint16)
    vals = finite.view(torch.bfloat16)                       # 65 280 finite values
    absbits = (finite.to(torch.int32) & 0x7FFF)
    amax_bits = torch.arange(0, 0x7F80, dtype=torch.int32, device=dev)     # every non-negative finite bf16
    K = 65536
    chunk = 128
    for start in range(0, amax_bits.numel(), chunk):
        a = amax_bits[start:start + chunk]
        x = torch.zeros((a.numel(), K), dtype=torch.bfloat16, device=dev)
        keep = absbits[None, :] <= a[:, None]                 # values not larger than this row's maximum
        x[:, : vals.numel()] = torch.where(keep, vals[None, :], torch.zeros((), dtype=torch.bfloat16, device=dev))
        x[:, -1] = a.to(torch.uint16).view(torch.bfloat16)    # make sure the maximum itself is present
        q, s = ops.fp8_quant_rowwise(x)
        wq, ws = ref.quant_rowwise(x)                         # torch ops on the device
        assert torch.equal(s, ws), f"scales differ for amax bits {start}..{start + chunk}"
        same = q.view(torch.uint8) == wq.view(torch.uint8)
        if not bool(same.all()):
            r, c = torch.nonzero(~same)[0].tolist()
            raise AssertionError(
                f"amax bits {int(a[r]):#06x}, x bits {int(x[r, c].view(torch.uint16)):#06x}: "
                f"got {int(q.view(torch.uint8)[r, c]):#04x} want {int(wq.view(torch.uint8)[r, c]):#04x}")


@pytest.mark.parametrize("M,N,K,force,gate_rows", [
    (50, 1024, 2048, "", 1), (50, 1024, 4096, "", 50), (200, 1024, 4096, "", 4), (70, 192, 272, "", 70),
    (816, 2048, 2048, "128", 816), (816, 2048, 2048, "256", 1), (300, 384, 4096, "128", 3), (9, 64, 128, "", 9),
    (816, 2048, 2048, "192", 816), (500, 640, 1024, "192", 5), (816, 2048, 2048, "224", 816), (500, 640, 1024, "224", 4), (816, 2048, 2048, "12864", 816), (500, 640, 1024, "12864", 1),
    (816, 2560, 2048, "", 816), (500, 640, 1024, "96", 1)])
def test_linear_gated_residual(dev, monkeypatch, M, N, K, force, gate_rows):
    """out = addcmul(residual, linear(x), gate) inside the GEMM epilogue, every kernel family; the result
    must equal torch.addcmul applied to the device's own plain linear output bit for bit."""
    ops = _ops()
    if force:
        monkeypatch.setenv("PHYAI_FP8_BIG", force)
    x, wq, ws, b = _problem(M, N, K, seed=M + N)
    res = seeded((M, N), seed=5)
    gate = seeded((gate_rows, N), seed=6, scale=0.5)
    xd, wd, sd, bd = x.to(dev), wq.to(dev), ws.to(dev), b.to(dev)
    y = ops.fp8_linear(xd, wd, sd, bd)
    got = ops.fp8_linear(xd, wd, sd, bd, residual=res.to(dev), gate=gate.to(dev))
    want = ref.addcmul(res, y.cpu(), gate)
    assert torch.equal(got.cpu(), want)
    # and through the quantized-input entry point, writing over the residual
    xq, xs = ops.fp8_quant_rowwise(xd)
    buf = res.to(dev).clone()
    ops.fp8_gemm(xq, xs, wd, sd, bd, residual=buf, gate=gate.to(dev), out=buf)
    assert torch.equal(buf.cpu(), want)
    # against the oracle's own linear, to the stated tolerance
    xq_c, xs_c = ref.quant_rowwise(x)
    y_ref = ref.gemm_f32(xq_c, xs_c, wq, ws, b)
    g_full = gate.repeat_interleave(M // gate_rows, dim=0).float()
    assert_close_to_ref(got, res.float() + y_ref.to(torch.bfloat16).float() * g_full, "gated residual")


def test_gated_residual_argument_errors(dev):
    ops = _ops()
    x, wq, ws, b = _problem(16, 64, 128, seed=1)
    xd, wd, sd = x.to(dev), wq.to(dev), ws.to(dev)
    r = torch.zeros(16, 64, dtype=torch.bfloat16, device=dev)
    with pytest.raises(RuntimeError, match="go together"):
        ops.fp8_linear(xd, wd, sd, None, residual=r)
    with pytest.raises(RuntimeError, match="excludes an activation"):
        ops.fp8_linear(xd, wd, sd, None, epilogue="gelu", residual=r, gate=r)
    with pytest.raises(RuntimeError, match="multiple of gate rows"):
        ops.fp8_linear(xd, wd, sd, None, residual=r, gate=r[:5])
    with pytest.raises(RuntimeError, match="residual must have shape"):
        ops.fp8_linear(xd, wd, sd, None, residual=r[:8], gate=r[:8])


# ---- against the reference's own GPU arithmetic (torch ops + torch._scaled_mm on this device) ----

def _torch_quantize_activation(x: torch.Tensor):
    """The three lines of Fp8Spec.quantize_activation (reference layers/quant/fp8.py:152-154), on the GPU."""
    a = x.abs().amax(dim=-1, keepdim=True).clamp_min(1e-12)
    s = (a / 448.0).to(torch.float32)
    return (x / s).to(torch.float8_e4m3fn), s


@pytest.mark.parametrize("shape", [(50, 1024), (816, 2048), (7, 4096), (300, 16384)])
def test_quantizer_bit_exact_with_reference_expressions_on_device(dev, shape):
    ops = _ops()
    x = seeded(shape, seed=shape[0], scale=1.5).to(dev)
    x[0, :16] = 0.0
    x[1 % shape[0], 3] = 300.0                                          # an outlier channel
    q_ref, s_ref = _torch_quantize_activation(x)
    q, s = ops.fp8_quant_rowwise(x)
    assert torch.equal(s, s_ref)
    assert torch.equal(q.view(torch.uint8), q_ref.view(torch.uint8))


@pytest.mark.parametrize("M,N,K,force", [(50, 2560, 1024, ""), (50, 1024, 4096, ""), (200, 1024, 2048, ""),
                                         (816, 2560, 2048, ""), (816, 2048, 16384, ""), (816, 4096, 2048, "256"),
                                         (816, 4096, 2048, "192"), (70, 192, 272, "")])
def test_gemm_against_torch_scaled_mm(dev, monkeypatch, M, N, K, force):
    """torch._scaled_mm with row-wise scales is the GEMM the reference calls
    (layers/linear/backends/torch.py:166-175).  Same codes, same scales, same bias on this GPU: the
    outputs must agree to the stated tolerance, and nearly all of them bit for bit."""
    ops = _ops()
    if force:
        monkeypatch.setenv("PHYAI_FP8_BIG", force)
    x, wq, ws, b = _problem(M, N, K, seed=M * 7 + N)
    xd, wd, sd, bd = x.to(dev), wq.to(dev), ws.to(dev), b.to(dev)
    xq, xs = ops.fp8_quant_rowwise(xd)
    try:
        want = torch._scaled_mm(xq, wd.t(), scale_a=xs, scale_b=sd.reshape(1, -1), bias=bd, out_dtype=torch.bfloat16)
        torch.cuda.synchronize()
    except Exception as e:  # noqa: BLE001
        pytest.skip(f"torch._scaled_mm does not run on this image: {str(e)[:100]}")
    got = ops.fp8_gemm(xq, xs, wd, sd, bd)
    assert_close_to_ref(got, want.float().cpu(), f"vs torch._scaled_mm {M}x{N}x{K}")
    step = want.float().abs().clamp_min(2.0 ** -126) * 2.0 ** -7
    assert bool(((got.float() - want.float()).abs() <= step).all()), "more than one bf16 step from torch._scaled_mm"
    assert float((got == want).float().mean()) > 0.97


def test_mfma_rate_probe_reports_a_plausible_machine(dev):
    """The hardware probe behind bench.py's measured MFMA peak: 64 cycles per 32 x 32 x 64 fp8 MFMA,
    a clock between 1 and 3 GHz, and a chip-wide rate that follows from the two."""
    ops = _ops()
    r = ops.mfma_rate_probe(workgroups=512, iters=400)
    assert 60.0 <= r["cycles_per_mfma"] <= 80.0, r
    assert 1.0 <= r["clock_GHz"] <= 3.0, r
    assert 1000.0 <= r["TFLOPs"] <= 6000.0, r
