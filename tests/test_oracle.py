"""Pins for the CPU oracle (no GPU needed).

Each test checks an oracle function against something that does not share its
code: the OCP closed form, torch's own casts, exact-integer arithmetic, textbook
activation routines, invariants of the quantizer, or the committed fixtures.
"""

from __future__ import annotations

import math
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as F

from conftest import seeded
from oracle import cport, ref

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp8_linear_golden.npz")


def bits(t):
    return t.contiguous().view(torch.uint16).numpy()


def codes(t):
    return t.contiguous().view(torch.uint8).numpy()


# ---------------------------------------------------------------------------
# e4m3fn
# ---------------------------------------------------------------------------

def ocp_value(c: int) -> float:
    s, e, m = c >> 7, (c >> 3) & 0xF, c & 7
    if e == 0xF and m == 7:
        return math.nan
    v = m * 2.0 ** -9 if e == 0 else (1 + m / 8) * 2.0 ** (e - 7)
    return -v if s else v


def test_e4m3_decode_all_codes_closed_form():
    got = cport.e4m3_to_f32(np.arange(256, dtype=np.uint8))
    for c in range(256):
        want = ocp_value(c)
        if math.isnan(want):
            assert math.isnan(got[c])
        else:
            assert got[c] == np.float32(want), c
    assert got[0x7E] == 448.0 and got[0x08] == 2.0 ** -6 and got[0x01] == 2.0 ** -9


def test_e4m3_decode_matches_torch():
    allc = torch.arange(256, dtype=torch.uint8)
    want = allc.view(torch.float8_e4m3fn).float().numpy()
    got = cport.e4m3_to_f32(allc.numpy())
    np.testing.assert_array_equal(np.nan_to_num(got, nan=-1.0), np.nan_to_num(want, nan=-1.0))


def test_e4m3_encode_roundtrip_and_ties():
    finite = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], np.uint8)
    vals = cport.e4m3_to_f32(finite)
    np.testing.assert_array_equal(cport.f32_to_e4m3(vals), finite)
    # midpoints between adjacent positive codes go to the even code; a hair above/below goes up/down
    pos = np.arange(0, 0x7E, dtype=np.uint8)
    lo, hi = cport.e4m3_to_f32(pos).astype(np.float64), cport.e4m3_to_f32(pos + 1).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)
    assert (mid.astype(np.float64) == (lo + hi) / 2).all()  # midpoints are exact in fp32
    even = np.where(pos % 2 == 0, pos, pos + 1).astype(np.uint8)
    np.testing.assert_array_equal(cport.f32_to_e4m3(mid), even)
    np.testing.assert_array_equal(cport.f32_to_e4m3(np.nextafter(mid, np.float32(np.inf))), pos + 1)
    np.testing.assert_array_equal(cport.f32_to_e4m3(np.nextafter(mid, np.float32(-np.inf))), pos)
    np.testing.assert_array_equal(cport.f32_to_e4m3(-mid), even | 0x80)


def test_e4m3_encode_overflow_rule():
    v = np.array([448.0, 463.99, 464.0, 464.01, 479.99, 480.0, 1e30, np.inf, -464.01, -np.inf], np.float32)
    want = np.array([0x7E, 0x7E, 0x7E, 0x7F, 0x7F, 0x7F, 0x7F, 0x7F, 0xFF, 0xFF], np.uint8)
    np.testing.assert_array_equal(cport.f32_to_e4m3(v), want)
    assert cport.f32_to_e4m3(np.array([np.nan], np.float32))[0] & 0x7F == 0x7F


def test_e4m3_encode_dense_sweep_vs_torch():
    hi = np.arange(0, 0x44000000 >> 12, dtype=np.uint32) << 12
    for tail in (0, 1, 0x7FF, 0x800, 0x801, 0xFFF):
        for sgn in (0, 0x80000000):
            b = (hi | np.uint32(tail) | np.uint32(sgn)).astype(np.uint32)
            v = b.view(np.float32)
            want = codes(torch.from_numpy(v.copy()).to(torch.float8_e4m3fn))
            got = cport.f32_to_e4m3(v)
            bad = np.nonzero(got != want)[0]
            assert bad.size == 0, (hex(int(b[bad[0]])), got[bad[0]], want[bad[0]])


def test_bf16_rne_exhaustive_upper_bits_vs_torch():
    hi = np.arange(0, 1 << 16, dtype=np.uint32) << 16
    for tail in (0, 1, 0x7FFF, 0x8000, 0x8001, 0xFFFF):
        v = (hi | np.uint32(tail)).view(np.float32)
        want = bits(torch.from_numpy(v.copy()).to(torch.bfloat16))
        got = cport.f32_to_bf16(v)
        nan = np.isnan(v)
        np.testing.assert_array_equal(got[~nan], want[~nan])
        assert ((got[nan] & 0x7F80) == 0x7F80).all() and ((got[nan] & 0x7F) != 0).all()


# ---------------------------------------------------------------------------
# quantizer
# ---------------------------------------------------------------------------

@pytest.mark.parametrize("M,K,seed,scale", [(8, 64, 0, 1.0), (50, 1024, 1, 1.0), (16, 2048, 2, 30.0),
                                           (5, 4096, 3, 1e-3), (3, 40, 4, 1.0)])
def test_quant_rowwise_c_equals_torch_closed_form(M, K, seed, scale):
    x = seeded((M, K), seed, scale)
    tq, ts = ref.quant_rowwise(x)
    cq, cs = cport.quant_rowwise(bits(x))
    np.testing.assert_array_equal(cq, codes(tq))
    np.testing.assert_array_equal(cs.view(np.uint32), ts.reshape(-1).numpy().view(np.uint32))


def test_quant_rowwise_invariants():
    x = seeded((64, 512), 9, 5.0)
    q, s = cport.quant_rowwise(bits(x))
    xf = x.float().numpy()
    arg = np.abs(xf).argmax(axis=1)
    top = q[np.arange(64), arg]
    assert ((top & 0x7F) == 0x7E).all()          # the row maximum always encodes to +-448
    assert (s > 0).all()
    # scale is bf16(amax/448) widened: low 16 bits of the fp32 pattern are zero
    assert ((s.view(np.uint32) & 0xFFFF) == 0).all()
    # sign of every code follows the sign bit of x
    assert (((q >> 7) & 1) == ((bits(x) >> 15) & 1)).all()
    # dequantized value within half an e4m3 step (relative 2^-4) of x, or within half a subnormal step
    deq = cport.e4m3_to_f32(q) * s[:, None]
    err = np.abs(deq - xf)
    assert (err <= np.maximum(np.abs(xf) * 2.0 ** -4, s[:, None] * 2.0 ** -10) * 1.001).all()


def test_quant_rowwise_all_zero_row_and_floor():
    x = torch.zeros(2, 32, dtype=torch.bfloat16)
    x[1, 3] = -0.0
    q, s = cport.quant_rowwise(bits(x))
    floor = torch.tensor([1e-12]).bfloat16()
    assert floor.view(torch.uint16).item() == 0x2B8D
    want = (floor.float() / 448.0).bfloat16().float().item()
    assert s[0] == np.float32(want) and s[1] == np.float32(want)
    assert (q[0] == 0).all() and q[1, 3] == 0x80


def test_scale_divide_equals_reciprocal_multiply_for_every_bf16_amax():
    """torch on a GPU computes tensor / python-scalar as a multiply by the reciprocal; for the
    scale (amax / 448 rounded to bf16) both forms agree on every finite non-negative bf16."""
    a = torch.arange(0, 0x7F80, dtype=torch.int32).to(torch.uint16).view(torch.bfloat16).float()
    div = (a / 448.0).bfloat16()
    mul = (a * torch.tensor(1.0 / 448.0, dtype=torch.float32)).bfloat16()
    assert torch.equal(div.view(torch.uint16), mul.view(torch.uint16))
    # and the largest |x / s| any row can produce stays below the NaN threshold of the cast
    s = div.float().clamp_min(torch.tensor([1e-12]).bfloat16().float() / 448.0)
    ratio = (a / s)[a >= 1e-12]
    assert ratio.max().item() < 464.0


def test_quant_static_c_equals_torch():
    x = seeded((7, 96), 12, 4.0)
    for sc in (1.0, 0.02, 0.37, 3.0):
        np.testing.assert_array_equal(cport.quant_static(bits(x), sc),
                                      codes(ref.quant_static(x, torch.tensor([sc]))))


def test_weight_quant_c_equals_torch_and_saturates():
    w = seeded((40, 128), 13, 0.02)
    w[3] = 0
    cq, cs = cport.weight_quant(bits(w))
    tq, ts = ref.weight_quant(w)
    np.testing.assert_array_equal(cq, codes(tq))
    np.testing.assert_array_equal(cs, ts.numpy())
    assert ((cq & 0x7F) <= 0x7E).all()
    assert (cq[3] == 0).all() and cs[3] > 0


# ---------------------------------------------------------------------------
# linear + epilogues
# ---------------------------------------------------------------------------

def test_linear_exact_integer_case():
    """Integer codes and power-of-two scales: every partial sum is exact in fp32, so the
    oracle must reproduce integer arithmetic bit for bit, whatever its summation order."""
    g = torch.Generator().manual_seed(0)
    M, N, K = 9, 24, 192
    xi = torch.randint(-8, 9, (M, K), generator=g)
    wi = torch.randint(-8, 9, (N, K), generator=g)
    bi = torch.randint(-4, 5, (N,), generator=g)
    xq = codes(xi.float().to(torch.float8_e4m3fn))
    wq = codes(wi.float().to(torch.float8_e4m3fn))
    xs = np.full(M, 0.5, np.float32)
    ws = np.full(N, 0.25, np.float32)
    out, f32 = cport.linear(xq, xs, wq, ws, bits(bi.to(torch.bfloat16)), 0, want_f32=True)
    want = (xi.double() @ wi.double().t()) * 0.125 + bi.double()
    np.testing.assert_array_equal(f32.astype(np.float64), want.numpy())
    np.testing.assert_array_equal(out, bits(want.to(torch.bfloat16)))


def test_linear_transposition_and_scale_axes_are_pinned():
    """One-hot activations pick single weight columns; distinct row / column scales show
    whether a scale was applied along the wrong axis."""
    M, N, K = 4, 6, 16
    x = torch.zeros(M, K)
    for m in range(M):
        x[m, 3 * m + 1] = 1.0
    w = (torch.arange(N * K).reshape(N, K) % 13 - 6).float()
    xs = np.array([1, 2, 4, 8], np.float32)
    ws = np.array([1, 0.5, 0.25, 2, 4, 8], np.float32)
    _, f32 = cport.linear(codes(x.to(torch.float8_e4m3fn)), xs, codes(w.to(torch.float8_e4m3fn)), ws,
                          None, 0, want_f32=True)
    want = np.array([[w[n, 3 * m + 1].item() * xs[m] * ws[n] for n in range(N)] for m in range(M)], np.float32)
    np.testing.assert_array_equal(f32, want)


@pytest.mark.parametrize("epi", [0, 1, 2, 3, 4, 5])
def test_linear_c_close_to_torch_closed_form(epi):
    x = seeded((12, 256), 21)
    w = seeded((64, 256), 22, 0.02)
    b = seeded((64,), 23, 0.01)
    tq, ts = ref.quant_rowwise(x)
    wq, ws = ref.weight_quant(w)
    y = ref.gemm_f32(tq, ts, wq, ws, b)
    out, f32 = cport.linear(codes(tq), ts.numpy(), codes(wq), ws.numpy(), bits(b), epi, want_f32=True)
    np.testing.assert_allclose(f32, y.numpy(), rtol=2e-5, atol=2e-6)
    want = ref.epilogue(y, epi).float().numpy()
    got = torch.from_numpy(out.copy()).view(torch.bfloat16).float().numpy()
    # two fp32 summation orders may round a value to neighbouring bf16 codes, never further
    assert np.abs(got - want).max() <= 2.0 ** -7 * np.abs(want).max()
    assert (got == want).mean() > 0.97


def test_activations_match_torch():
    v = torch.linspace(-12, 12, 4001)
    for epi, fn in ((4, lambda t: F.gelu(t, approximate="tanh")), (5, F.gelu), (3, F.silu)):
        np.testing.assert_allclose(cport.act(epi, v.numpy()), fn(v).numpy(), rtol=2e-6, atol=2e-6)
    # limits: gelu(-inf side) -> -0, gelu(+big) -> identity
    big = np.array([-50.0, 50.0], np.float32)
    assert cport.act(4, big)[0] == 0 and cport.act(4, big)[1] == 50.0


# ---------------------------------------------------------------------------
# committed fixtures
# ---------------------------------------------------------------------------

def test_golden_fixture_quantizer_and_linear():
    g = np.load(GOLDEN)
    for name in ("cfg1", "tiny", "edge"):
        q, s = cport.quant_rowwise(g[f"{name}_x"])
        np.testing.assert_array_equal(q, g[f"{name}_codes"])
        np.testing.assert_array_equal(s.view(np.uint32), g[f"{name}_scale"].view(np.uint32))
    np.testing.assert_array_equal(cport.quant_static(g["static_x"], float(g["static_scale"][0])), g["static_codes"])
    for name in ("cfg1", "tiny"):
        wq, ws = cport.weight_quant(g[f"{name}_w"])
        np.testing.assert_array_equal(wq, g[f"{name}_wq"])
        np.testing.assert_array_equal(ws, g[f"{name}_ws"])
        _, f32 = cport.linear(g[f"{name}_codes"], g[f"{name}_scale"], wq, ws, g[f"{name}_bias"], 0, want_f32=True)
        np.testing.assert_allclose(f32, g[f"{name}_out_f32"], rtol=2e-5, atol=2e-6)
    for epi in range(6):
        out = cport.linear(g["tiny_codes"], g["tiny_scale"], g["tiny_wq"], g["tiny_ws"], g["tiny_bias"], epi)
        a = torch.from_numpy(out.copy()).view(torch.bfloat16).float()
        b = torch.from_numpy(g[f"tiny_out_epi{epi}"].copy()).view(torch.bfloat16).float()
        assert (a - b).abs().max() <= 2.0 ** -7 * b.abs().max()


def test_golden_fixture_regenerates_identically(tmp_path):
    """The committed file is what tests/golden/make_fixtures.py writes today."""
    import importlib.util

    spec = importlib.util.spec_from_file_location(
        "make_fixtures", os.path.join(os.path.dirname(GOLDEN), "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    mod.OUT = str(tmp_path / "g.npz")
    mod.main()
    a, b = np.load(GOLDEN), np.load(mod.OUT)
    assert sorted(a.files) == sorted(b.files)
    for k in a.files:
        if "_out" in k:
            # matmul outputs: the order of an fp32 sum is the CPU BLAS's business and differs
            # between machines; inputs, codes and scales below are exact everywhere
            x, y = a[k], b[k]
            if x.dtype == np.uint16:                      # bf16 bit patterns
                x = torch.from_numpy(x.copy()).view(torch.bfloat16).float().numpy()
                y = torch.from_numpy(y.copy()).view(torch.bfloat16).float().numpy()
                np.testing.assert_allclose(x, y, rtol=2.0 ** -7, atol=1e-6, err_msg=k)
            else:
                np.testing.assert_allclose(x, y, rtol=2e-5, atol=2e-6, err_msg=k)
        else:
            np.testing.assert_array_equal(a[k], b[k], err_msg=k)


# ---- norm restatements (phyai-kernel triton/rms_norm.py, ada_rms_norm.py) -----------------------

def _bf16_ulp_diff(a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """Distance in bf16 steps between two bf16 tensors (sign-magnitude order)."""
    def key(t):
        u = t.view(torch.int16).to(torch.int32) & 0xFFFF
        return torch.where(u >= 0x8000, 0x8000 - u, u)
    return (key(a) - key(b)).abs()


@pytest.mark.parametrize("gemma", [False, True])
@pytest.mark.parametrize("D", [256, 1024, 3072])
def test_rmsnorm_oracle_against_float64_closed_form(D, gemma):
    x = seeded((17, D), seed=D, scale=0.5)
    w = seeded((D,), seed=D + 1, scale=0.3)
    got = ref.rmsnorm(x, w, 1e-6, gemma)
    x64, w64 = x.double(), w.double() + (1.0 if gemma else 0.0)
    want = (x64 / torch.sqrt((x64 * x64).mean(-1, keepdim=True) + 1e-6) * w64)
    d = _bf16_ulp_diff(got, want.to(torch.bfloat16))
    assert int(d.max()) <= 1 and float((d == 0).float().mean()) > 0.995
    # invariant: unit weight gives unit mean square
    ones = torch.ones(D, dtype=torch.bfloat16)
    o = ref.rmsnorm(x, ones if not gemma else torch.zeros(D, dtype=torch.bfloat16), 1e-6, gemma).double()
    assert torch.allclose((o * o).mean(-1), torch.ones(17, dtype=torch.float64), atol=5e-3)


def test_adarmsnorm_oracle_properties():
    D = 1024
    x = seeded((4, 13, D), seed=5, scale=0.5)
    mod = seeded((4, 3 * D), seed=6, scale=0.1)
    out, gate = ref.adarmsnorm(x, mod, 1e-6)
    assert out.shape == x.shape and gate.shape == (4, D)
    assert torch.equal(gate, mod[:, 2 * D:])                              # gate is a copy
    # float64 closed form, modulation row b serving x[b, :, :]
    x64 = x.double()
    sc, sh = mod[:, None, :D].double(), mod[:, None, D:2 * D].double()
    want = x64 / torch.sqrt((x64 * x64).mean(-1, keepdim=True) + 1e-6) * (1.0 + sc) + sh
    d = _bf16_ulp_diff(out, want.to(torch.bfloat16))
    assert int(d.max()) <= 1 and float((d == 0).float().mean()) > 0.995
    # zero modulation reduces to the plain norm with unit weight
    z = torch.zeros(4, 3 * D, dtype=torch.bfloat16)
    o0, g0 = ref.adarmsnorm(x, z, 1e-6)
    assert torch.equal(o0, ref.rmsnorm(x, torch.ones(D, dtype=torch.bfloat16), 1e-6, False))
    assert not bool(g0.any())
    # per-token mapping (one modulation row per x row) differs from the broadcast one only in rows
    mod_tok = mod.repeat_interleave(13, dim=0).reshape(4, 13, 3 * D)
    o_tok, g_tok = ref.adarmsnorm(x, mod_tok, 1e-6)
    assert torch.equal(o_tok, out) and g_tok.shape == (4, 13, D)


def test_addcmul_oracle_is_torch_addcmul_and_single_rounding():
    r, y, g = seeded((33, 64), 1), seeded((33, 64), 2), seeded((33, 64), 3, 0.3)
    got = ref.addcmul(r, y, g)
    assert torch.equal(got, torch.addcmul(r, y, g))                       # the library routine the reference calls
    want = (r.double() + y.double() * g.double()).to(torch.bfloat16)      # exact arithmetic, one rounding
    assert torch.equal(got, want)
    gb = seeded((3, 64), 4, 0.3)                                          # one gate row per 11 token rows
    assert torch.equal(ref.addcmul(r, y, gb), torch.addcmul(r.reshape(3, 11, 64), y.reshape(3, 11, 64),
                                                            gb.reshape(3, 1, 64)).reshape(33, 64))
