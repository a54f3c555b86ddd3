"""phyai_fp8_linear_static: the entry point that allocates nothing (scratch in a device array that is
part of the library) against phyai_fp8_linear with a caller-owned workspace.  Both run the same
kernels, so the outputs must be bit-identical.  Calls go straight through the C ABI.

Two calls in a row share the array, the second with a smaller input than the first: what the first
left behind (codes, scales, split-K partial sums) must not leak into the second.
"""

from __future__ import annotations

import pytest
import torch

pytestmark = pytest.mark.gpu

STATIC_BYTES = 32 * 1024 * 1024
EPI = {None: 0, "geglu_tanh": 1}


def _problem(dev, M, N, K, seed, bias):
    from phyai_amd import ops

    g = torch.Generator(device=dev).manual_seed(seed)
    x = torch.randn(M, K, generator=g, device=dev).to(torch.bfloat16)
    w = (torch.randn(N, K, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    b = (torch.randn(N, generator=g, device=dev) * 0.01).to(torch.bfloat16) if bias else None
    wq, ws = ops.fp8_weight_quant(w)
    return x, wq, ws, b


def _with_workspace(lib, x, wq, ws, b, epi, M, N, K, n_out):
    from phyai_amd import _lib

    need = lib.phyai_fp8_linear_workspace_bytes(M, N, K, epi)
    wsp = torch.zeros(need, dtype=torch.uint8, device=x.device)
    out = torch.empty(M, n_out, dtype=torch.bfloat16, device=x.device)
    rc = lib.phyai_fp8_linear(x.data_ptr(), K, wq.data_ptr(), ws.data_ptr(), b.data_ptr() if b is not None else None,
                              out.data_ptr(), n_out, M, N, K, epi, wsp.data_ptr(), need,
                              torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "phyai_fp8_linear")
    torch.cuda.synchronize()
    return out


def _static(lib, x, wq, ws, b, epi, M, N, K, n_out):
    from phyai_amd import _lib

    out = torch.full((M, n_out), float("nan"), dtype=torch.bfloat16, device=x.device)
    rc = lib.phyai_fp8_linear_static(x.data_ptr(), K, wq.data_ptr(), ws.data_ptr(),
                                     b.data_ptr() if b is not None else None, out.data_ptr(), n_out, M, N, K, epi,
                                     torch.cuda.current_stream().cuda_stream)
    _lib.check(rc, "phyai_fp8_linear_static")
    torch.cuda.synchronize()
    return out


# (first call, second smaller call): split-K tile kernel then weight streaming; generic split-K kernel
# (K not a multiple of 128) then a smaller generic split-K problem; gated epilogue then plain.
PAIRS = [
    ((816, 2048, 16384, None, False), (50, 1024, 4096, None, True)),
    ((200, 512, 1040, None, True), (40, 256, 528, None, False)),
    ((816, 4096, 2048, "geglu_tanh", False), (50, 8192, 1024, "geglu_tanh", False)),
    # the one-launch kernel (quantizes its own rows: the array is not touched at all), then a smaller one
    ((50, 2560, 1024, None, True), (16, 1024, 2048, None, False)),
]


@pytest.mark.parametrize("first,second", PAIRS)
def test_static_scratch_linear_equals_workspace_linear(dev, first, second):
    from phyai_amd import _lib

    lib = _lib.load()
    for i, (M, N, K, epi_name, bias) in enumerate((first, second)):
        epi = EPI[epi_name]
        n_out = N // 2 if epi else N
        x, wq, ws, b = _problem(dev, M, N, K, seed=900 + 7 * i + N, bias=bias)
        want = _with_workspace(lib, x, wq, ws, b, epi, M, N, K, n_out)
        got = _static(lib, x, wq, ws, b, epi, M, N, K, n_out)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), f"call {i}: {M}x{N}x{K} {epi_name}"
        # and once more on the array as that call left it
        again = _static(lib, x, wq, ws, b, epi, M, N, K, n_out)
        assert torch.equal(again.view(torch.int16), want.view(torch.int16)), f"call {i} repeated: {M}x{N}x{K}"


def test_static_scratch_linear_recorded_into_a_graph(dev):
    """The entry point is meant for code under graph capture (its first call on a device, which looks the array's
    address up, made outside): two calls are recorded into one graph - a split-K shape, whose recording holds the
    kernel that clears the arrival counters, the quantizer and the GEMM on the library's own array, and a shape that
    the one-launch kernel serves - and every replay must give the bits of phyai_fp8_linear, with eager calls that
    use the same array between the replays."""
    from phyai_amd import _lib
    from phyai_amd.runtime import HipGraph

    lib = _lib.load()
    shapes = [(816, 2048, 16384, 0), (50, 2560, 1024, 0)]
    probs, wants, outs = [], [], []
    for i, (M, N, K, epi) in enumerate(shapes):
        x, wq, ws, b = _problem(dev, M, N, K, seed=1234 + i, bias=True)
        probs.append((x, wq, ws, b))
        wants.append(_with_workspace(lib, x, wq, ws, b, epi, M, N, K, N))
        outs.append(torch.empty(M, N, dtype=torch.bfloat16, device=dev))
        _static(lib, x, wq, ws, b, epi, M, N, K, N)      # the call that looks the address up, outside capture

    def fn():
        st = torch.cuda.current_stream().cuda_stream
        for (M, N, K, epi), (x, wq, ws, b), out in zip(shapes, probs, outs):
            _lib.check(lib.phyai_fp8_linear_static(x.data_ptr(), K, wq.data_ptr(), ws.data_ptr(), b.data_ptr(), out.data_ptr(),
                                                   N, M, N, K, epi, st), "phyai_fp8_linear_static")

    g = HipGraph()
    g.capture(fn, {})
    for r in range(3):
        for out in outs:
            out.fill_(float("nan"))
        g.replay()
        torch.cuda.synchronize()
        for i, (out, want) in enumerate(zip(outs, wants)):
            assert torch.equal(out.view(torch.int16), want.view(torch.int16)), f"replay {r}, call {i}"
        # eager work on the same array between the replays: another split-K shape leaves other codes and partial sums
        M, N, K = 300, 384, 4096
        x, wq, ws, b = _problem(dev, M, N, K, seed=77 + r, bias=False)
        _static(lib, x, wq, ws, b, 0, M, N, K, N)


def test_static_scratch_linear_refuses_what_does_not_fit(dev):
    from phyai_amd import _lib

    lib = _lib.load()
    M, N, K = 4096, 2048, 16384     # 64 MiB of activation codes alone
    assert lib.phyai_fp8_linear_workspace_bytes(M, N, K, 0) > STATIC_BYTES
    x = torch.zeros(8, dtype=torch.bfloat16, device=dev)   # never dereferenced: the size check comes first
    rc = lib.phyai_fp8_linear_static(x.data_ptr(), K, x.data_ptr(), x.data_ptr(), None, x.data_ptr(), N, M, N, K, 0,
                                     torch.cuda.current_stream().cuda_stream)
    assert rc == -3
    assert b"static array holds" in lib.phyai_fp8_last_error()
    assert lib.phyai_fp8_linear_static(None, K, None, None, None, None, N, 0, N, K, 0, None) == 0   # empty input
