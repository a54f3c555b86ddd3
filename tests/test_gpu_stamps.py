"""The debug build of the library (`make -C phyai_amd/csrc stamps`: GEMM kernels that record time stamps of their
phases, phyai_amd/csrc/stamps.h) must compute exactly what the production build computes, and its stamps must make
sense: every wavefront of the launch leaves a record whose stamps increase."""

from __future__ import annotations

import os

import pytest
import torch

from conftest import seeded

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def libs():
    from phyai_amd import _lib

    if not os.path.exists(_lib.STAMPS_LIB_PATH):
        pytest.skip("debug build not present (make -C phyai_amd/csrc stamps)")
    return _lib.load(), _lib.open_library(_lib.STAMPS_LIB_PATH)


def _linear(lib, x, wq, ws, out, M, N, K, epi, flags=0):
    from phyai_amd import _lib

    need = lib.phyai_fp8_linear_workspace_bytes(M, N, K, epi)
    wsp = torch.zeros(need, dtype=torch.uint8, device=x.device)
    rc = lib.phyai_fp8_linear(x.data_ptr(), K, wq.data_ptr(), ws.data_ptr(), None, out.data_ptr(), out.shape[1], M, N, K,
                              epi | flags, wsp.data_ptr(), need, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, lib.phyai_fp8_last_error()
    torch.cuda.synchronize()


# waves: wavefronts of the launch (one-launch small-M kernel: 8 per workgroup, grid 32 x 7), 0: some multiple of four
@pytest.mark.parametrize("M,N,K,epi,waves", [(816, 4096, 2048, 1, 0), (50, 2560, 1024, 0, 8 * 32 * 7),
                                             (300, 512, 4096, 0, None)])
def test_stamped_kernels_give_the_same_bits_and_sane_stamps(dev, libs, M, N, K, epi, waves):
    from phyai_amd import ops

    main, stamped = libs
    assert main.phyai_fp8_debug_stamps(None, 0) == -2 and b"without time stamps" in main.phyai_fp8_last_error()
    x = seeded((M, K), seed=M + K).to(dev)
    wq, ws = ops.fp8_weight_quant(seeded((N, K), seed=N, scale=0.02).to(dev))
    wo = ops.fp8_weight_to_operand_order(wq, gated=bool(epi))
    n_out = N // 2 if epi else N
    want = torch.empty(M, n_out, dtype=torch.bfloat16, device=dev)
    _linear(main, x, wq, ws, want, M, N, K, epi)
    rec = torch.zeros(4096, 12, dtype=torch.int64, device=dev)
    assert stamped.phyai_fp8_debug_stamps(rec.data_ptr(), rec.shape[0]) == 0
    for w, flags in ((wq, 0), (wo, 0x600 if epi else 0x200)):
        rec.zero_()
        got = torch.full_like(want, float("nan"))
        _linear(stamped, x, w, ws, got, M, N, K, epi, flags)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16))
        r = rec.cpu()
        live = r[r[:, 0] > 0]
        if waves is not None:
            assert (live.shape[0] == waves) if waves else (live.shape[0] > 0 and live.shape[0] % 4 == 0), live.shape[0]
            taken = live[:, :10][:, (live[:, :10] > 0).all(dim=0)]
            assert taken.shape[1] >= 5 and bool((taken[:, 1:] >= taken[:, :-1]).all())
            assert bool((live[:, 11] > live[:, 10]).all())
    assert stamped.phyai_fp8_debug_stamps(None, 0) == 0
    rec.zero_()
    _linear(stamped, x, wq, ws, got, M, N, K, epi)
    assert int(rec.abs().max().item()) == 0      # recording switched off
