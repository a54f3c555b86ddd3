#!/usr/bin/env python3
"""Writes tests/golden/fp8_linear_golden.npz.

The reference holds no golden vectors for fp8 codes, scales or GEMM outputs (its
tests pin shapes and loose tolerances only), so these vectors are produced here
from the reference's own tensor expressions evaluated with torch CPU ops
(``oracle/ref.py``: quant/fp8.py:150-155, backends/torch.py:155-176,
mlp/dense_mlp.py:256-265) on seeded inputs.  The reference package itself is
not imported.  Run from the repo root: ``python tests/golden/make_fixtures.py``.
"""

from __future__ import annotations

import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import ref  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "fp8_linear_golden.npz")


def bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.uint16).numpy().copy()


def codes(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.uint8).numpy().copy()


def randn(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(*shape, generator=g) * scale).to(torch.bfloat16)


def main() -> None:
    d: dict[str, np.ndarray] = {}

    # -- benchmark configuration 1, activation side: X [50, 1024] ~ N(0,1), seed 0 ---------
    x = randn((50, 1024), 0)
    q, s = ref.quant_rowwise(x)
    d["cfg1_x"] = bits(x)
    d["cfg1_codes"] = codes(q)
    d["cfg1_scale"] = s.reshape(-1).numpy().copy()
    # ... and the first 64 output channels of its W [4096, 1024] ~ N(0, 0.02) (seed 1), bias seed 2
    w = randn((4096, 1024), 1, 0.02)[:64].contiguous()
    b = randn((4096,), 2, 0.01)[:64].contiguous()
    wq, ws = ref.weight_quant(w)
    y = ref.gemm_f32(q, s, wq, ws, b)
    d["cfg1_w"] = bits(w)
    d["cfg1_wq"] = codes(wq)
    d["cfg1_ws"] = ws.numpy().copy()
    d["cfg1_bias"] = bits(b)
    d["cfg1_out_f32"] = y.numpy().copy()
    d["cfg1_out"] = bits(y.to(torch.bfloat16))

    # -- a tiny full case: M=8, K=64, N=32, every epilogue ------------------------------------
    x = randn((8, 64), 10)
    w = randn((32, 64), 11, 0.02)
    b = randn((32,), 12, 0.01)
    q, s = ref.quant_rowwise(x)
    wq, ws = ref.weight_quant(w)
    y = ref.gemm_f32(q, s, wq, ws, b)
    d["tiny_x"], d["tiny_w"], d["tiny_bias"] = bits(x), bits(w), bits(b)
    d["tiny_codes"], d["tiny_scale"] = codes(q), s.reshape(-1).numpy().copy()
    d["tiny_wq"], d["tiny_ws"] = codes(wq), ws.numpy().copy()
    d["tiny_out_f32"] = y.numpy().copy()
    for epi in range(6):
        d[f"tiny_out_epi{epi}"] = bits(ref.epilogue(y, epi))

    # -- edge rows, K = 64 -------------------------------------------------------------------
    e = randn((8, 64), 20)
    e[0] = 0                                                   # all-zero row
    e[1] = 0; e[1, 0] = -0.0; e[1, 7] = 0.0                    # +-0 only
    e[2] = torch.full((64,), 9.2e-41).to(torch.bfloat16); e[2, 3] = -9.2e-41   # bf16 subnormals
    e[3] = e[3].clamp(-64, 64); e[3, 17] = 64.0                # amax a power of two
    e[4, 0] = torch.finfo(torch.bfloat16).max                   # amax at the bf16 maximum
    e[5, 40] = 2000.0                                          # outlier row
    e[6] = e[6] * 1e-20                                        # tiny magnitudes
    e[7] = -e[7].abs()                                         # all negative
    q, s = ref.quant_rowwise(e)
    d["edge_x"], d["edge_codes"], d["edge_scale"] = bits(e), codes(q), s.reshape(-1).numpy().copy()

    # -- static per-tensor quantizer -----------------------------------------------------------
    x = randn((5, 32), 30, 3.0)
    d["static_x"] = bits(x)
    d["static_scale"] = np.array([0.37], np.float32)
    d["static_codes"] = codes(ref.quant_static(x, torch.tensor([0.37])))

    np.savez_compressed(OUT, **d)
    print(f"wrote {OUT}: {len(d)} arrays, {os.path.getsize(OUT)} bytes")


if __name__ == "__main__":
    main()
