"""Host-side pieces of bench.py that need no GPU: the traffic figure it reports comes from the
committed counter summary and agrees with that summary's own table; the CPU description; the
single-GPU contract."""

from __future__ import annotations

import os
import re
import subprocess
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_reported_traffic_is_the_profiled_figure():
    import bench

    got = bench.profiled_layer_traffic()
    assert isinstance(got, int) and got > 0
    text = open(os.path.join(ROOT, "profiles", "expert_m50_hbm_traffic.md"), encoding="utf-8").read()
    rows = [ln for ln in text.splitlines() if ln.startswith(("| `gemm_fp8_skinny_kernel", "| `gemm_fp8_fusedq_kernel"))]
    assert len(rows) == 4                                   # qkv, o, gate_up, down
    total_mb = 0.0
    for ln in rows:
        cells = [c.strip() for c in ln.strip("|").split("|")]
        total_mb += float(cells[2]) + float(cells[4])       # fetched MB (calibrated) + written MB
    assert abs(got - total_mb * 1e6) <= 0.02e6, (got, total_mb)
    # more than the algorithmic bytes of the layer (bf16 token rows are fetched once per XCD, i.e. eight times:
    # 0.8 - 3.3 MB per linear beside 2.6 - 8.4 MB of weights), but not by much
    algorithmic = sum(bench.algorithmic_bytes(50, N, K, epi) for _, N, K, epi in bench.EXPERT_SET)
    assert algorithmic == 19_042_304 and algorithmic < got < 1.35 * algorithmic


def test_cpu_description():
    import bench

    model, cores = bench.cpu_info()
    assert isinstance(model, str) and model and isinstance(cores, int) and cores >= 1


def test_more_than_one_gpu_is_refused():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True,
                         timeout=300)
    assert out.returncode == 2 and re.search(r"ONE GPU", out.stderr)
