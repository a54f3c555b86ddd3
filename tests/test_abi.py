"""The C-ABI library loads and exports exactly what include/phyai_fp8.h declares.
No compute call is made here, so this runs without a GPU."""

from __future__ import annotations

import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "phyai_fp8.h")


def declared_functions() -> list[str]:
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(phyai_fp8_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for required in ("phyai_fp8_quant_rowwise", "phyai_fp8_quant_static", "phyai_fp8_weight_quant_rowwise",
                     "phyai_fp8_gemm", "phyai_fp8_linear", "phyai_fp8_linear_workspace_bytes",
                     "phyai_fp8_abi_version", "phyai_fp8_last_error"):
        assert required in names


def test_library_exports_every_declared_symbol():
    from phyai_amd import _lib

    lib = _lib.load()
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == declared_functions()
    assert lib.phyai_fp8_abi_version() == _lib.ABI_VERSION


def test_workspace_query_and_argument_validation_without_gpu():
    """Size queries and argument checks run entirely on the host."""
    from phyai_amd import _lib

    lib = _lib.load()
    hdr = 16384
    buf0 = (ctypes.c_char * 64)()
    assert lib.phyai_fp8_linear_workspace_bytes(50, 1024, 4096, 0) >= hdr + 50 * 4096
    assert lib.phyai_fp8_linear_workspace_bytes(0, 1024, 4096, 0) >= hdr
    # null pointers / bad shapes are rejected before anything is launched
    assert lib.phyai_fp8_quant_rowwise(None, 4, 64, 64, None, None, None) == -1
    assert lib.phyai_fp8_quant_rowwise(None, 0, 64, 64, None, None, None) == 0      # empty: nothing to do
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 4, 64, 60, 0, None, 0, None) == -2
    assert b"multiples of 16" in lib.phyai_fp8_last_error()
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 4, 64, 64, 9, None, 0, None) == -1
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 0, 64, 64, 0, None, 0, None) == 0
    # flag bits ride in the epilogue argument: the known one is accepted, others are not
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 0, 64, 64, 0x100 | 1, None, 0, None) == 0
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 4, 64, 64, 0x800, None, 0, None) == -1
    assert b"flag" in lib.phyai_fp8_last_error()
    # weight layout flags: operand order needs K % 128 == 0, the gated form goes with gated epilogues only
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 4, 64, 64, 0x200, None, 0, None) == -2
    assert b"K % 128" in lib.phyai_fp8_last_error()
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 0, 64, 128, 0x200, None, 0, None) == 0
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 0, 64, 128, 0x600 | 1, None, 0, None) == 0
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 4, 64, 128, 0x600, None, 0, None) == -1
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 4, 64, 128, 0x200 | 1, None, 0, None) == -1
    assert lib.phyai_fp8_gemm(None, None, 0, None, None, None, None, 64, 4, 64, 128, 0x400, None, 0, None) == -1
    assert lib.phyai_fp8_weight_to_operand_order(None, 0, 128, 0, None, None) == 0
    assert lib.phyai_fp8_weight_to_operand_order(None, 16, 128, 0, None, None) == -1
    assert lib.phyai_fp8_weight_to_operand_order(None, 16, 128, 1, None, None) == -1   # null before the N % 32 check
    assert lib.phyai_fp8_weight_to_operand_order(ctypes.addressof(buf0), 16, 64, 0, ctypes.addressof(buf0), None) == -2
    assert lib.phyai_fp8_linear_workspace_bytes(50, 1024, 4096, 0x100) == lib.phyai_fp8_linear_workspace_bytes(50, 1024, 4096, 0)
    buf = (ctypes.c_char * 64)()
    assert lib.phyai_fp8_linear(ctypes.addressof(buf), 64, None, None, None, None, 64, 4, 64, 64, 0, None, 0, None) == -3
    assert b"workspace" in lib.phyai_fp8_last_error()


def test_kernel_selection_for_the_benchmark_shapes(monkeypatch):
    """The dispatcher's choice, read back as text (host only).  The rules behind these cases were
    measured on the GPU: weight streaming up to 64 token rows; 256 x 256 tiles when they fill the
    chip and K is long or the last round of smaller tiles would be emptier; 192 x 128 tiles (two
    workgroups per CU) for K <= 8192 with enough tiles, or when they fit one round and 128 x 128 tiles
    would not; 128 x 128 tiles with a ring of two once there are more tiles than CUs, split along K
    for K >= 8192 with few tiles; weight streaming again up to 64 small tiles and 1024 rows, its
    workgroup shape chosen by (rounds of workgroups) x (operand blocks per workgroup)."""
    from phyai_amd import ops

    for var in ("PHYAI_FP8_BIG", "PHYAI_FP8_BIG_DEPTH", "PHYAI_FP8_BIG_SPLITS", "PHYAI_FP8_TILE",
                "PHYAI_FP8_SKINNY_PLAN", "PHYAI_FP8_SKINNY_MAXM"):
        monkeypatch.delenv(var, raising=False)
    d = ops.describe_plan
    # action expert, M = 50
    assert d(50, 2560, 1024) == "small-m nt=2 mb=2 kpw=1 rounds=1"    # 160 workgroups x 4 operand blocks
    assert d(50, 1024, 2048) == "small-m nt=1 mb=1 kpw=2 rounds=1"
    assert d(50, 8192, 1024, "geglu_tanh") == "small-m nt=2 mb=4 kpw=1 rounds=1"
    assert d(50, 1024, 4096) == "small-m nt=1 mb=1 kpw=4 rounds=1"
    assert d(1, 12288, 2048).startswith("small-m nt=1 mb=1")
    # prefix prefill, M = 816
    assert d(816, 2560, 2048) == "tile 96x128 depth=4 splits=1 tiles=180"      # 140 tiles of 128 x 128 idle 116 CUs, 280 of 128 x 64 need two rounds
    assert d(816, 2560, 2048, "gelu") == "tile 96x128 depth=4 splits=1 tiles=180"
    assert d(816, 2560, 2048, "geglu_tanh") == "tile 128x128 depth=4 splits=1 tiles=140"   # gated: no single-column-block tile
    assert d(816, 2560, 8192).startswith("tile 128x128 depth=4 splits=2")             # long K: split form
    assert d(1632, 2560, 2048) == "tile 128x128 depth=2 splits=1 tiles=260"             # the 128-row grid fills the chip
    assert d(816, 2048, 2048) == "tile 128x64 depth=4 splits=1 tiles=224"      # 112 tiles of 128 x 128 would idle half the CUs
    assert d(816, 32768, 2048, "geglu_tanh") == "tile 224x256 depth=2 splits=1 tiles=512"   # four tile rows either way: less padding
    assert d(816, 2048, 16384) == "tile 128x128 depth=4 splits=2 tiles=112"
    # batched serving and the DiT block
    assert d(1632, 32768, 2048, "geglu_tanh") == "tile 192x128 depth=2 splits=1 tiles=2304"
    assert d(4800, 8192, 2048, "gelu") == "tile 192x128 depth=2 splits=1 tiles=1600"
    assert d(6528, 2048, 2048) == "tile 256x256 depth=2 splits=1 tiles=208"
    assert d(13056, 2560, 2048) == "tile 192x128 depth=2 splits=1 tiles=1360"
    assert d(6528, 2560, 2048) == "tile 192x128 depth=2 splits=1 tiles=680"    # 260 large tiles: a nearly empty round
    assert d(6528, 2048, 16384) == "tile 256x256 depth=2 splits=1 tiles=208"
    assert d(800, 8192, 1024, "geglu_tanh") == "tile 128x128 depth=2 splits=1 tiles=448"
    assert d(1632, 2560, 2048) == "tile 128x128 depth=2 splits=1 tiles=260"   # more tiles than CUs
    assert d(1632, 2048, 2048) == "tile 128x128 depth=4 splits=1 tiles=208"   # fewer
    assert d(3264, 2560, 2048) == "tile 192x128 depth=2 splits=1 tiles=340"   # 520 small tiles would spill
    assert d(3264, 2048, 2048) == "tile 128x128 depth=2 splits=1 tiles=416"   # 416 do not
    assert d(200, 1024, 4096).startswith("small-m ")           # 16 small tiles: weight streaming wins
    assert d(800, 1024, 4096) == "small-m nt=4 mb=4 kpw=1 rounds=4"  # 56 small tiles: still weight streaming, 208 workgroups x 8 blocks
    assert d(400, 1024, 2048) == "small-m nt=2 mb=4 kpw=1 rounds=2"  # 224 workgroups x 6 blocks
    assert d(100, 2560, 1024) == "small-m nt=2 mb=3 kpw=1 rounds=1"  # 240 workgroups x 5 blocks
    assert d(100, 8192, 1024, "geglu_tanh") == "small-m nt=4 mb=4 kpw=1 rounds=1"
    assert d(1000, 1024, 4096) == "small-m nt=4 mb=4 kpw=1 rounds=4"
    assert d(1100, 1024, 4096) == "tile 128x64 depth=4 splits=1 tiles=144"
    assert d(816, 2048, 4096) == "tile 128x64 depth=4 splits=1 tiles=224"
    assert d(816, 2048, 8192) == "tile 128x128 depth=4 splits=2 tiles=112"     # long K: the split form is level or ahead
    assert d(816, 4096, 2048, "geglu_tanh") == "tile 128x128 depth=4 splits=1 tiles=224"   # gated: no 64-column tile
    # weights in operand order, K >= 4096: the 224 x 256 tile (weights straight into registers) where it has at least
    # 160 tiles and fills its rounds about as well as the shape chosen for row-major weights
    op, og = "operand", "operand_gated"
    R4, R8 = " weights in registers, ring of 4", " weights in registers, ring of 8"   # (and no barrier per stage)
    assert d(816, 32768, 2048, "geglu_tanh", og) == "tile 224x256 depth=2 splits=1 tiles=512" + R4
    assert d(816, 2560, 2048, None, op) == "tile 96x128 depth=4 splits=1 tiles=180"          # staged as they lie
    assert d(1632, 2048, 2048, None, op) == "tile 128x128 depth=4 splits=1 tiles=208" + R8
    assert d(1632, 2048, 2048 + 512, None, op) == "tile 128x128 depth=4 splits=1 tiles=208"  # K not a multiple of 1024
    assert d(816, 4096, 2048, "geglu_tanh", og) == "tile 128x128 depth=4 splits=1 tiles=224" # gated: staged
    assert d(1632, 2560, 2048, None, op) == "tile 128x128 depth=2 splits=1 tiles=260" + R4
    assert d(1632, 2560, 2048 + 128, None, op) == "tile 128x128 depth=2 splits=1 tiles=260"  # K not a multiple of 512
    assert d(800, 8192, 1024, "geglu_tanh", og) == "tile 128x128 depth=2 splits=1 tiles=448" # gated: staged
    assert d(6528, 2048, 16384, None, op) == "tile 224x256 depth=2 splits=1 tiles=240" + R4
    assert d(13056, 2048, 16384, None, op) == "tile 224x256 depth=2 splits=1 tiles=472" + R4
    assert d(4800, 2048, 8192, None, op) == "tile 224x256 depth=2 splits=1 tiles=176" + R4
    assert d(6528, 4096, 4096, "gelu", op) == "tile 224x256 depth=2 splits=1 tiles=480" + R4
    assert d(3264, 16384, 4096, "geglu_tanh", og) == "tile 224x256 depth=2 splits=1 tiles=960" + R4
    assert d(2048, 8192, 8192, None, op) == "tile 256x256 depth=2 splits=1 tiles=256"      # 320 tiles of 224 rows: a second round, mostly empty
    assert d(8000, 1024, 8192, None, op) == "tile 128x128 depth=2 splits=1 tiles=504" + R4  # 144 tiles of 224 x 256: too few
    assert d(3264, 2048, 16384, None, op) == "tile 128x128 depth=2 splits=1 tiles=416" + R4   # two workgroups per CU, each with its ring
    assert d(816, 2048, 16384, None, op) == "tile 128x128 depth=4 splits=2 tiles=112" + R8      # split launches stay
    assert d(6528, 32768, 2048, "geglu_tanh", og) == "tile 192x128 depth=2 splits=1 tiles=8704"   # K = 2048: two workgroups per CU keep their lead
    assert d(4800, 2048, 8192 + 128, None, op) == d(4800, 2048, 8192 + 128)                # K not a multiple of 512: no register path
    # what the fast kernels refuse goes to the generic one
    assert d(300, 384, 272).startswith("generic ")
    with pytest.raises(RuntimeError, match="multiples of 16"):
        d(50, 1000, 1024)


def test_whole_linear_selection_one_launch_or_two(monkeypatch):
    """phyai_fp8_linear runs one kernel that quantizes its own token rows where that was measured
    faster (up to 128 rows, K <= 4096, a grid of at most 256 workgroups), and quantizer + GEMM
    elsewhere.  Host only."""
    from phyai_amd import ops

    for var in ("PHYAI_FP8_FUSED", "PHYAI_FP8_FUSED_PLAN", "PHYAI_FP8_SKINNY_PLAN", "PHYAI_FP8_BIG"):
        monkeypatch.delenv(var, raising=False)
    d = ops.describe_linear_plan
    assert d(50, 2560, 1024) == "one launch: small-m rows=8 nt=5 kpw=1 grid=32x7"      # half the conversions of 16 x 4
    assert d(50, 1024, 2048) == "one launch: small-m rows=8 nt=2 kpw=2 grid=32x7"
    assert d(50, 8192, 1024, "geglu_tanh") == "one launch: small-m rows=16 nt=8 kpw=1 grid=64x4"
    assert d(50, 4096, 1024) == "one launch: small-m rows=16 nt=4 kpw=1 grid=64x4"
    assert d(1, 2048, 2048) == "one launch: small-m rows=8 nt=2 kpw=2 grid=64x1"
    assert d(50, 1024, 4096) == "one launch: small-m rows=8 nt=2 kpw=4 grid=32x7"      # four K steps per wavefront: 8 x 2 only
    assert d(50, 2048, 4096).startswith("quantizer + small-m")                          # ... whose grid must fit one round
    assert d(50, 2048, 4096, weight_layout="operand").startswith("quantizer + small-m")
    assert d(50, 1024, 4224).startswith("quantizer + ")                                 # K beyond 4096
    # the layout of the weight matrix is part of the question: with weights straight into registers more shapes fit
    assert d(50, 8192, 2048, "geglu_tanh").startswith("quantizer + ")
    assert d(50, 8192, 2048, "geglu_tanh", weight_layout="operand_gated") == "one launch: small-m rows=16 nt=8 kpw=2 grid=64x4"
    with pytest.raises(RuntimeError, match="does not go with"):
        d(50, 8192, 2048, "geglu_tanh", weight_layout="operand")
    m = ops.describe_mlp_plan
    assert m(50, 1024, 4096, 1024, "geglu_tanh") == ("row maxima handed over: one launch: small-m rows=16 nt=8 kpw=1 grid=64x4 | "
                                                     "one launch: small-m rows=8 nt=2 kpw=4 grid=32x7")
    assert m(50, 1024, 4096, 1024, "geglu_tanh", operand_order=True) == m(50, 1024, 4096, 1024, "geglu_tanh")
    assert not m(50, 2048, 8192, 2048, "geglu_tanh").startswith("row maxima")
    assert m(200, 1024, 4096, 1024, "geglu_tanh").count("quantizer + ") == 2
    assert d(50, 12288, 2048).startswith("quantizer + small-m")                       # more than one round of workgroups
    assert d(100, 2560, 1024) == "one launch: small-m rows=16 nt=8 kpw=1 grid=20x7"   # up to 128 rows, 16 per workgroup
    assert d(100, 8192, 1024, "geglu_tanh").startswith("quantizer + small-m")          # 16-row workgroups would need two rounds
    assert d(129, 1024, 1024).startswith("quantizer + small-m")
    assert d(50, 1024, 1040).startswith("quantizer + ")                               # K not a multiple of 128
    assert d(816, 2048, 2048) == "quantizer + tile 128x64 depth=4 splits=1 tiles=224"
    monkeypatch.setenv("PHYAI_FP8_FUSED", "0")
    assert d(50, 2560, 1024) == "quantizer + small-m nt=2 mb=2 kpw=1 rounds=1"
    monkeypatch.setenv("PHYAI_FP8_FUSED", "1")
    monkeypatch.setenv("PHYAI_FP8_FUSED_PLAN", "32,2")
    assert d(50, 2560, 1024) == "one launch: small-m rows=32 nt=2 kpw=1 grid=80x2"
    assert d(50, 1024, 4096).startswith("quantizer + ")                               # no such kernel at four K steps per wavefront
    monkeypatch.setenv("PHYAI_FP8_FUSED_PLAN", "16,1")
    assert d(50, 1024, 4096) == "one launch: small-m rows=16 nt=1 kpw=4 grid=64x4"    # exists, forced for tests only


def test_tuning_variables_are_ignored_without_the_switch():
    """A stray PHYAI_FP8_* variable must not change the kernel selection of a process that did not
    set PHYAI_FP8_TUNING (fresh processes: the switch is read once)."""
    import subprocess
    import sys

    code = ("from phyai_amd import ops; print(ops.describe_plan(816, 32768, 2048, 'geglu_tanh')); "
            "print(ops.describe_plan(50, 2560, 1024))")
    want = "tile 224x256 depth=2 splits=1 tiles=512\nsmall-m nt=2 mb=2 kpw=1 rounds=1\n"
    env = {k: v for k, v in os.environ.items() if not k.startswith("PHYAI_FP8_")}
    env.update(PHYAI_FP8_BIG="128", PHYAI_FP8_SKINNY_PLAN="1,4", PHYAI_FP8_TILE="128,128,2", PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert out.stdout == want
    env["PHYAI_FP8_TUNING"] = "1"
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
    assert out.returncode == 0, out.stderr
    assert out.stdout != want


C_CLIENT = r"""
#include <stdio.h>
#include <string.h>
#include "phyai_fp8.h"
int main(void) {
    char buf[96];
    if (phyai_fp8_abi_version() != PHYAI_FP8_ABI_VERSION) return 1;
    if (phyai_fp8_linear_workspace_bytes(50, 1024, 4096, PHYAI_FP8_EPI_NONE) < PHYAI_FP8_WORKSPACE_HEADER_BYTES) return 2;
    if (phyai_fp8_describe_plan(50, 8192, 1024, PHYAI_FP8_EPI_GEGLU_TANH, buf, sizeof buf) <= 0) return 3;
    if (strncmp(buf, "small-m", 7) != 0) return 4;
    if (phyai_fp8_gemm(NULL, NULL, 0, NULL, NULL, NULL, NULL, 64, 4, 64, 60, 0, NULL, 0, NULL) != PHYAI_FP8_EUNSUPPORTED) return 5;
    if (strstr(phyai_fp8_last_error(), "multiples of 16") == NULL) return 6;
    puts(buf);
    return 0;
}
"""


def test_header_and_library_serve_a_plain_c_client(tmp_path):
    """The header compiles as C99 and a C program linked against the library can call it (host-side
    entry points only: nothing here needs a GPU)."""
    import shutil
    import subprocess

    from phyai_amd import _lib

    _lib.load()
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    src = tmp_path / "client.c"
    src.write_text(C_CLIENT)
    exe = tmp_path / "client"
    libdir = os.path.dirname(_lib.LIB_PATH)
    subprocess.check_call([gcc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                           str(src), "-o", str(exe), "-L", libdir, "-lphyai_fp8", f"-Wl,-rpath,{libdir}"])
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, (out.returncode, out.stdout, out.stderr)
    assert out.stdout.startswith("small-m nt=2 mb=4")


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from phyai_amd import _lib

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.Fp8LibraryError, match="no non-HIP fallback"):
        _lib.load()


def test_product_package_never_imports_the_oracle():
    pkg = os.path.join(ROOT, "phyai_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".h")):
                text = open(os.path.join(base, f)).read()
                assert "oracle" not in text.replace("the oracle's", ""), f"{f} mentions the oracle"
