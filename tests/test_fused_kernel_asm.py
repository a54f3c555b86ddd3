"""The one-launch small-M linear loads its activation rows with inline-assembly loads the compiler cannot
see (phyai_amd/csrc/gemm_skinny_fused.hip).  What must hold of the code the compiler makes around them is
checked on the gfx950 assembly by phyai_amd/csrc/check_fused_asm.py (no GPU needed); the library's build
runs the same check.  Here: the check passes on the current sources, and it does catch each kind of
violation when one is planted in the assembly text."""

from __future__ import annotations

import importlib.util
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def guard():
    spec = importlib.util.spec_from_file_location("check_fused_asm", os.path.join(ROOT, "phyai_amd", "csrc", "check_fused_asm.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.fixture(scope="module")
def asm(guard):
    problems = guard.check_file(make=True)
    assert not problems, "\n".join(problems[:20])
    return open(guard.ASM, encoding="utf-8").read()


def test_every_instantiation_passes(guard, asm):
    kernels = guard.kernels_of(asm)
    assert len(kernels) >= 400
    # all variants are there: weights staged / straight into registers, own / handed-over row maxima
    names = "\n".join(k.split(":", 1)[0] for k in kernels)
    for tail in ("ELb0ELb0ELb0E", "ELb0ELb1ELb0E", "ELb0ELb0ELb1E", "ELb1ELb1ELb1E"):
        assert tail in names, tail


def test_planted_violations_are_caught(guard, asm):
    k = next(k for k in guard.kernels_of(asm) if "ILi8ELi2ELi4ELi0ELb0ELb1ELb1E" in k.split(":", 1)[0])
    name = k.split(":", 1)[0]
    rows = guard.rows_loaded(name)
    assert rows == 9 and not guard.check_kernel(k, rows)
    body, waited = guard.stretch(k)
    first = body[0]
    dest = re.search(r"v\[(\d+):\d+\]", first).group(1)
    lines = k.split("\n")
    at = next(i for i, line in enumerate(lines) if line.strip() == first)
    # a copy of a register in flight
    planted = "\n".join(lines[: at + 1] + [f"\tv_mov_b32_e32 v250, v{dest}"] + lines[at + 1:])
    assert any("touches a register" in p for p in guard.check_kernel(planted, rows))
    # a branch in the stretch
    planted = "\n".join(lines[: at + 1] + ["\ts_cbranch_scc1 .LBB0_99"] + lines[at + 1:])
    assert any("s_cbranch" in p for p in guard.check_kernel(planted, rows))
    # one more vector-memory instruction than the wait counts
    last = max(i for i, line in enumerate(lines[: at + 200]) if line.strip() in body and line.strip().startswith("global_load_dwordx4"))
    planted = "\n".join(lines[: last + 1] + ["\tglobal_load_dword v251, v252, s[0:1]"] + lines[last + 1:])
    assert any("vmcnt" in p for p in guard.check_kernel(planted, rows))
    # scratch
    planted = k + "\n\tscratch_store_dword off, v1, s0\n"
    assert any("scratch" in p for p in guard.check_kernel(planted, rows))


def test_tile_kernels_use_no_scratch(guard):
    """The pipelined tile kernels count their global -> LDS copies by hand (s_waitcnt vmcnt(N)): a spill would put
    scratch loads and stores of the compiler's among them.  The Makefile keeps the compiler's resource-usage remarks
    beside every object; the guard reads them (the library's build runs the same check)."""
    usage = os.path.join(ROOT, "phyai_amd", "csrc", "_obj", "gemm_big.o.usage")
    if not os.path.exists(usage):
        pytest.skip("no resource-usage remarks here (the library was built elsewhere)")
    assert not guard.check_tile_usage(), "\n".join(guard.check_tile_usage()[:20])
    planted = ("x.hip:1:1: remark: Function Name: _ZN5phyai19gemm_fp8_big_kernelILi2ELi2EEEvv [-Rpass-analysis=kernel-resource-usage]\n"
               "x.hip:1:1: remark:     ScratchSize [bytes/lane]: 268 [-Rpass-analysis=kernel-resource-usage]\n"
               "x.hip:1:1: remark: Function Name: _ZN5phyai5otherEv [-Rpass-analysis=kernel-resource-usage]\n"
               "x.hip:1:1: remark:     ScratchSize [bytes/lane]: 16 [-Rpass-analysis=kernel-resource-usage]\n")
    bad = guard.usage_problems(planted, min_kernels=1)
    assert len(bad) == 1 and "268 bytes" in bad[0]
    assert any("only 1" in p for p in guard.usage_problems(planted, min_kernels=2))
