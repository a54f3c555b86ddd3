"""The one-launch small-M linear loads its activation rows with inline-assembly loads the compiler
cannot see (phyai_amd/csrc/gemm_skinny_fused.hip): between such a load and the `s_waitcnt vmcnt`
that covers it the destination registers hold nothing yet.  A copy or any other use the compiler
schedules there reads stale registers, and the data that lands later overwrites whatever the
registers were reused for - addresses included.  This test compiles the file to gfx950 assembly
(no GPU needed) and checks every instantiation:

* no instruction between the first row load and the first vmcnt wait reads or writes a register
  that a row load writes (later loads' address operands included);
* no branch or label sits in that stretch (a join would let the compiler merge values with copies).
"""

from __future__ import annotations

import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CSRC = os.path.join(ROOT, "phyai_amd", "csrc")


def _vgprs(text: str) -> set[int]:
    out: set[int] = set()
    for m in re.finditer(r"v\[(\d+):(\d+)\]", text):
        out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"(?<![\w\[])v(\d+)\b", text):
        out.add(int(m.group(1)))
    return out


@pytest.fixture(scope="module")
def kernels():
    asm = os.path.join(CSRC, "_obj", "gemm_skinny_fused.s")
    r = subprocess.run(["make", "-C", CSRC, "_obj/gemm_skinny_fused.s"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr[-2000:]
    src = open(asm, encoding="utf-8").read()
    parts = re.split(r"\n(?=_Z\w*gemm_fp8_fusedq_kernel\w*:)", src)[1:]
    assert len(parts) >= 100, f"only {len(parts)} instantiations found"
    return parts


def _stretch(kernel: str):
    """instructions from the first row load up to (excluding) the first vmcnt wait"""
    started, body = False, []
    for line in kernel.split("\n")[1:]:
        t = line.strip()
        if not t or t.startswith(";"):
            continue
        is_row_load = t.startswith("global_load_dwordx4") and "lds" not in t.split()[0]
        if not started:
            if is_row_load:
                started = True
                body.append(t)
            continue
        if t.startswith("s_waitcnt") and "vmcnt" in t:
            return body
        body.append(t)
    raise AssertionError("no vmcnt wait after the row loads")


def test_nothing_touches_a_row_load_destination_before_the_wait(kernels):
    for k in kernels:
        name = k.split(":", 1)[0]
        dest: set[int] = set()
        for t in _stretch(k):
            if t.startswith("."):
                continue
            code = t.split(";")[0]
            if t.startswith("global_load_dwordx4") and "lds" not in t.split()[0]:
                ops = code.split(None, 1)[1].split(",")
                assert not (_vgprs(",".join(ops[1:])) & dest), f"{name}: address in flight: {t}"
                dest |= _vgprs(ops[0])
                continue
            assert not (_vgprs(code) & dest), f"{name}: `{t}` touches a register of a row load in flight"
        assert dest, f"{name}: no row load found"


def test_no_control_flow_between_the_row_loads_and_the_wait(kernels):
    for k in kernels:
        name = k.split(":", 1)[0]
        for t in _stretch(k):
            assert not t.startswith(("s_cbranch", "s_branch", "s_setpc", "s_call")), f"{name}: {t}"
            assert not re.match(r"\.LBB\d+_\d+:", t), f"{name}: label {t}"
