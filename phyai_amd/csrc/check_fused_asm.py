"""Build-time guard for gemm_skinny_fused.hip.

That kernel loads its activation rows (and, in one variant, row maxima handed over by an earlier launch)
with inline-assembly loads the compiler cannot see: between such a load and the ``s_waitcnt vmcnt(N)`` that
covers it the destination registers hold nothing yet.  A copy or any other use the compiler schedules there
reads stale registers, and the data that lands later overwrites whatever the registers were reused for -
addresses included, which faults the GPU.  The wait itself is counted by hand: ``N`` must be the number of
vector-memory instructions issued after the last such load, or registers are read before they are filled.

``check_file`` reads the gfx950 assembly of the file (``make _obj/gemm_skinny_fused.s``; no GPU needed) and
returns a list of violations over every instantiation of the kernel:

* an instruction between the first invisible load and the first vmcnt wait reads or writes a register that
  such a load writes (later loads' address operands included);
* a branch or a label sits in that stretch (a join would let the compiler merge values with copies);
* the number of vector-memory instructions between the last invisible load and that wait differs from the
  wait's ``N``;
* the kernel uses scratch memory (a spilled register in that stretch could be one of the loads').

``check_tile_usage`` is the guard of gemm_big.hip, whose global -> LDS copies are inline assembly too and whose
``s_waitcnt vmcnt(N)`` count, by hand, the vector-memory instructions of a wavefront in issue order: a kernel of that
file that spills has scratch loads and stores of the compiler's among them, and a wait would then let a stage be
read before it has landed.  It reads the compiler's resource-usage remarks that the Makefile keeps beside every
object (``_obj/gemm_big.o.usage``) and reports every instantiation with a scratch size other than zero.
"""

from __future__ import annotations

import os
import re
import subprocess

CSRC = os.path.dirname(os.path.abspath(__file__))
ASM = os.path.join(CSRC, "_obj", "gemm_skinny_fused.s")
KERNEL = r"_Z\w*gemm_fp8_fusedq_kernel\w*"
_VMEM = ("global_", "buffer_", "flat_", "scratch_")


def _vgprs(text: str) -> set[int]:
    out: set[int] = set()
    for m in re.finditer(r"v\[(\d+):(\d+)\]", text):
        out |= set(range(int(m.group(1)), int(m.group(2)) + 1))
    for m in re.finditer(r"(?<![\w\[])v(\d+)\b", text):
        out.add(int(m.group(1)))
    return out


def _is_invisible_load(t: str) -> bool:
    """The inline-assembly loads are the only plain `global_load_dwordx4` with an SGPR base and a VGPR offset that
    come before the first wait; the compiler's own weight loads in the same stretch are told apart by order: the
    invisible ones come first (they are issued first in the source)."""
    return t.startswith("global_load_dwordx4") and "lds" not in t.split()[0]


def kernels_of(asm_text: str) -> list[str]:
    return re.split(r"\n(?=" + KERNEL + r":)", asm_text)[1:]


def stretch(kernel: str) -> tuple[list[str], int]:
    """Instructions from the first 16-byte global load up to (excluding) the first vmcnt wait, and that wait's N."""
    started, body = False, []
    for line in kernel.split("\n")[1:]:
        t = line.strip()
        if not t or t.startswith(";"):
            continue
        if not started:
            if _is_invisible_load(t):
                started = True
                body.append(t)
            continue
        if t.startswith("s_waitcnt") and "vmcnt" in t:
            return body, int(re.search(r"vmcnt\((\d+)\)", t).group(1))
        body.append(t)
    raise AssertionError("no vmcnt wait after the row loads")


def check_kernel(kernel: str, younger_loads_are_rows: int) -> list[str]:
    """`younger_loads_are_rows`: how many 16-byte global loads at the head of the stretch are the invisible ones
    (the rest, if any, are the compiler's own weight loads into registers)."""
    name = kernel.split(":", 1)[0]
    bad: list[str] = []
    body, waited = stretch(kernel)
    dest: set[int] = set()
    seen_rows, after_last = 0, 0
    for t in body:
        if t.startswith("."):
            if re.match(r"\.LBB\d+_\d+:", t):
                bad.append(f"{name}: label {t} between the row loads and their wait")
            continue
        code = t.split(";")[0]
        if t.startswith(("s_cbranch", "s_branch", "s_setpc", "s_call")):
            bad.append(f"{name}: {t} between the row loads and their wait")
        if _is_invisible_load(t) and seen_rows < younger_loads_are_rows:
            ops = code.split(None, 1)[1].split(",")
            if _vgprs(",".join(ops[1:])) & dest:
                bad.append(f"{name}: address register of `{t}` is the destination of a load in flight")
            dest |= _vgprs(ops[0])
            seen_rows += 1
            after_last = 0
            continue
        if _vgprs(code) & dest:
            bad.append(f"{name}: `{t}` touches a register of a row load in flight")
        if t.startswith(_VMEM):
            after_last += 1
    if seen_rows != younger_loads_are_rows:
        bad.append(f"{name}: {seen_rows} invisible loads found, {younger_loads_are_rows} expected")
    if after_last != waited:
        bad.append(f"{name}: {after_last} vector-memory instructions follow the last row load, the wait says vmcnt({waited})")
    if re.search(r"^\s*scratch_", kernel, flags=re.M):
        bad.append(f"{name}: uses scratch memory")
    return bad


def rows_loaded(name: str) -> int:
    """Invisible loads of an instantiation, from its template arguments in the mangled name:
    <ROWS, NT, KPW, EPI, STREAM, DIRECT, AMAX_IN>: KPW x ceil(ROWS / 4) row loads (at most 4 per 16-row block)
    plus ceil(ROWS / 8) loads of handed-over maxima."""
    m = re.search(r"ILi(\d+)ELi(\d+)ELi(\d+)ELi(\d+)ELb([01])ELb([01])ELb([01])E", name)
    if not m:
        raise AssertionError(f"cannot read the template arguments of {name}")
    rows, _, kpw, _, _, _, amax_in = (int(g) for g in m.groups())
    per_step = sum(min(4, (min(16, rows - 16 * mb) + 3) // 4) for mb in range((rows + 15) // 16))
    return kpw * per_step + (((rows + 7) // 8) if amax_in else 0)


def check_text(asm_text: str, min_kernels: int = 100) -> list[str]:
    ks = kernels_of(asm_text)
    bad = [] if len(ks) >= min_kernels else [f"only {len(ks)} instantiations of the kernel found"]
    for k in ks:
        name = k.split(":", 1)[0]
        try:
            bad += check_kernel(k, rows_loaded(name))
        except AssertionError as e:
            bad.append(f"{name}: {e}")
    return bad


def check_file(make: bool = True, stamps: bool = False) -> list[str]:
    """stamps: the debug build with time stamps (make stamps), whose kernels must obey the same rules."""
    target = "_obj/stamps_gemm_skinny_fused.s" if stamps else "_obj/gemm_skinny_fused.s"
    if make:
        r = subprocess.run(["make", "-C", CSRC, target], capture_output=True, text=True)
        if r.returncode != 0:
            return [f"make {target} failed: {r.stderr[-2000:]}"]
    return check_text(open(os.path.join(CSRC, target), encoding="utf-8").read())


def usage_problems(text: str, kernel: str = "gemm_fp8_big_kernel", min_kernels: int = 50) -> list[str]:
    """Kernels named `kernel` whose resource-usage remarks (-Rpass-analysis=kernel-resource-usage) show scratch."""
    bad, seen, name = [], 0, None
    for line in text.split("\n"):
        m = re.search(r"remark: Function Name: (\S+)", line)
        if m:
            name = m.group(1) if kernel in m.group(1) else None
            seen += name is not None
            continue
        m = re.search(r"remark:\s+ScratchSize \[bytes/lane\]: (\d+)", line)
        if m and name is not None and int(m.group(1)) != 0:
            bad.append(f"{name}: {m.group(1)} bytes of scratch per lane")
    if seen < min_kernels:
        bad.append(f"only {seen} instantiations of {kernel} found in the resource-usage remarks")
    return bad


def check_tile_usage(stamps: bool = False) -> list[str]:
    """The pipelined tile kernels of the built library (or of the time-stamp build) use no scratch memory."""
    path = os.path.join(CSRC, "_obj", ("stamps_" if stamps else "") + "gemm_big.o.usage")
    if not os.path.exists(path):
        return [f"{path} is missing (make -C {CSRC} all stamps writes it)"]
    return usage_problems(open(path, encoding="utf-8", errors="replace").read())


if __name__ == "__main__":
    import sys

    problems = check_file(stamps="--stamps" in sys.argv) + check_tile_usage(stamps="--stamps" in sys.argv)
    for p in problems[:50]:
        print(p)
    print(f"{len(problems)} problem(s)")
    raise SystemExit(1 if problems else 0)
