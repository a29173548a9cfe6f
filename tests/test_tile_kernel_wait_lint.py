"""The prefill tile kernels issue their global loads as inline assembly and wait
for them with hand-written ``s_waitcnt vmcnt(n)`` (the compiler believes the
results ready at once).  This lint reads the generated gfx950 assembly of those
translation units and checks the one property the scheme rests on: between a
load and the wait that covers it, no instruction reads or writes the load's
destination registers (a register-allocator copy of a half-arrived value, or a
reuse of the registers, would be silent data corruption that a parity test
catches only by luck).

``vmcnt`` completes in order, so "covered" is positional: a wait for ``n``
leaves the youngest ``n`` vector-memory operations outstanding.  The scan is
linear in file order, which is execution order for the straight-line loop
bodies these kernels are made of.  CPU only: hipcc cross-compiles.
"""
import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
CSRC = ROOT / "mlx_amd" / "csrc"
UNITS = ("qmm_mfma.hip", "qmm_mfma_pairs.hip", "qmm_mfma_fp.hip", "qq_mfma.hip")

_REG = re.compile(r"\bv\[(\d+):(\d+)\]|\bv(\d+)\b")


def _regs(text):
    out = set()
    for m in _REG.finditer(text):
        if m.group(1):
            out.update(range(int(m.group(1)), int(m.group(2)) + 1))
        else:
            out.add(int(m.group(3)))
    return out


def lint(asm_text):
    """Returns (functions seen, loads tracked, list of violations)."""
    fn = None
    outstanding = []  # destination register sets of the vector-memory ops in flight, oldest first
    functions = loads = 0
    problems = []
    for ln, line in enumerate(asm_text.splitlines(), 1):
        t = line.strip()
        if not t or t.startswith(";") or t.startswith("."):
            continue
        if re.match(r"^_Z\w+:", t):
            fn, outstanding = t.split(":")[0], []
            functions += 1
            continue
        t = t.split(";")[0].strip()
        if not t:
            continue
        op = t.split()[0]
        args = t[len(op):]
        if op == "s_waitcnt":
            m = re.search(r"vmcnt\((\d+)\)", t)
            if m:
                n = int(m.group(1))
                outstanding = outstanding[-n:] if n else []
            continue
        if op == "s_endpgm":
            outstanding = []
            continue
        live = set().union(*outstanding) if outstanding else set()
        is_vmem = op.startswith(("global_", "buffer_", "flat_", "scratch_"))
        touched = _regs(args)
        if touched & live:
            problems.append(f"{fn} line {ln}: `{t}` touches in-flight v{sorted(touched & live)}")
        if is_vmem:
            if "load" in op and "lds" not in op:
                outstanding.append(_regs(args.split(",")[0]))
                loads += 1
            else:
                outstanding.append(set())  # stores and direct-to-LDS loads: counted, no registers
    return functions, loads, problems


def _assembly(unit):
    cmd = [
        os.environ.get("HIPCC", "hipcc"), "--offload-arch=gfx950", "-O3", "-std=c++17",
        "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
        "-I", str(ROOT / "include"), "-I", str(CSRC), "-S", "--cuda-device-only",
        str(CSRC / unit), "-o", "-",
    ]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    return unit, proc.returncode, proc.stdout, proc.stderr


def test_lint_catches_a_use_before_the_wait():
    bad = """
_Zkernel:
  global_load_dwordx4 v[4:7], v1, s[2:3]
  v_add_u32 v9, v5, v8
  s_waitcnt vmcnt(0)
  s_endpgm
"""
    good = bad.replace("v_add_u32 v9, v5, v8\n  s_waitcnt vmcnt(0)", "s_waitcnt vmcnt(0)\n  v_add_u32 v9, v5, v8")
    assert len(lint(bad)[2]) == 1
    assert lint(good)[2] == []
    # in-order completion: vmcnt(1) covers the older of two loads only
    two = """
_Zkernel:
  global_load_dword v4, v1, s[2:3]
  global_load_dword v5, v1, s[2:3] offset:4
  s_waitcnt vmcnt(1)
  v_mov_b32 v6, v4
  v_mov_b32 v7, v5
  s_endpgm
"""
    assert len(lint(two)[2]) == 1 and "v[5]" in lint(two)[2][0]


@pytest.mark.skipif(shutil.which(os.environ.get("HIPCC", "hipcc")) is None, reason="hipcc not present")
def test_no_load_destination_is_touched_before_its_wait():
    with ThreadPoolExecutor(max_workers=4) as pool:
        results = list(pool.map(_assembly, UNITS))
    for unit, rc, asm, err in results:
        assert rc == 0, f"{unit}:\n{err[-2000:]}"
        functions, loads, problems = lint(asm)
        assert functions > 0, unit
        if unit != "qq_mfma.hip":  # that kernel loads by DMA only: nothing lands in registers
            assert loads > 100, (unit, loads)
        assert not problems, f"{unit}:\n" + "\n".join(problems[:20])
