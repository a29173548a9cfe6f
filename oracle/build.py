"""Build recipe for the parity oracle (test infrastructure only).

  python oracle/build.py          # both targets (the second only if possible)

* ``oracle/libaffine_qref.so``  -- this repository's C restatement
  (``affine_qref.c`` and, for the floating-point modes, ``fp_qref.c``), always
  buildable with gcc.
* ``oracle/_ref/libmlx_cpu_qref.so`` -- the reference's own
  ``mlx/backend/cpu/quantized.cpp`` compiled as a single translation unit from
  where it lies in the reference checkout (``ref_harness.cpp`` includes it).
  Only possible where that checkout exists; the built library is kept out of
  git history and is used to validate the restatement and as the
  ``"reference"`` CPU baseline.
"""
from __future__ import annotations

import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE_ROOT = os.environ.get("MLX_REFERENCE_ROOT", "/root/reference")

QREF_SO = os.path.join(HERE, "libaffine_qref.so")
REF_DIR = os.path.join(HERE, "_ref")
REF_SO = os.path.join(REF_DIR, "libmlx_cpu_qref.so")


def _run(cmd):
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(
            "command failed: %s\n%s\n%s" % (" ".join(cmd), proc.stdout, proc.stderr)
        )


def build_qref() -> str:
    """Compile the C restatement.  No FMA contraction: the reference's scalar
    x86 build evaluates every multiply and add separately."""
    _run(
        [
            "gcc", "-std=c11", "-O3", "-fPIC", "-shared", "-ffp-contract=off",
            "-fno-fast-math", "-Wall", "-Wextra",
            os.path.join(HERE, "affine_qref.c"), os.path.join(HERE, "fp_qref.c"),
            "-lm", "-o", QREF_SO,
        ]
    )
    return QREF_SO


def reference_available() -> bool:
    return os.path.isfile(
        os.path.join(REFERENCE_ROOT, "mlx", "backend", "cpu", "quantized.cpp")
    )


def build_ref() -> str | None:
    """Compile the reference translation unit, if the checkout is present."""
    if not reference_available():
        return None
    os.makedirs(REF_DIR, exist_ok=True)
    _run(
        [
            "g++", "-std=c++20", "-O3", "-fPIC", "-shared", "-fvisibility=hidden",
            "-ffunction-sections", "-fdata-sections", "-ffp-contract=off",
            "-I", REFERENCE_ROOT,
            os.path.join(HERE, "ref_harness.cpp"),
            "-Wl,--gc-sections",
            "-Wl,--version-script=" + os.path.join(HERE, "ref_exports.map"),
            "-o", REF_SO,
        ]
    )
    return REF_SO


def main() -> int:
    print("built", build_qref())
    ref = build_ref()
    print("built" if ref else "skipped (no reference checkout):", ref or REF_SO)
    return 0


if __name__ == "__main__":
    sys.exit(main())
