"""Writes tests/golden/fp_modes_ref.npz from the reference's own code.

Run in a container that has the reference checkout:

    python oracle/build.py            # builds oracle/_ref/libmlx_cpu_qref.so
    python tests/golden/make_fp_golden.py

Every output is produced by the reference translation unit
(mlx/backend/cpu/quantized.cpp compiled as-is): the fp8 converters ``ToFP8`` /
``FromFP8``, ``to_fp8_e8m0``, ``to_fp4_e2m1`` and ``fp_qmm_dispatch_transpose<T,
group_size, bits>`` through raw pointers.  The packed weights and scale bytes
the products read are inputs (written by the oracle's quantizer, stored beside
the outputs).  Data only: seeded inputs and the reference's outputs as raw bit
patterns.
"""
from __future__ import annotations

import os
import struct
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import fp_qref, qref  # noqa: E402

DTYPES = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
MODES = ("mxfp4", "mxfp8", "nvfp4")


def bits_of(t: torch.Tensor) -> np.ndarray:
    t = t.contiguous()
    if t.dtype == torch.uint32:
        return t.numpy().copy()
    if t.dtype == torch.uint8:
        return t.numpy().copy()
    if t.element_size() == 2:
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.view(torch.int32).numpy().view(np.uint32).copy()


def probe_floats() -> np.ndarray:
    """float32 bit patterns: random magnitudes over 40 binades, every e4m3 value
    and every midpoint between neighbours, the e2m1 decision points, specials."""
    rng = np.random.default_rng(0)
    mag = np.exp(rng.uniform(-20.0, 8.0, size=12000)).astype(np.float32)
    sign = np.where(rng.uniform(size=12000) < 0.5, -1.0, 1.0).astype(np.float32)
    table = sorted(set(abs(float(v)) for v in fp_qref._e4m3_values()))
    mids = [(a + b) / 2 for a, b in zip(table, table[1:])]
    e2m1 = [0.0, 0.25, 0.5, 0.75, 1.0, 1.25, 1.5, 1.75, 2.0, 2.5, 3.0, 3.5, 4.0, 5.0, 6.0, 7.0]
    near = [v + e for v in e2m1 for e in (0.0, 1e-6, -1e-6)]
    special = [448.0, 464.0, 465.0, 479.9, 480.0, 1e6, 2.0 ** -10, 2.0 ** -11, 2.0 ** -127, 3e38]
    pos = np.array(table + mids + near + special, dtype=np.float32)
    vals = np.concatenate([mag * sign, pos, -pos])
    return vals.view(np.uint32).copy()


def main() -> int:
    if not qref.reference_built():
        print("oracle/_ref is not built; run python oracle/build.py first", file=sys.stderr)
        return 1
    ref = fp_qref.FpOracle("reference")
    out = {}
    out["from_fp8"] = np.array(
        [np.array([ref.ref.ref_from_fp8(c)], dtype=np.float32).view(np.uint32)[0] for c in range(256)],
        dtype=np.uint32)
    probes = probe_floats()
    out["probe_bits"] = probes
    to_fp8 = np.empty(probes.shape, dtype=np.uint8)
    e8m0 = np.empty(probes.shape, dtype=np.uint8)
    e2m1 = np.empty(probes.shape, dtype=np.uint8)
    for i, u in enumerate(probes):
        f = struct.unpack("f", struct.pack("I", int(u)))[0]
        to_fp8[i] = ref.ref.ref_to_fp8(f)
        e8m0[i] = ref.ref.ref_e8m0(f)
        e2m1[i] = ref.ref.ref_e2m1(f)
    out["to_fp8"], out["e8m0"], out["e2m1"] = to_fp8, e8m0, e2m1

    for mode in MODES:
        gs = fp_qref.GROUP_SIZE[mode]
        for dname, dtype in DTYPES.items():
            for transpose in (True, False):
                tag = f"{mode}_{dname}_{'t' if transpose else 'n'}"
                M, N, K = 3, 2 * 32, 4 * 32
                seed = 100 * MODES.index(mode) + 10 * list(DTYPES).index(dname) + int(transpose)
                g = torch.Generator().manual_seed(seed)
                w = (torch.randn((N, K) if transpose else (K, N), generator=g) * 0.3).to(dtype)
                w.reshape(-1)[: gs] = 0.0  # a zero group
                wq, scales = ref.quantize(w, mode)  # the oracle's quantizer: an input of the product
                x = torch.randn((M, K), generator=g).to(dtype)
                y = ref.qmm(x, wq, scales, mode, transpose)
                out[tag + "_wq"] = bits_of(wq)
                out[tag + "_scales"] = bits_of(scales)
                out[tag + "_x"] = bits_of(x)
                out[tag + "_y"] = bits_of(y)
    np.savez_compressed(os.path.join(HERE, "fp_modes_ref.npz"), **out)
    print("wrote fp_modes_ref.npz:", len(out), "arrays")
    return 0


if __name__ == "__main__":
    sys.exit(main())
