"""Writes the golden vectors under tests/golden/ from the reference's own code.

Run in a container that has the reference checkout:

    python oracle/build.py            # builds oracle/_ref/libmlx_cpu_qref.so
    python tests/golden/make_golden.py

Every output below is produced by the reference translation unit
(mlx/backend/cpu/quantized.cpp compiled as-is): ``quantize<T,U>`` and the
pointer overload of ``_qmm_dispatch_typed<T>``, plus the reference's software
float16 / bfloat16 conversions.  The fixtures are data only: seeded inputs and
the reference's outputs, stored as raw bit patterns in ``.npz`` files.
"""
from __future__ import annotations

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from oracle import qref  # noqa: E402

DTYPES = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}
BITS = (2, 3, 4, 5, 6, 8)
GROUPS = (32, 64, 128)


def bits_of(t: torch.Tensor) -> np.ndarray:
    t = t.contiguous()
    if t.dtype == torch.uint32:
        return t.numpy().copy()
    if t.element_size() == 2:
        return t.view(torch.int16).numpy().view(np.uint16).copy()
    return t.view(torch.int32).numpy().view(np.uint32).copy()


def weights(seed: int, shape, dtype) -> torch.Tensor:
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(shape, generator=g) * 0.02
    # a few special groups: zeros, constant, one spike, tiny range
    w[0, :32] = 0.0
    w[1, :32] = 0.5
    w[2, :64] = 0.0
    w[2, 7] = -1.25
    w[3, :32] = torch.linspace(-3e-8, 2e-8, 32)
    return w.to(dtype)


def main() -> int:
    if not qref.reference_built():
        print("oracle/_ref is not built; run python oracle/build.py first", file=sys.stderr)
        return 1
    ref = qref.Oracle("reference")
    assert ref.ref.ref_simd_max_size(0) == 1  # scalar path, as on any x86 build

    out = {}
    for dname, dtype in DTYPES.items():
        for bits in BITS:
            for gs in GROUPS:
                tag = f"{dname}_b{bits}_g{gs}"
                seed = bits * 1000 + gs
                w = weights(seed, (6, 256), dtype)
                wq, s, b = ref.quantize(w, gs, bits)
                g = torch.Generator().manual_seed(seed + 1)
                x = torch.randn((3, 256), generator=g).to(dtype)
                y_t = ref.qmm(x, wq, s, b, True, gs, bits)
                # transpose=false: the same packed array read as [K=6, N=256]
                x_n = torch.randn((2, 6), generator=g).to(dtype)
                y_n = ref.qmm(x_n, wq, s, b, False, gs, bits)
                out[tag + "_w"] = bits_of(w)
                out[tag + "_wq"] = bits_of(wq)
                out[tag + "_scales"] = bits_of(s)
                out[tag + "_biases"] = bits_of(b)
                out[tag + "_x"] = bits_of(x)
                out[tag + "_y_t"] = bits_of(y_t)
                out[tag + "_xn"] = bits_of(x_n)
                out[tag + "_y_n"] = bits_of(y_n)
    np.savez_compressed(os.path.join(HERE, "affine_quantized_ref.npz"), **out)

    # software half types of the reference: every binary16 value widened, and a
    # sample of float32 bit patterns narrowed to both 16-bit types
    rng = np.random.default_rng(0)
    f32_bits = np.concatenate([
        rng.integers(0, 2**32, size=20000, dtype=np.uint64).astype(np.uint32),
        np.array([0, 0x80000000, 0x7F800000, 0xFF800000, 0x7FC00000, 0x00000001,
                  0x007FFFFF, 0x00800000, 0x33000000, 0x33000001, 0x32FFFFFF,
                  0x387FC000, 0x387FE000, 0x38800000, 0x477FE000, 0x477FEFFF,
                  0x477FF000, 0x47800000, 0x3F808000, 0x3F818000, 0x3F800001],
                 dtype=np.uint32),
    ])
    f16_out = np.empty(f32_bits.shape, dtype=np.uint16)
    bf16_out = np.empty(f32_bits.shape, dtype=np.uint16)
    for i, u in enumerate(f32_bits):
        f = float(np.array([u], dtype=np.uint32).view(np.float32)[0])
        f16_out[i] = ref.ref.ref_f16_from_f32(f)
        bf16_out[i] = ref.ref.ref_bf16_from_f32(f)
    widen = np.empty(65536, dtype=np.uint32)
    for h in range(65536):
        widen[h] = np.array([ref.ref.ref_f16_to_f32(h)], dtype=np.float32).view(np.uint32)[0]
    np.savez_compressed(
        os.path.join(HERE, "half_types_ref.npz"),
        f32_bits=f32_bits, f16_from_f32=f16_out, bf16_from_f32=bf16_out, f16_to_f32=widen,
    )
    print("wrote", os.listdir(HERE))
    return 0


if __name__ == "__main__":
    sys.exit(main())
