"""Helpers shared by the GGUF tests: block construction as in the reference's
known-answer test (python/tests/test_load.py:203-281) and a minimal GGUF v3
writer."""
from __future__ import annotations

import struct

import numpy as np

Q4_0, Q4_1, Q8_0 = 2, 3, 8
BITS = {Q4_0: 4, Q4_1: 4, Q8_0: 8}


def packed_nibbles(q):
    # GGML nibble order: byte j = element j | element j + 16 << 4
    return (q[:, :16] | (q[:, 16:] << 4)).astype(np.uint8)


def make_blocks(ggml_type, n_blocks, rng, d=None, m=None):
    """Random GGML blocks.  Returns (blocks uint8 [n, block_bytes], expected
    float32 [n, 32]) with expected = d (q - 8) | d q + m | d q computed from the
    float16 d, m in float32 -- what the format prescribes."""
    if d is None:
        d = (rng.standard_normal((n_blocks, 1)) * 0.05).astype(np.float16)
    if m is None:
        m = (rng.standard_normal((n_blocks, 1)) * 0.1).astype(np.float16)
    d32, m32 = d.astype(np.float32), m.astype(np.float32)
    if ggml_type == Q8_0:
        q8 = rng.integers(-128, 128, size=(n_blocks, 32)).astype(np.int8)
        blocks = np.concatenate([d.view(np.uint8), q8.view(np.uint8)], axis=1)
        return blocks, d32 * q8.astype(np.float32)
    q4 = rng.integers(0, 16, size=(n_blocks, 32)).astype(np.uint8)
    if ggml_type == Q4_0:
        blocks = np.concatenate([d.view(np.uint8), packed_nibbles(q4)], axis=1)
        return blocks, d32 * (q4.astype(np.float32) - 8)
    blocks = np.concatenate([d.view(np.uint8), m.view(np.uint8), packed_nibbles(q4)], axis=1)
    return blocks, d32 * q4.astype(np.float32) + m32


def write_gguf(path, tensors, metadata=(), alignment=None):
    """tensors: list of (name, shape (row-major), ggml_type_id, bytes);
    metadata: list of (key, value_type_id, packed value bytes)."""
    with open(path, "wb") as f:
        f.write(b"GGUF")
        f.write(struct.pack("<IQQ", 3, len(tensors), len(metadata)))
        for key, vtype, payload in metadata:
            k = key.encode()
            f.write(struct.pack("<Q", len(k)) + k + struct.pack("<I", vtype) + payload)
        offset = 0
        align = alignment or 32
        offsets = []
        for name, shape, type_id, data in tensors:
            nm = name.encode()
            f.write(struct.pack("<Q", len(nm)) + nm)
            dims = list(reversed(shape))  # GGML order: innermost first
            f.write(struct.pack("<I", len(dims)))
            for dim in dims:
                f.write(struct.pack("<Q", dim))
            f.write(struct.pack("<IQ", type_id, offset))
            offsets.append(offset)
            offset += (len(data) + align - 1) // align * align
        f.write(b"\x00" * (-f.tell() % align))
        base = f.tell()
        for (name, shape, type_id, data), off in zip(tensors, offsets):
            f.write(b"\x00" * (base + off - f.tell()))
            f.write(data)


def dequantize_np(wq, scales, biases, bits):
    """Closed form of the affine dequantize in float16 with two roundings
    (mlx/ops.cpp:5320-5324) for bits 4 / 8, group size 32."""
    wq = np.asarray(wq, dtype=np.uint32)
    per_word = 32 // bits
    shifts = (bits * np.arange(per_word)).astype(np.uint32)
    codes = (wq[..., None] >> shifts) & np.uint32((1 << bits) - 1)
    codes = codes.reshape(wq.shape[:-1] + (wq.shape[-1] * per_word,)).astype(np.float16)
    s = np.repeat(np.asarray(scales, dtype=np.float16), 32, axis=-1)
    b = np.repeat(np.asarray(biases, dtype=np.float16), 32, axis=-1)
    return ((codes * s).astype(np.float16) + b).astype(np.float16)
