"""CPU restatement of the GGUF block -> affine triplet conversion (test
infrastructure only: tests, the smoke check and the benchmark's cpu_baseline
leg may import this module, nothing else).

Follows mlx/io/gguf_quants.cpp: ``unpack_32_4`` (:13-31), ``extract_q4_0_data``
(:33-52), ``extract_q4_1_data`` (:54-74), ``extract_q8_0_data`` (:76-100) and
the shapes of ``gguf_load_quantized`` (:102-166).  That file needs gguflib (a
dependency the reference's build downloads) and MLX's array type, so it is
not compiled here; the restatement is pinned by the reference's own
known-answer test (python/tests/test_load.py:203-281: a loaded Q4_0 / Q4_1 /
Q8_0 tensor dequantizes to d (q - 8), d q + m, d q) and by the nibble order
that test states (byte j = element j | element j + 16 << 4).
"""
from __future__ import annotations

import numpy as np

Q4_0, Q4_1, Q8_0 = 2, 3, 8  # GGML type ids as stored in a GGUF file

BLOCK_BYTES = {Q4_0: 18, Q4_1: 20, Q8_0: 34}
BITS = {Q4_0: 4, Q4_1: 4, Q8_0: 8}
WEIGHTS_PER_BLOCK = 32


def repack(blocks: np.ndarray, ggml_type: int):
    """blocks: uint8 [n_blocks, BLOCK_BYTES] -> (wq uint32 [n_blocks, 4 | 8],
    scales fp16 [n_blocks], biases fp16 [n_blocks]); group size 32."""
    if ggml_type not in BLOCK_BYTES:
        raise ValueError(f"GGML type {ggml_type} is not kept quantized")
    blocks = np.ascontiguousarray(blocks, dtype=np.uint8).reshape(-1, BLOCK_BYTES[ggml_type])
    n = blocks.shape[0]
    d = blocks[:, 0:2].copy().view(np.float16).reshape(n)
    if ggml_type == Q4_1:
        biases = blocks[:, 2:4].copy().view(np.float16).reshape(n)
        q = blocks[:, 4:]
    else:
        # float16 * int is evaluated in float and rounded back (exact here)
        factor = -8.0 if ggml_type == Q4_0 else -128.0
        with np.errstate(over="ignore", invalid="ignore"):
            biases = (d.astype(np.float32) * np.float32(factor)).astype(np.float16)
        q = blocks[:, 2:]
    if ggml_type == Q8_0:
        codes = q ^ np.uint8(0x80)  # int8 + 128
        wq = codes.copy().view("<u4").reshape(n, 8)
    else:
        lo = q & np.uint8(0x0F)  # elements 0..15
        hi = q >> np.uint8(4)    # elements 16..31
        elems = np.concatenate([lo, hi], axis=1).astype(np.uint32)  # [n, 32] in element order
        shifts = (4 * (np.arange(32) % 8)).astype(np.uint32)
        wq = (elems << shifts).reshape(n, 4, 8).sum(axis=2, dtype=np.uint32)
    return wq.astype(np.uint32), d.copy(), biases


def triplet_shapes(shape, ggml_type: int):
    """Shapes of (weight, scales, biases) for a GGUF tensor of logical `shape`
    (gguf_quants.cpp:113-137)."""
    shape = tuple(int(s) for s in shape)
    if shape[-1] % WEIGHTS_PER_BLOCK != 0:
        raise ValueError(f"last dim {shape[-1]} is not a multiple of {WEIGHTS_PER_BLOCK}")
    per_word = 32 // BITS[ggml_type]
    return (
        shape[:-1] + (shape[-1] // per_word,),
        shape[:-1] + (shape[-1] // WEIGHTS_PER_BLOCK,),
        shape[:-1] + (shape[-1] // WEIGHTS_PER_BLOCK,),
    )
