"""The GGUF repack oracle against the reference's known-answer test and a
literal loop form of its nibble shuffle; the GGUF header parser.  No GPU."""
import struct

import numpy as np
import pytest

from oracle import gguf_ref

from gguf_util import BITS, Q4_0, Q4_1, Q8_0, dequantize_np, make_blocks, packed_nibbles, write_gguf


def test_known_answer_of_the_reference_test():
    # python/tests/test_load.py:203-281: rows, cols = 2, 64; seed 7; d = 0.5, m = -1.25
    rows, cols = 2, 64
    n_blocks = rows * cols // 32
    np.random.seed(7)
    d = np.full((n_blocks, 1), 0.5, dtype=np.float16)
    m = np.full((n_blocks, 1), -1.25, dtype=np.float16)
    q4 = np.random.randint(0, 16, size=(n_blocks, 32)).astype(np.uint8)
    q8 = np.random.randint(-128, 128, size=(n_blocks, 32)).astype(np.int8)
    d32, m32 = d.astype(np.float32), m.astype(np.float32)
    cases = [
        (Q4_0, np.concatenate([d.view(np.uint8), packed_nibbles(q4)], axis=1), d32 * (q4.astype(np.float32) - 8)),
        (Q4_1, np.concatenate([d.view(np.uint8), m.view(np.uint8), packed_nibbles(q4)], axis=1),
         d32 * q4.astype(np.float32) + m32),
        (Q8_0, np.concatenate([d.view(np.uint8), q8.view(np.uint8)], axis=1), d32 * q8.astype(np.float32)),
    ]
    for ggml_type, blocks, expected in cases:
        wq, scales, biases = gguf_ref.repack(blocks, ggml_type)
        w_shape, s_shape, b_shape = gguf_ref.triplet_shapes((rows, cols), ggml_type)
        assert wq.dtype == np.uint32 and wq.size == np.prod(w_shape)
        assert s_shape == (rows, cols // 32) and b_shape == (rows, cols // 32)
        deq = dequantize_np(wq.reshape(w_shape), scales.reshape(s_shape), biases.reshape(b_shape), BITS[ggml_type])
        assert np.array_equal(deq.astype(np.float32), expected.reshape(rows, cols))


def _unpack_32_4_loops(data):
    # the two loops of mlx/io/gguf_quants.cpp:13-31, byte for byte
    dst = [0] * 16
    for j in range(16):
        x = data[j] & 0x0F
        if j % 2 != 0:
            x = (x << 4) & 0xFF
        dst[j // 2] = (dst[j // 2] + x) & 0xFF
    for j in range(16):
        x = data[j] >> 4
        if j % 2 != 0:
            x = (x << 4) & 0xFF
        dst[8 + j // 2] = (dst[8 + j // 2] + x) & 0xFF
    return bytes(dst)


@pytest.mark.parametrize("ggml_type", [Q4_0, Q4_1])
def test_nibble_shuffle_matches_the_loop_form(ggml_type):
    rng = np.random.default_rng(3)
    blocks, _ = make_blocks(ggml_type, 37, rng)
    wq, scales, biases = gguf_ref.repack(blocks, ggml_type)
    header = 2 if ggml_type == Q4_0 else 4
    for i in range(blocks.shape[0]):
        want = _unpack_32_4_loops(bytes(blocks[i, header:]))
        assert wq[i].astype("<u4").tobytes() == want
        d = blocks[i, 0:2].copy().view(np.float16)[0]
        assert scales[i] == d
        if ggml_type == Q4_0:
            assert biases[i] == np.float16(-8) * d
        else:
            assert biases[i] == blocks[i, 2:4].copy().view(np.float16)[0]


def test_q8_0_codes_are_int8_plus_128():
    rng = np.random.default_rng(5)
    blocks, expected = make_blocks(Q8_0, 19, rng)
    wq, scales, biases = gguf_ref.repack(blocks, Q8_0)
    codes = wq.astype("<u4").view(np.uint8).reshape(19, 32).astype(np.int32)
    q8 = blocks[:, 2:].view(np.int8).astype(np.int32)
    assert np.array_equal(codes, q8 + 128)
    assert np.array_equal(biases, (scales.astype(np.float32) * -128).astype(np.float16))
    deq = dequantize_np(wq, scales[:, None], biases[:, None], 8).astype(np.float32)
    # d q is exact in float32; the float16 affine form T(T(code) d) - 128 d rounds
    # twice at magnitudes up to 255 |d|: half an ulp (2^-11 relative) each time
    bound = 2.0 ** -10 * 256 * np.abs(scales.astype(np.float32))[:, None]
    assert np.all(np.abs(deq - expected) <= bound)


def test_rejects_other_types_and_ragged_rows():
    with pytest.raises(ValueError):
        gguf_ref.repack(np.zeros((1, 18), np.uint8), 12)
    with pytest.raises(ValueError):
        gguf_ref.triplet_shapes((4, 48), Q4_0)


def test_header_parser(tmp_path):
    from mlx_amd import gguf

    rng = np.random.default_rng(0)
    blocks, _ = make_blocks(Q4_1, 6, rng)
    f32 = rng.standard_normal((3, 5)).astype(np.float32)
    name_kv = ("general.name", 8, struct.pack("<Q", 4) + b"tiny")
    arr_kv = ("tokenizer.scores", 9, struct.pack("<IQ", 6, 3) + struct.pack("<3f", 1.0, 2.0, 3.0))
    u32_kv = ("general.alignment", 4, struct.pack("<I", 64))
    path = tmp_path / "t.gguf"
    write_gguf(
        path,
        [("blk.0.weight", (3, 64), Q4_1, blocks.tobytes()), ("norm.weight", (3, 5), 0, f32.tobytes())],
        metadata=[name_kv, arr_kv, u32_kv],
        alignment=64,
    )
    buf = path.read_bytes()
    metadata, tensors, data_offset = gguf.read_header(buf)
    assert metadata == {"general.name": "tiny", "tokenizer.scores": [1.0, 2.0, 3.0], "general.alignment": 64}
    assert data_offset % 64 == 0
    (n0, s0, t0, o0), (n1, s1, t1, o1) = tensors
    assert (n0, s0, t0, o0) == ("blk.0.weight", (3, 64), Q4_1, 0)
    assert (n1, s1, t1) == ("norm.weight", (3, 5), 0) and o1 % 64 == 0
    assert buf[data_offset + o0: data_offset + o0 + blocks.size] == blocks.tobytes()
    assert np.array_equal(np.frombuffer(buf, np.float32, 15, data_offset + o1).reshape(3, 5), f32)
    with pytest.raises(ValueError):
        gguf.read_header(b"GGML" + buf[4:])
    with pytest.raises(ValueError):
        gguf.read_header(buf[:40])
