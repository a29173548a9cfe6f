"""GGUF Q4_0 / Q4_1 / Q8_0 -> affine triplet on the GPU: bit-exact against the
CPU oracle, the reference's known-answer test end to end (file -> load ->
dequantize), and the repacked weights in a quantized matmul."""
import numpy as np
import pytest
import torch

import mlx_amd
from mlx_amd import gguf
from oracle import gguf_ref

from gguf_util import BITS, Q4_0, Q4_1, Q8_0, make_blocks, packed_nibbles, write_gguf

pytestmark = pytest.mark.gpu

TYPES = (Q4_0, Q4_1, Q8_0)


def _repack_gpu(blocks, ggml_type, shape):
    dev_blocks = torch.from_numpy(blocks.reshape(-1).copy()).cuda()
    w, s, b = gguf.repack(dev_blocks, ggml_type, shape)
    torch.cuda.synchronize()
    return w.cpu().numpy(), s.cpu().numpy(), b.cpu().numpy()


@pytest.mark.parametrize("ggml_type", TYPES)
@pytest.mark.parametrize("n_blocks", [1, 7, 255, 256, 257, 1000, 70001])
def test_repack_bit_exact(ggml_type, n_blocks):
    rng = np.random.default_rng(100 + n_blocks)
    blocks, _ = make_blocks(ggml_type, n_blocks, rng)
    # a few extreme scales: zero, subnormal, largest finite, infinity
    extremes = np.array([0x0000, 0x8000, 0x0001, 0x03FF, 0x7BFF, 0xFBFF, 0x7C00], dtype=np.uint16)
    k = min(n_blocks, extremes.size)
    blocks[:k, 0:2] = extremes[:k].view(np.uint8).reshape(k, 2)
    want_w, want_s, want_b = gguf_ref.repack(blocks, ggml_type)
    got_w, got_s, got_b = _repack_gpu(blocks, ggml_type, (n_blocks, 32))
    assert got_w.dtype == np.uint32 and got_s.dtype == np.float16
    assert np.array_equal(got_w.reshape(want_w.shape), want_w)
    assert np.array_equal(got_s.reshape(-1).view(np.uint16), want_s.view(np.uint16))
    assert np.array_equal(got_b.reshape(-1).view(np.uint16), want_b.view(np.uint16))


def test_known_answer_file_round_trip(tmp_path):
    # python/tests/test_load.py:203-281, through this package's loader and kernels
    rows, cols = 2, 64
    n_blocks = rows * cols // 32
    np.random.seed(7)
    d = np.full((n_blocks, 1), 0.5, dtype=np.float16)
    m = np.full((n_blocks, 1), -1.25, dtype=np.float16)
    q4 = np.random.randint(0, 16, size=(n_blocks, 32)).astype(np.uint8)
    q8 = np.random.randint(-128, 128, size=(n_blocks, 32)).astype(np.int8)
    d32, m32 = d.astype(np.float32), m.astype(np.float32)
    cases = [
        ("Q4_0", Q4_0, np.concatenate([d.view(np.uint8), packed_nibbles(q4)], axis=1),
         d32 * (q4.astype(np.float32) - 8)),
        ("Q4_1", Q4_1, np.concatenate([d.view(np.uint8), m.view(np.uint8), packed_nibbles(q4)], axis=1),
         d32 * q4.astype(np.float32) + m32),
        ("Q8_0", Q8_0, np.concatenate([d.view(np.uint8), q8.view(np.uint8)], axis=1),
         d32 * q8.astype(np.float32)),
    ]
    for name, type_id, blocks, expected in cases:
        path = tmp_path / f"quant_{name}.gguf"
        write_gguf(path, [("tensor.weight", (rows, cols), type_id, blocks.tobytes())])
        arrays, metadata = gguf.load_gguf(path)
        assert metadata == {}
        assert arrays["tensor.weight"].dtype == torch.uint32
        assert tuple(arrays["tensor.scales"].shape) == (rows, cols // 32)
        assert tuple(arrays["tensor.biases"].shape) == (rows, cols // 32)
        deq = mlx_amd.dequantize(
            arrays["tensor.weight"], arrays["tensor.scales"], arrays["tensor.biases"],
            group_size=32, bits=BITS[type_id],
        )
        assert np.array_equal(deq.float().cpu().numpy(), expected.reshape(rows, cols))


def test_loader_mixed_file_and_errors(tmp_path):
    rng = np.random.default_rng(11)
    blocks, _ = make_blocks(Q4_0, 8 * 4, rng)
    f16 = rng.standard_normal((8,)).astype(np.float16)
    path = tmp_path / "m.gguf"
    write_gguf(path, [("l.weight", (8, 128), Q4_0, blocks.tobytes()), ("l.bias", (8,), 1, f16.tobytes())])
    arrays, _ = gguf.load_gguf(path)
    assert sorted(arrays) == ["l.bias", "l.biases", "l.scales", "l.weight"]
    assert np.array_equal(arrays["l.bias"].cpu().numpy(), f16)
    assert tuple(arrays["l.weight"].shape) == (8, 16)
    # a type the loader would have to dequantize (Q5_0 = 6) is refused by name
    bad = tmp_path / "bad.gguf"
    write_gguf(bad, [("x.weight", (1, 32), 6, b"\x00" * 22)])
    with pytest.raises(RuntimeError, match="GGML type 6"):
        gguf.load_gguf(bad)
    # last dim not a multiple of 32 (gguf_quants.cpp:115-120)
    ragged = tmp_path / "ragged.gguf"
    write_gguf(ragged, [("x.weight", (2, 16), Q4_0, b"\x00" * 18)])
    with pytest.raises(RuntimeError, match="incompatible last dim"):
        gguf.load_gguf(ragged)
    # two tensors that map to the same scales name
    dup = tmp_path / "dup.gguf"
    write_gguf(dup, [("a.weight", (1, 32), Q4_0, blocks[:1].tobytes()),
                     ("a.scales", (1,), 0, np.zeros(1, np.float32).tobytes())])
    with pytest.raises(RuntimeError, match="Duplicate parameter name"):
        gguf.load_gguf(dup)


@pytest.mark.parametrize("ggml_type", TYPES)
def test_repacked_weights_in_a_matmul(ggml_type):
    # y = x W^T with W given by the block format's own formula, in float64
    N, K, M = 96, 256, 5
    rng = np.random.default_rng(21)
    blocks, expected = make_blocks(ggml_type, N * K // 32, rng)
    w, s, b = gguf.repack(torch.from_numpy(blocks.reshape(-1).copy()).cuda(), ggml_type, (N, K))
    x = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float16)).cuda()
    y = mlx_amd.quantized_matmul(x, w, s, b, transpose=True, group_size=32, bits=BITS[ggml_type])
    want = x.double().cpu().numpy() @ expected.reshape(N, K).astype(np.float64).T
    wmax = np.abs(expected).max()
    tol = 2e-2 * np.sqrt(K) * float(x.abs().max()) * wmax
    assert np.abs(y.double().cpu().numpy() - want).max() <= tol


def test_full_size_layer_matches_oracle():
    # a 14336 x 4096 Q4_0 tensor (1.8 M blocks): whole-tensor equality against the oracle
    N, K = 14336, 4096
    rng = np.random.default_rng(5)
    n_blocks = N * K // 32
    blocks = rng.integers(0, 256, size=(n_blocks, 18), dtype=np.uint8)
    blocks[:, 1] &= 0x3B  # keep d finite and small (no NaN payloads)
    want_w, want_s, want_b = gguf_ref.repack(blocks, Q4_0)
    got_w, got_s, got_b = _repack_gpu(blocks, Q4_0, (N, K))
    assert got_w.shape == (N, K // 8) and got_s.shape == (N, K // 32)
    assert np.array_equal(got_w.reshape(-1, 4), want_w)
    assert np.array_equal(got_s.reshape(-1).view(np.uint16), want_s.view(np.uint16))
    assert np.array_equal(got_b.reshape(-1).view(np.uint16), want_b.view(np.uint16))
