"""Pins the CPU oracle (oracle/affine_qref.c) -- no GPU involved.

1. byte-for-byte against golden vectors produced by the reference's own
   translation unit (tests/golden/*.npz, written by tests/golden/make_golden.py);
2. byte-for-byte against that translation unit directly, when oracle/_ref is
   built in this checkout;
3. against what the mathematics fixes: closed-form special groups, the ramp test
   of the reference's C++ suite, an independent bit-stream unpacker, the fp64
   GEMM on dequantized weights, brute-force loops for the batched and gathered
   entry points, and the GGUF d*q+m known-answer layout.
"""
import os

import numpy as np
import pytest
import torch

from oracle import qref
from tests.util import ALL_BITS, ALL_GROUPS, DTYPES, bits_equal, normal_weights, activations

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
NAMES = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}


def from_bits(arr: np.ndarray, dtype: torch.dtype) -> torch.Tensor:
    if dtype == torch.uint32:
        return torch.from_numpy(arr.astype(np.uint32))
    if dtype == torch.float32:
        return torch.from_numpy(arr.view(np.int32).copy()).view(torch.float32)
    return torch.from_numpy(arr.view(np.int16).copy()).view(dtype)


@pytest.fixture(scope="module")
def golden():
    return np.load(os.path.join(GOLDEN, "affine_quantized_ref.npz"), allow_pickle=False)


@pytest.mark.parametrize("dname", list(NAMES))
@pytest.mark.parametrize("bits", ALL_BITS)
@pytest.mark.parametrize("gs", ALL_GROUPS)
def test_port_reproduces_reference_golden_vectors(port_oracle, golden, dname, bits, gs):
    dtype = NAMES[dname]
    tag = f"{dname}_b{bits}_g{gs}"
    w = from_bits(golden[tag + "_w"], dtype)
    wq, s, b = port_oracle.quantize(w, gs, bits)
    assert bits_equal(wq, from_bits(golden[tag + "_wq"], torch.uint32))
    assert bits_equal(s, from_bits(golden[tag + "_scales"], dtype))
    assert bits_equal(b, from_bits(golden[tag + "_biases"], dtype))
    x = from_bits(golden[tag + "_x"], dtype)
    y = port_oracle.qmm(x, wq, s, b, True, gs, bits)
    assert bits_equal(y, from_bits(golden[tag + "_y_t"], dtype))
    xn = from_bits(golden[tag + "_xn"], dtype)
    yn = port_oracle.qmm(xn, wq, s, b, False, gs, bits)
    assert bits_equal(yn, from_bits(golden[tag + "_y_n"], dtype))


def test_half_type_conversions_match_reference(port_oracle):
    g = np.load(os.path.join(GOLDEN, "half_types_ref.npz"), allow_pickle=False)
    lib = port_oracle.port
    f32 = g["f32_bits"].view(np.float32)
    for i in range(0, len(f32)):
        f = float(f32[i])
        if f != f:  # NaN payloads do not survive the Python float round trip
            continue
        assert lib.qref_f16_from_f32(f) == int(g["f16_from_f32"][i]), hex(int(g["f32_bits"][i]))
        assert lib.qref_bf16_from_f32(f) == int(g["bf16_from_f32"][i]), hex(int(g["f32_bits"][i]))
    widened = g["f16_to_f32"]
    for h in range(0, 65536):
        got = np.array([lib.qref_f16_to_f32(h)], dtype=np.float32).view(np.uint32)[0]
        exp = widened[h]
        if (h & 0x7C00) == 0x7C00 and (h & 0x3FF):
            continue  # NaN
        assert got == exp, hex(h)


@pytest.mark.skipif(not qref.reference_built(), reason="oracle/_ref not built here")
@pytest.mark.parametrize("dtype", DTYPES)
def test_port_matches_reference_translation_unit(port_oracle, dtype):
    ref = qref.Oracle("reference")
    assert [ref.ref.ref_simd_max_size(i) for i in range(3)] == [1, 1, 1]
    for bits in ALL_BITS:
        for gs in ALL_GROUPS:
            w = normal_weights((9, 384), dtype, seed=bits + gs)
            a, b = port_oracle.quantize(w, gs, bits), ref.quantize(w, gs, bits)
            assert all(bits_equal(p, r) for p, r in zip(a, b))
            x = activations((5, 384), dtype)
            assert bits_equal(port_oracle.qmm(x, *a, True, gs, bits), ref.qmm(x, *a, True, gs, bits))
            xn = activations((5, 9), dtype)
            assert bits_equal(port_oracle.qmm(xn, *a, False, gs, bits), ref.qmm(xn, *a, False, gs, bits))


@pytest.mark.parametrize("bits", ALL_BITS)
def test_quantize_closed_form_groups(port_oracle, bits):
    gs, n_bins = 32, float(2**bits - 1)
    # all-zero group: codes 0, bias 0, scale = -max(0, 1e-7)
    wq, s, b = port_oracle.quantize(torch.zeros(1, gs), gs, bits)
    assert int(wq.view(torch.int32).abs().sum()) == 0
    assert float(b) == 0.0 and float(s) == pytest.approx(-1e-7, rel=1e-6)
    # constant positive group c: edge = c, q0 = rint(c / -1e-7) != 0 -> bias = c, codes 0
    wq, s, b = port_oracle.quantize(torch.full((1, gs), 0.75), gs, bits)
    assert int(wq.view(torch.int32).abs().sum()) == 0 and float(b) == 0.75
    # integers spanning exactly 0..n_bins: |scale| = 1 and an exact round trip
    ramp = (torch.arange(128, dtype=torch.float32) * 2).remainder(n_bins + 1)
    ramp[-1] = n_bins
    ramp = ramp.reshape(1, 128)
    wq, s, b = port_oracle.quantize(ramp, 128, bits)
    codes = qref.unpack_codes(wq, bits).float()
    assert abs(float(s)) == 1.0
    assert torch.equal(codes * float(s) + float(b), ramp)


def test_quantize_dequantize_ramp_of_reference_cpp_suite(port_oracle):
    # tests/ops_tests.cpp:3376-3395: x[r, c] = c, 128 x 512, group 128
    x = torch.arange(512, dtype=torch.float32).repeat(128, 1)
    for bits in (2, 4, 8):
        wq, s, b = port_oracle.quantize(x, 128, bits)
        assert wq.shape == (128, 512 * bits // 32) and s.shape == (128, 4)
        x_hat = port_oracle.dequantize(wq, s, b, 128, bits)
        assert float((x - x_hat).abs().max()) <= 127.0 / (1 << bits)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits", ALL_BITS)
@pytest.mark.parametrize("gs", ALL_GROUPS)
def test_dequantize_against_independent_unpacker(port_oracle, dtype, bits, gs):
    """qref_dequantize == T(T(code) * s) + b with codes from a pure-torch
    bit-stream reader; also the error bound and zero round trip of
    python/tests/test_quantized.py:22-39."""
    w = normal_weights((7, 512), dtype, seed=11)
    wq, s, b = port_oracle.quantize(w, gs, bits)
    got = port_oracle.dequantize(wq, s, b, gs, bits)
    codes = qref.unpack_codes(wq, bits).to(dtype)
    se = s.repeat_interleave(gs, dim=-1)
    be = b.repeat_interleave(gs, dim=-1)
    exp = (codes * se) + be  # torch rounds each op to dtype, as MLX's Multiply / Add do
    assert bits_equal(got, exp)
    if dtype == torch.float32:  # the reference states this bound for float32 inputs
        assert bool(((w - got).abs() <= se.abs() + 1e-6).all())
    z = port_oracle.quantize(torch.zeros(2, 256, dtype=dtype), gs, bits)
    assert bool((port_oracle.dequantize(*z, gs, bits) == 0).all())


@pytest.mark.parametrize("transpose", (True, False))
@pytest.mark.parametrize("bits", ALL_BITS)
def test_qmm_against_fp64_gemm(port_oracle, bits, transpose):
    gs = 64
    N, K, M = 128, 256, 5
    w = normal_weights((N, K) if transpose else (K, N), torch.float32, seed=bits)
    wq, s, b = port_oracle.quantize(w, gs, bits)
    w_hat = port_oracle.dequantize(wq, s, b, gs, bits).double()
    x = activations((M, K), torch.float32)
    y = port_oracle.qmm(x, wq, s, b, transpose, gs, bits).double()
    exact = x.double() @ (w_hat.T if transpose else w_hat)
    assert float((y - exact).abs().max()) < 1e-4
    # a dropped bias term or a wrong group index would fail this by orders of magnitude
    assert float(exact.abs().max()) > 0.05


def test_batched_and_gather_are_loops_over_qmm(port_oracle):
    gs, bits = 32, 5
    w = normal_weights((4, 48, 128), torch.float32, seed=3)
    wq, s, b = port_oracle.quantize(w, gs, bits)
    x = activations((4, 3, 128), torch.float32)
    yb = port_oracle.port_qmm_batched(x, wq, s, b, True, gs, bits)
    for i in range(4):
        assert bits_equal(yb[i], port_oracle.qmm(x[i], wq[i], s[i], b[i], True, gs, bits))
    # one weight shared by every batch
    ys = port_oracle.port_qmm_batched(x, wq[1], s[1], b[1], True, gs, bits)
    for i in range(4):
        assert bits_equal(ys[i], port_oracle.qmm(x[i], wq[1], s[1], b[1], True, gs, bits))
    lhs = torch.tensor([3, 0, 0, 2, 1])
    rhs = torch.tensor([1, 1, 3, 0, 2])
    yg = port_oracle.port_gather_qmm(x, wq, s, b, lhs, rhs, True, gs, bits)
    assert bits_equal(yg, port_oracle.gather_qmm(x, wq, s, b, lhs, rhs, True, gs, bits))
    for i in range(5):
        li, ri = int(lhs[i]), int(rhs[i])
        assert bits_equal(yg[i], port_oracle.qmm(x[li], wq[ri], s[ri], b[ri], True, gs, bits))


def test_gguf_q4_known_answer_layout(port_oracle):
    """python/tests/test_load.py:203-281: a Q4_0-style block d*(q-8) and a
    Q4_1-style block d*q+m, group 32, float16, low nibble first."""
    q = torch.arange(32) % 16
    words = torch.zeros(4, dtype=torch.int64)
    for i in range(32):
        words[i // 8] |= int(q[i]) << (4 * (i % 8))
    wq = words.to(torch.uint32).reshape(1, 4)
    d, m = 0.5, -1.25
    s = torch.tensor([[d]], dtype=torch.float16)
    out = port_oracle.dequantize(wq, s, torch.tensor([[-8 * d]], dtype=torch.float16), 32, 4)
    assert torch.equal(out.float().reshape(-1), d * (q.float() - 8))
    out = port_oracle.dequantize(wq, s, torch.tensor([[m]], dtype=torch.float16), 32, 4)
    assert torch.equal(out.float().reshape(-1), d * q.float() + m)


def test_pack_factor_tables(port_oracle):
    # mlx/backend/common/quantized.h:5-12
    lib = port_oracle.port
    assert [lib.qref_pack_factor(b, 8) for b in ALL_BITS] == [4, 8, 2, 8, 4, 1]
    assert [lib.qref_pack_factor(b, 32) for b in ALL_BITS] == [16, 8, 8, 8, 4, 4]
    assert [lib.qref_bytes_per_pack(b, 8) for b in ALL_BITS] == [1, 3, 1, 5, 3, 1]
