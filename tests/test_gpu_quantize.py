"""GPU parity of affine quantize / dequantize against the CPU oracle:
packed words, scales and biases must be bit-identical."""
import pytest
import torch

import mlx_amd
from tests.util import (
    ALL_BITS, ALL_GROUPS, DTYPES, bits_equal, count_mismatch, normal_weights,
    student_t_weights,
)

pytestmark = pytest.mark.gpu


def _check_quantize(oracle, gpu, w, gs, bits):
    ref = oracle.quantize(w, gs, bits)
    got = mlx_amd.quantize(w.to(gpu), gs, bits)
    torch.cuda.synchronize()
    for name, r, g in zip(("wq", "scales", "biases"), ref, got):
        assert g.device.type == "cuda"
        assert bits_equal(r, g), (
            f"{name} differs in {count_mismatch(r, g)} of {r.numel()} elements "
            f"(dtype={w.dtype}, gs={gs}, bits={bits}, shape={tuple(w.shape)})"
        )
    return got


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits", ALL_BITS)
@pytest.mark.parametrize("gs", ALL_GROUPS)
def test_quantize_all_widths(oracle, gpu, dtype, bits, gs):
    # 3 rows x 1280: not a multiple of the 256-lane block, exercises the tail
    w = normal_weights((3, 1280), dtype, seed=bits * 131 + gs)
    _check_quantize(oracle, gpu, w, gs, bits)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits", ALL_BITS)
def test_quantize_special_groups(oracle, gpu, dtype, bits):
    """All-zero, constant, single-spike, tiny, and sign-mixed groups."""
    gs = 32
    rows = []
    rows.append(torch.zeros(gs))
    rows.append(torch.full((gs,), 0.75))
    rows.append(torch.full((gs,), -0.3))
    spike = torch.zeros(gs); spike[5] = 2.5; rows.append(spike)
    spike = torch.zeros(gs); spike[31] = -1e-3; rows.append(spike)
    rows.append(torch.linspace(-1, 1, gs))
    rows.append(torch.linspace(0, 1e-9, gs))
    rows.append(torch.linspace(-3e-8, 2e-8, gs))
    rows.append(torch.arange(gs, dtype=torch.float32))
    rows.append(-torch.arange(gs, dtype=torch.float32) * 1e3)
    neg0 = torch.zeros(gs); neg0[3] = -0.0; rows.append(neg0)
    w = torch.stack(rows).reshape(1, -1).to(dtype)
    _check_quantize(oracle, gpu, w, gs, bits)


def test_quantize_config1_fp32_and_round_trip(oracle, gpu):
    """W fp32 [4096,4096] ~ N(0,0.02), seed 0, 4-bit g64, plus dequantize."""
    w = normal_weights((4096, 4096), torch.float32, seed=0)
    wq, s, b = _check_quantize(oracle, gpu, w, 64, 4)
    w_hat = mlx_amd.dequantize(wq, s, b, 64, 4)
    ref_hat = oracle.dequantize(wq.cpu(), s.cpu(), b.cpu(), 64, 4)
    assert bits_equal(ref_hat, w_hat)
    # python/tests/test_quantized.py:29-31
    err = (w - w_hat.cpu()).abs().reshape(4096, 64, 64)
    assert bool((err <= s.cpu().abs().unsqueeze(-1) + 1e-6).all())


@pytest.mark.parametrize("bits,gs", [(4, 64), (8, 128)])
def test_quantize_decode_shapes_bf16(oracle, gpu, bits, gs):
    """Llama-3-8B MLP weights, bf16 scales/biases."""
    for shape in ((14336, 4096), (4096, 14336)):
        w = normal_weights(shape, torch.bfloat16, seed=0)
        _check_quantize(oracle, gpu, w, gs, bits)


@pytest.mark.parametrize("bits", (2, 3, 5, 6))
@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16))
def test_quantize_odd_width_stress(oracle, gpu, dtype, bits):
    """[11008,4096] and [4096,11008], group 32, normal and heavy-tailed."""
    for shape in ((11008, 4096), (4096, 11008)):
        for make in (normal_weights, student_t_weights):
            w = make(shape, dtype, seed=bits)
            wq, s, b = _check_quantize(oracle, gpu, w, 32, bits)
    # dequantize of the last one, bit-exact against the two-rounding formula
    w_hat = mlx_amd.dequantize(wq, s, b, 32, bits)
    ref_hat = oracle.dequantize(wq.cpu(), s.cpu(), b.cpu(), 32, bits)
    assert bits_equal(ref_hat, w_hat)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits", ALL_BITS)
@pytest.mark.parametrize("gs", ALL_GROUPS)
def test_dequantize_all_widths(oracle, gpu, dtype, bits, gs):
    w = normal_weights((5, 768), dtype, seed=7 + bits)
    wq, s, b = oracle.quantize(w, gs, bits)
    ref = oracle.dequantize(wq, s, b, gs, bits)
    got = mlx_amd.dequantize(wq.to(gpu), s.to(gpu), b.to(gpu), gs, bits)
    assert bits_equal(ref, got)
    # zeros stay exact zeros (python/tests/test_quantized.py:33-39)
    z = torch.zeros((2, 256), dtype=dtype, device=gpu)
    zq = mlx_amd.quantize(z, gs, bits)
    z_hat = mlx_amd.dequantize(*zq, gs, bits)
    assert bool((z_hat == 0).all())


def test_dequantize_output_dtype(gpu):
    w = normal_weights((4, 256), torch.bfloat16).to(gpu)
    wq, s, b = mlx_amd.quantize(w)
    out = mlx_amd.dequantize(wq, s, b, dtype=torch.float32)
    assert out.dtype == torch.float32
    assert torch.equal(out, mlx_amd.dequantize(wq, s, b).float())


def test_quantize_batched_and_empty(oracle, gpu):
    w = normal_weights((2, 3, 4, 128), torch.float16, seed=3)
    got = _check_quantize(oracle, gpu, w, 64, 4)
    assert got[0].shape == (2, 3, 4, 16) and got[1].shape == (2, 3, 4, 2)
    e = torch.zeros((0, 64), dtype=torch.float32, device=gpu)
    wq, s, b = mlx_amd.quantize(e)
    assert wq.shape == (0, 8) and s.shape == (0, 1)


@pytest.mark.parametrize("bits", (2, 4, 5, 8))
def test_quantize_division_corner_magnitudes(oracle, gpu, bits):
    """Every code is a correctly rounded fp32 quotient rounded to an integer: run
    many groups whose quotients sit on or next to the rounding ties (values on a
    half-integer grid of the scale), at magnitudes from 1e-30 to 1e30, with
    heavy tails, and with infinities / NaNs in some groups."""
    g = torch.Generator().manual_seed(bits)
    n_bins = (1 << bits) - 1
    rows = []
    for exp in (-30, -20, -7, -3, 0, 4, 20, 30):
        base = torch.rand((64, 64), generator=g) * 2 - 1
        # half-integer grid: quotients k + 0.5 exactly where representable
        grid = (torch.randint(0, 2 * n_bins + 1, (64, 64), generator=g).float() / 2) / n_bins - 0.5
        tails = torch.distributions.StudentT(2.0).sample((64, 64)).clamp(-1e4, 1e4) * 0.01
        rows += [base * 10.0 ** exp, grid * 10.0 ** exp, tails * 10.0 ** exp]
    w = torch.cat(rows).float()
    _check_quantize(oracle, gpu, w, 64, bits)
    _check_quantize(oracle, gpu, w.reshape(-1, 128), 32, bits)
    # non-finite members: the group is garbage in the reference too, but it must
    # be the same garbage wherever the reference's result is well defined
    w2 = w[:64].clone()
    w2[3, 5] = float("inf")
    w2[7, 9] = float("-inf")
    ref = oracle.quantize(w2, 64, bits)
    got = mlx_amd.quantize(w2.to(gpu), 64, bits)
    clean = torch.ones(64, dtype=torch.bool)
    clean[3] = clean[7] = False
    for r, t in zip(ref, got):
        assert bits_equal(r[clean], t.cpu()[clean])
