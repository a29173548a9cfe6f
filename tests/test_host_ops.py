"""Argument validation of the Python operator mirror: same conditions and the
same exception type (std::invalid_argument -> ValueError) as the reference's
ops, python/tests/test_quantized.py:877-956.  Runs on the CPU: every check
comes before the first device call."""
import pytest
import torch

import mlx_amd


def _triple(N=64, K=512, gs=64, bits=4, dtype=torch.float32):
    wq = torch.zeros((N, K * bits // 32), dtype=torch.uint32)
    s = torch.ones((N, K // gs), dtype=dtype)
    return wq, s, torch.zeros_like(s)


def test_quantize_errors():
    with pytest.raises(ValueError, match="floating"):
        mlx_amd.quantize(torch.zeros((4, 64), dtype=torch.int32))
    with pytest.raises(ValueError, match="at least 2"):
        mlx_amd.quantize(torch.zeros(64))
    with pytest.raises(ValueError, match="divisible"):
        mlx_amd.quantize(torch.zeros((4, 65)))
    with pytest.raises(ValueError, match="group size"):
        mlx_amd.quantize(torch.zeros((4, 96)), group_size=48)
    with pytest.raises(ValueError, match="bits"):
        mlx_amd.quantize(torch.zeros((4, 64)), bits=7)
    with pytest.raises(ValueError, match="mode"):
        mlx_amd.quantize(torch.zeros((4, 64)), mode="bogus")
    with pytest.raises(RuntimeError, match="GPU"):
        mlx_amd.quantize(torch.zeros((4, 64)), mode="mxfp4")  # valid, but not on the device
    with pytest.raises(RuntimeError, match="GPU"):
        mlx_amd.quantize(torch.zeros((4, 64)))  # valid, but not on the device


def test_quantized_matmul_errors():
    wq, s, b = _triple()
    x = torch.zeros((2, 512))
    with pytest.raises(ValueError, match="Biases must be provided"):
        mlx_amd.quantized_matmul(x, wq, s, None)
    with pytest.raises(ValueError, match="uint32"):
        mlx_amd.quantized_matmul(x, wq.view(torch.int32), s, b)
    with pytest.raises(ValueError, match="same shape"):
        mlx_amd.quantized_matmul(x, wq, s, b[:, :4])
    with pytest.raises(ValueError, match="incompatible"):
        mlx_amd.quantized_matmul(x, wq, s, b, group_size=32)
    with pytest.raises(ValueError, match="does not match"):
        mlx_amd.quantized_matmul(torch.zeros((2, 256)), wq, s, b)
    with pytest.raises(ValueError, match="does not match"):
        mlx_amd.quantized_matmul(x, wq, s, b, transpose=False)
    with pytest.raises(ValueError, match="floating"):
        mlx_amd.quantized_matmul(x, wq, s.to(torch.int32), b.to(torch.int32))
    with pytest.raises(RuntimeError, match="GPU"):
        mlx_amd.quantized_matmul(x, wq, s, b)


def test_dequantize_errors():
    wq, s, b = _triple()
    with pytest.raises(ValueError, match="uint32"):
        mlx_amd.dequantize(wq.view(torch.int32), s, b)
    with pytest.raises(ValueError, match="does not match"):
        mlx_amd.dequantize(wq, s[:32], b[:32])
    with pytest.raises(ValueError, match="does not match"):
        mlx_amd.dequantize(wq, s, b, group_size=128)
    with pytest.raises(ValueError, match="floating"):
        mlx_amd.dequantize(wq, s, b, dtype=torch.int32)
    with pytest.raises(ValueError, match="at least 2"):
        mlx_amd.dequantize(wq[0], s[0], b[0])


def test_gather_qmm_errors_and_defaults():
    wq, s, b = _triple()
    wq3, s3, b3 = wq.reshape(1, 64, 64), s.reshape(1, 64, 8), b.reshape(1, 64, 8)
    x = torch.zeros((3, 1, 512))
    with pytest.raises(ValueError, match="integral"):
        mlx_amd.gather_qmm(x, wq3, s3, b3, rhs_indices=torch.zeros(3))
    with pytest.raises(ValueError, match="at least two"):
        mlx_amd.gather_qmm(torch.zeros(512), wq3, s3, b3, rhs_indices=torch.zeros(3, dtype=torch.int64))
    # without indices it is quantized_matmul (mlx/ops.cpp:5566-5569)
    with pytest.raises(RuntimeError, match="GPU"):
        mlx_amd.gather_qmm(x, wq, s, b)


def test_broadcast_shape_matches_numpy():
    """The plain-Python shape broadcast used for default gather indices agrees
    with numpy on every pair, errors included."""
    import itertools

    import numpy as np

    from mlx_amd.ops import _broadcast_shape

    shapes = [(), (1,), (3,), (2, 3), (1, 3), (2, 1), (4, 2, 3), (4, 1, 1), (0,), (2, 0)]
    for a, b in itertools.product(shapes, repeat=2):
        try:
            want = tuple(np.broadcast_shapes(a, b))
        except ValueError:
            with pytest.raises(ValueError):
                _broadcast_shape(a, b)
            continue
        assert _broadcast_shape(a, b) == want, (a, b)


def test_fp_mode_errors():
    """Argument checks of the floating-point modes (mlx/ops.cpp:4704-4782,
    5108-5123, 5351-5390; python/tests/test_quantized.py:41-181) run before any
    device work."""
    w = torch.zeros((8, 64))
    for mode, gs, bits in (("mxfp4", 32, 4), ("mxfp8", 32, 8), ("nvfp4", 16, 4)):
        with pytest.raises(ValueError, match="requires group size"):
            mlx_amd.quantize(w, group_size=64, mode=mode)
        with pytest.raises(ValueError, match="requires bits"):
            mlx_amd.quantize(w, bits=2 if bits != 2 else 4, mode=mode)
        with pytest.raises(RuntimeError, match="GPU"):
            mlx_amd.quantize(w, mode=mode)
        wq = torch.zeros((8, 64 * bits // 32), dtype=torch.uint32)
        sc = torch.zeros((8, 64 // gs), dtype=torch.uint8)
        with pytest.raises(ValueError, match="Scale type must be uint8"):
            mlx_amd.dequantize(wq, sc.to(torch.float32), mode=mode)
        with pytest.raises(ValueError, match="Biases must be null"):
            mlx_amd.dequantize(wq, sc, sc, mode=mode)
        with pytest.raises(ValueError, match="does not match"):
            mlx_amd.dequantize(wq, sc[:, :1], mode=mode)
        with pytest.raises(ValueError, match="output dtype"):
            mlx_amd.dequantize(wq, sc, mode=mode, dtype=torch.int32)
        with pytest.raises(ValueError, match="requires group size"):
            mlx_amd.dequantize(wq, sc, group_size=64, mode=mode)
        x = torch.zeros((2, 64))
        with pytest.raises(ValueError, match="Biases must be null"):
            mlx_amd.quantized_matmul(x, wq, sc, sc, mode=mode)
        with pytest.raises(ValueError, match="does not match"):
            mlx_amd.quantized_matmul(x[:, :32], wq, sc, mode=mode)
        with pytest.raises(ValueError, match="real floating"):
            mlx_amd.quantized_matmul(x.to(torch.int32), wq, sc, mode=mode)
        with pytest.raises(RuntimeError, match="GPU"):
            mlx_amd.quantized_matmul(x, wq, sc, mode=mode)
        with pytest.raises(RuntimeError, match="GPU"):
            mlx_amd.gather_qmm(x, wq[None], sc[None], rhs_indices=torch.zeros(1, dtype=torch.int32),
                               mode=mode)
    with pytest.raises(ValueError, match="only supported for 'nvfp4'"):
        mlx_amd.quantize(w, mode="mxfp8", global_scale=torch.ones(()))
    with pytest.raises(ValueError, match="scalar"):
        mlx_amd.quantize(w, mode="nvfp4", global_scale=torch.ones(2))
    with pytest.raises(ValueError, match="dtype float32"):
        mlx_amd.quantize(w, mode="nvfp4", global_scale=torch.ones((), dtype=torch.float16))
    with pytest.raises(RuntimeError, match="GPU"):  # valid arguments: only the device is wrong
        mlx_amd.quantize(w, mode="nvfp4", global_scale=torch.ones(()))


def test_qqmm_errors():
    # validate_qqmm_inputs, mlx/ops.cpp:4836-4894
    x = torch.zeros((2, 64))
    wq = torch.zeros((8, 8), dtype=torch.uint32)
    sc = torch.zeros((8, 4), dtype=torch.uint8)
    with pytest.raises(ValueError, match="Only 2D"):
        mlx_amd.qqmm(x, wq[None], sc[None])
    with pytest.raises(ValueError, match="Scales must be provided"):
        mlx_amd.qqmm(x, wq)
    with pytest.raises(ValueError, match="second argument dtype"):
        mlx_amd.qqmm(x, wq.view(torch.int32), sc)
    with pytest.raises(ValueError, match="first argument dtype"):
        mlx_amd.qqmm(x.to(torch.float64), wq, sc)
    with pytest.raises(ValueError, match="either both"):
        mlx_amd.qqmm(x, wq, sc, global_scale_x=torch.ones(()))
    with pytest.raises(ValueError, match="must match last dimension"):
        mlx_amd.qqmm(x, torch.zeros((8, 32)))
    with pytest.raises(RuntimeError, match="GPU"):
        mlx_amd.qqmm(x, wq, sc)


def test_gather_qqmm_errors():
    # gather_qqmm, mlx/ops.cpp:5631-5681 (extract_qqmm_dims :4896-4924)
    x = torch.zeros((2, 4, 64))
    wq = torch.zeros((3, 8, 8), dtype=torch.uint32)
    sc = torch.zeros((3, 8, 4), dtype=torch.uint8)
    idx = torch.zeros(2, dtype=torch.int32)
    with pytest.raises(ValueError, match="Affine quantization is not supported"):
        mlx_amd.gather_qqmm(x, wq, sc, rhs_indices=idx, mode="affine")
    with pytest.raises(ValueError, match="Scales must be provided"):
        mlx_amd.gather_qqmm(x, wq, rhs_indices=idx)
    with pytest.raises(ValueError, match="first argument dtype"):
        mlx_amd.gather_qqmm(x.to(torch.float64), wq, sc, rhs_indices=idx)
    with pytest.raises(ValueError, match="either both"):
        mlx_amd.gather_qqmm(x, wq, sc, rhs_indices=idx, global_scale_w=torch.ones(()))
    with pytest.raises(ValueError, match="only supported for 'nvfp4'"):
        mlx_amd.gather_qqmm(x, wq, sc, rhs_indices=idx, mode="mxfp4",
                            global_scale_x=torch.ones(()), global_scale_w=torch.ones(()))
    with pytest.raises(ValueError, match="must match last dimension"):
        mlx_amd.gather_qqmm(x, torch.zeros((3, 8, 32)), rhs_indices=idx)
    with pytest.raises(ValueError, match="integral"):
        mlx_amd.gather_qqmm(x, wq, sc, rhs_indices=idx.float())
    with pytest.raises(ValueError, match="at least two dimensions"):
        mlx_amd.gather_qqmm(x[0, 0], wq, sc, rhs_indices=idx)
    with pytest.raises(RuntimeError, match="GPU"):
        mlx_amd.gather_qqmm(x, wq, sc, rhs_indices=idx)


def test_fp8_conversion_errors():
    # mlx/ops.cpp:5519-5552
    with pytest.raises(ValueError, match="Only real floating types"):
        mlx_amd.to_fp8(torch.zeros(4, dtype=torch.int32))
    with pytest.raises(ValueError, match="must have type uint8"):
        mlx_amd.from_fp8(torch.zeros(4))
    with pytest.raises(ValueError, match="Only real floating types"):
        mlx_amd.from_fp8(torch.zeros(4, dtype=torch.uint8), torch.int32)
    with pytest.raises(RuntimeError, match="GPU"):
        mlx_amd.to_fp8(torch.zeros(4))
    with pytest.raises(RuntimeError, match="GPU"):
        mlx_amd.from_fp8(torch.zeros(4, dtype=torch.uint8))


def test_vjp_wrt_scales_is_refused():
    # python/tests/test_quantized.py:1668-1694 (test_fp_vjp_scales_throws) and
    # mlx/primitives.cpp:3556-3567
    x = torch.zeros((2, 64))
    wq = torch.zeros((8, 8), dtype=torch.uint32)
    for mode, match, exc in (("mxfp4", "no gradient wrt scales in mxfp4", ValueError),
                             ("mxfp8", "no gradient wrt scales in mxfp8", ValueError)):
        sc = torch.zeros((8, 2), dtype=torch.float32, requires_grad=True)
        with pytest.raises(exc, match=match):
            mlx_amd.quantized_matmul(x, wq if mode == "mxfp4" else torch.zeros((8, 16), dtype=torch.uint32),
                                     sc, mode=mode)
    s = torch.zeros((8, 1), requires_grad=True)
    b = torch.zeros((8, 1))
    with pytest.raises(NotImplementedError, match="scales and biases"):
        mlx_amd.quantized_matmul(x, wq, s, b)
    with torch.no_grad():  # no graph is being recorded: the ordinary checks apply
        with pytest.raises(RuntimeError, match="GPU"):
            mlx_amd.quantized_matmul(x, wq, s, b)
