"""Host-side mirror of MLX's affine quantization operators for MI355X.

Same names, argument meaning, defaults and error behaviour as
``mx.quantize`` / ``mx.dequantize`` / ``mx.quantized_matmul`` /
``mx.gather_qmm`` (reference: ``mlx/ops.cpp:4784-4834, 5035-5099, 5208-5246,
5465-5517, 5553-5629``; Python binding ``python/src/ops.cpp:4622-4866``).
Tensors are torch tensors resident on the GPU; torch only supplies device
memory and the current HIP stream -- every computation is done by the HIP
kernels behind the C ABI of ``include/mlx_rocm_qmm.h``.  Invalid arguments
raise ``ValueError`` exactly where the reference throws
``std::invalid_argument``.
"""
from __future__ import annotations

import functools
from typing import Optional, Tuple

import torch

from . import _lib
from ._copy import astype as _astype, contiguous as _contiguous

_DTYPE_CODE = {
    torch.float32: _lib.FLOAT32,
    torch.float16: _lib.FLOAT16,
    torch.bfloat16: _lib.BFLOAT16,
}
_FLOATING = tuple(_DTYPE_CODE)
_MODES = ("affine", "mxfp4", "mxfp8", "nvfp4")
_INTEGER = (
    torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64,
    torch.uint16, torch.uint32, torch.uint64,
)


def _stream_ptr(t: torch.Tensor) -> int:
    return torch.cuda.current_stream(t.device).cuda_stream


def _require_gpu(tag: str, *tensors: torch.Tensor) -> None:
    for t in tensors:
        if t.device.type != "cuda":
            raise RuntimeError(
                f"[{tag}] mlx_amd runs on the GPU only; got a tensor on {t.device}"
            )


def _mode(tag: str, mode: str) -> str:
    # string_to_quantization_mode, mlx/primitives.cpp
    if mode not in _MODES:
        raise ValueError(f"[{tag}] Invalid quantization mode '{mode}'.")
    return mode


def _params_from_mode(mode: str, group_size, bits) -> Tuple[int, int]:
    # quantization_params_from_mode, mlx/ops.cpp:4675-4702
    defaults = {"affine": (64, 4), "nvfp4": (16, 4), "mxfp4": (32, 4), "mxfp8": (32, 8)}
    dg, db = defaults[mode]
    return (dg if group_size is None else int(group_size),
            db if bits is None else int(bits))


_MODE_CODE = {"mxfp4": _lib.MXFP4, "mxfp8": _lib.MXFP8, "nvfp4": _lib.NVFP4}


def _check_fp_params(tag: str, mode: str, group_size: int, bits: int) -> None:
    # fp_quantize / fp_dequantize, mlx/ops.cpp:5108-5123, 5351-5366
    want_gs = 16 if mode == "nvfp4" else 32
    want_bits = 8 if mode == "mxfp8" else 4
    if group_size != want_gs:
        raise ValueError(
            f"[{tag}] {mode} quantization requires group size {want_gs} but got {group_size}."
        )
    if bits != want_bits:
        raise ValueError(
            f"[{tag}] {mode} quantization requires bits to be {want_bits} but got {bits}."
        )


def _global_scale(tag: str, mode: str, g, like: torch.Tensor):
    """validate_global_scale, mlx/ops.cpp:4756-4782; returns the scale as one
    float32 on ``like``'s device, or None."""
    if g is None:
        return None
    if mode != "nvfp4":
        raise ValueError(
            f"[{tag}] Global scale is only supported for 'nvfp4' quantization mode."
        )
    if g.numel() != 1:
        raise ValueError(
            f"[{tag}] Global scale must be a scalar but got shape {tuple(g.shape)}."
        )
    if g.dtype != torch.float32:
        raise ValueError(
            f"[{tag}] Global scale must have dtype float32 but got {g.dtype}."
        )
    return g.detach().reshape(1).to(like.device).contiguous()


def _validate_mode_with_type(tag, scales, biases, out_type, mode):
    # mlx/ops.cpp:4704-4754
    mode = _mode(tag, mode)
    if out_type is not None and out_type not in _FLOATING:
        raise ValueError(
            f"[{tag}] Only real floating types are supported but output dtype == {out_type}."
        )
    if mode == "affine":
        if biases is None:
            raise ValueError(f"[{tag}] Biases must be provided for affine quantization.")
        dtype = torch.promote_types(scales.dtype, biases.dtype)
        if dtype not in _FLOATING:
            raise ValueError(
                f"[{tag}] Only real floating types are supported but scales.dtype() == "
                f"{scales.dtype} and biases.dtype() == {biases.dtype}."
            )
        return (out_type if out_type is not None else dtype), mode
    if scales.dtype != torch.uint8:
        raise ValueError(
            f"[{tag}] Scale type must be uint8 but received type {scales.dtype}."
        )
    if biases is not None:
        raise ValueError(
            f"[{tag}] Biases must be null for quantization mode '{mode}'."
        )
    return (out_type if out_type is not None else torch.bfloat16), mode


def _validate_quantized_input(tag, w, scales, group_size, bits, biases):
    # mlx/ops.cpp:110-150
    if w.dtype != torch.uint32:
        raise ValueError(
            f"[{tag}] The weight matrix should be uint32 but received {w.dtype}"
        )
    if biases is not None and scales.shape != biases.shape:
        raise ValueError(
            f"[{tag}] Scales and biases should have the same shape. Received scales "
            f"with shape {tuple(scales.shape)} and biases with {tuple(biases.shape)}"
        )
    if w.dim() < 2 or scales.dim() < 2 or tuple(w.shape[:-2]) != tuple(
        scales.shape[: w.dim() - 2]
    ):
        raise ValueError(
            f"[{tag}] Weight and scales should have the same batch shape. Received "
            f"weight with shape {tuple(w.shape)}, scales with {tuple(scales.shape)}."
        )
    if w.shape[-1] * 32 // bits != scales.shape[-1] * group_size:
        raise ValueError(
            f"[{tag}] The shapes of the weight and scales are incompatible based on "
            f"bits and group_size. w.shape() == {tuple(w.shape)} and scales.shape() "
            f"== {tuple(scales.shape)} with group_size={group_size} and bits={bits}"
        )


def _extract_dims(tag, x, w, scales, biases, transpose, group_size, bits):
    # extract_quantized_matmul_dims, mlx/ops.cpp:152-181
    _validate_quantized_input(tag, w, scales, group_size, bits, biases)
    if x.dim() < 1:
        raise ValueError(f"[{tag}] x must have at least one dimension")
    x_inner = x.shape[-1]
    w_inner = w.shape[-1] * 32 // bits if transpose else w.shape[-2]
    w_outer = w.shape[-2] if transpose else w.shape[-1] * 32 // bits
    if w_inner != x_inner:
        raise ValueError(
            f"[{tag}] Last dimension of first input with shape (..., {x_inner}) does "
            f"not match the expanded quantized matrix ({w_inner}, {w_outer}) computed "
            f"from shape {tuple(w.shape)} with group_size={group_size}, bits={bits} "
            f"and transpose={str(bool(transpose)).lower()}"
        )
    return w_inner, w_outer


def _check_affine_params(tag: str, group_size: int, bits: int) -> None:
    # affine_quantize, mlx/ops.cpp:5038-5050
    if group_size not in (32, 64, 128):
        raise ValueError(
            f"[{tag}] The requested group size {group_size} is not supported. "
            "The supported group sizes are 32, 64, and 128."
        )
    if bits < 2 or bits > 8 or bits == 7:
        raise ValueError(
            f"[{tag}] The requested number of bits {bits} is not supported. "
            "The supported bits are 2, 3, 4, 5, 6 and 8."
        )


def _last_two_dense(t: torch.Tensor) -> bool:
    """Rows of the trailing matrix are contiguous (what the CPU backend
    requires of w / scales / biases, mlx/backend/cpu/quantized.cpp:974-990)."""
    return t.stride(-1) == 1 and t.stride(-2) == t.shape[-1]


# --------------------------------------------------------------------------
def quantize(
    w: torch.Tensor,
    group_size: Optional[int] = None,
    bits: Optional[int] = None,
    mode: str = "affine",
    global_scale: Optional[torch.Tensor] = None,
):
    """``mx.quantize``: returns ``(w_q uint32, scales, biases)`` for
    ``mode="affine"`` (mlx/ops.cpp:5208-5246 -> affine_quantize :5035-5099) and
    ``(w_q uint32, scales uint8)`` for the floating-point modes (fp_quantize
    :5101-5205)."""
    mode = _mode("quantize", mode)
    group_size, bits = _params_from_mode(mode, group_size, bits)
    if w.dtype not in _FLOATING:
        raise ValueError(
            f"[quantize] Only real floating types can be quantized but w has type {w.dtype}."
        )
    if w.dim() < 2:
        raise ValueError(
            "[quantize] The matrix to be quantized must have at least 2 dimension "
            f"but it has only {w.dim()}."
        )
    if w.shape[-1] % group_size != 0:
        raise ValueError(
            "[quantize] The last dimension of the matrix needs to be divisible by the "
            f"quantization group size {group_size}. However the provided  matrix has "
            f"shape {tuple(w.shape)}"
        )
    gscale = _global_scale("quantize", mode, global_scale, w)
    if mode == "affine":
        _check_affine_params("quantize", group_size, bits)
    else:
        _check_fp_params("quantize", mode, group_size, bits)
    _require_gpu("quantize", w)
    lib = _lib.load()
    w = _contiguous(w)  # ensure_row_contiguous, cpu/quantized.cpp:1233
    lead = tuple(w.shape[:-1])
    K = w.shape[-1]
    wq = torch.empty(lead + (K * bits // 32,), dtype=torch.uint32, device=w.device)
    if mode != "affine":
        # fp_quantize, mlx/ops.cpp:5101-5205: two outputs, one scale byte per group
        scales = torch.empty(lead + (K // group_size,), dtype=torch.uint8, device=w.device)
        if gscale is not None:
            # the reference's GPU-only variant, mlx/backend/cuda/quantized/fp_quantize.cuh:147-215
            _lib.check(
                lib.mlxrocm_nvfp4_quantize_global(
                    w.data_ptr(), gscale.data_ptr(), wq.data_ptr(), scales.data_ptr(), w.numel(),
                    _DTYPE_CODE[w.dtype], _stream_ptr(w),
                )
            )
            return wq, scales
        _lib.check(
            lib.mlxrocm_fp_quantize(
                w.data_ptr(), wq.data_ptr(), scales.data_ptr(), w.numel(),
                _MODE_CODE[mode], _DTYPE_CODE[w.dtype], _stream_ptr(w),
            )
        )
        return wq, scales
    scales = torch.empty(lead + (K // group_size,), dtype=w.dtype, device=w.device)
    biases = torch.empty_like(scales)
    _lib.check(
        lib.mlxrocm_affine_quantize(
            w.data_ptr(), wq.data_ptr(), scales.data_ptr(), biases.data_ptr(),
            w.numel(), group_size, bits, _DTYPE_CODE[w.dtype], _stream_ptr(w),
        )
    )
    return wq, scales, biases


def dequantize(
    w: torch.Tensor,
    scales: torch.Tensor,
    biases: Optional[torch.Tensor] = None,
    group_size: Optional[int] = None,
    bits: Optional[int] = None,
    mode: str = "affine",
    global_scale: Optional[torch.Tensor] = None,
    dtype: Optional[torch.dtype] = None,
):
    """``mx.dequantize`` (mlx/ops.cpp:5465-5517 -> affine_dequantize :5248-5340,
    fp_dequantize :5342-5462)."""
    out_type, mode = _validate_mode_with_type("dequantize", scales, biases, dtype, mode)
    group_size, bits = _params_from_mode(mode, group_size, bits)
    gscale = _global_scale("dequantize", mode, global_scale, w)
    if mode != "affine":
        return _fp_dequantize(w, scales, group_size, bits, mode, out_type, gscale)
    if bits <= 0:
        raise ValueError(f"[dequantize] Invalid value for bits: {bits}")
    if group_size <= 0:
        raise ValueError(f"[dequantize] Invalid value for group_size: {group_size}")
    if w.dtype != torch.uint32:
        raise ValueError("[dequantize] The matrix should be given as a uint32")
    if w.dim() < 2:
        raise ValueError(
            "[dequantize] The matrix to be dequantized must have at least 2 dimension "
            f"but it has only {w.dim()}."
        )
    if (
        w.dim() != scales.dim()
        or w.dim() != biases.dim()
        or tuple(w.shape[:-1]) != tuple(scales.shape[:-1])
        or tuple(w.shape[:-1]) != tuple(biases.shape[:-1])
    ):
        raise ValueError(
            "[dequantize] Shape of scales and biases does not match the matrix"
        )
    out_size = w.shape[-1] * 32 // bits
    if out_size != scales.shape[-1] * group_size or scales.shape != biases.shape:
        raise ValueError(
            "[dequantize] Shape of scales and biases does not match the matrix given "
            f"the quantization parameters. Provided matrix of shape {tuple(w.shape)} "
            f"and scales/biases of shape {tuple(scales.shape)} with "
            f"group_size={group_size} and bits={bits}."
        )
    _check_affine_params("dequantize", group_size, bits)
    _require_gpu("dequantize", w, scales, biases)
    lib = _lib.load()
    # The affine step runs in scales' dtype (mlx/ops.cpp:5322-5323); biases are
    # promoted to it the way the Add primitive would.
    sdt = torch.promote_types(scales.dtype, biases.dtype)
    w = _contiguous(w)
    scales = _contiguous(_astype(scales, sdt))
    biases = _contiguous(_astype(biases, sdt))
    out = torch.empty(tuple(w.shape[:-1]) + (out_size,), dtype=sdt, device=w.device)
    _lib.check(
        lib.mlxrocm_affine_dequantize(
            w.data_ptr(), scales.data_ptr(), biases.data_ptr(), out.data_ptr(),
            out.numel(), group_size, bits, _DTYPE_CODE[sdt], _stream_ptr(w),
        )
    )
    return _astype(out, out_type)  # astype, :5502-5505


def _fp_dequantize(w, scales, group_size, bits, mode, out_type, gscale=None):
    # fp_dequantize, mlx/ops.cpp:5342-5462
    if bits <= 0:
        raise ValueError(f"[dequantize] Invalid value for bits: {bits}")
    if group_size <= 0:
        raise ValueError(f"[dequantize] Invalid value for group_size: {group_size}")
    if w.dtype != torch.uint32:
        raise ValueError("[dequantize] The matrix should be given as a uint32")
    if w.dim() < 2:
        raise ValueError(
            "[dequantize] The matrix to be dequantized must have at least 2 dimension "
            f"but it has only {w.dim()}."
        )
    _check_fp_params("dequantize", mode, group_size, bits)
    if w.dim() != scales.dim() or tuple(w.shape[:-1]) != tuple(scales.shape[:-1]):
        raise ValueError("[dequantize] Shape of scales does not match the matrix")
    out_size = w.shape[-1] * 32 // bits
    if out_size != scales.shape[-1] * group_size:
        raise ValueError(
            "[dequantize] Shape of scales does not match the matrix given the "
            f"quantization parameters. Provided matrix of shape {tuple(w.shape)} and "
            f"scales of shape {tuple(scales.shape)}."
        )
    _require_gpu("dequantize", w, scales)
    lib = _lib.load()
    w = _contiguous(w)
    scales = _contiguous(scales)
    out = torch.empty(tuple(w.shape[:-1]) + (out_size,), dtype=out_type, device=w.device)
    if gscale is not None:
        # mlx/backend/cuda/quantized/fp_quantize.cuh:548-592
        _lib.check(
            lib.mlxrocm_nvfp4_dequantize_global(
                w.data_ptr(), scales.data_ptr(), gscale.data_ptr(), out.data_ptr(), out.numel(),
                _DTYPE_CODE[out_type], _stream_ptr(w),
            )
        )
        return out
    _lib.check(
        lib.mlxrocm_fp_dequantize(
            w.data_ptr(), scales.data_ptr(), out.data_ptr(), out.numel(),
            _MODE_CODE[mode], _DTYPE_CODE[out_type], _stream_ptr(w),
        )
    )
    return out


def _dense_batches(t: torch.Tensor, batch_shape: Tuple[int, ...]):
    """Expand the leading dims of ``t`` to ``batch_shape``; returns the tensor
    and its batch stride in elements (0 when one matrix serves every batch)."""
    if t.dim() == 2:
        return (t if _last_two_dense(t) else _contiguous(t)), 0
    t = t.expand(*batch_shape, *t.shape[-2:])
    t = _contiguous(t)
    return t, t.shape[-1] * t.shape[-2]


def quantized_swiglu(
    x: torch.Tensor,
    gate: tuple,
    up: tuple,
    group_size: Optional[int] = None,
    bits: Optional[int] = None,
):
    """``silu(quantized_matmul(x, *gate)) * quantized_matmul(x, *up)`` for decode
    (at most 8 rows of x), both projections in one launch.  ``gate`` and ``up``
    are ``(weight, scales, biases)`` triplets of equal shape, as
    ``nn.QuantizedLinear`` holds them (python/mlx/nn/layers/quantized.py:205-307);
    the reference has no fused primitive for the gated MLP, so more rows of x, or
    a device other than the GPU, raise instead of taking another route."""
    wg, sg, bg = gate
    wu, su, bu = up
    dtype, mode = _validate_mode_with_type("quantized_swiglu", sg, bg, None, "affine")
    group_size, bits = _params_from_mode(mode, group_size, bits)
    _, n_gate = _extract_dims("quantized_swiglu", x, wg, sg, bg, True, group_size, bits)
    _, n_up = _extract_dims("quantized_swiglu", x, wu, su, bu, True, group_size, bits)
    if n_gate != n_up or wg.shape != wu.shape or wg.dim() != 2:
        raise ValueError(
            "[quantized_swiglu] gate and up must be 2-D weights of one shape; got "
            f"{tuple(wg.shape)} and {tuple(wu.shape)}."
        )
    dtype = torch.promote_types(x.dtype, dtype)
    if dtype not in _FLOATING:
        raise ValueError(
            f"[quantized_swiglu] Only real floating types are supported but x.dtype() == {x.dtype}."
        )
    _check_affine_params("quantized_swiglu", group_size, bits)
    _require_gpu("quantized_swiglu", x, wg, sg, bg, wu, su, bu)
    lib = _lib.load()
    K = x.shape[-1]
    M = 1
    for d in x.shape[:-1]:
        M *= d
    xb = _contiguous(_astype(x, dtype)).reshape(M, K)
    sg, bg, su, bu = (_contiguous(_astype(t, dtype)) for t in (sg, bg, su, bu))
    wg, wu = _contiguous(wg), _contiguous(wu)
    code = _DTYPE_CODE[dtype]
    ws_bytes = lib.mlxrocm_qmm_swiglu_workspace_size(M, n_gate, code)
    workspace = torch.empty(max(int(ws_bytes), 16), dtype=torch.uint8, device=x.device)
    out = torch.empty(tuple(x.shape[:-1]) + (n_gate,), dtype=dtype, device=x.device)
    _lib.check(
        lib.mlxrocm_qmm_swiglu(
            xb.data_ptr(), wg.data_ptr(), sg.data_ptr(), bg.data_ptr(),
            wu.data_ptr(), su.data_ptr(), bu.data_ptr(), out.data_ptr(), workspace.data_ptr(),
            M, n_gate, K, group_size, bits, code, _stream_ptr(x),
        )
    )
    return out


class _QuantizedMatmulVjp(torch.autograd.Function):
    """The vector-Jacobian product of QuantizedMatmul with respect to x
    (mlx/primitives.cpp:3532-3555): the cotangent times the same quantized
    matrix with ``transpose`` flipped."""

    @staticmethod
    def forward(ctx, x, w, scales, biases, transpose, group_size, bits, mode, sb_image):
        ctx.save_for_backward(w, scales, biases if biases is not None else scales)
        ctx.args = (bool(transpose), group_size, bits, mode, biases is None, x.shape, x.dtype)
        return _quantized_matmul(x, w, scales, biases, transpose, group_size, bits, mode, sb_image)

    @staticmethod
    def backward(ctx, cotangent):
        w, scales, biases = ctx.saved_tensors
        transpose, group_size, bits, mode, no_biases, x_shape, x_dtype = ctx.args
        dx = _quantized_matmul(cotangent, w, scales, None if no_biases else biases,
                               not transpose, group_size, bits, mode, None)
        if tuple(dx.shape) != tuple(x_shape):
            raise NotImplementedError(
                "[QuantizedMatmul::vjp] x was broadcast against a batched weight: "
                f"cotangent of shape {tuple(dx.shape)} for x of shape {tuple(x_shape)}"
            )
        return (_astype(dx, x_dtype),) + (None,) * 8


def quantized_matmul(
    x: torch.Tensor,
    w: torch.Tensor,
    scales: torch.Tensor,
    biases: Optional[torch.Tensor] = None,
    transpose: bool = True,
    group_size: Optional[int] = None,
    bits: Optional[int] = None,
    mode: str = "affine",
    *,
    sb_image: Optional[torch.Tensor] = None,
):
    """``mx.quantized_matmul`` (mlx/ops.cpp:4784-4834).  ``sb_image`` (not in
    the reference): the result of :func:`quantized_matmul_sb_image` for these
    scales and biases, which saves prefill calls their transposition pre-pass;
    results do not depend on it.  Under autograd the gradient with respect to x
    is the reference's (QuantizedMatmul::vjp, mlx/primitives.cpp:3532-3555);
    gradients with respect to scales and biases are not provided."""
    if torch.is_grad_enabled():
        wants = [t is not None and t.requires_grad for t in (scales, biases)]
        if any(wants):
            if mode != "affine":
                # mlx/primitives.cpp:3562-3567
                raise ValueError(
                    f"[QuantizedMatmul::vjp] no gradient wrt scales in {mode} quantization."
                )
            raise NotImplementedError(
                "[QuantizedMatmul::vjp] gradients wrt scales and biases are not provided "
                "by mlx_amd (they need a dense matmul, which is outside this path)"
            )
        if x.requires_grad:
            return _QuantizedMatmulVjp.apply(
                x, w, scales, biases, transpose, group_size, bits, mode, sb_image
            )
    return _quantized_matmul(x, w, scales, biases, transpose, group_size, bits, mode, sb_image)


def _quantized_matmul(x, w, scales, biases, transpose, group_size, bits, mode, sb_image):
    dtype, mode = _validate_mode_with_type("quantized_matmul", scales, biases, None, mode)
    group_size, bits = _params_from_mode(mode, group_size, bits)
    _, w_outer = _extract_dims(
        "quantized_matmul", x, w, scales, biases, transpose, group_size, bits
    )
    affine = mode == "affine"
    dtype = torch.promote_types(x.dtype, dtype) if affine else x.dtype  # :4803-4807
    if dtype not in _FLOATING:
        raise ValueError(
            "[quantized_matmul] Only real floating types are supported but "
            f"x.dtype() == {x.dtype}."
        )
    if affine:
        _check_affine_params("quantized_matmul", group_size, bits)
        _require_gpu("quantized_matmul", x, w, scales, biases)
    else:
        _check_fp_params("quantized_matmul", mode, group_size, bits)
        _require_gpu("quantized_matmul", x, w, scales)
        if sb_image is not None:
            raise ValueError("[quantized_matmul] sb_image belongs to mode='affine'")
    lib = _lib.load()

    if affine:
        x = _astype(x, dtype)
        scales = _astype(scales, dtype)
        biases = _astype(biases, dtype)
    K = x.shape[-1]
    M = x.shape[-2] if x.dim() > 1 else 1
    x_batch = tuple(x.shape[:-2]) if x.dim() > 2 else ()
    if x.dim() > 2 and w.dim() > 2:
        # broadcast_arrays(inputs, {-2, -1}), :4823-4825
        batch_shape = tuple(torch.broadcast_shapes(x_batch, tuple(w.shape[:-2])))
    else:
        batch_shape = x_batch
        if w.dim() > 2:
            raise ValueError(
                "[quantized_matmul] a batched weight needs a batched first input"
            )
    out_shape = (tuple(x.shape[:-1]) if x.dim() <= 2 else batch_shape + (M,)) + (w_outer,)
    L = 1
    for d in batch_shape:
        L *= d
    xb = x.reshape(1, M, K) if x.dim() <= 2 else x.expand(*batch_shape, M, K)
    xb = _contiguous(xb)
    if w.dim() == 2 and L > 1:
        # one weight matrix for every batch entry: the batch folds into the rows
        # of x, so W is read once for all of them (the GPU backends do the same,
        # metal/quantized.cpp:1799-1801, cuda/quantized/qmm/qmm.cu:143-146)
        M, L = M * L, 1
    wb, w_stride = _dense_batches(w, batch_shape)
    sb, sb_stride = _dense_batches(scales, batch_shape)
    out = torch.empty(out_shape, dtype=dtype, device=x.device)
    code = _DTYPE_CODE[dtype]
    if not affine:
        ws_bytes = lib.mlxrocm_fp_qmm_workspace_size(
            M, w_outer, K, L, int(sb_stride != 0), _MODE_CODE[mode], code, int(bool(transpose)))
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
        _lib.check(
            lib.mlxrocm_fp_qmm(
                xb.data_ptr(), wb.data_ptr(), sb.data_ptr(), out.data_ptr(),
                M, w_outer, K, L, M * K, w_stride, sb_stride, _MODE_CODE[mode], code,
                int(bool(transpose)), ws.data_ptr() if ws is not None else None, ws_bytes,
                _stream_ptr(x),
            )
        )
        return out
    bb, _ = _dense_batches(biases, batch_shape)
    ws_bytes = lib.mlxrocm_qmm_workspace_size(
        M, w_outer, K, L, int(w_stride != 0), group_size, bits, code, int(bool(transpose))
    )
    # a temporary of the call, like the ones eval_gpu hands to add_temporary
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    if sb_image is not None:
        want = lib.mlxrocm_qmm_sb_image_size(
            w_outer, K, L if sb_stride else 1, group_size, code)
        if (not transpose or sb_image.dtype != dtype or sb_image.device != x.device
                or not sb_image.is_contiguous() or sb_image.numel() * sb_image.element_size() != want):
            raise ValueError(
                "[quantized_matmul] sb_image does not belong to these scales and biases "
                "(quantized_matmul_sb_image with the same dtype, transpose=True)"
            )
    _lib.check(
        lib.mlxrocm_qmm_prepacked(
            xb.data_ptr(), wb.data_ptr(), sb.data_ptr(), bb.data_ptr(),
            sb_image.data_ptr() if sb_image is not None else None, out.data_ptr(),
            M, w_outer, K, L, M * K, w_stride, sb_stride, group_size, bits,
            code, int(bool(transpose)),
            ws.data_ptr() if ws is not None else None, ws_bytes, _stream_ptr(x),
        )
    )
    return out


def quantized_matmul_sb_image(
    scales: torch.Tensor,
    biases: torch.Tensor,
    group_size: int = 64,
    dtype: Optional[torch.dtype] = None,
) -> torch.Tensor:
    """Scales and biases of ``[..., N, K / group_size]`` weights transposed to the
    ``[K / group_size][N]`` image the prefill kernels read, to be kept beside a
    weight and passed to ``quantized_matmul(..., sb_image=...)``.  ``dtype``: the
    type the product will run in (that of x after promotion; default: that of
    the scales).  No counterpart in the reference."""
    dtype = dtype or scales.dtype
    _require_gpu("quantized_matmul_sb_image", scales, biases)
    if scales.shape != biases.shape or scales.dim() < 2:
        raise ValueError("[quantized_matmul_sb_image] scales and biases must have one shape")
    lib = _lib.load()
    s = _contiguous(_astype(scales, dtype))
    b = _contiguous(_astype(biases, dtype))
    N, G = s.shape[-2], s.shape[-1]
    batches = s.numel() // (N * G)
    code = _DTYPE_CODE[dtype]
    nbytes = lib.mlxrocm_qmm_sb_image_size(N, G * group_size, batches, group_size, code)
    image = torch.empty(nbytes // s.element_size(), dtype=dtype, device=s.device)
    _lib.check(
        lib.mlxrocm_qmm_sb_image(
            s.data_ptr(), b.data_ptr(), image.data_ptr(), N, G * group_size, batches,
            N * G, group_size, code, _stream_ptr(s),
        )
    )
    return image


def _indices_or_default(tag, indices, t):
    # mlx/ops.cpp:79-108
    if t.dim() < 2:
        raise ValueError(
            f"{tag} Input must have at least two dimensions but got input with shape "
            f"{tuple(t.shape)}."
        )
    if indices is not None:
        if indices.dtype not in _INTEGER:
            raise ValueError(
                f"{tag} Got indices with invalid dtype. Indices must be integral."
            )
        return indices
    shape = tuple(t.shape[:-2])
    total = 1
    for d in shape:
        total *= d
    return torch.arange(total, dtype=torch.int32, device=t.device).reshape(shape)


def _broadcast_shape(a: tuple, b: tuple) -> tuple:
    """Numpy broadcasting of two shapes in plain Python (the library routine
    costs more than the rest of a decode-sized call)."""
    if a == b:
        return a
    if len(a) < len(b):
        a, b = b, a
    out = list(a)
    off = len(a) - len(b)
    for i, d in enumerate(b):
        e = out[off + i]
        if e == d or d == 1:
            continue
        if e != 1:
            raise ValueError(f"Shapes {a} and {b} cannot be broadcast.")
        out[off + i] = d
    return tuple(out)


@functools.lru_cache(maxsize=64)
def _default_lhs_uint32(batch_shape: tuple, like_shape: tuple, device: torch.device) -> torch.Tensor:
    """The default ``lhs_indices`` (``arange`` over the batch dims of x,
    mlx/ops.cpp:100-107) broadcast against ``like_shape`` and flattened to
    uint32.  It depends on shapes only, so it is built once per shape and kept:
    a decode step then issues no kernel for it.  Callers only read it."""
    total = 1
    for d in batch_shape:
        total *= d
    lhs = torch.arange(total, dtype=torch.int32, device=device).reshape(batch_shape)
    shape = _broadcast_shape(batch_shape, like_shape)
    flat = lhs.expand(shape).reshape(-1).contiguous().view(torch.uint32)
    torch.cuda.current_stream(device).synchronize()  # later calls may run on other streams
    return flat


def _as_uint32(indices: torch.Tensor) -> torch.Tensor:
    """Flat uint32 view or copy of an index tensor: what ``astype(indices,
    uint32)`` gives (mlx/ops.cpp:5600-5601) -- two's-complement truncation, so
    32-bit indices are reinterpreted without a kernel."""
    flat = _contiguous(indices).reshape(-1)
    if flat.dtype == torch.uint32:
        return flat
    if flat.dtype == torch.int32:
        return flat.view(torch.uint32)
    return _astype(flat, torch.uint32)


def gather_qmm(
    x: torch.Tensor,
    w: torch.Tensor,
    scales: torch.Tensor,
    biases: Optional[torch.Tensor] = None,
    lhs_indices: Optional[torch.Tensor] = None,
    rhs_indices: Optional[torch.Tensor] = None,
    transpose: bool = True,
    group_size: Optional[int] = None,
    bits: Optional[int] = None,
    mode: str = "affine",
    sorted_indices: bool = False,
):
    """``mx.gather_qmm`` (mlx/ops.cpp:5553-5629)."""
    if lhs_indices is None and rhs_indices is None:
        return quantized_matmul(x, w, scales, biases, transpose, group_size, bits, mode)
    out_type, mode = _validate_mode_with_type("gather_qmm", scales, biases, None, mode)
    group_size, bits = _params_from_mode(mode, group_size, bits)
    _, w_outer = _extract_dims(
        "gather_qmm", x, w, scales, biases, transpose, group_size, bits
    )
    affine = mode == "affine"
    out_type = torch.promote_types(x.dtype, out_type) if affine else x.dtype
    if out_type not in _FLOATING:
        raise ValueError(
            f"[gather_qmm] Only real floating types are supported but x.dtype() == {x.dtype}."
        )
    lhs = None if lhs_indices is None and rhs_indices is not None else \
        _indices_or_default("[gather_qmm]", lhs_indices, x)
    rhs = _indices_or_default("[gather_qmm]", rhs_indices, w)
    if lhs is None:
        # default lhs against given rhs: shapes decide everything
        if x.dim() < 2:
            raise ValueError(
                "[gather_qmm] Input must have at least two dimensions but got input with "
                f"shape {tuple(x.shape)}."
            )
        lhs_shape = _broadcast_shape(tuple(x.shape[:-2]), tuple(rhs.shape))
    if affine:
        _check_affine_params("gather_qmm", group_size, bits)
    else:
        _check_fp_params("gather_qmm", mode, group_size, bits)
    _require_gpu("gather_qmm", x, w, scales, rhs, *(() if biases is None else (biases,)),
                 *(() if lhs is None else (lhs,)))
    lib = _lib.load()
    if lhs is None:
        if tuple(rhs.shape) != lhs_shape:
            rhs = rhs.expand(lhs_shape)
    elif lhs.shape != rhs.shape:
        lhs, rhs = torch.broadcast_tensors(lhs, rhs)
    right_sorted = bool(sorted_indices) and lhs_indices is None

    if affine:
        x = _astype(x, out_type)
        scales = _astype(scales, out_type)
        biases = _astype(biases, out_type)
    M, K = x.shape[-2], x.shape[-1]
    xb = _contiguous(x).reshape(-1, M, K)
    # Only the trailing matrices must be dense; a sliced expert stack keeps its
    # stride (python/tests/test_quantized.py:1567-1593).
    def experts(t):
        if t.dim() == 3 and _last_two_dense(t):
            return t, t.stride(0)
        t = _contiguous(t).reshape(-1, *t.shape[-2:])
        return t, t.shape[-1] * t.shape[-2]
    wb, w_stride = experts(w)
    sb, sb_stride = experts(scales)
    if not affine:
        n_idx = rhs.numel()
        if lhs is None:
            lhs_u = _default_lhs_uint32(tuple(x.shape[:-2]), tuple(rhs.shape), x.device)
        else:
            lhs_u = _as_uint32(lhs) if n_idx else lhs.reshape(-1)
        rhs_u = _as_uint32(rhs) if n_idx else rhs.reshape(-1)
        out = torch.empty(tuple(rhs.shape) + (M, w_outer), dtype=out_type, device=x.device)
        ws_bytes = lib.mlxrocm_fp_gather_qmm_workspace_size(
            M, w_outer, K, n_idx, wb.shape[0], int(sb_stride != 0), _MODE_CODE[mode],
            _DTYPE_CODE[out_type], int(bool(transpose)),
        )
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
        _lib.check(
            lib.mlxrocm_fp_gather_qmm(
                xb.data_ptr(), wb.data_ptr(), sb.data_ptr(),
                lhs_u.data_ptr() if n_idx else None, rhs_u.data_ptr() if n_idx else None,
                out.data_ptr(), M, w_outer, K, n_idx, xb.shape[0], wb.shape[0],
                M * K, w_stride, sb_stride, _MODE_CODE[mode], _DTYPE_CODE[out_type],
                int(bool(transpose)), ws.data_ptr() if ws is not None else None, ws_bytes,
                _stream_ptr(x),
            )
        )
        return out
    bb, bb_stride = experts(biases)
    if bb_stride != sb_stride:
        bb = _contiguous(bb)
        sb = _contiguous(sb)
        sb_stride = sb.shape[-1] * sb.shape[-2]
    n_idx = rhs.numel()
    if lhs is None:
        lhs_u = _default_lhs_uint32(tuple(x.shape[:-2]), tuple(rhs.shape), x.device)
    else:
        lhs_u = _as_uint32(lhs) if n_idx else lhs.reshape(-1)
    rhs_u = _as_uint32(rhs) if n_idx else rhs.reshape(-1)
    out = torch.empty(tuple(rhs.shape) + (M, w_outer), dtype=out_type, device=x.device)
    code = _DTYPE_CODE[out_type]
    ws_bytes = lib.mlxrocm_gather_qmm_workspace_size(
        M, w_outer, K, n_idx, wb.shape[0], group_size, bits, code,
        int(bool(transpose)), int(right_sorted),
    )
    ws = (
        torch.empty(ws_bytes, dtype=torch.uint8, device=x.device) if ws_bytes else None
    )
    _lib.check(
        lib.mlxrocm_gather_qmm(
            xb.data_ptr(), wb.data_ptr(), sb.data_ptr(), bb.data_ptr(),
            lhs_u.data_ptr() if n_idx else None, rhs_u.data_ptr() if n_idx else None,
            out.data_ptr(), M, w_outer, K, n_idx, xb.shape[0], wb.shape[0],
            M * K, w_stride, sb_stride, group_size, bits, code,
            int(bool(transpose)), int(right_sorted),
            ws.data_ptr() if ws is not None else None, ws_bytes, _stream_ptr(x),
        )
    )
    return out


def qqmm(
    x: torch.Tensor,
    w: torch.Tensor,
    scales: Optional[torch.Tensor] = None,
    group_size: Optional[int] = None,
    bits: Optional[int] = None,
    mode: str = "nvfp4",
    global_scale_x: Optional[torch.Tensor] = None,
    global_scale_w: Optional[torch.Tensor] = None,
):
    """``mx.qqmm`` (mlx/ops.cpp:4926-4990): x is quantized and dequantized on
    the fly, then multiplied by the transposed quantized w.  Like the CPU backend
    (QQMatmul::eval_cpu, mlx/backend/cpu/quantized.cpp:1322-1360) this takes a
    quantized w; unlike it, any number of rows of x.  A floating-point w, which
    the CPU backend does not take either, is quantized first as the CUDA backend
    does (mlx/backend/cuda/quantized/qqmm.cpp)."""
    mode = _mode("qqmm", mode)
    group_size, bits = _params_from_mode(mode, group_size, bits)
    in_shape = tuple(x.shape)
    if x.dim() == 1:
        x = x.unsqueeze(0)
    elif w.dim() == 2 and x.dim() > 2:
        x = x.reshape(-1, x.shape[-1])
    # validate_qqmm_inputs, mlx/ops.cpp:4836-4894
    if x.dim() > 2 or w.dim() > 2:
        raise ValueError(
            f"[qqmm] Only 2D inputs are supported but x.ndim() == {x.dim()} and "
            f"w.ndim() == {w.dim()}."
        )
    if w.dtype == torch.uint32:
        if scales is None:
            raise ValueError("[qqmm] Scales must be provided if second argument is quantized.")
        _validate_quantized_input("qqmm", w, scales, group_size, bits, None)
    elif w.dtype not in _FLOATING:
        raise ValueError(
            "[qqmm] Only real floating types except float64 are supported but "
            f"second argument dtype == {w.dtype}."
        )
    if x.dtype not in _FLOATING:
        raise ValueError(
            "[qqmm] Only real floating types except float64 are supported but "
            f"first argument dtype == {x.dtype}."
        )
    if mode == "affine":
        raise ValueError("[qqmm] Affine quantization is not supported for qqmm.")
    if mode == "nvfp4" and (global_scale_x is None) != (global_scale_w is None):
        raise ValueError(
            "[qqmm] For nvfp4 mode, either both global_scale_x and global_scale_w "
            "must be provided, or neither."
        )
    gx = _global_scale("qqmm", mode, global_scale_x, x)
    gw = _global_scale("qqmm", mode, global_scale_w, x)
    _check_fp_params("qqmm", mode, group_size, bits)
    if w.dtype != torch.uint32:
        # extract_qqmm_dims, :4896-4924
        if x.shape[-1] != w.shape[-1]:
            raise ValueError(
                f"[qqmm] Last dimension of first input with shape {tuple(x.shape)} must "
                f"match last dimension of second input with shape {tuple(w.shape)}."
            )
        w, scales = quantize(_astype(w, x.dtype), group_size, bits, mode, global_scale=gw)
    else:
        _extract_dims("qqmm", x, w, scales, None, True, group_size, bits)
    if scales.dtype != torch.uint8:
        raise ValueError(f"[qqmm] Scale type must be uint8 but received type {scales.dtype}.")
    _require_gpu("qqmm", x, w, scales)
    lib = _lib.load()
    xc = _contiguous(x)
    wc = w if _last_two_dense(w) else _contiguous(w)
    sc = scales if _last_two_dense(scales) else _contiguous(scales)
    M, K = xc.shape
    N = wc.shape[0]
    code = _DTYPE_CODE[xc.dtype]
    out = torch.empty((M, N), dtype=xc.dtype, device=xc.device)
    ws_bytes = lib.mlxrocm_fp_qqmm_workspace_size(M, N, K, _MODE_CODE[mode], code)
    ws = torch.empty(max(int(ws_bytes), 256), dtype=torch.uint8, device=xc.device)
    if gx is not None:
        _lib.check(
            lib.mlxrocm_nvfp4_qqmm_global(
                xc.data_ptr(), wc.data_ptr(), sc.data_ptr(), gx.data_ptr(), gw.data_ptr(),
                out.data_ptr(), M, N, K, code, ws.data_ptr(), ws_bytes, _stream_ptr(xc),
            )
        )
    else:
        _lib.check(
            lib.mlxrocm_fp_qqmm(
                xc.data_ptr(), wc.data_ptr(), sc.data_ptr(), out.data_ptr(), M, N, K,
                _MODE_CODE[mode], code, ws.data_ptr(), ws_bytes, _stream_ptr(xc),
            )
        )
    if len(in_shape) > 2:
        return out.reshape(in_shape[:-1] + (out.shape[-1],))
    if len(in_shape) == 1:
        return out.squeeze(0)
    return out


def gather_qqmm(
    x: torch.Tensor,
    w: torch.Tensor,
    scales: Optional[torch.Tensor] = None,
    lhs_indices: Optional[torch.Tensor] = None,
    rhs_indices: Optional[torch.Tensor] = None,
    group_size: Optional[int] = None,
    bits: Optional[int] = None,
    mode: str = "nvfp4",
    global_scale_x: Optional[torch.Tensor] = None,
    global_scale_w: Optional[torch.Tensor] = None,
    sorted_indices: bool = False,
):
    """``mx.gather_qqmm`` (mlx/ops.cpp:5631-5681; GatherQQMM::eval_gpu,
    mlx/backend/cuda/quantized/qqmm.cpp:210-281 -- the CPU backend has none):
    every matrix of x is quantized and dequantized in its own type, then pair i
    multiplies ``x_hat[lhs_indices[i]]`` by the transposed quantized
    ``w[rhs_indices[i]]``.  A floating-point w is quantized first."""
    mode = _mode("gather_qqmm", mode)
    group_size, bits = _params_from_mode(mode, group_size, bits)
    if mode == "affine":
        raise ValueError("[gather_qqmm] Affine quantization is not supported for qqmm.")
    if x.dtype not in _FLOATING:
        raise ValueError(
            "[gather_qqmm] Only real floating types except float64 are supported but "
            f"first argument dtype == {x.dtype}."
        )
    if (global_scale_x is None) != (global_scale_w is None):
        raise ValueError(
            "[gather_qqmm] For nvfp4 mode, either both global_scale_x and global_scale_w "
            "must be provided, or neither."
        )
    gx = _global_scale("gather_qqmm", mode, global_scale_x, x)
    gw = _global_scale("gather_qqmm", mode, global_scale_w, x)
    _check_fp_params("gather_qqmm", mode, group_size, bits)
    if x.dim() < 2:
        raise ValueError(
            "[gather_qqmm] Input must have at least two dimensions but got input with "
            f"shape {tuple(x.shape)}."
        )
    if w.dtype != torch.uint32:
        # extract_qqmm_dims, mlx/ops.cpp:4896-4924
        if w.dtype not in _FLOATING:
            raise ValueError(
                "[gather_qqmm] Only real floating types except float64 are supported but "
                f"second argument dtype == {w.dtype}."
            )
        if x.shape[-1] != w.shape[-1]:
            raise ValueError(
                f"[gather_qqmm] Last dimension of first input with shape {tuple(x.shape)} must "
                f"match last dimension of second input with shape {tuple(w.shape)}."
            )
        w, scales = quantize(_astype(w, x.dtype), group_size, bits, mode, global_scale=gw)
    else:
        if scales is None:
            raise ValueError(
                "[gather_qqmm] Scales must be provided if second argument is quantized."
            )
        _extract_dims("gather_qqmm", x, w, scales, None, True, group_size, bits)
    if scales.dtype != torch.uint8:
        raise ValueError(
            f"[gather_qqmm] Scale type must be uint8 but received type {scales.dtype}."
        )
    w_outer = w.shape[-2]
    lhs = _indices_or_default("[gather_qqmm]", lhs_indices, x)
    rhs = _indices_or_default("[gather_qqmm]", rhs_indices, w)
    _require_gpu("gather_qqmm", x, w, scales, lhs, rhs)
    lib = _lib.load()
    if lhs.shape != rhs.shape:
        lhs, rhs = torch.broadcast_tensors(lhs, rhs)
    M, K = x.shape[-2], x.shape[-1]
    xb = _contiguous(x).reshape(-1, M, K)

    def experts(t):
        if t.dim() == 3 and _last_two_dense(t):
            return t, t.stride(0)
        t = _contiguous(t).reshape(-1, *t.shape[-2:])
        return t, t.shape[-1] * t.shape[-2]

    wb, w_stride = experts(w)
    sb, sb_stride = experts(scales)
    n_idx = rhs.numel()
    lhs_u = _as_uint32(lhs) if n_idx else lhs.reshape(-1)
    rhs_u = _as_uint32(rhs) if n_idx else rhs.reshape(-1)
    out = torch.empty(tuple(rhs.shape) + (M, w_outer), dtype=x.dtype, device=x.device)
    code = _DTYPE_CODE[x.dtype]
    ws_bytes = lib.mlxrocm_fp_gather_qqmm_workspace_size(
        M, w_outer, K, n_idx, xb.shape[0], wb.shape[0], int(sb_stride != 0), _MODE_CODE[mode], code
    )
    ws = torch.empty(max(int(ws_bytes), 256), dtype=torch.uint8, device=x.device)
    _lib.check(
        lib.mlxrocm_fp_gather_qqmm(
            xb.data_ptr(), wb.data_ptr(), sb.data_ptr(),
            lhs_u.data_ptr() if n_idx else None, rhs_u.data_ptr() if n_idx else None,
            gx.data_ptr() if gx is not None else None,
            gw.data_ptr() if gw is not None else None,
            out.data_ptr(), M, w_outer, K, n_idx, xb.shape[0], wb.shape[0],
            M * K, w_stride, sb_stride, _MODE_CODE[mode], code,
            ws.data_ptr(), ws_bytes, _stream_ptr(x),
        )
    )
    return out


def to_fp8(x: torch.Tensor) -> torch.Tensor:
    """``mx.to_fp8`` (mlx/ops.cpp:5539-5552): elementwise conversion to e4m3
    bytes, round to nearest even, saturating at 448."""
    if x.dtype not in _FLOATING:
        raise ValueError(
            f"[to_fp8] Only real floating types are supported but x.dtype() == {x.dtype}."
        )
    _require_gpu("to_fp8", x)
    lib = _lib.load()
    xc = _contiguous(x)
    out = torch.empty(xc.shape, dtype=torch.uint8, device=xc.device)
    _lib.check(
        lib.mlxrocm_to_fp8(xc.data_ptr(), out.data_ptr(), xc.numel(), _DTYPE_CODE[xc.dtype],
                           _stream_ptr(xc))
    )
    return out


def from_fp8(x: torch.Tensor, dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """``mx.from_fp8`` (mlx/ops.cpp:5519-5537): e4m3 bytes to ``dtype``."""
    if x.dtype != torch.uint8:
        raise ValueError(f"[from_fp8] Input must have type uint8 but x.dtype() == {x.dtype}.")
    if dtype not in _FLOATING:
        raise ValueError(
            f"[from_fp8] Only real floating types are supported but dtype == {dtype}."
        )
    _require_gpu("from_fp8", x)
    lib = _lib.load()
    xc = _contiguous(x)
    out = torch.empty(xc.shape, dtype=dtype, device=xc.device)
    _lib.check(
        lib.mlxrocm_from_fp8(xc.data_ptr(), out.data_ptr(), xc.numel(), _DTYPE_CODE[dtype],
                             _stream_ptr(xc))
    )
    return out
