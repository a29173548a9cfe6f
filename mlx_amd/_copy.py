"""Element copies through the HIP copy kernels of the C ABI
(``mlxrocm_copy_contiguous`` / ``mlxrocm_copy_strided``): the host-side
counterpart of ``copy_gpu`` / ``contiguous_copy_gpu`` / ``astype``
(reference: ``mlx/backend/gpu/copy.cpp:11-44``).  torch supplies the output
allocation and the current stream only."""
from __future__ import annotations

import ctypes

import torch

from . import _lib

DTYPE_CODE = {
    torch.float32: 0, torch.float16: 1, torch.bfloat16: 2, torch.bool: 3,
    torch.uint8: 4, torch.uint16: 5, torch.uint32: 6, torch.uint64: 7,
    torch.int8: 8, torch.int16: 9, torch.int32: 10, torch.int64: 11,
    torch.float64: 12, torch.complex64: 13,
}


def _code(dtype: torch.dtype) -> int:
    try:
        return DTYPE_CODE[dtype]
    except KeyError:
        raise ValueError(f"[copy] dtype {dtype} has no ROCm copy kernel") from None


def _i64_array(values):
    return (ctypes.c_int64 * max(1, len(values)))(*values)


def copy(t: torch.Tensor, dtype: torch.dtype | None = None) -> torch.Tensor:
    """A new row-contiguous tensor with ``t``'s values converted to ``dtype``."""
    if t.device.type != "cuda":
        raise RuntimeError(f"[copy] mlx_amd runs on the GPU only; got a tensor on {t.device}")
    dtype = t.dtype if dtype is None else dtype
    out = torch.empty(t.shape, dtype=dtype, device=t.device)
    if out.numel() == 0:
        return out
    lib = _lib.load()
    stream = torch.cuda.current_stream(t.device).cuda_stream
    if t.is_contiguous():
        _lib.check(lib.mlxrocm_copy_contiguous(
            t.data_ptr(), _code(t.dtype), out.data_ptr(), _code(dtype), t.numel(), 0, stream))
    else:
        _lib.check(lib.mlxrocm_copy_strided(
            t.data_ptr(), _code(t.dtype), _i64_array(t.stride()),
            out.data_ptr(), _code(dtype), None,
            t.dim(), _i64_array(t.shape), stream))
    return out


def contiguous(t: torch.Tensor) -> torch.Tensor:
    """``t`` itself when it is row-contiguous, else a contiguous copy."""
    return t if t.is_contiguous() else copy(t)


def astype(t: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """``t`` itself when it already has ``dtype``, else a converted (contiguous) copy."""
    return t if t.dtype == dtype else copy(t, dtype)


def full_like(t: torch.Tensor, value: torch.Tensor) -> torch.Tensor:
    """A tensor shaped like ``t`` filled with the one-element device tensor
    ``value`` converted to ``t``'s dtype (``fill_gpu``)."""
    out = torch.empty_like(t, memory_format=torch.contiguous_format)
    if out.numel():
        lib = _lib.load()
        stream = torch.cuda.current_stream(t.device).cuda_stream
        _lib.check(lib.mlxrocm_copy_contiguous(
            value.data_ptr(), _code(value.dtype), out.data_ptr(), _code(out.dtype),
            out.numel(), 1, stream))
    return out
