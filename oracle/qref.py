"""ctypes front end of the CPU parity oracle (test infrastructure only).

Two interchangeable back ends with the same call signatures:

* ``Oracle("port")``      -- ``libaffine_qref.so``, this repository's C
  restatement of the reference's CPU algorithm (``affine_qref.c``).
* ``Oracle("reference")`` -- ``_ref/libmlx_cpu_qref.so``, the reference's own
  ``mlx/backend/cpu/quantized.cpp`` compiled as one translation unit.  It has
  no dequantize / batched / gather entry points (the reference expresses those
  with array objects), so those calls always go to the port, which loops over
  the selected back end's ``qmm``.

All functions take and return CPU torch tensors; float16 / bfloat16 travel as
raw 16-bit storage.  Only tests, the smoke check and the benchmark's
cpu_baseline leg may import this module.
"""
from __future__ import annotations

import ctypes
import os

import torch

HERE = os.path.dirname(os.path.abspath(__file__))
QREF_SO = os.path.join(HERE, "libaffine_qref.so")
REF_SO = os.path.join(HERE, "_ref", "libmlx_cpu_qref.so")

DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}

_c_int = ctypes.c_int
_c_size = ctypes.c_size_t
_c_ptr = ctypes.c_void_p


def _ptr(t: torch.Tensor) -> int:
    assert t.device.type == "cpu" and t.is_contiguous()
    return t.data_ptr()


def _load(path: str) -> ctypes.CDLL:
    if not os.path.isfile(path):
        raise FileNotFoundError(
            f"{path} is not built; run `python oracle/build.py` first"
        )
    return ctypes.CDLL(path)


def reference_built() -> bool:
    return os.path.isfile(REF_SO)


class Oracle:
    def __init__(self, kind: str = "port"):
        if kind not in ("port", "reference"):
            raise ValueError(kind)
        self.kind = kind
        self.port = _load(QREF_SO)
        self._declare_port(self.port)
        self.ref = None
        if kind == "reference":
            self.ref = _load(REF_SO)
            self._declare_ref(self.ref)

    @staticmethod
    def _declare_port(lib):
        lib.qref_quantize.argtypes = [_c_ptr] * 4 + [_c_int, _c_int, _c_size, _c_int]
        lib.qref_quantize.restype = _c_int
        lib.qref_dequantize.argtypes = [_c_ptr] * 4 + [_c_size, _c_int, _c_int, _c_int]
        lib.qref_dequantize.restype = _c_int
        lib.qref_qmm.argtypes = [_c_ptr] * 5 + [_c_int] * 7
        lib.qref_qmm.restype = _c_int
        lib.qref_qmm_batched.argtypes = (
            [_c_ptr] * 5 + [_c_int] * 4 + [_c_size] * 3 + [_c_int] * 4
        )
        lib.qref_qmm_batched.restype = _c_int
        lib.qref_gather_qmm.argtypes = (
            [_c_ptr] * 7 + [_c_int] * 4 + [_c_size] * 3 + [_c_int] * 4
        )
        lib.qref_gather_qmm.restype = _c_int
        lib.qref_bf16_from_f32.argtypes = [ctypes.c_float]
        lib.qref_bf16_from_f32.restype = ctypes.c_uint16
        lib.qref_bf16_to_f32.argtypes = [ctypes.c_uint16]
        lib.qref_bf16_to_f32.restype = ctypes.c_float
        lib.qref_f16_from_f32.argtypes = [ctypes.c_float]
        lib.qref_f16_from_f32.restype = ctypes.c_uint16
        lib.qref_f16_to_f32.argtypes = [ctypes.c_uint16]
        lib.qref_f16_to_f32.restype = ctypes.c_float
        lib.qref_pack_factor.argtypes = [_c_int, _c_int]
        lib.qref_bytes_per_pack.argtypes = [_c_int, _c_int]

    @staticmethod
    def _declare_ref(lib):
        lib.ref_quantize.argtypes = [_c_ptr] * 4 + [_c_int, _c_int, _c_size, _c_int]
        lib.ref_quantize.restype = _c_int
        lib.ref_qmm.argtypes = [_c_ptr] * 5 + [_c_int] * 7
        lib.ref_qmm.restype = _c_int
        lib.ref_simd_max_size.argtypes = [_c_int]
        lib.ref_bf16_from_f32.argtypes = [ctypes.c_float]
        lib.ref_bf16_from_f32.restype = ctypes.c_uint16
        lib.ref_bf16_to_f32.argtypes = [ctypes.c_uint16]
        lib.ref_bf16_to_f32.restype = ctypes.c_float
        lib.ref_f16_from_f32.argtypes = [ctypes.c_float]
        lib.ref_f16_from_f32.restype = ctypes.c_uint16
        lib.ref_f16_to_f32.argtypes = [ctypes.c_uint16]
        lib.ref_f16_to_f32.restype = ctypes.c_float

    # ------------------------------------------------------------------ ops
    def quantize(self, w: torch.Tensor, group_size: int = 64, bits: int = 4):
        """w [..., K] -> (wq uint32 [..., K*bits/32], scales, biases [..., K/gs])."""
        w = w.contiguous()
        K = w.shape[-1]
        assert K % group_size == 0 and (K * bits) % 32 == 0
        lead = tuple(w.shape[:-1])
        wq = torch.zeros(lead + (K * bits // 32,), dtype=torch.uint32)
        scales = torch.empty(lead + (K // group_size,), dtype=w.dtype)
        biases = torch.empty_like(scales)
        fn = self.ref.ref_quantize if self.ref is not None else self.port.qref_quantize
        rc = fn(
            _ptr(w), _ptr(wq), _ptr(scales), _ptr(biases), bits, group_size,
            w.numel(), DTYPE_CODE[w.dtype],
        )
        if rc != 0:
            raise ValueError(f"oracle quantize rejected bits={bits} gs={group_size}")
        return wq, scales, biases

    def dequantize(self, wq, scales, biases, group_size: int = 64, bits: int = 4):
        wq, scales, biases = wq.contiguous(), scales.contiguous(), biases.contiguous()
        K = wq.shape[-1] * 32 // bits
        out = torch.empty(tuple(wq.shape[:-1]) + (K,), dtype=scales.dtype)
        rc = self.port.qref_dequantize(
            _ptr(wq), _ptr(scales), _ptr(biases), _ptr(out), out.numel(),
            group_size, bits, DTYPE_CODE[scales.dtype],
        )
        if rc != 0:
            raise ValueError("oracle dequantize rejected arguments")
        return out

    def _qmm_ptr(self, y, x, w, s, b, M, N, K, group_size, bits, transpose, code):
        fn = self.ref.ref_qmm if self.ref is not None else self.port.qref_qmm
        rc = fn(y, x, w, s, b, M, N, K, group_size, bits, int(transpose), code)
        if rc != 0:
            raise ValueError("oracle qmm rejected arguments")

    def qmm(self, x, wq, scales, biases, transpose=True, group_size=64, bits=4):
        """x [M, K]; wq/scales/biases 2-D.  Returns [M, N] in x.dtype."""
        x, wq = x.contiguous(), wq.contiguous()
        scales, biases = scales.contiguous(), biases.contiguous()
        assert x.dim() == 2 and wq.dim() == 2
        M, K = x.shape
        N = wq.shape[0] if transpose else wq.shape[1] * 32 // bits
        y = torch.empty((M, N), dtype=x.dtype)
        self._qmm_ptr(
            _ptr(y), _ptr(x), _ptr(wq), _ptr(scales), _ptr(biases), M, N, K,
            group_size, bits, transpose, DTYPE_CODE[x.dtype],
        )
        return y

    def qmm_batched(self, x, wq, scales, biases, transpose=True, group_size=64, bits=4):
        """x [L, M, K]; wq either 2-D (shared by every batch) or [L, ., .]."""
        x, wq = x.contiguous(), wq.contiguous()
        scales, biases = scales.contiguous(), biases.contiguous()
        L, M, K = x.shape
        N = wq.shape[-2] if transpose else wq.shape[-1] * 32 // bits
        y = torch.empty((L, M, N), dtype=x.dtype)
        es = x.element_size()
        w_stride = 0 if wq.dim() == 2 else wq.shape[-1] * wq.shape[-2]
        sb_stride = 0 if wq.dim() == 2 else scales.shape[-1] * scales.shape[-2]
        for i in range(L):
            self._qmm_ptr(
                _ptr(y) + i * M * N * es, _ptr(x) + i * M * K * es,
                _ptr(wq) + i * w_stride * 4, _ptr(scales) + i * sb_stride * es,
                _ptr(biases) + i * sb_stride * es, M, N, K, group_size, bits,
                transpose, DTYPE_CODE[x.dtype],
            )
        return y

    def gather_qmm(
        self, x, wq, scales, biases, lhs_indices, rhs_indices, transpose=True,
        group_size=64, bits=4,
    ):
        """x [Bx, M, K]; wq [E, ., .]; flat index vectors of equal length."""
        x, wq = x.contiguous(), wq.contiguous()
        scales, biases = scales.contiguous(), biases.contiguous()
        Bx, M, K = x.shape
        N = wq.shape[-2] if transpose else wq.shape[-1] * 32 // bits
        lhs = lhs_indices.reshape(-1).tolist()
        rhs = rhs_indices.reshape(-1).tolist()
        assert len(lhs) == len(rhs)
        y = torch.empty((len(lhs), M, N), dtype=x.dtype)
        es = x.element_size()
        w_stride = wq.shape[-1] * wq.shape[-2]
        sb_stride = scales.shape[-1] * scales.shape[-2]
        for i, (xi, wi) in enumerate(zip(lhs, rhs)):
            assert 0 <= xi < Bx and 0 <= wi < wq.shape[0]
            self._qmm_ptr(
                _ptr(y) + i * M * N * es, _ptr(x) + xi * M * K * es,
                _ptr(wq) + wi * w_stride * 4, _ptr(scales) + wi * sb_stride * es,
                _ptr(biases) + wi * sb_stride * es, M, N, K, group_size, bits,
                transpose, DTYPE_CODE[x.dtype],
            )
        return y

    # The port's own C loops (exercised by the oracle self-tests).
    def port_qmm_batched(self, x, wq, scales, biases, transpose, group_size, bits):
        x, wq = x.contiguous(), wq.contiguous()
        scales, biases = scales.contiguous(), biases.contiguous()
        L, M, K = x.shape
        N = wq.shape[-2] if transpose else wq.shape[-1] * 32 // bits
        y = torch.empty((L, M, N), dtype=x.dtype)
        w_stride = 0 if wq.dim() == 2 else wq.shape[-1] * wq.shape[-2]
        sb_stride = 0 if wq.dim() == 2 else scales.shape[-1] * scales.shape[-2]
        rc = self.port.qref_qmm_batched(
            _ptr(y), _ptr(x), _ptr(wq), _ptr(scales), _ptr(biases), M, N, K, L,
            M * K, w_stride, sb_stride, group_size, bits, int(transpose),
            DTYPE_CODE[x.dtype],
        )
        assert rc == 0
        return y

    def port_gather_qmm(
        self, x, wq, scales, biases, lhs_indices, rhs_indices, transpose,
        group_size, bits,
    ):
        x, wq = x.contiguous(), wq.contiguous()
        scales, biases = scales.contiguous(), biases.contiguous()
        Bx, M, K = x.shape
        N = wq.shape[-2] if transpose else wq.shape[-1] * 32 // bits
        lhs = lhs_indices.reshape(-1).to(torch.int64).to(torch.uint32).contiguous()
        rhs = rhs_indices.reshape(-1).to(torch.int64).to(torch.uint32).contiguous()
        y = torch.empty((lhs.numel(), M, N), dtype=x.dtype)
        rc = self.port.qref_gather_qmm(
            _ptr(y), _ptr(x), _ptr(wq), _ptr(scales), _ptr(biases), _ptr(lhs),
            _ptr(rhs), lhs.numel(), M, N, K, M * K,
            wq.shape[-1] * wq.shape[-2], scales.shape[-1] * scales.shape[-2],
            group_size, bits, int(transpose), DTYPE_CODE[x.dtype],
        )
        assert rc == 0
        return y


def unpack_codes(wq: torch.Tensor, bits: int) -> torch.Tensor:
    """Integer codes [..., K] of a packed tensor, by the bit-stream definition
    (code e of a row occupies bits [e*bits, (e+1)*bits) of the row's
    little-endian bit stream; python/src/ops.cpp:4738-4742).  Pure torch; an
    independent statement used to cross-check the C code paths."""
    words = wq.contiguous().view(torch.int32).to(torch.int64) & 0xFFFFFFFF
    shifts = torch.arange(32, dtype=torch.int64)
    bitsream = (words.unsqueeze(-1) >> shifts) & 1  # [..., W, 32]
    bitsream = bitsream.reshape(*wq.shape[:-1], -1, bits)
    weights = 1 << torch.arange(bits, dtype=torch.int64)
    return (bitsream * weights).sum(-1)
