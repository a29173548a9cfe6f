"""ctypes front end of the CPU parity oracle for the floating-point
quantization modes mxfp4 / mxfp8 / nvfp4 (test infrastructure only).

``FpOracle("port")`` runs ``fp_qref.c`` (in ``libaffine_qref.so``);
``FpOracle("reference")`` sends what the reference's translation unit can
compute through raw pointers -- the quantized matmul and the scalar converters --
to ``_ref/libmlx_cpu_qref.so`` and everything else to the port.  All functions
take and return CPU torch tensors.
"""
from __future__ import annotations

import ctypes

import torch

from oracle.qref import DTYPE_CODE, QREF_SO, REF_SO, _load, _ptr, reference_built  # noqa: F401

MODES = {"mxfp4": 0, "mxfp8": 1, "nvfp4": 2}
GROUP_SIZE = {"mxfp4": 32, "mxfp8": 32, "nvfp4": 16}
BITS = {"mxfp4": 4, "mxfp8": 8, "nvfp4": 4}
FP4_VALUES = (0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0)

_i, _sz, _p = ctypes.c_int, ctypes.c_size_t, ctypes.c_void_p


class FpOracle:
    def __init__(self, kind: str = "port"):
        if kind not in ("port", "reference"):
            raise ValueError(kind)
        self.kind = kind
        self.port = _load(QREF_SO)
        p = self.port
        p.fpq_to_fp8.argtypes, p.fpq_to_fp8.restype = [ctypes.c_float], ctypes.c_uint8
        p.fpq_from_fp8.argtypes, p.fpq_from_fp8.restype = [ctypes.c_uint8], ctypes.c_float
        p.fpq_e8m0.argtypes, p.fpq_e8m0.restype = [ctypes.c_float], ctypes.c_uint8
        p.fpq_e2m1.argtypes, p.fpq_e2m1.restype = [ctypes.c_float], ctypes.c_uint8
        p.fpq_quantize.argtypes, p.fpq_quantize.restype = [_p, _p, _p, _sz, _i, _i], _i
        p.fpq_dequantize.argtypes, p.fpq_dequantize.restype = [_p, _p, _p, _sz, _i, _i], _i
        p.fpq_quantize_dequantize.argtypes = [_p, _p, _sz, _i, _i]
        p.fpq_quantize_dequantize.restype = _i
        p.fpq_qmm.argtypes, p.fpq_qmm.restype = [_p] * 4 + [_i] * 6, _i
        self.ref = None
        if kind == "reference":
            self.ref = _load(REF_SO)
            r = self.ref
            r.ref_to_fp8.argtypes, r.ref_to_fp8.restype = [ctypes.c_float], ctypes.c_uint8
            r.ref_from_fp8.argtypes, r.ref_from_fp8.restype = [ctypes.c_uint8], ctypes.c_float
            r.ref_e8m0.argtypes, r.ref_e8m0.restype = [ctypes.c_float], ctypes.c_uint8
            r.ref_e2m1.argtypes, r.ref_e2m1.restype = [ctypes.c_float], ctypes.c_uint8
            r.ref_fp_qmm.argtypes, r.ref_fp_qmm.restype = [_p] * 4 + [_i] * 6, _i

    def quantize(self, w: torch.Tensor, mode: str):
        """w [..., K] -> (wq uint32 [..., K*bits/32], scales uint8 [..., K/gs])."""
        w = w.contiguous()
        gs, bits = GROUP_SIZE[mode], BITS[mode]
        K = w.shape[-1]
        assert K % gs == 0 and (K * bits) % 32 == 0
        wq = torch.zeros(tuple(w.shape[:-1]) + (K * bits // 32,), dtype=torch.uint32)
        scales = torch.zeros(tuple(w.shape[:-1]) + (K // gs,), dtype=torch.uint8)
        rc = self.port.fpq_quantize(_ptr(w), _ptr(wq), _ptr(scales), w.numel(), MODES[mode],
                                    DTYPE_CODE[w.dtype])
        assert rc == 0
        return wq, scales

    def dequantize(self, wq, scales, mode: str, dtype=torch.float32):
        wq, scales = wq.contiguous(), scales.contiguous()
        K = wq.shape[-1] * 32 // BITS[mode]
        out = torch.empty(tuple(wq.shape[:-1]) + (K,), dtype=dtype)
        rc = self.port.fpq_dequantize(_ptr(wq), _ptr(scales), _ptr(out), out.numel(), MODES[mode],
                                      DTYPE_CODE[dtype])
        assert rc == 0
        return out

    def quantize_dequantize(self, x: torch.Tensor, mode: str):
        x = x.contiguous()
        out = torch.empty_like(x)
        rc = self.port.fpq_quantize_dequantize(_ptr(x), _ptr(out), x.numel(), MODES[mode],
                                               DTYPE_CODE[x.dtype])
        assert rc == 0
        return out

    def qmm(self, x, wq, scales, mode: str, transpose: bool = True):
        """x [M, K]; wq / scales 2-D.  Returns [M, N] in x.dtype."""
        x, wq, scales = x.contiguous(), wq.contiguous(), scales.contiguous()
        M, K = x.shape
        N = wq.shape[0] if transpose else wq.shape[1] * 32 // BITS[mode]
        y = torch.empty((M, N), dtype=x.dtype)
        fn = self.ref.ref_fp_qmm if self.ref is not None else self.port.fpq_qmm
        rc = fn(_ptr(y), _ptr(x), _ptr(wq), _ptr(scales), M, N, K, MODES[mode], int(transpose),
                DTYPE_CODE[x.dtype])
        assert rc == 0
        return y

    def port_qmm(self, x, wq, scales, mode: str, transpose: bool = True):
        saved, self.ref = self.ref, None
        try:
            return self.qmm(x, wq, scales, mode, transpose)
        finally:
            self.ref = saved

    def qqmm(self, x, wq, scales, mode: str):
        """QQMatmul::eval_cpu (mlx/backend/cpu/quantized.cpp:1322-1356): x is
        quantized and dequantized in its own type, then multiplied."""
        return self.qmm(self.quantize_dequantize(x, mode), wq, scales, mode, True)


def exact_fp_weights(wq: torch.Tensor, scales: torch.Tensor, mode: str) -> torch.Tensor:
    """fp64 values of a quantized tensor by the definition of the formats
    (independent of the C code): e2m1 / e4m3 code value times the group's scale
    (2^(s-127) for e8m0, the e4m3 value for nvfp4)."""
    bits, gs = BITS[mode], GROUP_SIZE[mode]
    raw = wq.contiguous().view(torch.uint8).to(torch.int64)
    if bits == 4:
        codes = torch.stack((raw & 0xF, raw >> 4), dim=-1).reshape(*wq.shape[:-1], -1)
        vals = torch.tensor(FP4_VALUES, dtype=torch.float64)[codes]
    else:
        vals = _e4m3_values()[raw.reshape(*wq.shape[:-1], -1)]
    if mode == "nvfp4":
        s = _e4m3_values()[scales.to(torch.int64)]
    else:
        s = torch.pow(torch.tensor(2.0, dtype=torch.float64), scales.to(torch.float64) - 127.0)
    return vals * s.repeat_interleave(gs, dim=-1)


def _e4m3_values() -> torch.Tensor:
    """All 256 e4m3 codes as the reference decodes them (bias 7, subnormals, no
    NaN or infinity codes)."""
    out = []
    for c in range(256):
        e, m = (c >> 3) & 0xF, c & 7
        v = (m / 8.0) * 2.0 ** -6 if e == 0 else (1.0 + m / 8.0) * 2.0 ** (e - 7)
        out.append(-v if c & 0x80 else v)
    return torch.tensor(out, dtype=torch.float64)
