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

import numpy as np
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


# ---- nvfp4 with a tensor-wide scale ------------------------------------------
# The reference computes this on the GPU only (mlx/ops.cpp:4760-4766), so there is
# no CPU function to compile: the functions below restate the CUDA kernels' fp32
# arithmetic (mlx/backend/cuda/quantized/fp_quantize.cuh:73-145 quantize-dequantize,
# :147-215 quantize, :548-592 dequantize; nvfp4_quantize.cuh:13-24 for the codes)
# in numpy, every operation rounded to float32 as the kernels' are.  Parity
# unpinned for exact bits: no run of the reference backs them; they are checked
# against the formats' definitions (nearest code, ties to even), against the C
# port's converters and against the properties the reference's tests assert
# (python/tests/test_quantized.py:183-190, 192-300).

NVFP4_SPAN = np.float32(448.0 * 6.0)
_F32 = np.float32


def e4m3_round(v: np.ndarray) -> np.ndarray:
    """float32 >= 0 -> e4m3 byte: nearest, ties to the even code, saturating at
    448 (cvt.rn.satfinite.e4m3x2.f32; cutlass::float_e4m3_t(float))."""
    table = _e4m3_values()[:127].numpy()  # codes 0 .. 0x7E, ascending
    v64 = v.astype(np.float64)
    hi = np.clip(np.searchsorted(table, v64, side="left"), 1, 126)
    lo = hi - 1
    d_lo, d_hi = v64 - table[lo], table[hi] - v64
    pick_hi = (d_hi < d_lo) | ((d_hi == d_lo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo)
    code = np.where(v64 >= 448.0, 126, code)
    code = np.where(v64 <= 0.0, 0, code)
    return code.astype(np.uint8)


def e2m1_round(v: np.ndarray) -> np.ndarray:
    """float32 -> e2m1 code: nearest, ties to the even code, saturating at 6; a
    NaN gives +6 (cvt.rn.satfinite.e2m1x2.f32)."""
    table = np.array(FP4_VALUES[:8], dtype=np.float64)
    a = np.abs(v.astype(np.float64))
    nan = np.isnan(a)
    a = np.where(nan, 0.0, a)
    hi = np.clip(np.searchsorted(table, a, side="left"), 1, 7)
    lo = hi - 1
    d_lo, d_hi = a - table[lo], table[hi] - a
    pick_hi = (d_hi < d_lo) | ((d_hi == d_lo) & (hi % 2 == 0))
    code = np.where(pick_hi, hi, lo)
    code = np.where(a >= 6.0, 7, code)
    code = code | np.where(np.signbit(v), 8, 0)
    return np.where(nan, 7, code).astype(np.uint8)


def _nvfp4_global_codes(w: torch.Tensor, global_scale: float):
    """(codes [..., K] uint8, scale bytes [..., K/16], scale values float32,
    scale_enc float32) by fp_quantize.cuh:147-215."""
    x = w.detach().float().numpy().astype(_F32)
    scale_enc = _F32(NVFP4_SPAN / _F32(global_scale))
    groups = x.reshape(*x.shape[:-1], -1, 16)
    amax = np.abs(groups).max(axis=-1).astype(_F32)
    scale_dec_b = (amax / _F32(6.0)).astype(_F32)
    scale_dec_b = (scale_dec_b * scale_enc).astype(_F32)
    sbytes = e4m3_round(scale_dec_b)
    svals = _e4m3_values().numpy()[sbytes].astype(_F32)
    with np.errstate(divide="ignore", invalid="ignore"):
        scale_enc_b = (scale_enc / svals).astype(_F32)
        scaled = (groups * scale_enc_b[..., None]).astype(_F32)
    codes = e2m1_round(scaled).reshape(x.shape)
    return codes, sbytes, svals, scale_enc


def nvfp4_global_quantize(w: torch.Tensor, global_scale: float):
    """-> (wq uint32 [..., K/8], scales uint8 [..., K/16])."""
    codes, sbytes, _, _ = _nvfp4_global_codes(w, global_scale)
    pairs = codes.reshape(*codes.shape[:-1], -1, 2).astype(np.uint8)
    packed = (pairs[..., 0] | (pairs[..., 1] << 4)).astype(np.uint8)
    wq = torch.from_numpy(np.ascontiguousarray(packed)).view(torch.uint32)
    return wq, torch.from_numpy(np.ascontiguousarray(sbytes))


def nvfp4_global_dequantize(wq, scales, global_scale: float, dtype=torch.float32):
    """fp_quantize.cuh:548-592: T(code value * (scale value * (global / 2688)))."""
    raw = wq.contiguous().view(torch.uint8).numpy()
    codes = np.stack((raw & 0xF, raw >> 4), axis=-1).reshape(*wq.shape[:-1], -1)
    vals = np.array(FP4_VALUES, dtype=_F32)[codes]
    inv_scale_enc = _F32(_F32(global_scale) / NVFP4_SPAN)
    s = (_e4m3_values().numpy()[scales.numpy()].astype(_F32) * inv_scale_enc).astype(_F32)
    out = (np.repeat(s, 16, axis=-1) * vals).astype(_F32)
    return torch.from_numpy(out).to(dtype)


def nvfp4_global_quantize_dequantize(x: torch.Tensor, global_scale: float):
    """fp_quantize.cuh:73-145, in x's type."""
    codes, _, svals, scale_enc = _nvfp4_global_codes(x, global_scale)
    inv_scale_enc = _F32(_F32(1.0) / scale_enc)
    scale_dec = (svals * inv_scale_enc).astype(_F32)
    vals = np.array(FP4_VALUES, dtype=_F32)[codes]
    out = (vals * np.repeat(scale_dec, 16, axis=-1)).astype(_F32)
    return torch.from_numpy(out).to(x.dtype)


def nvfp4_global_qqmm_f64(x, wq, scales, global_scale_x: float, global_scale_w: float):
    """What qqmm with both tensor-wide scales approximates, in float64: x_hat (in
    x's type) times the block-scaled codes, times global_scale_w / 2688
    (mlx/backend/cuda/quantized/qqmm.cpp:139-170, qmm/qmv.cu:163-165).  Also
    returns sum |x_hat w| for error bounds."""
    x_hat = nvfp4_global_quantize_dequantize(x, global_scale_x).double()
    w = exact_fp_weights(wq, scales, "nvfp4")
    factor = float(_F32(_F32(global_scale_w) / NVFP4_SPAN))
    return (x_hat @ w.T) * factor, (x_hat.abs() @ w.abs().T) * factor
