"""ctypes binding of ``libmlx_rocm_qmm.so`` (the C ABI in
``include/mlx_rocm_qmm.h``).  There is no CPU fallback: if the library is not
built, importing an operator raises."""
from __future__ import annotations

import ctypes
import os

HERE = os.path.dirname(os.path.abspath(__file__))
# MLX_ROCM_QMM_LIBRARY names another build of the library (e.g. one under test).
LIB_PATH = os.environ.get("MLX_ROCM_QMM_LIBRARY") or os.path.join(HERE, "lib", "libmlx_rocm_qmm.so")

OK = 0
INVALID_ARGUMENT = -1
UNSUPPORTED = -2
HIP_ERROR = -3
OUT_OF_MEMORY = -4

FLOAT32, FLOAT16, BFLOAT16 = 0, 1, 2
MXFP4, MXFP8, NVFP4 = 0, 1, 2  # mlxrocm_fp_mode

_i = ctypes.c_int
_i64 = ctypes.c_int64
_sz = ctypes.c_size_t
_p = ctypes.c_void_p

# name -> (restype, argtypes); the list the symbol-export test walks.
SIGNATURES = {
    "mlxrocm_abi_version": (_i, []),
    "mlxrocm_last_error": (ctypes.c_char_p, []),
    "mlxrocm_affine_quantize": (_i, [_p, _p, _p, _p, _sz, _i, _i, _i, _p]),
    "mlxrocm_affine_dequantize": (_i, [_p, _p, _p, _p, _sz, _i, _i, _i, _p]),
    "mlxrocm_gguf_repack": (_i, [_p, _p, _p, _p, _sz, _i, _p]),
    "mlxrocm_qmm_workspace_size": (_sz, [_i] * 9),
    "mlxrocm_qmm": (
        _i,
        [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i64, _i64, _i64, _i, _i, _i, _i, _p, _sz, _p],
    ),
    "mlxrocm_qmm_sb_image_size": (_sz, [_i] * 5),
    "mlxrocm_qmm_sb_image": (_i, [_p, _p, _p, _i, _i, _i, _i64, _i, _i, _p]),
    "mlxrocm_qmm_prepacked": (
        _i,
        [_p, _p, _p, _p, _p, _p, _i, _i, _i, _i, _i64, _i64, _i64, _i, _i, _i, _i, _p, _sz, _p],
    ),
    "mlxrocm_qmm_static": (
        _i,
        [_p, _p, _p, _p, _p, _i, _i, _i, _i, _i64, _i64, _i64, _i, _i, _i, _i, _p],
    ),
    "mlxrocm_qmm_swiglu_workspace_size": (_sz, [_i, _i, _i]),
    "mlxrocm_qmm_swiglu": (_i, [_p] * 9 + [_i] * 6 + [_p]),
    "mlxrocm_gather_qmm": (
        _i,
        [_p] * 7 + [_i] * 6 + [_i64] * 3 + [_i] * 5 + [_p, _sz, _p],
    ),
    "mlxrocm_gather_qmm_workspace_size": (_sz, [_i] * 10),
    "mlxrocm_fp_quantize": (_i, [_p, _p, _p, _sz, _i, _i, _p]),
    "mlxrocm_fp_dequantize": (_i, [_p, _p, _p, _sz, _i, _i, _p]),
    "mlxrocm_fp_quantize_dequantize": (_i, [_p, _p, _sz, _i, _i, _p]),
    "mlxrocm_fp_qmm_workspace_size": (_sz, [_i] * 8),
    "mlxrocm_fp_qmm": (_i, [_p] * 4 + [_i] * 4 + [_i64] * 3 + [_i] * 3 + [_p, _sz, _p]),
    "mlxrocm_fp_qqmm_workspace_size": (_sz, [_i] * 5),
    "mlxrocm_fp_qqmm": (_i, [_p] * 4 + [_i] * 5 + [_p, _sz, _p]),
    "mlxrocm_fp_qmm_plan": (_i, [_i] * 8 + [_sz, ctypes.c_char_p, _sz]),
    "mlxrocm_fp_qqmm_plan": (_i, [_i] * 5 + [_sz, ctypes.c_char_p, _sz]),
    "mlxrocm_fp_gather_qmm_workspace_size": (_sz, [_i] * 9),
    "mlxrocm_fp_gather_qmm": (_i, [_p] * 6 + [_i] * 6 + [_i64] * 3 + [_i] * 3 + [_p, _sz, _p]),
    "mlxrocm_fp_gather_qqmm_workspace_size": (_sz, [_i] * 9),
    "mlxrocm_fp_gather_qqmm": (_i, [_p] * 8 + [_i] * 6 + [_i64] * 3 + [_i] * 2 + [_p, _sz, _p]),
    "mlxrocm_nvfp4_quantize_global": (_i, [_p] * 4 + [_sz, _i, _p]),
    "mlxrocm_nvfp4_dequantize_global": (_i, [_p] * 4 + [_sz, _i, _p]),
    "mlxrocm_nvfp4_quantize_dequantize_global": (_i, [_p] * 3 + [_sz, _i, _p]),
    "mlxrocm_nvfp4_qqmm_global": (_i, [_p] * 6 + [_i] * 4 + [_p, _sz, _p]),
    "mlxrocm_to_fp8": (_i, [_p, _p, _sz, _i, _p]),
    "mlxrocm_from_fp8": (_i, [_p, _p, _sz, _i, _p]),
    "mlxrocm_qmm_kernel_name": (ctypes.c_char_p, [_i] * 8),
    "mlxrocm_qmm_plan": (_i, [_i] * 9 + [_sz, ctypes.c_char_p, _sz]),
    "mlxrocm_gather_qmm_plan": (_i, [_i] * 10 + [_sz, ctypes.c_char_p, _sz]),
    "mlxrocm_qmm_rule_count": (_i, []),
    "mlxrocm_qmm_rule_name": (ctypes.c_char_p, [_i]),
    "mlxrocm_qmm_rule_evidence": (ctypes.c_char_p, [_i]),
    "mlxrocm_malloc": (_i, [ctypes.POINTER(_p), _sz]),
    "mlxrocm_free": (_i, [_p]),
    "mlxrocm_buffer_size": (_sz, [_p]),
    "mlxrocm_get_active_memory": (_sz, []),
    "mlxrocm_get_peak_memory": (_sz, []),
    "mlxrocm_reset_peak_memory": (None, []),
    "mlxrocm_get_cache_memory": (_sz, []),
    "mlxrocm_set_cache_limit": (_sz, [_sz]),
    "mlxrocm_set_memory_limit": (_sz, [_sz]),
    "mlxrocm_get_memory_limit": (_sz, []),
    "mlxrocm_clear_cache": (None, []),
    "mlxrocm_host_malloc": (_i, [ctypes.POINTER(_p), _sz]),
    "mlxrocm_host_free": (_i, [_p]),
    "mlxrocm_memcpy_h2d": (_i, [_p, _p, _sz, _p]),
    "mlxrocm_memcpy_d2h": (_i, [_p, _p, _sz, _p]),
    "mlxrocm_memcpy_d2d": (_i, [_p, _p, _sz, _p]),
    "mlxrocm_stream_create": (_i, [ctypes.POINTER(_p)]),
    "mlxrocm_stream_destroy": (_i, [_p]),
    "mlxrocm_stream_synchronize": (_i, [_p]),
    "mlxrocm_event_create": (_i, [ctypes.POINTER(_p)]),
    "mlxrocm_event_create_blocking": (_i, [ctypes.POINTER(_p)]),
    "mlxrocm_event_destroy": (_i, [_p]),
    "mlxrocm_dtype_size": (ctypes.c_size_t, [_i]),
    "mlxrocm_copy_contiguous": (_i, [_p, _i, _p, _i, ctypes.c_size_t, _i, _p]),
    "mlxrocm_copy_strided": (_i, [_p, _i, ctypes.POINTER(ctypes.c_int64), _p, _i,
                                  ctypes.POINTER(ctypes.c_int64), _i,
                                  ctypes.POINTER(ctypes.c_int64), _p]),
    "mlxrocm_event_record": (_i, [_p, _p]),
    "mlxrocm_event_wait": (_i, [_p, _p]),
    "mlxrocm_event_synchronize": (_i, [_p]),
    "mlxrocm_event_query": (_i, [_p]),
    "mlxrocm_event_elapsed_ms": (_i, [ctypes.POINTER(ctypes.c_float), _p, _p]),
    "mlxrocm_device_count": (_i, []),
    "mlxrocm_device_info": (
        _i,
        [_i, ctypes.c_char_p, ctypes.POINTER(_i), ctypes.POINTER(_sz), ctypes.POINTER(_i)],
    ),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the HIP library; raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.isfile(LIB_PATH):
        raise ImportError(
            f"{LIB_PATH} not found: build it with `python -m mlx_amd._build` "
            "(hipcc, gfx950).  mlx_amd has no CPU fallback."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    if lib.mlxrocm_abi_version() != 4:
        raise ImportError("libmlx_rocm_qmm.so ABI version mismatch")
    _lib = lib
    return lib


def qmm_plan(M, N, K, L=1, batched_weights=False, group_size=64, bits=4, dtype=BFLOAT16,
             transpose=True, workspace_bytes=None):
    """(status, record) of a rehearsed mlxrocm_qmm call: the dispatch rules it
    takes and the kernels it would launch, e.g.
    "[qmm_t_tile_sb_transposed]+transpose_sb+qmm_t_tile(nt=7)".  Runs without a
    GPU.  workspace_bytes=None rehearses with exactly mlxrocm_qmm_workspace_size."""
    lib = load()
    args = (M, N, K, L, int(batched_weights), group_size, bits, dtype, int(transpose))
    if workspace_bytes is None:
        workspace_bytes = lib.mlxrocm_qmm_workspace_size(*args)
    buf = ctypes.create_string_buffer(1024)
    rc = lib.mlxrocm_qmm_plan(*args, workspace_bytes, buf, len(buf))
    return rc, buf.value.decode()


def gather_qmm_plan(M, N, K, n_indices, x_batches, n_experts, group_size=64, bits=4,
                    dtype=BFLOAT16, transpose=True, workspace_bytes=None):
    """The same for mlxrocm_gather_qmm."""
    lib = load()
    if workspace_bytes is None:
        workspace_bytes = lib.mlxrocm_gather_qmm_workspace_size(
            M, N, K, n_indices, n_experts, group_size, bits, dtype, int(transpose), 0)
    buf = ctypes.create_string_buffer(1024)
    rc = lib.mlxrocm_gather_qmm_plan(M, N, K, n_indices, x_batches, n_experts, group_size, bits,
                                     dtype, int(transpose), workspace_bytes, buf, len(buf))
    return rc, buf.value.decode()


def fp_qmm_plan(M, N, K, L=1, batched_weights=False, mode=MXFP4, dtype=BFLOAT16, transpose=True,
                workspace_bytes=None):
    """(status, plan) of mlxrocm_fp_qmm for these arguments; the workspace
    defaults to what mlxrocm_fp_qmm_workspace_size asks for."""
    lib = load()
    if workspace_bytes is None:
        workspace_bytes = lib.mlxrocm_fp_qmm_workspace_size(
            M, N, K, L, int(batched_weights), mode, dtype, int(transpose))
    buf = ctypes.create_string_buffer(512)
    rc = lib.mlxrocm_fp_qmm_plan(M, N, K, L, int(batched_weights), mode, dtype, int(transpose),
                                 workspace_bytes, buf, len(buf))
    return rc, buf.value.decode()


def fp_qqmm_plan(M, N, K, mode=MXFP4, dtype=BFLOAT16, workspace_bytes=None):
    lib = load()
    if workspace_bytes is None:
        workspace_bytes = lib.mlxrocm_fp_qqmm_workspace_size(M, N, K, mode, dtype)
    buf = ctypes.create_string_buffer(512)
    rc = lib.mlxrocm_fp_qqmm_plan(M, N, K, mode, dtype, workspace_bytes, buf, len(buf))
    return rc, buf.value.decode()


def dispatch_rules():
    """[(name, evidence)] of the dispatch table of mlxrocm_qmm, in match order."""
    lib = load()
    return [(lib.mlxrocm_qmm_rule_name(i).decode(), lib.mlxrocm_qmm_rule_evidence(i).decode())
            for i in range(lib.mlxrocm_qmm_rule_count())]


def last_error() -> str:
    return load().mlxrocm_last_error().decode("utf-8", "replace")


def check(status: int) -> None:
    """Turn a status into the exception MLX's C++ glue would throw:
    std::invalid_argument -> ValueError, runtime_error -> RuntimeError."""
    if status == OK:
        return
    msg = last_error()
    if status == INVALID_ARGUMENT:
        raise ValueError(msg)
    if status == OUT_OF_MEMORY:
        raise MemoryError(msg)
    raise RuntimeError(msg)
