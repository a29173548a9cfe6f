"""The C ABI library loads, exports every symbol the header declares, and its
argument checks (which run before any HIP call) behave -- no GPU needed."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from mlx_amd import _build, _lib

    if not os.path.isfile(_lib.LIB_PATH):
        _build.build()
    return _lib.load()


def declared_functions():
    text = open(os.path.join(ROOT, "include", "mlx_rocm_qmm.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mlxrocm_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(lib):
    from mlx_amd import _lib

    names = declared_functions()
    assert len(names) >= 30
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in the header but not exported"
    assert sorted(_lib.SIGNATURES) == names, "ctypes table and header disagree"


def test_abi_version(lib):
    assert lib.mlxrocm_abi_version() == 4


def test_invalid_arguments_are_reported_not_thrown(lib):
    from mlx_amd import _lib

    one = ctypes.c_void_p(16)  # never dereferenced: the checks come first
    rc = lib.mlxrocm_affine_quantize(one, one, one, one, 64, 64, 7, 0, None)
    assert rc == _lib.INVALID_ARGUMENT and b"bits" in lib.mlxrocm_last_error()
    rc = lib.mlxrocm_affine_quantize(one, one, one, one, 64, 48, 4, 0, None)
    assert rc == _lib.INVALID_ARGUMENT and b"group size" in lib.mlxrocm_last_error()
    rc = lib.mlxrocm_affine_quantize(one, one, one, one, 100, 64, 4, 0, None)
    assert rc == _lib.INVALID_ARGUMENT
    rc = lib.mlxrocm_affine_dequantize(one, one, one, one, 64, 64, 4, 9, None)
    assert rc == _lib.INVALID_ARGUMENT and b"dtype" in lib.mlxrocm_last_error()
    # quantized axis not a multiple of the group size
    rc = lib.mlxrocm_qmm(one, one, one, one, one, 1, 32, 96, 1, 96, 0, 0, 64, 4, 0, 1, None, 0, None)
    assert rc == _lib.INVALID_ARGUMENT
    rc = lib.mlxrocm_qmm(None, one, one, one, one, 1, 32, 128, 1, 128, 0, 0, 64, 4, 0, 1, None, 0, None)
    assert rc == _lib.INVALID_ARGUMENT and b"null" in lib.mlxrocm_last_error()
    with pytest.raises(ValueError):
        _lib.check(rc)
    # empty problems succeed without touching the device
    assert lib.mlxrocm_affine_quantize(None, None, None, None, 0, 64, 4, 0, None) == 0
    assert lib.mlxrocm_qmm(None, None, None, None, None, 0, 32, 128, 1, 0, 0, 0, 64, 4, 0, 1, None, 0, None) == 0


def test_kernel_choice(lib):
    name = lambda *a: lib.mlxrocm_qmm_kernel_name(*a)  # noqa: E731
    assert name(1, 14336, 4096, 1, 64, 4, 2, 1) == b"qmv"
    assert name(8, 4096, 14336, 1, 128, 8, 2, 1) == b"qmv"
    assert name(2048, 14336, 4096, 1, 64, 4, 2, 1) == b"qmm_t"
    assert name(2048, 14336, 4096, 1, 64, 4, 0, 1) == b"qmm_t"        # float32: split bf16
    assert name(2048, 14336, 4000, 1, 32, 4, 0, 1) == b"qmm_generic"  # K not a multiple of 64
    assert name(64, 512, 256, 1, 64, 4, 2, 0) == b"qmm_n"             # transpose=False, 4/8-bit
    assert name(64, 512, 256, 1, 64, 3, 2, 0) == b"qmm_n"             # ... odd width: repacked at 4 bits
    assert name(64, 512, 256, 1, 64, 3, 0, 0) == b"qmm_generic"       # ... odd width, float32, many rows
    assert name(64, 512, 256, 1, 64, 4, 0, 0) == b"qmm_generic"       # transpose=False, float32
    assert name(64, 512, 250, 1, 64, 4, 2, 1) is None


def test_memory_counters_without_device(lib):
    assert lib.mlxrocm_get_active_memory() == 0
    assert lib.mlxrocm_malloc(None, 16) != 0
    p = ctypes.c_void_p()
    assert lib.mlxrocm_malloc(ctypes.byref(p), 0) == 0 and not p.value
    assert lib.mlxrocm_free(None) == 0
