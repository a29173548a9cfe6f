"""Element copies with dtype conversion (mlxrocm_copy_contiguous /
mlxrocm_copy_strided), bit for bit against numpy / torch-on-CPU conversions of
the same values.

The reference tests the same movement through `astype`, `contiguous`, slicing
and broadcasting in python/tests/test_ops.py and tests/ops_tests.cpp; here the
kernels are driven directly through the C ABI and through `mlx_amd._copy`.
Values are chosen inside every target type's range (C++ leaves out-of-range
float -> integer conversions undefined), and 64-bit sources are exactly
representable in fp32 so that one- and two-step roundings agree.
"""
import ctypes

import numpy as np
import pytest
import torch

from mlx_amd import _copy, _lib

pytestmark = pytest.mark.gpu

DEV = "cuda:0"

NP = {
    torch.float32: np.float32, torch.float16: np.float16, torch.bool: np.bool_,
    torch.uint8: np.uint8, torch.uint16: np.uint16, torch.uint32: np.uint32,
    torch.uint64: np.uint64, torch.int8: np.int8, torch.int16: np.int16,
    torch.int32: np.int32, torch.int64: np.int64, torch.float64: np.float64,
    torch.complex64: np.complex64,
}
ALL = list(_copy.DTYPE_CODE)


def _source(dtype, n, seed):
    """n values of `dtype` (a CPU torch tensor), small enough for every target."""
    rng = np.random.default_rng(seed)
    if dtype == torch.bool:
        return torch.from_numpy(rng.integers(0, 2, n).astype(np.bool_))
    if dtype == torch.complex64:
        re = rng.integers(0, 100, n).astype(np.float32) + rng.integers(0, 4, n).astype(np.float32) / 4
        im = rng.integers(-3, 4, n).astype(np.float32)
        re[::7] = 0
        return torch.from_numpy((re + 1j * im).astype(np.complex64))
    if dtype.is_floating_point:
        # non-negative, below 127, with fractions that fp16/bf16 must round
        v = rng.uniform(0, 126, n).astype(np.float32)
        v[::5] = 0
        v[1::11] = np.floor(v[1::11])
        t = torch.from_numpy(v)
        return t.to(dtype)
    v = rng.integers(0, 127, n)
    v[::5] = 0
    return torch.from_numpy(v.astype(NP[dtype]))


def _to_f32(t):
    if t.dtype == torch.complex64:
        return t.real.contiguous()
    return t.to(torch.float32)


def _expected(src, dst_dtype):
    """Conversion of CPU tensor `src` to `dst_dtype` by numpy (bf16 through torch)."""
    if src.dtype == dst_dtype:
        return src.clone()
    if dst_dtype == torch.bool:
        if src.dtype == torch.complex64:
            return (src.real != 0) | (src.imag != 0)
        return _to_f32(src) != 0 if src.dtype.is_floating_point else torch.from_numpy(
            src.numpy() != 0)
    if torch.bfloat16 in (src.dtype, dst_dtype) or torch.float16 in (src.dtype, dst_dtype):
        mid = _to_f32(src) if src.dtype != torch.float64 else torch.from_numpy(
            src.numpy().astype(np.float32))
        if not src.dtype.is_floating_point and src.dtype not in (torch.bool, torch.complex64):
            mid = torch.from_numpy(src.numpy().astype(np.float32))
        if dst_dtype in (torch.bfloat16, torch.float16):
            return mid.to(dst_dtype)
        return _expected(mid, dst_dtype)
    a = src.numpy()
    if src.dtype == torch.complex64 and dst_dtype != torch.complex64:
        a = a.real
    return torch.from_numpy(np.ascontiguousarray(a).astype(NP[dst_dtype]))


def _bytes(t):
    return t.contiguous().cpu().view(torch.uint8).numpy().tobytes()


@pytest.mark.parametrize("src_dtype", ALL, ids=lambda d: str(d).split(".")[-1])
def test_contiguous_conversion_to_every_type(src_dtype):
    n = 5000 + 3  # a ragged tail after the 16-byte vectors
    src = _source(src_dtype, n, seed=ALL.index(src_dtype))
    dev = src.to(DEV)
    for dst_dtype in ALL:
        got = _copy.copy(dev, dst_dtype)
        assert got.dtype == dst_dtype and got.shape == dev.shape
        want = _expected(src, dst_dtype)
        assert _bytes(got) == _bytes(want), f"{src_dtype} -> {dst_dtype}"


@pytest.mark.parametrize("pair", [(torch.bfloat16, torch.float32), (torch.float32, torch.float16),
                                  (torch.uint8, torch.int64), (torch.float32, torch.float32)])
def test_unaligned_views_take_the_elementwise_path(pair):
    s, d = pair
    src = _source(s, 4099, seed=3)
    dev = src.to(DEV)
    lib = _lib.load()
    out = torch.zeros(4099, dtype=d, device=DEV)
    # both ends start one element past an aligned address
    _lib.check(lib.mlxrocm_copy_contiguous(
        dev[1:].data_ptr(), _copy.DTYPE_CODE[s], out[1:].data_ptr(), _copy.DTYPE_CODE[d],
        4098, 0, torch.cuda.current_stream().cuda_stream))
    want = torch.zeros(4099, dtype=d)
    want[1:] = _expected(src[1:], d)
    assert _bytes(out) == _bytes(want)


def _views(t):
    yield "transpose", t.transpose(0, 2)
    yield "permute", t.permute(2, 0, 3, 1)
    yield "step", t[::2, 1:, ::3, :5]
    yield "expand", t[:, :1, :, :1].expand(-1, 4, -1, 6)
    yield "inner_slice", t[..., 2:7]
    yield "row", t[1, 2]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.uint32, torch.int64,
                                   torch.uint8, torch.complex64],
                         ids=lambda d: str(d).split(".")[-1])
def test_strided_sources_gather_into_rows(dtype):
    src = _source(dtype, 6 * 5 * 9 * 8, seed=11).reshape(6, 5, 9, 8)
    dev = src.to(DEV)
    for (name, v_dev), (_, v_cpu) in zip(_views(dev), _views(src)):
        got = _copy.contiguous(v_dev)
        assert got.is_contiguous()
        assert _bytes(got) == _bytes(v_cpu.contiguous()), name
        if dtype != torch.complex64:
            got = _copy.copy(v_dev, torch.float32)
            assert _bytes(got) == _bytes(_expected(v_cpu.contiguous(), torch.float32)), name


def _strided(src, sst, dst, dstr, shape, sdt=None, ddt=None):
    lib = _lib.load()
    arr = lambda v: (ctypes.c_int64 * max(1, len(v)))(*v)
    return lib.mlxrocm_copy_strided(
        src.data_ptr(), _copy.DTYPE_CODE[sdt or src.dtype], arr(sst),
        dst.data_ptr(), _copy.DTYPE_CODE[ddt or dst.dtype],
        None if dstr is None else arr(dstr), len(shape), arr(shape),
        torch.cuda.current_stream().cuda_stream)


def test_negative_and_destination_strides():
    src = torch.arange(7 * 12, dtype=torch.int32).reshape(7, 12)
    dev = src.to(DEV)
    # reversed rows: start at the last row, walk backwards
    out = torch.empty_like(dev)
    _lib.check(_strided(dev[6], (-12, 1), out, None, (7, 12), torch.int32, torch.int32))
    assert torch.equal(out.cpu(), src.flip(0))
    # scatter into a transposed destination (general -> general)
    out = torch.full((12, 7), -1, dtype=torch.int64, device=DEV)
    _lib.check(_strided(dev, (12, 1), out, (1, 7), (7, 12)))
    assert torch.equal(out.cpu(), src.t().to(torch.int64))
    # destination with gaps keeps what lies between the written elements
    out = torch.full((7, 24), -1, dtype=torch.int32, device=DEV)
    _lib.check(_strided(dev, (12, 1), out, (24, 2), (7, 12)))
    want = torch.full((7, 24), -1, dtype=torch.int32)
    want[:, ::2] = src
    assert torch.equal(out.cpu(), want)


def test_many_dimensions_merge_or_are_refused():
    src = torch.arange(2 ** 10, dtype=torch.int32)
    dev = src.to(DEV)
    out = torch.empty_like(dev)
    # ten extent-2 dimensions of a dense array merge into one run
    shape = (2,) * 10
    strides = tuple(2 ** (9 - d) for d in range(10))
    _lib.check(_strided(dev, strides, out, None, shape))
    assert torch.equal(out.cpu(), src)
    # reversed order of ten dimensions cannot merge: refused, not truncated
    rc = _strided(dev, strides[::-1], out, None, shape)
    assert rc == _lib.UNSUPPORTED and "dimensions" in _lib.last_error()
    # eight is the limit and works
    src8 = src[:256].reshape((2,) * 8)
    perm = src8.permute(*range(7, -1, -1))
    got = _copy.contiguous(src8.to(DEV).permute(*range(7, -1, -1)))
    assert torch.equal(got.cpu(), perm.contiguous())


@pytest.mark.parametrize("dtype", [torch.uint8, torch.bfloat16, torch.float32, torch.int64],
                         ids=lambda d: str(d).split(".")[-1])
def test_row_slices_take_the_widened_path_and_its_fallbacks(dtype):
    """Same-type copies whose rows are contiguous move 16, 8 or 4 bytes per lane
    when extents, strides and addresses allow, and single elements otherwise: every
    alignment of the column window must give the same bytes."""
    src = _source(dtype, 64 * 96, seed=21).reshape(64, 96)
    dev = src.to(DEV)
    for lo, hi in ((0, 64), (16, 80), (8, 72), (4, 36), (2, 50), (1, 33), (3, 96)):
        got = _copy.contiguous(dev[:, lo:hi])
        assert _bytes(got) == _bytes(src[:, lo:hi].contiguous()), (lo, hi)
        got = _copy.contiguous(dev[5:61:3, lo:hi])
        assert _bytes(got) == _bytes(src[5:61:3, lo:hi].contiguous()), (lo, hi)


@pytest.mark.parametrize("dtype", [torch.uint8, torch.bfloat16, torch.float32, torch.complex64],
                         ids=lambda d: str(d).split(".")[-1])
def test_transposed_sources_take_the_tiled_path(dtype):
    """A same-type copy whose source runs along another dimension than the last
    goes through 32 x 32 LDS tiles: ragged extents, batch dimensions on either
    side of the transposed pair, a batch dimension with its own stride."""
    base = _source(dtype, 7 * 45 * 70, seed=31).reshape(7, 45, 70)
    dev = base.to(DEV)
    views = {
        "2d": lambda t: t[0].t(),                       # [70, 45]
        "batched": lambda t: t.transpose(1, 2),         # [7, 70, 45]
        "batch_inside": lambda t: t.permute(2, 0, 1),   # [70, 7, 45]: last = dim 1, unit stride = dim 2
        "outer_to_last": lambda t: t.permute(1, 2, 0),  # [45, 70, 7]: too short a last dim -> generic
        "sliced": lambda t: t[1:6, 3:40, 5:69].transpose(1, 2),
        "stepped_batch": lambda t: t[::2].transpose(1, 2),
    }
    for name, view in views.items():
        got = _copy.contiguous(view(dev))
        assert _bytes(got) == _bytes(view(base).contiguous()), name
    # into a destination with its own row stride (general -> general)
    lib = _lib.load()
    arr = lambda v: (ctypes.c_int64 * len(v))(*v)
    src2 = dev[0]                                           # [45, 70]
    out = torch.zeros((70, 64), dtype=dtype, device=DEV)
    code = _copy.DTYPE_CODE[dtype]
    _lib.check(lib.mlxrocm_copy_strided(
        src2.data_ptr(), code, arr((1, 70)), out.data_ptr(), code, arr((64, 1)),
        2, arr((70, 45)), torch.cuda.current_stream().cuda_stream))
    want = torch.zeros((70, 64), dtype=dtype)
    want[:, :45] = base[0].t()
    assert _bytes(out) == _bytes(want)


def test_fill_broadcasts_one_device_scalar():
    like = torch.empty((33, 77), dtype=torch.bfloat16, device=DEV)
    value = torch.tensor([1.2345], dtype=torch.float32, device=DEV)
    got = _copy.full_like(like, value)
    assert torch.equal(got.cpu(), torch.full((33, 77), 1.2345, dtype=torch.float32).to(torch.bfloat16))
    like = torch.empty(1001, dtype=torch.int64, device=DEV)
    got = _copy.full_like(like, torch.tensor([7], dtype=torch.uint8, device=DEV))
    assert torch.equal(got.cpu(), torch.full((1001,), 7, dtype=torch.int64))


def test_large_copy_moves_every_element():
    n = (1 << 27) + 5  # 256 MiB of bf16 -> 512 MiB of fp32
    g = torch.Generator(device=DEV).manual_seed(5)
    src = torch.randn(n, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    got = _copy.copy(src, torch.float32)
    assert torch.equal(got, src.float())
    back = _copy.copy(got, torch.bfloat16)
    assert torch.equal(back.view(torch.int16), src.view(torch.int16))


def test_bad_arguments():
    lib = _lib.load()
    t = torch.zeros(8, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    assert lib.mlxrocm_copy_contiguous(t.data_ptr(), 99, t.data_ptr(), 0, 8, 0, s) == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_copy_contiguous(None, 0, t.data_ptr(), 0, 8, 0, s) == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_copy_contiguous(None, 0, None, 0, 0, 0, s) == _lib.OK  # empty is fine
    assert _strided(t, (1,), t, None, (-1,)) == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_dtype_size(2) == 2 and lib.mlxrocm_dtype_size(13) == 8
    assert lib.mlxrocm_dtype_size(14) == 0
    with pytest.raises(RuntimeError):
        _copy.copy(torch.zeros(3))  # a CPU tensor
