"""GPU tests of the runtime part of the C ABI: the device allocator with its
cache, limits and counters (the contract of mlx/allocator.h:52-75 and
mlx/memory.h; model mlx/backend/cuda/allocator.cpp:165-250), pinned host
memory and explicit copies, and the stream / event calls behind
mlx::core::Stream and mlx::core::Event (mlx/backend/cuda/event.cu:330-420)."""
import ctypes

import pytest
import torch

from mlx_amd import _lib

pytestmark = pytest.mark.gpu

PAGE = 16384


@pytest.fixture()
def lib(gpu):
    lib = _lib.load()
    lib.mlxrocm_clear_cache()
    prev = lib.mlxrocm_set_cache_limit(ctypes.c_size_t(-1).value)
    yield lib
    lib.mlxrocm_clear_cache()
    lib.mlxrocm_set_cache_limit(prev)


def _malloc(lib, size):
    p = ctypes.c_void_p()
    rc = lib.mlxrocm_malloc(ctypes.byref(p), size)
    return rc, p.value


def test_size_classes_and_counters(lib):
    base = lib.mlxrocm_get_active_memory()
    lib.mlxrocm_reset_peak_memory()
    sizes = {1: 8, 8: 8, 9: 16, 100: 128, 5000: 8192, PAGE - 1: PAGE, PAGE: PAGE,
             PAGE + 1: 2 * PAGE, 1 << 20: 1 << 20}
    live = []
    total = 0
    for want, cls in sizes.items():
        rc, p = _malloc(lib, want)
        assert rc == 0 and p
        assert lib.mlxrocm_buffer_size(p) == cls
        total += cls
        live.append(p)
        assert lib.mlxrocm_get_active_memory() == base + total
    assert lib.mlxrocm_get_peak_memory() >= base + total
    for p in live:
        assert lib.mlxrocm_free(p) == 0
    assert lib.mlxrocm_get_active_memory() == base
    assert lib.mlxrocm_get_cache_memory() == total
    assert lib.mlxrocm_get_peak_memory() >= base + total  # the peak stays
    lib.mlxrocm_reset_peak_memory()
    assert lib.mlxrocm_get_peak_memory() <= base
    # an empty request is an empty buffer, an unknown pointer an error
    rc, p = _malloc(lib, 0)
    assert rc == 0 and p is None
    assert lib.mlxrocm_free(None) == 0
    assert lib.mlxrocm_free(ctypes.c_void_p(0x1000)) == _lib.INVALID_ARGUMENT
    assert "not a live buffer" in _lib.last_error()
    assert lib.mlxrocm_buffer_size(ctypes.c_void_p(0x1000)) == 0


def test_cache_reuse_and_trim(lib):
    rc, a = _malloc(lib, 3 * PAGE)
    assert rc == 0
    assert lib.mlxrocm_free(a) == 0
    assert lib.mlxrocm_get_cache_memory() == 3 * PAGE
    # a request of at least half the cached size takes the cached buffer ...
    rc, b = _malloc(lib, 2 * PAGE)
    assert rc == 0 and b == a and lib.mlxrocm_buffer_size(b) == 3 * PAGE
    assert lib.mlxrocm_get_cache_memory() == 0
    assert lib.mlxrocm_free(b) == 0
    # ... a much smaller one does not
    rc, c = _malloc(lib, PAGE)
    assert rc == 0 and c != a and lib.mlxrocm_buffer_size(c) == PAGE
    assert lib.mlxrocm_get_cache_memory() == 3 * PAGE
    assert lib.mlxrocm_free(c) == 0
    assert lib.mlxrocm_get_cache_memory() == 4 * PAGE
    # the limit trims the least recently freed buffer first (the 3-page one)
    prev = lib.mlxrocm_set_cache_limit(PAGE)
    assert prev == ctypes.c_size_t(-1).value
    assert lib.mlxrocm_get_cache_memory() == PAGE
    rc, d = _malloc(lib, PAGE)
    assert rc == 0 and d == c
    assert lib.mlxrocm_free(d) == 0
    # limit 0: nothing is kept
    assert lib.mlxrocm_set_cache_limit(0) == PAGE
    assert lib.mlxrocm_get_cache_memory() == 0
    rc, e = _malloc(lib, PAGE)
    assert rc == 0
    assert lib.mlxrocm_free(e) == 0
    assert lib.mlxrocm_get_cache_memory() == 0


def test_memory_limit_releases_the_cache(lib):
    total = ctypes.c_size_t()
    assert lib.mlxrocm_device_info(0, None, None, ctypes.byref(total), None) == 0
    default = lib.mlxrocm_get_memory_limit()
    assert 0 < default <= total.value
    rc, a = _malloc(lib, 64 * PAGE)
    assert rc == 0 and lib.mlxrocm_free(a) == 0
    assert lib.mlxrocm_get_cache_memory() == 64 * PAGE
    # with the limit at what is in use now, the next fresh allocation must give
    # the cached buffer back first
    prev = lib.mlxrocm_set_memory_limit(lib.mlxrocm_get_active_memory() + PAGE)
    assert prev == default
    rc, b = _malloc(lib, 8 * PAGE)  # too small to reuse the 64-page buffer
    assert rc == 0
    assert lib.mlxrocm_get_cache_memory() == 0
    assert lib.mlxrocm_free(b) == 0
    lib.mlxrocm_set_memory_limit(default)
    assert lib.mlxrocm_get_memory_limit() == default


def test_absurd_request_is_out_of_memory(lib):
    before = lib.mlxrocm_get_active_memory()
    for size in (1 << 50, ctypes.c_size_t(-1).value - 5):
        rc, p = _malloc(lib, size)
        assert rc == _lib.OUT_OF_MEMORY and p is None
        assert "unable to allocate" in _lib.last_error()
    assert lib.mlxrocm_get_active_memory() == before
    # the device still works afterwards
    rc, p = _malloc(lib, 1 << 20)
    assert rc == 0 and lib.mlxrocm_free(p) == 0
    with pytest.raises(MemoryError):
        _lib.check(_lib.OUT_OF_MEMORY)


def test_host_memory_and_copies(lib):
    n = (1 << 20) + 12  # not a multiple of anything interesting
    src, dst = ctypes.c_void_p(), ctypes.c_void_p()
    assert lib.mlxrocm_host_malloc(ctypes.byref(src), n) == 0
    assert lib.mlxrocm_host_malloc(ctypes.byref(dst), n) == 0
    host_src = (ctypes.c_uint8 * n).from_address(src.value)
    host_dst = (ctypes.c_uint8 * n).from_address(dst.value)
    pattern = bytes((i * 131 + 7) & 0xFF for i in range(4096)) * (n // 4096 + 1)
    ctypes.memmove(src.value, pattern, n)
    ctypes.memset(dst.value, 0, n)
    rc, d1 = _malloc(lib, n)
    assert rc == 0
    rc, d2 = _malloc(lib, n)
    assert rc == 0
    s = ctypes.c_void_p()
    assert lib.mlxrocm_stream_create(ctypes.byref(s)) == 0
    assert lib.mlxrocm_memcpy_h2d(d1, src, n, s) == 0
    assert lib.mlxrocm_memcpy_d2d(d2, d1, n, s) == 0
    assert lib.mlxrocm_memcpy_d2h(dst, d2, n, s) == 0
    assert lib.mlxrocm_stream_synchronize(s) == 0
    assert bytes(host_dst) == bytes(host_src) == pattern[:n]
    # zero-length copies are accepted and do nothing
    assert lib.mlxrocm_memcpy_h2d(d1, src, 0, s) == 0
    # a kernel of the library reads what the copies wrote: dequantize one group
    assert lib.mlxrocm_stream_destroy(s) == 0
    assert lib.mlxrocm_free(d1) == 0 and lib.mlxrocm_free(d2) == 0
    assert lib.mlxrocm_host_free(src) == 0 and lib.mlxrocm_host_free(dst) == 0
    rc = lib.mlxrocm_host_malloc(ctypes.byref(src), 0)
    assert rc == 0 and src.value is None


def test_allocator_buffers_feed_the_kernels(lib):
    """Buffers of the allocator and explicit copies around one operator call:
    quantize 64 x 256 float32 values uploaded from pinned memory, read the
    packed words back, compare with the same operator on torch memory."""
    import mlx_amd

    rows, K, gs, bits = 64, 256, 64, 4
    w = torch.randn(rows, K, generator=torch.Generator().manual_seed(0))
    n = w.numel()
    host = ctypes.c_void_p()
    assert lib.mlxrocm_host_malloc(ctypes.byref(host), n * 4) == 0
    ctypes.memmove(host.value, w.numpy().ctypes.data, n * 4)
    bufs = []
    for size in (n * 4, n * bits // 8, n // gs * 4, n // gs * 4):
        rc, p = _malloc(lib, size)
        assert rc == 0
        bufs.append(p)
    dw, dq, ds, db = bufs
    s = ctypes.c_void_p()
    assert lib.mlxrocm_stream_create(ctypes.byref(s)) == 0
    assert lib.mlxrocm_memcpy_h2d(dw, host, n * 4, s) == 0
    assert lib.mlxrocm_affine_quantize(dw, dq, ds, db, n, gs, bits, _lib.FLOAT32, s) == 0
    out = ctypes.c_void_p()
    assert lib.mlxrocm_host_malloc(ctypes.byref(out), n * bits // 8) == 0
    assert lib.mlxrocm_memcpy_d2h(out, dq, n * bits // 8, s) == 0
    assert lib.mlxrocm_stream_synchronize(s) == 0
    got = bytes((ctypes.c_uint8 * (n * bits // 8)).from_address(out.value))
    wq, _, _ = mlx_amd.quantize(w.cuda(), gs, bits)
    torch.cuda.synchronize()
    assert got == wq.cpu().numpy().tobytes()
    assert lib.mlxrocm_stream_destroy(s) == 0
    for p in bufs:
        assert lib.mlxrocm_free(p) == 0
    assert lib.mlxrocm_host_free(host) == 0 and lib.mlxrocm_host_free(out) == 0


def test_events_order_two_streams(lib):
    """Producer stream: fill A, record; consumer stream: wait, copy A -> B.
    Without the wait nothing orders the two non-blocking streams."""
    n = 64 << 20
    s1, s2 = ctypes.c_void_p(), ctypes.c_void_p()
    assert lib.mlxrocm_stream_create(ctypes.byref(s1)) == 0
    assert lib.mlxrocm_stream_create(ctypes.byref(s2)) == 0
    ev, done = ctypes.c_void_p(), ctypes.c_void_p()
    assert lib.mlxrocm_event_create(ctypes.byref(ev)) == 0
    assert lib.mlxrocm_event_create(ctypes.byref(done)) == 0
    rc, a = _malloc(lib, n)
    assert rc == 0
    rc, b = _malloc(lib, n)
    assert rc == 0
    host = ctypes.c_void_p()
    assert lib.mlxrocm_host_malloc(ctypes.byref(host), n) == 0
    back = ctypes.c_void_p()
    assert lib.mlxrocm_host_malloc(ctypes.byref(back), n) == 0
    for round_ in range(3):
        ctypes.memset(host.value, 0x30 + round_, n)
        ctypes.memset(back.value, 0, n)
        assert lib.mlxrocm_memcpy_h2d(a, host, n, s1) == 0
        assert lib.mlxrocm_event_record(ev, s1) == 0
        assert lib.mlxrocm_event_wait(ev, s2) == 0
        assert lib.mlxrocm_memcpy_d2d(b, a, n, s2) == 0
        assert lib.mlxrocm_memcpy_d2h(back, b, n, s2) == 0
        assert lib.mlxrocm_event_record(done, s2) == 0
        q = lib.mlxrocm_event_query(done)
        assert q in (0, 1)
        assert lib.mlxrocm_event_synchronize(done) == 0
        assert lib.mlxrocm_event_query(done) == 1
        assert lib.mlxrocm_event_query(ev) == 1  # the producer finished before the consumer
        view = (ctypes.c_uint8 * n).from_address(back.value)
        assert view[0] == view[n // 2] == view[n - 1] == 0x30 + round_
        assert bytes(view[:4096]) == bytes([0x30 + round_]) * 4096
    ms = ctypes.c_float(-1.0)
    assert lib.mlxrocm_event_record(ev, s1) == 0
    assert lib.mlxrocm_memcpy_h2d(a, host, n, s1) == 0
    assert lib.mlxrocm_event_record(done, s1) == 0
    assert lib.mlxrocm_event_synchronize(done) == 0
    assert lib.mlxrocm_event_elapsed_ms(ctypes.byref(ms), ev, done) == 0
    assert ms.value > 0.0
    assert lib.mlxrocm_event_elapsed_ms(None, ev, done) == _lib.INVALID_ARGUMENT
    for e in (ev, done):
        assert lib.mlxrocm_event_destroy(e) == 0
    for s in (s1, s2):
        assert lib.mlxrocm_stream_destroy(s) == 0
    assert lib.mlxrocm_free(a) == 0 and lib.mlxrocm_free(b) == 0
    assert lib.mlxrocm_host_free(host) == 0 and lib.mlxrocm_host_free(back) == 0


def test_device_info(lib):
    assert lib.mlxrocm_device_count() >= 1
    name = ctypes.create_string_buffer(256)
    cus, clock = ctypes.c_int(), ctypes.c_int()
    total = ctypes.c_size_t()
    assert lib.mlxrocm_device_info(0, name, ctypes.byref(cus), ctypes.byref(total),
                                   ctypes.byref(clock)) == 0
    assert b"gfx950" in name.value
    assert cus.value >= 64 and total.value > (64 << 30) and clock.value > 0
