"""GPU test of mlxrocm_qmm_static, the entry point that allocates nothing: its
results must be those of mlxrocm_qmm with a caller-provided workspace, bit for
bit, on two calls in a row (the second with a smaller input, which finds the
first call's contents in the shared scratch array), for every kind of shape
that uses scratch; shapes beyond the built-in buffer are refused."""
import pytest
import torch

import mlx_amd
from mlx_amd import _lib
from tests.util import activations, normal_weights

pytestmark = pytest.mark.gpu

CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _both(lib, gpu, x, q, gs, bits, transpose):
    """(mlxrocm_qmm with a workspace, mlxrocm_qmm_static) on the same operands."""
    wq, s, b = q
    M, K = x.shape
    N = wq.shape[0] if transpose else wq.shape[1] * 32 // bits
    code = CODE[x.dtype]
    stream = torch.cuda.current_stream().cuda_stream
    need = lib.mlxrocm_qmm_workspace_size(M, N, K, 1, 0, gs, bits, code, int(transpose))
    ws = torch.empty(max(need, 256), dtype=torch.uint8, device=gpu)
    ref = torch.full((M, N), float("nan"), dtype=x.dtype, device=gpu)
    got = torch.full((M, N), float("nan"), dtype=x.dtype, device=gpu)
    args = (M, N, K, 1, M * K, 0, 0, gs, bits, code, int(transpose))
    _lib.check(lib.mlxrocm_qmm(x.data_ptr(), wq.data_ptr(), s.data_ptr(), b.data_ptr(),
                               ref.data_ptr(), *args, ws.data_ptr(), need, stream))
    _lib.check(lib.mlxrocm_qmm_static(x.data_ptr(), wq.data_ptr(), s.data_ptr(), b.data_ptr(),
                                      got.data_ptr(), *args, stream))
    torch.cuda.synchronize()
    return ref, got, need


# (dtype, bits, gs, transpose, first shape (M, N, K), second, smaller shape)
CASES = (
    # 16-bit prefill: transposed scales and biases, K split into fp32 partial planes
    (torch.bfloat16, 4, 64, True, (640, 4096, 4096), (520, 1024, 2048)),
    (torch.float16, 8, 128, True, (2048, 2048, 1024), (512, 600, 512)),
    # float32 prefill: x split into two bfloat16 parts
    (torch.float32, 4, 64, True, (300, 1024, 2048), (40, 200, 256)),
    # transpose == 0 on the matrix cores and on the streaming kernel's planes
    (torch.bfloat16, 4, 64, False, (600, 2048, 1024), (70, 512, 384)),
    (torch.bfloat16, 8, 64, False, (3, 4096, 4096), (1, 1024, 2050)),
)


def _memory_state(lib):
    """(bytes the library's allocator holds, its peak, its cache, free device
    memory as the driver reports it)."""
    free, total = torch.cuda.mem_get_info()
    return (lib.mlxrocm_get_active_memory(), lib.mlxrocm_get_peak_memory(),
            lib.mlxrocm_get_cache_memory(), free)


def test_static_entry_point_allocates_nothing(gpu):
    """The property in the entry point's name: around calls of every kind of
    shape that uses scratch, the library's allocator counters (active, peak,
    cache) and the driver's free-memory figure do not move.  The array's
    address is resolved by an empty call first, as documented."""
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.mlxrocm_qmm_static(None, None, None, None, None, 0, 32, 128, 1, 0, 0, 0,
                                  64, 4, 2, 1, stream) == 0
    prepared = []
    for dtype, bits, gs, transpose, first, second in CASES:
        for M, N, K in (first, second):
            w = normal_weights((N, K) if transpose else (K, N), dtype, seed=M + N).to(gpu)
            wq, s, b = mlx_amd.quantize(w, gs, bits)
            x = activations((M, K), dtype, seed=K).to(gpu)
            out = torch.empty((M, N), dtype=dtype, device=gpu)
            prepared.append((x, wq, s, b, out, (M, N, K, 1, M * K, 0, 0, gs, bits, CODE[dtype],
                                                int(transpose))))
            del w
    def run_all():
        for x, wq, s, b, out, args in prepared:
            _lib.check(lib.mlxrocm_qmm_static(x.data_ptr(), wq.data_ptr(), s.data_ptr(),
                                              b.data_ptr(), out.data_ptr(), *args, stream))
        torch.cuda.synchronize()

    run_all()  # the runtime loads each kernel's code on its first launch
    before = _memory_state(lib)
    run_all()
    after = _memory_state(lib)
    assert after == before, (before, after)


@pytest.mark.parametrize("dtype,bits,gs,transpose,first,second", CASES)
def test_static_scratch_matches_workspace_call(gpu, dtype, bits, gs, transpose, first, second):
    lib = _lib.load()
    used = 0
    for M, N, K in (first, second):
        w = normal_weights((N, K) if transpose else (K, N), dtype, seed=M + N).to(gpu)
        q = mlx_amd.quantize(w, gs, bits)
        x = activations((M, K), dtype, seed=K).to(gpu)
        ref, got, need = _both(lib, gpu, x, q, gs, bits, transpose)
        used = max(used, need)
        assert not bool(torch.isnan(ref.float()).any())
        assert torch.equal(ref.view(torch.int16 if dtype != torch.float32 else torch.int32),
                           got.view(torch.int16 if dtype != torch.float32 else torch.int32))
    assert used > 0  # the case does exercise the scratch array


def test_static_scratch_decode_and_empty_calls(gpu):
    """Shapes that need no scratch run the same kernels; an empty call is the
    documented way to resolve the array's address ahead of time."""
    lib = _lib.load()
    stream = torch.cuda.current_stream().cuda_stream
    assert lib.mlxrocm_qmm_static(None, None, None, None, None, 0, 32, 128, 1, 0, 0, 0,
                                  64, 4, 2, 1, stream) == 0
    w = normal_weights((4096, 4096), torch.bfloat16).to(gpu)
    q = mlx_amd.quantize(w, 64, 4)
    x = activations((1, 4096), torch.bfloat16).to(gpu)
    ref, got, need = _both(lib, gpu, x, q, 64, 4, True)
    assert need == 0 and torch.equal(ref.view(torch.int16), got.view(torch.int16))


def test_static_scratch_refuses_what_does_not_fit(gpu):
    lib = _lib.load()
    M, N, K = 8192, 16384, 4096  # float32: the split x alone is 192 MiB
    assert lib.mlxrocm_qmm_workspace_size(M, N, K, 1, 0, 64, 4, 0, 1) > (64 << 20)
    one = torch.zeros(64, dtype=torch.uint8, device=gpu)
    rc = lib.mlxrocm_qmm_static(one.data_ptr(), one.data_ptr(), one.data_ptr(), one.data_ptr(),
                                one.data_ptr(), M, N, K, 1, M * K, 0, 0, 64, 4, 0, 1,
                                torch.cuda.current_stream().cuda_stream)
    assert rc == _lib.UNSUPPORTED
    assert "built-in" in _lib.last_error()
    with pytest.raises(RuntimeError):
        _lib.check(rc)
