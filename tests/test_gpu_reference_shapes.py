"""The shape grids of the reference's own quantized-matmul tests
(python/tests/test_quantized.py), run the way they are written there: quantize,
dequantize, and compare ``quantized_matmul`` with the dense product of the
dequantized matrix under the reference's absolute tolerance.  The other GPU
tests check the same kernels against the oracle at full sizes; these add the
small, ragged and lopsided shapes the reference walks -- N of 3 .. 99, K of 3,
8, 33 and 67 with ``transpose=False``, N beyond 2^15, M beyond 2^15, stacks of
1, 3 and 8 weight matrices.  The dense product is float64 on the CPU."""
import itertools

import pytest
import torch

import mlx_amd

pytestmark = pytest.mark.gpu

FP_MODES = ("mxfp4", "nvfp4", "mxfp8")


def _randn(shape, g, dtype=torch.float32, scale=1.0):
    return (torch.randn(shape, generator=g) * scale).to(dtype)


def _check(gpu, x, w, transpose, tol, group_size=None, bits=None, mode="affine"):
    """quantized_matmul(x, quantize(w)) against x @ dequantize(quantize(w))."""
    kw = dict(group_size=group_size, bits=bits, mode=mode)
    q = mlx_amd.quantize(w.to(gpu), **kw)
    if mode == "affine":
        w_hat = mlx_amd.dequantize(*q, **kw)
        y_q = mlx_amd.quantized_matmul(x.to(gpu), *q, transpose=transpose, **kw)
    else:
        w_hat = mlx_amd.dequantize(*q, **kw, dtype=torch.float32)
        y_q = mlx_amd.quantized_matmul(x.to(gpu), *q, transpose=transpose, **kw)
    w_hat = w_hat.cpu().double()
    y_hat = x.double() @ (w_hat.transpose(-1, -2) if transpose else w_hat)
    assert tuple(y_q.shape) == tuple(y_hat.shape), (x.shape, w.shape, transpose)
    err = (y_q.cpu().double() - y_hat).abs().max().item() if y_hat.numel() else 0.0
    assert err < tol, (tuple(x.shape), tuple(w.shape), transpose, group_size, bits, mode, err)


def test_qmm_large_dims(gpu):
    # :325-357 -- N beyond 2^15 and not a tile multiple; M beyond 2^15
    g = torch.Generator().manual_seed(0)
    K = 128
    for M, N in ((16, 32840), (32, 32840), (33, 32840), (33000, 64)):
        x = _randn((M, K), g, torch.float16, K ** -0.5)
        w = _randn((N, K), g, torch.float16, K ** -0.5)
        _check(gpu, x, w, True, 1.5e-3, 64, 4)


def test_qmv_wide_grid(gpu):
    # :678-753 -- 2..9 rows of x, ragged N, one and three weight matrices, every
    # width and group size; then the fp modes; then tiny shapes
    g = torch.Generator().manual_seed(1)
    Ms, Ns, Bs = (2, 3, 4, 5, 6, 7, 9), (256, 67), (1, 3)
    for gs, bits, K in itertools.product((32, 64, 128), (2, 3, 4, 5, 6, 8), (128, 512)):
        for M, N, B in itertools.product(Ms, Ns, Bs):
            x = _randn((M, K) if B == 1 else (B, M, K), g)
            w = _randn((N, K) if B == 1 else (B, N, K), g)
            _check(gpu, x, w, True, 1e-3, gs, bits)
    for mode, K in itertools.product(FP_MODES, (128, 512)):
        for M, N, B in itertools.product(Ms, Ns, Bs):
            x = _randn((M, K) if B == 1 else (B, M, K), g)
            w = _randn((N, K) if B == 1 else (B, N, K), g)
            _check(gpu, x, w, True, 1e-3, mode=mode)
    for M, K, N in ((2, 32, 10), (4, 32, 7), (3, 64, 5), (5, 64, 3)):
        for bits, gs, mode in ((4, 32, "affine"), (6, 32, "affine"), (4, 16, "nvfp4")):
            _check(gpu, _randn((M, K), g), _randn((N, K), g), True, 1e-3, gs, bits, mode)


def test_small_matrix_and_non_multiples(gpu):
    # :958-992 (test_small_matrix), :994-1066 (test_non_multiples)
    g = torch.Generator().manual_seed(2)
    for w_shape in ((8, 256), (1, 8, 256), (3, 8, 256)):
        w = _randn(w_shape, g)
        for x_shape in ((3, 1, 256), (3, 4, 256), (3, 10, 256)):
            _check(gpu, _randn(x_shape, g), w, True, 1e-3)
        for x_shape in ((3, 1, 8), (3, 10, 8)):
            _check(gpu, _randn(x_shape, g), w, False, 1e-3)
    for rows in (33, 3):
        w = _randn((rows, 256), g)
        for M in (1, 10):
            _check(gpu, _randn((M, 256), g), w, True, 1e-3)
            _check(gpu, _randn((M, rows), g), w, False, 1e-3)
    _check(gpu, _randn((129, 256), g), _randn((99, 256), g), True, 1e-3)


def test_qmv_small_non_multiples(gpu):
    # :1068-1125 -- very small K and N, with and without a batch of weights
    g = torch.Generator().manual_seed(3)
    for M, K, N in ((1, 32, 3), (2, 32, 10), (1, 32, 5), (4, 32, 7)):
        for bits, gs, mode in ((4, 32, "affine"), (6, 32, "affine"), (4, 16, "nvfp4")):
            _check(gpu, _randn((M, K), g), _randn((N, K), g), True, 1e-3, gs, bits, mode)
            _check(gpu, _randn((3, M, K), g), _randn((3, N, K), g), True, 1e-3, gs, bits, mode)


def test_qvm_grid(gpu):
    # :755-780 (test_qvm), :844-875 (test_fp_qvm): one row of x against [K, N]
    # weights, K of 128, 256 and 67, stacks of 1, 3 and 8 matrices
    g = torch.Generator().manual_seed(4)
    for gs, bits, M, N, B in itertools.product(
            (128, 64, 32), (2, 3, 4, 5, 6, 8), (32, 128, 256), (128, 256, 67), (0, 1, 3, 8)):
        if M < gs:
            continue
        x = _randn((1, N) if B == 0 else (B, 1, N), g)
        w = _randn((N, M) if B == 0 else (B, N, M), g)
        _check(gpu, x, w, False, 1e-3, gs, bits)
    cases = list(itertools.product((32, 128, 256), (128, 256, 67), (0, 1, 3, 8))) + [(128, 16384, 0)]
    for (M, N, B), mode in itertools.product(cases, FP_MODES):
        x = _randn((1, N) if B == 0 else (B, 1, N), g)
        w = _randn((N, M) if B == 0 else (B, N, M), g)
        _check(gpu, x, w, False, 2e-3, mode=mode)


def test_qvm_split_k(gpu):
    # :782-842 -- long K with transpose=False: one row and 2..3 rows of x; a 1-D x
    g = torch.Generator().manual_seed(5)
    for gs, bits, B in itertools.product((128, 64, 32), (2, 4, 8), (1, 3)):
        x = _randn((B, 1, 16384), g, scale=0.1)
        w = _randn((B, 16384, 128), g, scale=0.1)
        _check(gpu, x, w, False, 2e-3, gs, bits)
    _check(gpu, _randn((2048,), g, scale=0.1), _randn((2048, 2048), g, scale=0.1), False, 2e-3, 32, 8)
    for gs, bits, K, M in itertools.product((64, 32), (4, 8), (2048, 4096), (2, 3)):
        _check(gpu, _randn((M, K), g, scale=0.1), _randn((K, 128), g, scale=0.1), False, 2e-3, gs, bits)


def test_qmm_grid(gpu):
    # :288-323 (test_qmm) -- both values of transpose, float16 as on the GPU there
    g = torch.Generator().manual_seed(6)
    for gs, bits, M, N, K, transposed in itertools.product(
            (128, 64, 32), (2, 4, 8), (8, 32, 33, 64), (128, 256), (128, 256), (True, False)):
        x = _randn((M, K), g, torch.float16, K ** -0.5)
        w = _randn((N, K) if transposed else (K, N), g, torch.float16, K ** -0.5)
        _check(gpu, x, w, transposed, 1.5e-3, gs, bits)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16), ids=str)
def test_qmm_non_transposed(gpu, dtype):
    # :359-442 -- [K, N] weights over transformer-sized K / N and M values that
    # leave partial tiles; affine and the fp modes; batched x; M beyond 2^15.
    # bfloat16 results are compared at their own resolution.
    g = torch.Generator().manual_seed(7)
    tol = 1.5e-3 if dtype == torch.float16 else 1.2e-2

    def affine(M, K, N, gs, bits, batch=()):
        x = _randn(batch + (M, K), g, dtype, K ** -0.5)
        _check(gpu, x, _randn((K, N), g, dtype, K ** -0.5), False, tol, gs, bits)

    def fp(M, K, N, mode, batch=()):
        x = _randn(batch + (M, K), g, dtype, K ** -0.5)
        _check(gpu, x, _randn((K, N), g, dtype, K ** -0.5), False, tol, mode=mode)

    for M in (1, 2, 31, 32, 33, 63, 64, 65, 96, 97, 100, 127, 128, 129):
        for gs, bits in ((64, 4), (128, 4), (64, 8)):
            affine(M, 512, 1024, gs, bits)
        for mode in FP_MODES:
            fp(M, 512, 1024, mode)
    for K, N in ((2048, 2048), (512, 2048), (2048, 512), (11008, 2048)):
        for M in (100, 256):
            affine(M, K, N, 64, 4)
    for batch in ((2,), (2, 3)):
        for M in (33, 250):
            affine(M, 512, 1024, 64, 4, batch)
            for mode in FP_MODES:
                fp(M, 512, 1024, mode, batch)
    affine(33000, 128, 64, 64, 4)
    fp(33000, 128, 64, "mxfp8")
    for M, K in itertools.product((8, 33, 65), (64, 128, 256)):
        for bits in (2, 4, 8):
            affine(M, K, 128, 32, bits)
        for mode in FP_MODES:
            fp(M, K, 128, mode)


def test_qmm_small_m_block_and_shapes(gpu):
    # :444-478 (batched weights / an fp mode at 14 rows), :540-563 (test_qmm_shapes)
    g = torch.Generator().manual_seed(8)
    K = 1024
    x = _randn((2, 14, K), g, torch.float16, K ** -0.5)
    _check(gpu, x, _randn((2, 8256, K), g, torch.float16, K ** -0.5), True, 1e-3, 64, 4)
    x = _randn((14, K), g, torch.bfloat16, K ** -0.5)
    _check(gpu, x, _randn((8256, K), g, torch.bfloat16, K ** -0.5), True, 8e-3, mode="mxfp4")
    for w_shape, transposed in (((32, 256), True), ((256, 256), False)):
        w = _randn(w_shape, g)
        for s in ((3, 256), (2, 1, 7, 256)):
            _check(gpu, _randn(s, g), w, transposed, 1e-3, 64, 4)


def test_qmv_grid(gpu):
    # :565-590 (test_qmv), :592-641 (test_fp_qmv): one row of x per matrix, N of
    # 256, 512, 67, 5 and 7, stacks of 1, 3 and 8 matrices, every width
    g = torch.Generator().manual_seed(9)
    for gs, bits, M, N, B in itertools.product(
            (128, 64, 32), (2, 3, 4, 5, 6, 8), (256, 512, 67), (64, 256), (0, 1, 3, 8)):
        if gs > N:
            continue
        x = _randn((3, 1, N) if B == 0 else (B, 1, N), g, scale=N ** -0.5)
        w = _randn((M, N) if B == 0 else (B, M, N), g, scale=N ** -0.5)
        _check(gpu, x, w, True, 1e-3, gs, bits)
    for (M, N, B), mode in itertools.product(
            itertools.product((256, 512, 67, 5, 7), (64, 256), (0, 1, 3, 8)), FP_MODES):
        x = _randn((3, 1, N) if B == 0 else (B, 1, N), g)
        w = _randn((M, N) if B == 0 else (B, M, N), g)
        _check(gpu, x, w, True, 1e-3, mode=mode)
    _check(gpu, _randn((1, 48), g), _randn((128, 48), g), True, 1e-3, mode="nvfp4")


def test_qmm_fp_type_and_strided_scales(gpu):
    # :1362-1379 (test_qmm_fp_type): the result has the type of x, also through
    # gather_qmm with a 2-D x and [3, 1] expert indices; :1696-1706
    # (test_quantize_strided): scales that are a broadcast view
    g = torch.Generator().manual_seed(10)
    indices = torch.tensor([[2], [0], [1]], dtype=torch.int32, device=gpu)
    for mode in ("mxfp8", "mxfp4"):
        for t in (torch.bfloat16, torch.float16, torch.float32):
            x = _randn((32, 256), g, t).to(gpu)
            wq, s = mlx_amd.quantize(_randn((32, 256), g).to(gpu), mode=mode)
            assert mlx_amd.quantized_matmul(x, wq, s, mode=mode).dtype == t
            wq, s = mlx_amd.quantize(_randn((4, 32, 256), g).to(gpu), mode=mode)
            out = mlx_amd.gather_qmm(x, wq, s, rhs_indices=indices, mode=mode)
            assert out.dtype == t and tuple(out.shape) == (3, 1, 32, 32)
            w_hat = mlx_amd.dequantize(wq, s, mode=mode, dtype=torch.float32).cpu().double()
            for i, e in enumerate((2, 0, 1)):
                want = x.cpu().double() @ w_hat[e].T
                tol = {torch.float32: 1e-3, torch.float16: 3e-2, torch.bfloat16: 2.5e-1}[t]
                assert (out[i, 0].cpu().double() - want).abs().max().item() < tol, (mode, t, i)
    w_q, scales = mlx_amd.quantize(_randn((64, 64), g).to(gpu), mode="nvfp4")
    flat = torch.tensor(56, dtype=torch.uint8, device=gpu).expand(scales.shape)
    w_hat = mlx_amd.dequantize(w_q, flat, mode="nvfp4")
    expected = mlx_amd.dequantize(w_q, flat.contiguous(), mode="nvfp4")
    assert torch.equal(w_hat, expected)


def test_more_rows_of_x_than_a_grid_is_deep(gpu):
    """70,000 rows of x through the kernels that use one grid row per row of x
    (K not a multiple of 64, [K, N] weights with an odd K, the fp modes' streaming
    kernels): the launches are cut into slices of rows on the host."""
    g = torch.Generator().manual_seed(11)
    M = 70000
    _check(gpu, _randn((M, 32), g), _randn((40, 32), g), True, 1e-3, 32, 4)
    _check(gpu, _randn((M, 5), g), _randn((5, 64), g), False, 1e-3, 32, 4)
    _check(gpu, _randn((2, M, 5), g), _randn((2, 5, 64), g), False, 1e-3, 32, 8)
    _check(gpu, _randn((M, 64), g), _randn((24, 64), g), True, 1e-3, mode="mxfp4")
    _check(gpu, _randn((M, 48), g), _randn((24, 48), g), True, 1e-3, mode="nvfp4")
    _check(gpu, _randn((M, 7), g), _randn((7, 64), g), False, 1e-3, mode="mxfp8")
    _check(gpu, _randn((M, 64), g, torch.bfloat16), _randn((24, 64), g, torch.bfloat16), True, 0.15,
           mode="mxfp8")


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16), ids=str)
def test_stacks_with_unaligned_rows_sixteen_bit(gpu, dtype):
    """Stacks of [K, N] weights with K = 67 and of x [B, M, 67] in the 16-bit
    types (batch strides of 134 and 1340 bytes), and stacks of tiny packed
    matrices (18 words each): accepted and right."""
    g = torch.Generator().manual_seed(12)
    tol = 4e-3 if dtype == torch.float16 else 3e-2  # results of magnitude ~1 at their own resolution
    for M in (1, 3, 10):
        def x_of(K):
            return _randn((3, M, K), g, dtype, K ** -0.5)

        for bits, gs in ((4, 64), (3, 32), (8, 128)):
            _check(gpu, x_of(67), _randn((3, 67, 128), g, dtype), False, tol, gs, bits)
        _check(gpu, x_of(67), _randn((3, 67, 128), g, dtype), False, tol, mode="mxfp4")
        _check(gpu, x_of(32), _randn((3, 3, 32), g, dtype), True, tol, 32, 6)
        _check(gpu, x_of(48), _randn((3, 5, 48), g, dtype), True, tol, mode="nvfp4")
