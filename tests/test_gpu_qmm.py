"""GPU parity of quantized_matmul against the CPU oracle and the fp64 product."""
import math

import pytest
import torch

import mlx_amd
from tests.util import (
    ALL_BITS, ALL_GROUPS, DTYPES, activations, exact_affine_weights,
    exact_affine_weights_on, exact_product_error, exact_tolerance,
    exact_tolerance_from, matmul_tolerance, normal_weights, student_t_weights,
)

pytestmark = pytest.mark.gpu


def _check_qmm(oracle, gpu, x, w, gs, bits, transpose=True, rows=None, quantized=None):
    """x [M, K]; w dense weights (quantized on the CPU by the oracle) or a
    ready (wq, s, b) triple.  Every row of the result is compared with the fp64
    product of the exact affine weights (torch float64 on the GPU); `rows` is
    the subset of x rows the scalar CPU oracle is run on (all rows if None)."""
    wq, s, b = quantized if quantized is not None else oracle.quantize(w, gs, bits)
    got = mlx_amd.quantized_matmul(
        x.to(gpu), wq.to(gpu), s.to(gpu), b.to(gpu), transpose, gs, bits
    )
    torch.cuda.synchronize()
    K = x.shape[-1]
    w_hat = exact_affine_weights_on(gpu, wq, s, b, gs, bits)
    w_absmax, x_absmax = float(w_hat.abs().max()), float(x.abs().max())
    assert got.shape == (x.shape[0], w_hat.shape[0] if transpose else w_hat.shape[1])
    assert got.dtype == x.dtype
    # strict check, every row: fp64 product
    err_exact, y_absmax = exact_product_error(got, x, w_hat, transpose)
    tol_exact = exact_tolerance_from(x.dtype, K, x_absmax, w_absmax, y_absmax)
    assert err_exact <= tol_exact, f"vs fp64 (all rows): {err_exact} > {tol_exact}"
    # the CPU oracle on the sampled rows
    sel = slice(None) if rows is None else rows
    xs = x[sel]
    ref = oracle.qmm(xs, wq, s, b, transpose, gs, bits).double()
    exact = (xs.to(gpu).double() @ (w_hat.T if transpose else w_hat)).cpu()
    g = got.cpu()[sel].double()
    err_ref = float((g - ref).abs().max())
    c = 1e-5 if x.dtype == torch.float32 else 2e-2
    bare = c * math.sqrt(K) * x_absmax * w_absmax  # the stated bound
    tol_ref = bare
    discount = 0.0
    if x.dtype != torch.float32:
        # The x86 CPU reference accumulates 16-bit types in the element type
        # (cpu/quantized.cpp:177-206); at K >= 4096 its own distance from the
        # exact product already exceeds the bound, so that measured distance is
        # discounted.  The fp64 check above is the strict one.
        discount = float((ref - exact).abs().max())
        tol_ref += discount
    print(f"qmm M={x.shape[0]} K={K} b{bits} g{gs} {x.dtype}: |gpu-oracle|={err_ref:.3e} "
          f"bare bound={bare:.3e} (margin {bare - err_ref:+.3e}) |oracle-fp64|={discount:.3e}; "
          f"|gpu-fp64|={err_exact:.3e} bound={tol_exact:.3e}")
    assert err_ref <= tol_ref, f"vs oracle: {err_ref} > {tol_ref}"
    return got.cpu()


def _spread_rows(M):
    """Rows of x for the scalar oracle: first, last, and one in each quarter of a
    256-row tile (rows 65, 130 and 195 of different tiles)."""
    picks = {0, M - 1}
    for i, off in enumerate((65, 130, 195)):
        r = 256 * (i * max(1, M // 256) // 3) + off
        if r < M:
            picks.add(r)
    return torch.tensor(sorted(picks))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits", ALL_BITS)
@pytest.mark.parametrize("gs", ALL_GROUPS)
def test_qmv_all_widths(oracle, gpu, dtype, bits, gs):
    # python/tests/test_quantized.py:565-590 (N = 67 is not a tile multiple)
    for M, N, K in ((1, 67, 512), (3, 128, 256)):
        w = normal_weights((N, K), dtype, seed=bits + gs)
        x = activations((M, K), dtype)
        _check_qmm(oracle, gpu, x, w, gs, bits)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits", ALL_BITS)
@pytest.mark.parametrize("gs", ALL_GROUPS)
@pytest.mark.parametrize("transpose", (True, False))
def test_qmm_all_widths(oracle, gpu, dtype, bits, gs, transpose):
    # python/tests/test_quantized.py:288-323: M in {8, 32, 33, 64}
    for M in (33, 64):
        N, K = 256, 384
        w = normal_weights((N, K) if transpose else (K, N), dtype, seed=bits * gs)
        x = activations((M, K), dtype)
        _check_qmm(oracle, gpu, x, w, gs, bits, transpose)


def test_qmv_config1_fp32(oracle, gpu):
    w = normal_weights((4096, 4096), torch.float32, seed=0)
    x = activations((1, 4096), torch.float32, seed=0)
    _check_qmm(oracle, gpu, x, w, 64, 4)


@pytest.mark.parametrize("bits,gs", [(4, 64), (8, 128)])
@pytest.mark.parametrize("B", (1, 4, 8))
def test_qmv_decode_shapes_bf16(oracle, gpu, bits, gs, B):
    for N, K in ((14336, 4096), (4096, 14336)):
        w = normal_weights((N, K), torch.bfloat16, seed=0)
        x = activations((B, K), torch.bfloat16)
        _check_qmm(oracle, gpu, x, w, gs, bits)


@pytest.mark.parametrize("bits", (4, 8))
@pytest.mark.parametrize("gs", (64, 128))
def test_qmm_t_prefill_shapes_bf16(oracle, gpu, bits, gs):
    """Full prefill shapes on the GPU, M in {512, 2048, 8192}: every row against
    the fp64 product; the scalar oracle sees a few rows spread over the quarters
    of a 256-row tile (each output row depends only on its own x row)."""
    for N, K in ((4096, 4096), (14336, 4096), (4096, 14336)):
        w = normal_weights((N, K), torch.bfloat16, seed=0)
        q = oracle.quantize(w, gs, bits)
        for M in (512, 2048, 8192):
            x = activations((M, K), torch.bfloat16)
            _check_qmm(oracle, gpu, x, None, gs, bits, rows=_spread_rows(M), quantized=q)


@pytest.mark.parametrize("bits", (2, 3, 5, 6))
@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16))
@pytest.mark.parametrize("tails", ("normal", "student_t"))
def test_odd_width_stress_matmul(oracle, gpu, dtype, bits, tails):
    """Codes that straddle words, groups of 32, normal and heavy-tailed
    (Student-t, 3 degrees of freedom) weights through the decode GEMV (x
    [1, K]) and the prefill GEMM (x [1024, K]), float32 and bfloat16."""
    make = normal_weights if tails == "normal" else student_t_weights
    for N, K in ((11008, 4096), (4096, 11008)):
        w = make((N, K), dtype, seed=bits)
        q = oracle.quantize(w, 32, bits)
        _check_qmm(oracle, gpu, activations((1, K), dtype), None, 32, bits, quantized=q)
        x = activations((1024, K), dtype)
        _check_qmm(oracle, gpu, x, None, 32, bits, rows=_spread_rows(1024), quantized=q)


@pytest.mark.parametrize("bits", (2, 3, 5, 6))
@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16))
@pytest.mark.parametrize("tails", ("normal", "student_t"))
def test_odd_width_stress_matmul_weight_as_k_by_n(oracle, gpu, dtype, bits, tails):
    """The other reading of the [4096, 11008] stress weight: x of width 4096
    only fits it with transpose=False, i.e. W is [K = 4096, N = 11008] with
    the groups of 32 along n (`_qmm`, cpu/quantized.cpp:96-152).  Full size,
    x [1, 4096] and [1024, 4096], every row against the fp64 product, spread
    rows against the scalar oracle."""
    make = normal_weights if tails == "normal" else student_t_weights
    K, N = 4096, 11008
    w = make((K, N), dtype, seed=bits)
    q = oracle.quantize(w, 32, bits)
    assert q[0].shape == (K, N * bits // 32) and q[1].shape == (K, N // 32)
    _check_qmm(oracle, gpu, activations((1, K), dtype), None, 32, bits, transpose=False,
               quantized=q)
    x = activations((1024, K), dtype)
    _check_qmm(oracle, gpu, x, None, 32, bits, transpose=False, rows=_spread_rows(1024),
               quantized=q)


def test_qmm_batched_shapes(oracle, gpu):
    # python/tests/test_quantized.py:540-563
    gs, bits = 64, 4
    w = normal_weights((32, 256), torch.float32)
    wq, s, b = oracle.quantize(w, gs, bits)
    x = activations((3, 5, 256), torch.float32)
    got = mlx_amd.quantized_matmul(x.to(gpu), wq.to(gpu), s.to(gpu), b.to(gpu), True, gs, bits)
    assert got.shape == (3, 5, 32)
    ref = oracle.qmm_batched(x, wq, s, b, True, gs, bits)
    assert float((got.cpu() - ref).abs().max()) < 1e-4
    # batched weights
    w3 = normal_weights((3, 32, 256), torch.float32, seed=5)
    wq3, s3, b3 = oracle.quantize(w3, gs, bits)
    got = mlx_amd.quantized_matmul(x.to(gpu), wq3.to(gpu), s3.to(gpu), b3.to(gpu), True, gs, bits)
    ref = oracle.qmm_batched(x, wq3, s3, b3, True, gs, bits)
    assert float((got.cpu() - ref).abs().max()) < 1e-4
    # 1-D x
    x1 = activations((256,), torch.float32)
    got = mlx_amd.quantized_matmul(x1.to(gpu), wq.to(gpu), s.to(gpu), b.to(gpu))
    assert got.shape == (32,)
    ref = oracle.qmm(x1.reshape(1, -1), wq, s, b, True, gs, bits)[0]
    assert float((got.cpu() - ref).abs().max()) < 1e-4


def test_qmm_type_promotion(gpu):
    """x, scales, biases are cast to the promoted type (mlx/ops.cpp:4816-4818)."""
    w = normal_weights((64, 128), torch.bfloat16).to(gpu)
    wq, s, b = mlx_amd.quantize(w)
    x = activations((2, 128), torch.float32).to(gpu)
    out = mlx_amd.quantized_matmul(x, wq, s, b)
    assert out.dtype == torch.float32
    out16 = mlx_amd.quantized_matmul(x.to(torch.float16), wq, s, b)
    assert out16.dtype == torch.float32  # float16 x bfloat16 -> float32


def test_qmm_t_fp32_runs_on_the_matrix_path(oracle, gpu):
    """fp32 prefill (M > 8, K a multiple of 64) is computed on the bf16 matrix
    cores from operands split into high and low parts: the fp32 bound still
    holds, also for batched x, batched weights, ragged M / N and heavy-tailed
    weights (Student-t, 3 degrees of freedom)."""
    from mlx_amd import _lib
    lib = _lib.load()
    assert lib.mlxrocm_qmm_kernel_name(1024, 11008, 4096, 1, 32, 3, 0, 1) == b"qmm_t"
    g = torch.Generator().manual_seed(3)
    for (M, N, K, bits, gs) in ((9, 50, 64, 4, 32), (300, 232, 1024, 8, 128), (513, 67, 448, 5, 64)):
        t = torch.distributions.StudentT(3.0).sample((N, K)) * 0.02
        w = t.clamp(-1.0, 1.0).float()
        x = activations((M, K), torch.float32, seed=M)
        _check_qmm(oracle, gpu, x, w, gs, bits)
    # batched x against one weight and against batched weights
    gs, bits = 64, 4
    x = activations((3, 40, 256), torch.float32)
    w3 = normal_weights((3, 96, 256), torch.float32, seed=7)
    wq3, s3, b3 = oracle.quantize(w3, gs, bits)
    for q in ((wq3[0], s3[0], b3[0]), (wq3, s3, b3)):
        got = mlx_amd.quantized_matmul(x.to(gpu), *(t.to(gpu) for t in q), True, gs, bits)
        ref = oracle.qmm_batched(x, *q, True, gs, bits)
        assert got.shape == (3, 40, 96)
        assert float((got.cpu() - ref).abs().max()) <= matmul_tolerance(
            torch.float32, 256, x, exact_affine_weights(wq3, s3, b3, gs, bits))


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
@pytest.mark.parametrize("bits", ALL_BITS)
def test_qmm_few_rows_kernels(oracle, gpu, dtype, bits):
    """3 <= M <= 32 goes to the few-row kernels (K split over wavefronts up to 16
    rows and, for a narrow N, twice for up to 32; 64-row LDS-staged tiles for
    17..32 rows over a wide N): ragged N, K of one and of several steps, every
    group size."""
    for gs in ALL_GROUPS:
        for M, N, K in ((5, 67, 128), (12, 130, 1280), (16, 48, 8704), (17, 200, 256), (32, 67, 1792),
                        (20, 8224, 384), (32, 8192, 128)):
            w = normal_weights((N, K), dtype, seed=bits + gs + M)
            x = activations((M, K), dtype, seed=M)
            _check_qmm(oracle, gpu, x, w, gs, bits)


@pytest.mark.parametrize("dtype,gs", ((torch.bfloat16, 128), (torch.float16, 64)))
def test_qmm_few_rows_of_8_bit_over_many_bytes(oracle, gpu, dtype, gs):
    """3..8 rows over 64 MB of 8-bit codes or more take the LDS-staged 32-row
    kernel (as 9..32 rows do): ragged N, every row checked against fp64, the
    first and the last against the CPU reference."""
    N, K = 8200, 8192
    w = normal_weights((N, K), dtype, std=0.05)
    quantized = oracle.quantize(w, gs, 8)
    for M in (3, 8):
        x = activations((M, K), dtype, seed=M)
        _check_qmm(oracle, gpu, x, None, gs, 8, rows=torch.tensor([0, M - 1]), quantized=quantized)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("bits,gs", ((4, 32), (4, 64), (8, 64), (8, 128)))
def test_qmm_n_on_the_matrix_path(oracle, gpu, dtype, bits, gs):
    # transpose=False (w [K, N], groups along n; cpu/quantized.cpp:96-152) with
    # K % 64 == 0 runs on the matrix cores: one row (qvm), a ragged M, a width
    # that is not a tile multiple, and a K long enough to be cut into ranges
    from mlx_amd import _lib

    code = {torch.float16: 1, torch.bfloat16: 2}[dtype]
    for M, K, N in ((1, 256, 384), (300, 192, 640), (70, 2048, 128), (5, 64, 256)):
        assert _lib.load().mlxrocm_qmm_kernel_name(M, N, K, 1, gs, bits, code, 0) == b"qmm_n"
        w = normal_weights((K, N), dtype, seed=bits + gs + M)
        x = activations((M, K), dtype, seed=M)
        _check_qmm(oracle, gpu, x, w, gs, bits, transpose=False)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits,gs", ((4, 32), (4, 64), (4, 128), (8, 32), (8, 64), (8, 128)))
def test_qvm_streaming_kernel(oracle, gpu, dtype, bits, gs):
    """transpose=False with 1..4 rows of x (cpu/quantized.cpp:96-152, the "qvm"
    case) runs on the row-streaming kernel: one K range and many, a K that is
    not a multiple of the four wavefronts or of the eight rows in flight, an N
    that leaves lanes (and whole wavefronts of the last column block) idle."""
    for M, K, N in ((1, 40, 128), (2, 257, 1152), (3, 1024, 640), (4, 4096, 2048), (1, 2050, 4096)):
        w = normal_weights((K, N), dtype, seed=bits + gs + M)
        x = activations((M, K), dtype, seed=K)
        _check_qmm(oracle, gpu, x, w, gs, bits, transpose=False)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits,gs", ((4, 64), (8, 128), (3, 32)))
def test_qvm_streaming_kernel_twice_for_5_to_8_rows(oracle, gpu, dtype, bits, gs):
    """transpose=False with 5..8 rows of x: the row-streaming kernel runs twice
    (four rows, then the rest) over the same planes of the workspace."""
    from mlx_amd import _lib

    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    K, N = 1088, 1152
    w = normal_weights((K, N), dtype, seed=bits + gs)
    quantized = oracle.quantize(w, gs, bits)
    for M in (5, 7, 8):
        x = activations((M, K), dtype, seed=M)
        _check_qmm(oracle, gpu, x, None, gs, bits, transpose=False, quantized=quantized)
        ws4 = _lib.load().mlxrocm_qmm_workspace_size(4, N, K, 1, 0, gs, bits, code, 0)
        ws = _lib.load().mlxrocm_qmm_workspace_size(M, N, K, 1, 0, gs, bits, code, 0)
        assert ws == ws4 and ws > 0, "the call is not sized like its four-row pass"


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits,gs", ((2, 32), (3, 64), (5, 32), (6, 128)))
def test_transpose_false_odd_widths_are_repacked(oracle, gpu, dtype, bits, gs):
    """transpose=False at 2/3/5/6 bits: the codes are repacked at 4 or 8 bits
    into the workspace first (same values, same scales) and the call goes on on
    the kernels of that width -- one row and four (streaming kernel, every
    element type), a ragged M and a long K on the matrix cores (16-bit types;
    float32 with more than eight rows stays on the scalar kernel)."""
    from mlx_amd import _lib

    code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
    lib = _lib.load()
    for M, K, N in ((1, 512, 384), (4, 1000, 1152), (70, 2048, 640), (9, 64, 4096)):
        w = normal_weights((K, N), dtype, seed=bits + gs + M)
        x = activations((M, K), dtype, seed=M)
        _check_qmm(oracle, gpu, x, w, gs, bits, transpose=False)
        ws = lib.mlxrocm_qmm_workspace_size(M, N, K, 1, 0, gs, bits, code, 0)
        repacked = K * N * (4 if bits < 4 else 8) // 8
        if M <= 8 or (dtype != torch.float32 and K % 64 == 0):
            assert ws >= repacked, "the call did not repack the codes"
        else:
            assert ws == 0


def test_transpose_false_odd_width_batched_weights(oracle, gpu):
    """Three problems with their own 3-bit [K, N] weights: every matrix is
    repacked, the batch stride of the repacked stack is the new one; the same
    with a strided (every other) selection of a larger stack."""
    dtype = torch.bfloat16
    L, M, K, N = 3, 20, 256, 320
    w = normal_weights((2 * L, K, N), dtype, seed=1)
    wq, s, b = oracle.quantize(w, 64, 3)
    x = activations((L, M, K), dtype, seed=2)
    for sel in (slice(0, L), slice(0, 2 * L, 2)):
        got = mlx_amd.quantized_matmul(
            x.to(gpu), wq.to(gpu)[sel], s.to(gpu)[sel], b.to(gpu)[sel], False, 64, 3).cpu()
        w_hat = exact_affine_weights(wq[sel], s[sel], b[sel], 64, 3)  # [L, K, N]
        exact = torch.einsum("lmk,lkn->lmn", x.double(), w_hat)
        assert float((got.double() - exact).abs().max()) <= exact_tolerance(dtype, K, x, w_hat, exact)


@pytest.mark.parametrize("dtype", DTYPES)
def test_transpose_false_odd_k(oracle, gpu, dtype):
    # K need not be a multiple of anything when w is [K, N]: rows of x then start
    # at unaligned addresses (7 rows: the generic kernel; 3 rows: the streaming one)
    for M, K, N in ((7, 257, 128), (3, 101, 96)):
        w = normal_weights((K, N), dtype, seed=K)
        x = activations((M, K), dtype, seed=M)
        _check_qmm(oracle, gpu, x, w, 32, 4, transpose=False)


def test_qvm_streaming_kernel_batched(oracle, gpu):
    dtype, gs, bits, L, M, K, N = torch.bfloat16, 64, 4, 3, 2, 1536, 256
    ws = [normal_weights((K, N), dtype, seed=20 + l) for l in range(L)]
    qs = [oracle.quantize(w, gs, bits) for w in ws]
    wq = torch.stack([q[0] for q in qs]).to(gpu)
    s = torch.stack([q[1] for q in qs]).to(gpu)
    b = torch.stack([q[2] for q in qs]).to(gpu)
    x = activations((L, M, K), dtype, seed=5)
    got = mlx_amd.quantized_matmul(x.to(gpu), wq, s, b, False, gs, bits).cpu()
    for l in range(L):
        ref = oracle.qmm(x[l], *qs[l], False, gs, bits)
        w_hat = exact_affine_weights(*qs[l], gs, bits)
        exact = x[l].double() @ w_hat
        tol = matmul_tolerance(dtype, K, x[l], w_hat) + float((ref.double() - exact).abs().max())
        assert float((got[l].double() - ref.double()).abs().max()) <= tol


def test_qmm_n_batched_and_full_size(oracle, gpu):
    # a batch of problems with one shared weight matrix, and the benchmark's
    # gate/up shape read the other way round, checked on sampled rows
    dtype = torch.bfloat16
    K, N = 128, 256
    w = normal_weights((K, N), dtype, seed=3)
    wq, s, b = oracle.quantize(w, 64, 4)
    x = activations((3, 40, K), dtype, seed=5)
    got = mlx_amd.quantized_matmul(x.to(gpu), wq.to(gpu), s.to(gpu), b.to(gpu), False, 64, 4).cpu()
    for l in range(3):
        ref = oracle.qmm(x[l], wq, s, b, False, 64, 4)
        tol = matmul_tolerance(dtype, K, x[l], exact_affine_weights(wq, s, b, 64, 4))
        assert float((got[l].double() - ref.double()).abs().max()) <= 2 * tol
    K, N, M = 4096, 14336, 512
    w = normal_weights((K, N), dtype, seed=0)
    x = activations((M, K), dtype, seed=0)
    _check_qmm(oracle, gpu, x, w, 64, 4, transpose=False, rows=_spread_rows(M))


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
@pytest.mark.parametrize("gs", ALL_GROUPS)
def test_qmv_matrix_instruction_gemv(oracle, gpu, dtype, gs):
    """4-bit decode with 2..4 rows of x (and 1 or 5..8 rows where K is long or the
    groups are 32 wide) runs on the 4x4x4 matrix-instruction GEMV: K of one slot,
    of a slot count that leaves the last wavefront's slots empty (1536, 14336),
    of every k-wave split, ragged N, both operand sets of x."""
    shapes = (
        (2, 67, 512), (3, 100, 1024), (4, 36, 1536), (2, 64, 2048), (4, 130, 4096),
        (3, 40, 8192), (1, 24, 14336), (4, 24, 14336), (8, 20, 14336), (7, 33, 16384),
    )
    if gs == 32:
        shapes += ((5, 67, 1024), (8, 40, 4096))
    for M, N, K in shapes:
        w = normal_weights((N, K), dtype, seed=gs + M + K)
        x = activations((M, K), dtype, seed=M + K)
        _check_qmm(oracle, gpu, x, w, gs, 4)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16))
def test_qmv_launch_plans(oracle, gpu, dtype):
    """Shapes that select each launch plan of the decode kernels: workgroups of
    four and of eight waves with the dot products on the matrix instruction
    (one row of x, 4-bit, groups of 64 / 128), four rows per wave for a long K
    that is not a whole number of chunks (11008, one and two rows of x; 8-bit at
    14336), and two row quads per wave on the 4x4x4 GEMV (8192 rows)."""
    cases = (
        (1, 6144, 4096, 4, 64), (1, 8192, 4096, 4, 128), (1, 4104, 2048, 4, 64),
        (1, 4096, 11008, 4, 64), (2, 4096, 11008, 4, 64), (1, 4096, 14336, 8, 128),
        (2, 4096, 8192, 8, 64), (3, 8192, 4096, 4, 64), (2, 8200, 4096, 4, 32),
        # 5..8 rows: the 4x4x4 GEMV with two operand sets (K = 8192; a single
        # round of workgroups) and the 32-row MFMA GEMV (a half-empty last round)
        (6, 4096, 8192, 4, 64), (8, 1024, 4096, 4, 128), (5, 6144, 4096, 4, 64),
    )
    for M, N, K, bits, gs in cases:
        w = normal_weights((N, K), dtype, seed=M + N + K)
        x = activations((M, K), dtype, seed=N + bits)
        _check_qmm(oracle, gpu, x, w, gs, bits)


def test_qmv_matrix_instruction_gemv_batched(oracle, gpu):
    # a batch of problems, each with its own weights: blockIdx.y walks the batch
    dtype, gs, L, M, N, K = torch.bfloat16, 64, 3, 3, 48, 1024
    ws = [normal_weights((N, K), dtype, seed=10 + l) for l in range(L)]
    qs = [oracle.quantize(w, gs, 4) for w in ws]
    wq = torch.stack([q[0] for q in qs]).to(gpu)
    s = torch.stack([q[1] for q in qs]).to(gpu)
    b = torch.stack([q[2] for q in qs]).to(gpu)
    x = activations((L, M, K), dtype, seed=4)
    got = mlx_amd.quantized_matmul(x.to(gpu), wq, s, b, True, gs, 4).cpu()
    for l in range(L):
        ref = oracle.qmm(x[l], *qs[l], True, gs, 4)
        w_hat = exact_affine_weights(*qs[l], gs, 4)
        exact = x[l].double() @ w_hat.T
        tol = matmul_tolerance(dtype, K, x[l], w_hat) + float((ref.double() - exact).abs().max())
        assert float((got[l].double() - ref.double()).abs().max()) <= tol


@pytest.mark.parametrize("bits", ALL_BITS)
def test_qmv_float32_streaming(oracle, gpu, bits):
    """One row of float32 x runs on the fp32 streaming GEMV: K of a partial chunk,
    of several k-waves with an unused tail (11008), ragged N, every group size."""
    for gs, N, K in ((32, 67, 2080), (64, 40, 11008), (128, 130, 4096), (32, 9, 16384)):
        w = normal_weights((N, K), torch.float32, seed=bits + gs)
        x = activations((1, K), torch.float32, seed=K)
        _check_qmm(oracle, gpu, x, w, gs, bits)


@pytest.mark.parametrize("bits", ALL_BITS)
def test_qmv_float32_few_rows(oracle, gpu, bits):
    """2..4 rows of float32 x in one launch of the fp32 streaming GEMV (K up to
    8192), and the shapes beyond it (5..16 rows, K > 8192 with two rows, a batch
    of problems with five rows) on the generic kernels; 9..16 rows run them
    twice (eight rows, then the rest) and need no workspace, 17 rows take the
    matrix path."""
    cases = ((64, 2, 100, 512), (32, 3, 70, 4096), (128, 4, 33, 8192), (64, 7, 64, 2048),
             (64, 16, 48, 4096), (32, 13, 40, 6144), (64, 2, 24, 10240))
    for gs, M, N, K in cases:
        w = normal_weights((N, K), torch.float32, seed=bits + gs + M)
        x = activations((M, K), torch.float32, seed=K + M)
        _check_qmm(oracle, gpu, x, w, gs, bits)
    from mlx_amd import _lib
    assert _lib.load().mlxrocm_qmm_workspace_size(13, 4096, 4096, 1, 0, 64, bits, 0, 1) == 0
    assert _lib.load().mlxrocm_qmm_workspace_size(17, 4096, 4096, 1, 0, 64, bits, 0, 1) > 0
    # batched, five rows
    L, M, N, K, gs = 2, 5, 40, 1024, 64
    ws = [normal_weights((N, K), torch.float32, seed=30 + l) for l in range(L)]
    qs = [oracle.quantize(w, gs, bits) for w in ws]
    wq = torch.stack([q[0] for q in qs]).to(gpu)
    s = torch.stack([q[1] for q in qs]).to(gpu)
    b = torch.stack([q[2] for q in qs]).to(gpu)
    x = activations((L, M, K), torch.float32, seed=6)
    got = mlx_amd.quantized_matmul(x.to(gpu), wq, s, b, True, gs, bits).cpu()
    for l in range(L):
        ref = oracle.qmm(x[l], *qs[l], True, gs, bits)
        w_hat = exact_affine_weights(*qs[l], gs, bits)
        tol = matmul_tolerance(torch.float32, K, x[l], w_hat)
        assert float((got[l].double() - ref.double()).abs().max()) <= tol


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("bits,gs", ((4, 64), (8, 128), (3, 32)))
def test_quantized_swiglu_matches_the_unfused_chain(oracle, gpu, dtype, bits, gs):
    """silu(gate(x)) * up(x) in one call against the same chain built from the
    oracle's two products, with every intermediate rounded to the element type as
    `x * sigmoid(x)` and the multiply round it; 1..8 rows of x, ragged N."""
    # one row at 4 bits runs with the gate inside the GEMV (K of a partial chunk,
    # of exactly one wave's chunks, a grid of four- and of eight-wave workgroups)
    for M, N, K in ((1, 200, 512), (1, 1000, 4096), (1, 6144, 4096), (2, 96, 4096), (4, 64, 1024),
                    (8, 130, 2048), (1, 40, 8192), (1, 48, 14336)):
        wg = normal_weights((N, K), dtype, seed=bits + M)
        wu = normal_weights((N, K), dtype, seed=bits + M + 100)
        x = activations((M, K), dtype, seed=K + M)
        qg = oracle.quantize(wg, gs, bits)
        qu = oracle.quantize(wu, gs, bits)
        got = mlx_amd.quantized_swiglu(
            x.to(gpu), tuple(t.to(gpu) for t in qg), tuple(t.to(gpu) for t in qu), gs, bits
        ).cpu()
        assert got.shape == (M, N) and got.dtype == dtype
        # the chain in fp64 from the exact products, and its unfused form on the GPU
        eg = x.double() @ exact_affine_weights(*qg, gs, bits).T
        eu = x.double() @ exact_affine_weights(*qu, gs, bits).T
        exact = eg * torch.sigmoid(eg) * eu
        g = mlx_amd.quantized_matmul(x.to(gpu), *(t.to(gpu) for t in qg), True, gs, bits)
        u = mlx_amd.quantized_matmul(x.to(gpu), *(t.to(gpu) for t in qu), True, gs, bits)
        unfused = ((g * torch.sigmoid(g)) * u).cpu()
        eps = {torch.float32: 2.0 ** -22, torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
        scale = float(unfused.double().abs().max()) + 1e-30
        # same products, same roundings: a few units in the last place of T
        assert float((got.double() - unfused.double()).abs().max()) <= 4 * eps * scale
        # and within the matmul tolerance (propagated through the gate) of fp64
        w_hat = exact_affine_weights(*qg, gs, bits)
        tol = matmul_tolerance(dtype, K, x, w_hat)
        bound = tol * (float(eu.abs().max()) + 1.1 * float(eg.abs().max()) + tol) + 8 * eps * scale
        assert float((got.double() - exact).abs().max()) <= bound


def test_quantized_swiglu_rejects_prefill_and_mismatched_weights(oracle, gpu):
    w = normal_weights((64, 256), torch.bfloat16, seed=1)
    q = tuple(t.to(gpu) for t in oracle.quantize(w, 64, 4))
    x = activations((9, 256), torch.bfloat16).to(gpu)
    with pytest.raises(RuntimeError, match="M <= 8"):
        mlx_amd.quantized_swiglu(x, q, q, 64, 4)
    w2 = normal_weights((32, 256), torch.bfloat16, seed=2)
    q2 = tuple(t.to(gpu) for t in oracle.quantize(w2, 64, 4))
    with pytest.raises(ValueError, match="one shape"):
        mlx_amd.quantized_swiglu(x[:1], q, q2, 64, 4)


def test_batched_x_with_one_weight_folds_into_rows(oracle, gpu):
    """x [B, 1, K] against a 2-D weight (the decode call of nn.QuantizedLinear)
    runs as one M = B product, and gives what B separate products give."""
    gs, bits, dtype = 64, 4, torch.bfloat16
    w = normal_weights((4096, 4096), dtype, seed=2)
    q = oracle.quantize(w, gs, bits)
    x = activations((8, 1, 4096), dtype, seed=9)
    gq = [t.to(gpu) for t in q]
    got = mlx_amd.quantized_matmul(x.to(gpu), *gq, True, gs, bits)
    assert got.shape == (8, 1, 4096)
    flat = _check_qmm(oracle, gpu, x.reshape(8, 4096), None, gs, bits, quantized=q)
    assert torch.equal(got.cpu().reshape(8, 4096).view(torch.int16), flat.view(torch.int16))
    # more batch entries than a grid dimension holds
    xs = activations((70000, 1, 64), torch.float32, seed=1)
    w2 = normal_weights((8, 64), torch.float32, seed=3)
    q2 = oracle.quantize(w2, 64, 4)
    got = mlx_amd.quantized_matmul(xs.to(gpu), *(t.to(gpu) for t in q2), True, 64, 4).cpu()
    ref = oracle.qmm(xs.reshape(-1, 64), *q2, True, 64, 4).reshape(70000, 1, 8)
    assert float((got - ref).abs().max()) < 1e-4


def test_workspace_contract(oracle, gpu):
    """mlxrocm_qmm takes its scratch from the caller: the size query names it,
    a missing or short workspace is an invalid argument, a misaligned one too."""
    from mlx_amd import _lib
    lib = _lib.load()
    M, N, K = 2048, 4096, 4096
    need = lib.mlxrocm_qmm_workspace_size(M, N, K, 1, 0, 64, 4, 2, 1)
    assert need >= 4 * N * K // 64
    assert lib.mlxrocm_qmm_workspace_size(1, N, K, 1, 0, 64, 4, 2, 1) == 0
    assert lib.mlxrocm_qmm_workspace_size(M, N, K, 1, 0, 64, 7, 2, 1) == 0  # invalid bits
    w = normal_weights((N, K), torch.bfloat16).to(gpu)
    wq, s, b = mlx_amd.quantize(w, 64, 4)
    x = activations((M, K), torch.bfloat16).to(gpu)
    out = torch.empty((M, N), dtype=torch.bfloat16, device=gpu)
    ws = torch.empty(need + 256, dtype=torch.uint8, device=gpu)
    stream = torch.cuda.current_stream().cuda_stream

    def call(ptr, nbytes):
        return lib.mlxrocm_qmm(x.data_ptr(), wq.data_ptr(), s.data_ptr(), b.data_ptr(),
                               out.data_ptr(), M, N, K, 1, M * K, 0, 0, 64, 4, 2, 1,
                               ptr, nbytes, stream)

    assert call(None, 0) == _lib.INVALID_ARGUMENT and "workspace" in _lib.last_error()
    assert call(ws.data_ptr(), need - 1) == _lib.INVALID_ARGUMENT
    assert call(ws.data_ptr() + 16, need) == _lib.INVALID_ARGUMENT
    assert "aligned" in _lib.last_error()
    assert call(ws.data_ptr(), need) == 0
    torch.cuda.synchronize()


def test_prefill_call_replays_from_a_hip_graph(oracle, gpu):
    """An M = 2048 mlxrocm_qmm (transposed scales in the workspace) captured in a
    HIP graph: nothing in the call allocates, locks or synchronizes.  Replayed
    several times with eager work and synchronizations in between, every replay
    equals the eager result, also after x has changed."""
    from mlx_amd import _lib
    lib = _lib.load()
    M, N, K = 2048, 4096, 4096
    need = lib.mlxrocm_qmm_workspace_size(M, N, K, 1, 0, 64, 4, 2, 1)
    w = normal_weights((N, K), torch.bfloat16).to(gpu)
    wq, s, b = mlx_amd.quantize(w, 64, 4)
    x = activations((M, K), torch.bfloat16).to(gpu)
    out = torch.zeros((M, N), dtype=torch.bfloat16, device=gpu)
    ws = torch.empty(need, dtype=torch.uint8, device=gpu)

    def call(stream):
        _lib.check(lib.mlxrocm_qmm(x.data_ptr(), wq.data_ptr(), s.data_ptr(), b.data_ptr(),
                                   out.data_ptr(), M, N, K, 1, M * K, 0, 0, 64, 4, 2, 1,
                                   ws.data_ptr(), need, stream))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(side.cuda_stream)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        call(torch.cuda.current_stream().cuda_stream)
    for i in range(4):
        x.copy_(activations((M, K), torch.bfloat16, seed=100 + i).to(gpu))
        eager = mlx_amd.quantized_matmul(x, wq, s, b, True, 64, 4)
        out.fill_(-1.0)  # a fill kernel, not a memset node
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out.view(torch.int16), eager.view(torch.int16)), f"replay {i}"


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
def test_qmm_prepacked_scale_image(gpu, dtype):
    """A prefill call that is handed the transposed (scale, bias) pair image of its
    weight skips the pre-pass and returns the bits of the plain call; shapes that
    read no image ignore it; an image of another weight shape is refused."""
    N, K, gs = 1024, 2048, 64
    w = normal_weights((N, K), dtype, std=0.05).to(gpu)
    wq, s, b = mlx_amd.quantize(w, gs, 4)
    image = mlx_amd.quantized_matmul_sb_image(s, b, gs)
    assert image.numel() == 2 * N * (K // gs) and image.dtype == dtype
    # the image is [K / gs][N] pairs: a row's scale, then its bias
    pairs = image.reshape(K // gs, N, 2)
    assert torch.equal(pairs[..., 0], s.T.contiguous())
    assert torch.equal(pairs[..., 1], b.T.contiguous())
    for M in (1, 8, 600, 2048):
        x = activations((M, K), dtype).to(gpu)
        plain = mlx_amd.quantized_matmul(x, wq, s, b, True, gs, 4)
        packed = mlx_amd.quantized_matmul(x, wq, s, b, True, gs, 4, sb_image=image)
        assert torch.equal(plain, packed), M
    with pytest.raises(ValueError):
        mlx_amd.quantized_matmul(x, wq, s, b, True, gs, 4, sb_image=image[:-8])
    # the layer keeps the image and drops it when the weights are replaced
    lin = mlx_amd.nn.QuantizedLinear(K, N, bias=False, device=gpu, dtype=dtype)
    x = activations((640, K), dtype).to(gpu)
    before = lin(x)
    assert torch.equal(lin.prepack()(x), before)
    lin._set_quantized(w)
    assert torch.equal(lin(x), mlx_amd.quantized_matmul(x, wq, s, b, True, gs, 4))


@pytest.mark.parametrize("dtype", (torch.float32, torch.bfloat16), ids=str)
def test_vjp_with_respect_to_x(gpu, dtype):
    """python/tests/test_quantized.py:480-508 (test_qmm_vjp): the gradient with
    respect to x is the cotangent times the same quantized matrix with transpose
    flipped; here under torch autograd, through the operator and the layer."""
    g = torch.Generator().manual_seed(0)
    M, N, K = 64, 1024, 512
    c = torch.ones((2, M, N), dtype=dtype, device=gpu)
    for transposed in (True, False):
        w = torch.randn((N, K) if transposed else (K, N), generator=g).to(dtype).to(gpu)
        wq, scales, biases = mlx_amd.quantize(w, 64, 8)
        x = torch.randn((2, M, K), generator=g).to(dtype).to(gpu).requires_grad_(True)
        y = mlx_amd.quantized_matmul(x, wq, scales, biases, transposed, 64, 8)
        assert y.requires_grad
        y.backward(c)
        want = mlx_amd.quantized_matmul(c, wq, scales, biases, not transposed, 64, 8)
        assert x.grad.shape == x.shape and x.grad.dtype == dtype
        assert torch.equal(x.grad, want)
    # the floating-point modes take the same route
    wq, scales = mlx_amd.quantize(torch.randn((N, K), generator=g).to(dtype).to(gpu), mode="mxfp4")
    x = torch.randn((3, K), generator=g).to(dtype).to(gpu).requires_grad_(True)
    mlx_amd.quantized_matmul(x, wq, scales, mode="mxfp4").sum().backward()
    want = mlx_amd.quantized_matmul(torch.ones((3, N), dtype=dtype, device=gpu), wq, scales,
                                    transpose=False, mode="mxfp4")
    assert torch.equal(x.grad, want)
    # a frozen quantized layer between two trainable ones passes gradients through
    lin = mlx_amd.nn.QuantizedLinear.from_linear(
        torch.nn.Linear(K, N, bias=True).to(gpu).to(dtype), group_size=64, bits=4)
    x = torch.randn((5, K), generator=g).to(dtype).to(gpu).requires_grad_(True)
    lin(x).sum().backward()
    assert x.grad is not None and float(x.grad.abs().max()) > 0
