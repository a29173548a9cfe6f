"""GPU parity of the few-row kernel that streams packed 4-bit rows through LDS
with x resident per K range (5..32 rows of a plain call, small expert groups of
a gather): against the CPU oracle and the fp64 product of the exact weights."""
import pytest
import torch

import mlx_amd
from mlx_amd import _lib
from tests.test_gpu_qmm import _check_qmm
from tests.util import (
    activations, exact_affine_weights, exact_tolerance, matmul_tolerance, normal_weights,
)

pytestmark = pytest.mark.gpu

CODE = {torch.float16: 1, torch.bfloat16: 2}


def _planes_bytes(M, N, K, L=1):
    return -(-K // 1024) * L * M * N * 4 if K > 1024 else 0


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
@pytest.mark.parametrize("gs", (32, 64, 128))
@pytest.mark.parametrize("M", (5, 9, 16, 17, 32))
def test_slab_rows_and_groups(oracle, gpu, dtype, gs, M):
    """[8192, 4096]: four K ranges x 32 slabs.  32-wide groups have no two-tile
    form and stay on the older kernels from 17 rows on (still checked)."""
    N, K = 8192, 4096
    w = normal_weights((N, K), dtype, std=0.05)
    x = activations((M, K), dtype)
    _check_qmm(oracle, gpu, x, w, gs, 4, rows=torch.tensor([0, M - 1]))
    if M >= 9 and (gs != 32 or M <= 16):  # (5..8 rows: only where the 4x4x4 kernel is not chosen)
        ws = _lib.load().mlxrocm_qmm_workspace_size(M, N, K, 1, 0, gs, 4, CODE[dtype], 1)
        assert ws == _planes_bytes(M, N, K), "the shape did not take the slab kernel"


@pytest.mark.parametrize("N,K", ((8000, 4096), (32772, 1024), (4096, 14336), (32000, 2048)))
def test_slab_ragged_and_single_range(oracle, gpu, N, K):
    """N that is no multiple of the 256-row slab (the last slab's rows are
    clamped and never written), a single K range (written directly, no planes),
    a long K (14 ranges) and a tall matrix (more workgroups than the kernel
    with all of K in LDS is used for, so 5..8 rows come here as well)."""
    dtype = torch.bfloat16
    w = normal_weights((N, K), dtype, std=0.05)
    for M in (6, 9, 24):
        x = activations((M, K), dtype, seed=M)
        _check_qmm(oracle, gpu, x, w, 64, 4, rows=torch.tensor([M - 1]))
        ws = _lib.load().mlxrocm_qmm_workspace_size(M, N, K, 1, 0, 64, 4, 2, 1)
        if M >= 9 or K >= 8192 or N >= 32000:  # (5..8 rows: a long K or many rows of W)
            assert ws == _planes_bytes(M, N, K)


@pytest.mark.parametrize("dtype,gs", ((torch.bfloat16, 64), (torch.float16, 128), (torch.bfloat16, 32)))
@pytest.mark.parametrize("N,K", ((16384, 1536), (8200, 3584), (4096, 11008)))
def test_slab_short_last_range(oracle, gpu, dtype, gs, N, K):
    """K a multiple of 256 but not of 1024: the last K range has two or three
    steps instead of four (1536 = 4 + 2, 3584 = 4 + 4 + 4 + 2, 11008 = 10 x 4 + 3);
    its scales are fetched from a window that ends with the row, x beyond K
    stays zero in LDS."""
    w = normal_weights((N, K), dtype, std=0.05)
    quantized = oracle.quantize(w, gs, 4)
    for M in (9, 16):
        x = activations((M, K), dtype, seed=M)
        _check_qmm(oracle, gpu, x, None, gs, 4, rows=torch.tensor([M - 1]), quantized=quantized)
        ws = _lib.load().mlxrocm_qmm_workspace_size(M, N, K, 1, 0, gs, 4, CODE[dtype], 1)
        assert ws == _planes_bytes(M, N, K), "the shape did not take the slab kernel"


@pytest.mark.parametrize("dtype,gs", ((torch.bfloat16, 64), (torch.float16, 128)))
def test_slab_two_passes_for_33_to_64_rows(oracle, gpu, dtype, gs):
    """33..64 rows run the kernel twice (32 rows, then the rest) over the same
    planes; 65 rows and 32-wide groups stay on the tile GEMM."""
    N, K = 8200, 3584
    w = normal_weights((N, K), dtype, std=0.05)
    quantized = oracle.quantize(w, gs, 4)
    lib = _lib.load()
    for M in (33, 47, 64):
        x = activations((M, K), dtype, seed=M)
        _check_qmm(oracle, gpu, x, None, gs, 4, rows=torch.tensor([0, 31, 32, M - 1]),
                   quantized=quantized)
        ws = lib.mlxrocm_qmm_workspace_size(M, N, K, 1, 0, gs, 4, CODE[dtype], 1)
        assert ws == _planes_bytes(32, N, K), "the shape did not take the slab kernel twice"
    assert lib.mlxrocm_qmm_workspace_size(65, N, K, 1, 0, gs, 4, CODE[dtype], 1) != _planes_bytes(32, N, K)
    assert lib.mlxrocm_qmm_workspace_size(40, N, K, 1, 0, 32, 4, CODE[dtype], 1) != _planes_bytes(32, N, K)


def test_slab_below_half_occupancy_for_large_weights(oracle, gpu):
    """Fewer units than half the compute units, but weights large enough that
    the kernels it replaces would be slower than its floor: 17..32 rows at
    6144 x 4096 (96 units) and 2048 x 8192 (64 units, long K) take it; 4096 x
    4096 (64 units) and 12 rows at 6144 x 4096 do not."""
    lib = _lib.load()
    dtype = torch.bfloat16
    for (N, K) in ((6144, 4096), (2048, 8192)):
        w = normal_weights((N, K), dtype, std=0.05)
        x = activations((24, K), dtype)
        _check_qmm(oracle, gpu, x, w, 64, 4, rows=torch.tensor([0, 23]))
        assert lib.mlxrocm_qmm_workspace_size(24, N, K, 1, 0, 64, 4, 2, 1) == _planes_bytes(24, N, K)
    assert lib.mlxrocm_qmm_workspace_size(24, 4096, 4096, 1, 0, 64, 4, 2, 1) == 0
    assert lib.mlxrocm_qmm_workspace_size(12, 6144, 4096, 1, 0, 64, 4, 2, 1) == 0


def test_slab_one_step_last_range_is_refused(gpu):
    """A last range of a single step (K = 1280, 5376 ...) is not built: such
    shapes stay on the other kernels and ask for no planes."""
    for K in (1280, 5376):
        assert _lib.load().mlxrocm_qmm_workspace_size(16, 16384, K, 1, 0, 64, 4, 2, 1) == 0


def test_slab_batched_weights(oracle, gpu):
    """Eight problems of [4096, 1024] with their own weights: the unit list runs
    over problems, every workgroup restages x when it crosses into the next one."""
    L, M, N, K = 8, 9, 4096, 1024
    dtype = torch.float16
    w = normal_weights((L, N, K), dtype, std=0.05)
    wq, s, b = oracle.quantize(w, 64, 4)
    x = activations((L, M, K), dtype)
    got = mlx_amd.quantized_matmul(x.to(gpu), wq.to(gpu), s.to(gpu), b.to(gpu), True, 64, 4).cpu()
    ref = oracle.qmm_batched(x, wq, s, b, True, 64, 4)
    w_hat = exact_affine_weights(wq, s, b, 64, 4)
    exact = torch.einsum("lmk,lnk->lmn", x.double(), w_hat)
    assert float((got.double() - exact).abs().max()) <= exact_tolerance(dtype, K, x, w_hat, exact)
    assert float((got.double() - ref.double()).abs().max()) <= matmul_tolerance(dtype, K, x, w_hat)


@pytest.mark.parametrize("K", (2048, 1792))
@pytest.mark.parametrize("E,T", ((8, 6), (8, 64), (16, 320)))
@pytest.mark.parametrize("dtype,gs", ((torch.bfloat16, 64), (torch.float16, 64), (torch.bfloat16, 128),
                                      (torch.bfloat16, 32)))
def test_slab_grouped_gather(oracle, gpu, dtype, gs, E, T, K):
    """T tokens x top-2 of E experts of [520, K] (two K ranges, the second one
    short at K = 1792; a ragged slab).  6 tokens: grouping pays from 8 pairs on over large experts, these small
    ones are multiplied pair by pair; 64 tokens over 8
    experts: the kernel groups the pairs itself, experts end up with fewer and
    with more than 16 rows; 320 tokens over 16 experts: the planning kernel runs
    first, experts have more than one tile.  One pair names
    an expert that does not exist (zero row), and the run on expert-sorted pairs
    reproduces the unsorted one bit for bit."""
    N = 520
    w = normal_weights((E, N, K), dtype, std=0.5)
    wq, s, b = oracle.quantize(w, gs, 4)
    x = activations((T, 1, 1, K), dtype)
    g = torch.Generator().manual_seed(3)
    idx = torch.randint(0, E, (T, 2), generator=g)
    idx[:12, 0] = 5  # one expert with well over 16 rows
    counts = torch.bincount(idx.reshape(-1), minlength=E)
    if T == 64:
        assert int(counts.max()) > 16 and int(counts.min()) <= 16
    elif T == 320:
        assert int(counts.max()) > 32
    gx, gwq, gsc, gb, gidx = (t.to(gpu) for t in (x, wq, s, b, idx))
    ws = _lib.load().mlxrocm_gather_qmm_workspace_size(1, N, K, 2 * T, E, gs, 4, CODE[dtype], 1, 0)
    if T == 6:
        # 12 pairs: grouped only over experts of 4 MB and more (one GEMV over a
        # smaller one takes about a microsecond); these stay on one GEMV per pair
        assert ws == 0
        big = _lib.load().mlxrocm_gather_qmm_workspace_size(1, 4096, 4096, 12, E, gs, 4, CODE[dtype], 1, 0)
        assert big >= 4 * 12 * 4096 * 4, "12 pairs over large experts are not grouped"
    elif gs != 32 or 2 * T <= 512:  # (32-wide groups: only where the kernel groups the pairs itself)
        assert ws >= -(-K // 1024) * 2 * T * N * 4, "the call did not take the slab kernel"
    got = mlx_amd.gather_qmm(gx, gwq, gsc, gb, rhs_indices=gidx, transpose=True,
                             group_size=gs, bits=4)
    assert got.shape == (T, 2, 1, N)
    ref = oracle.gather_qmm(
        x.reshape(T, 1, K), wq, s, b,
        torch.arange(T).repeat_interleave(2), idx.reshape(-1), True, gs, 4,
    ).reshape(T, 2, 1, N)
    w_hat = exact_affine_weights(wq, s, b, gs, 4)
    exact = torch.einsum("tk,tjnk->tjn", x.reshape(T, K).double(), w_hat[idx]).reshape(T, 2, 1, N)
    assert float((got.cpu().double() - exact).abs().max()) <= exact_tolerance(
        dtype, K, x, w_hat, exact)
    # (the CPU reference accumulates 16-bit types in the element type,
    # cpu/quantized.cpp:177-206: its own distance from the exact product is
    # discounted; the fp64 check above is the strict one)
    tol_ref = matmul_tolerance(dtype, K, x, w_hat) + float((ref.double() - exact).abs().max())
    assert float((got.cpu().double() - ref.double()).abs().max()) <= tol_ref
    # sorted by expert: same rows, bit for bit
    flat = gidx.reshape(-1)
    order = torch.argsort(flat, stable=True)
    xs = gx.reshape(T, 1, K)[order // 2]
    ys = mlx_amd.gather_qmm(xs, gwq, gsc, gb, rhs_indices=flat[order].contiguous(),
                            transpose=True, group_size=gs, bits=4, sorted_indices=True)
    assert torch.equal(ys[torch.argsort(order)].reshape(T, 2, 1, N), got)
    # an expert index out of range: that row is zero, the others unchanged
    bad = gidx.clone()
    bad[min(7, T - 1), 1] = E + 3
    got_bad = mlx_amd.gather_qmm(gx, gwq, gsc, gb, rhs_indices=bad, transpose=True,
                                 group_size=gs, bits=4)
    torch.cuda.synchronize()
    assert bool((got_bad[min(7, T - 1), 1] == 0).all())
    keep = torch.ones((T, 2), dtype=torch.bool, device=gpu)
    keep[min(7, T - 1), 1] = False
    assert torch.equal(got_bad[keep], got[keep])


@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
@pytest.mark.parametrize("gs,K", ((64, 4096), (64, 2048), (32, 1024), (128, 4096)))
def test_rows8_all_of_k_resident(oracle, gpu, dtype, gs, K):
    """5..8 rows of x (up to 16 at K <= 2048) kept in LDS for the whole of K, the
    K steps split over the wavefronts of a tile; N with a ragged last workgroup."""
    N = 8200
    w = normal_weights((N, K), dtype, std=0.05)
    quantized = oracle.quantize(w, gs, 4)
    rows = (5, 8) + ((12, 16) if K <= 2048 else ())  # M * K * 2 bytes <= 64 KiB
    for M in rows:
        x = activations((M, K), dtype, seed=M)
        _check_qmm(oracle, gpu, x, None, gs, 4, rows=torch.tensor([M - 1]), quantized=quantized)
        ws = _lib.load().mlxrocm_qmm_workspace_size(M, N, K, 1, 0, gs, 4, CODE[dtype], 1)
        assert ws == 0, "the shape did not take the kernel without K ranges"


def test_rows8_batched(oracle, gpu):
    L, M, N, K = 3, 7, 4096, 4096
    dtype = torch.bfloat16
    w = normal_weights((L, N, K), dtype, std=0.05)
    wq, s, b = oracle.quantize(w, 64, 4)
    x = activations((L, M, K), dtype)
    got = mlx_amd.quantized_matmul(x.to(gpu), wq.to(gpu), s.to(gpu), b.to(gpu), True, 64, 4).cpu()
    w_hat = exact_affine_weights(wq, s, b, 64, 4)
    exact = torch.einsum("lmk,lnk->lmn", x.double(), w_hat)
    assert float((got.double() - exact).abs().max()) <= exact_tolerance(dtype, K, x, w_hat, exact)
