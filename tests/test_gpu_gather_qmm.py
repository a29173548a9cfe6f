"""GPU parity of gather_qmm (expert-routed quantized matmul)."""
import pytest
import torch

import mlx_amd
from tests.util import (
    activations, exact_affine_weights, exact_affine_weights_on, exact_tolerance,
    exact_tolerance_from, matmul_tolerance, normal_weights,
)

pytestmark = pytest.mark.gpu


def _to(gpu, *ts):
    return [None if t is None else t.to(gpu) for t in ts]


def _gather_case(oracle, gpu, M, N, K, batch_A, batch_B, lhs, rhs, transpose,
                 gs=64, bits=4, dtype=torch.float32):
    x = activations(batch_A + (M, K), dtype)
    w = normal_weights(batch_B + ((N, K) if transpose else (K, N)), dtype, std=1.0)
    wq, s, b = oracle.quantize(w, gs, bits)
    lhs_t = None if lhs is None else torch.tensor(lhs, dtype=torch.int64)
    rhs_t = None if rhs is None else torch.tensor(rhs, dtype=torch.int64)
    gx, gwq, gs_, gb, glhs, grhs = _to(gpu, x, wq, s, b, lhs_t, rhs_t)
    got = mlx_amd.gather_qmm(gx, gwq, gs_, gb, glhs, grhs, transpose, gs, bits).cpu()
    # expected: per-pair oracle qmm on broadcast indices (cpu/quantized.cpp:727-746)
    nA = 1
    for d in batch_A:
        nA *= d
    nB = 1
    for d in batch_B:
        nB *= d
    li = torch.arange(nA).reshape(batch_A) if lhs_t is None else lhs_t
    ri = torch.arange(nB).reshape(batch_B) if rhs_t is None else rhs_t
    li, ri = torch.broadcast_tensors(li, ri)
    ref = oracle.gather_qmm(
        x.reshape(-1, M, K), wq.reshape(-1, *wq.shape[-2:]),
        s.reshape(-1, *s.shape[-2:]), b.reshape(-1, *b.shape[-2:]),
        li, ri, transpose, gs, bits,
    ).reshape(tuple(li.shape) + (M, N))
    assert got.shape == ref.shape
    w_hat = exact_affine_weights(wq, s, b, gs, bits)
    tol = matmul_tolerance(dtype, K, x, w_hat)
    assert float((got.double() - ref.double()).abs().max()) <= tol


CASES = (
    dict(batch_A=(1,), lhs=(0,), batch_B=(3,), rhs=(2, 1)),
    dict(batch_A=(1,), lhs=None, batch_B=(3,), rhs=(2, 1)),
    dict(batch_A=(2,), lhs=None, batch_B=(3,), rhs=(2, 1)),
    dict(batch_A=(3,), lhs=(0, 2), batch_B=(1,), rhs=(0,)),
    dict(batch_A=(5,), lhs=(0, 2), batch_B=(3,), rhs=(2, 1)),
    dict(batch_A=(4, 2), lhs=((7, 6), (5, 4), (1, 2)), batch_B=(4, 1),
         rhs=((2,), (0,), (1,))),
)


@pytest.mark.parametrize("case", CASES)
def test_gather_qmm_index_broadcasting(oracle, gpu, case):
    # python/tests/test_quantized.py:1127-1266
    for M, N, K, transpose in (
        (1, 32, 128, True), (32, 32, 256, True), (1, 32, 512, True),
        (32, 256, 32, False), (1, 512, 32, False),
    ):
        _gather_case(oracle, gpu, M, N, K, transpose=transpose, **case)


@pytest.mark.parametrize("dtype", (torch.float32, torch.float16, torch.bfloat16))
def test_gather_qmm_sorted_moe(oracle, gpu, dtype):
    """L tokens x top-2 of 4 experts, sorted vs unsorted
    (python/tests/test_quantized.py:1451-1565)."""
    E, N, K, T = 4, 96, 128, 40
    gs, bits = 64, 4
    w = normal_weights((E, N, K), dtype, std=0.5)
    wq, s, b = oracle.quantize(w, gs, bits)
    x = activations((T, 1, 1, K), dtype)
    g = torch.Generator().manual_seed(0)
    idx = torch.randint(0, E, (T, 2), generator=g)
    gx, gwq, gsc, gb, gidx = _to(gpu, x, wq, s, b, idx)
    unsorted = mlx_amd.gather_qmm(gx, gwq, gsc, gb, rhs_indices=gidx,
                                  transpose=True, group_size=gs, bits=bits)
    assert unsorted.shape == (T, 2, 1, N)
    # sorted: gather tokens by expert, run with sorted_indices, un-permute
    flat = gidx.reshape(-1)
    order = torch.argsort(flat, stable=True)
    inv = torch.argsort(order)
    xs = gx.reshape(T, 1, K)[order // 2]
    ys = mlx_amd.gather_qmm(xs, gwq, gsc, gb, rhs_indices=flat[order], transpose=True,
                            group_size=gs, bits=bits, sorted_indices=True)
    assert ys.shape == (2 * T, 1, N)
    resorted = ys[inv].reshape(T, 2, 1, N)
    ref = oracle.gather_qmm(
        x.reshape(T, 1, K), wq, s, b,
        torch.arange(T).repeat_interleave(2), idx.reshape(-1), True, gs, bits,
    ).reshape(T, 2, 1, N)
    w_hat = exact_affine_weights(wq, s, b, gs, bits)
    tol = matmul_tolerance(dtype, K, x, w_hat)
    exact = torch.einsum(
        "tk,tjnk->tjn", x.reshape(T, K).double(), w_hat[idx]
    ).reshape(T, 2, 1, N)
    assert float((unsorted.cpu().double() - exact).abs().max()) <= exact_tolerance(
        dtype, K, x, w_hat, exact)
    assert float((unsorted.cpu().double() - ref.double()).abs().max()) <= tol
    assert float((resorted.cpu().double() - ref.double()).abs().max()) <= tol


def test_gather_qmm_sliced_expert_stack(oracle, gpu):
    """Non-contiguous expert stacks need no copy
    (python/tests/test_quantized.py:1567-1593)."""
    E, N, K = 6, 64, 128
    w = normal_weights((E, N, K), torch.float32, std=0.5)
    wq, s, b = oracle.quantize(w, 64, 4)
    x = activations((8, 1, K), torch.float32)
    idx = torch.tensor([0, 1, 2, 0, 1, 2, 2, 1])
    gx, gwq, gs_, gb, gidx = _to(gpu, x, wq, s, b, idx)
    got = mlx_amd.gather_qmm(gx, gwq[::2], gs_[::2], gb[::2], rhs_indices=gidx)
    ref = oracle.gather_qmm(x, wq[::2].contiguous(), s[::2].contiguous(),
                            b[::2].contiguous(), torch.arange(8), idx, True, 64, 4)
    assert float((got.cpu() - ref).abs().max()) < 1e-4


def test_gather_qmm_out_of_range_index_is_contained(gpu):
    w = normal_weights((2, 32, 64), torch.float32).to(gpu)
    wq, s, b = mlx_amd.quantize(w)
    x = activations((1, 1, 64), torch.float32).to(gpu)
    idx = torch.tensor([1, 7], device=gpu)  # 7 is not an expert
    out = mlx_amd.gather_qmm(x, wq, s, b, rhs_indices=idx)
    torch.cuda.synchronize()
    assert bool((out[1] == 0).all()) and bool(out[0].abs().sum() > 0)


def _grouped_ws_bytes(M, N, K, n_idx, E, gs, bits, dtype_code=2):
    from mlx_amd import _lib
    return _lib.load().mlxrocm_gather_qmm_workspace_size(
        M, N, K, n_idx, E, gs, bits, dtype_code, 1, 0)


@pytest.mark.parametrize("bits,gs", ((4, 64), (8, 128), (3, 32), (6, 64)))
@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
def test_gather_qmm_grouped_by_expert(oracle, gpu, dtype, bits, gs):
    """Many index pairs per expert take the grouped matrix-core path: a skewed
    routing (one expert with more than one 256-row tile, one expert unused), x
    rows reused by several pairs, N not a multiple of the tile."""
    E, N, K, T = 5, 200, 256, 700
    assert _grouped_ws_bytes(1, N, K, T, E, gs, bits) > 0  # the grouped path is taken
    w = normal_weights((E, N, K), dtype, std=0.5)
    wq, s, b = oracle.quantize(w, gs, bits)
    X = 64
    x = activations((X, 1, K), dtype)
    g = torch.Generator().manual_seed(1)
    rhs = torch.multinomial(torch.tensor([0.6, 0.0, 0.25, 0.1, 0.05]), T,
                            replacement=True, generator=g)
    lhs = torch.randint(0, X, (T,), generator=g)
    assert int((rhs == 0).sum()) > 256 and int((rhs == 1).sum()) == 0
    gx, gwq, gsc, gb, glhs, grhs = _to(gpu, x, wq, s, b, lhs, rhs)
    got = mlx_amd.gather_qmm(gx, gwq, gsc, gb, glhs, grhs, True, gs, bits).cpu()
    assert got.shape == (T, 1, N)
    w_hat = exact_affine_weights(wq, s, b, gs, bits)
    exact = torch.einsum("tk,tnk->tn", x.reshape(X, K).double()[lhs], w_hat[rhs])
    err = float((got.reshape(T, N).double() - exact).abs().max())
    assert err <= exact_tolerance(dtype, K, x, w_hat, exact)
    # and against the oracle on a subsample of the pairs (the oracle is scalar)
    sub = torch.arange(0, T, 23)
    ref = oracle.gather_qmm(x, wq, s, b, lhs[sub], rhs[sub], True, gs, bits)
    tol = matmul_tolerance(dtype, K, x, w_hat)
    assert float((got[sub].double() - ref.double()).abs().max()) <= tol


@pytest.mark.parametrize("bits,gs", ((4, 64), (8, 32), (4, 128)))
@pytest.mark.parametrize("dtype", (torch.bfloat16, torch.float16))
def test_gather_qmm_grouped_by_expert_not_transposed(oracle, gpu, dtype, bits, gs):
    """transpose=False (weights [K, N], what GatherQMM::vjp asks for,
    mlx/primitives.cpp:3718-3837) with many pairs per expert: sorted by expert
    into 256-row tiles of the column-loading tile GEMM.  Skewed routing (one
    expert with more than one tile, one unused), x rows reused, N no multiple
    of the tile width, one expert index out of range (zero row); a shared
    scale/bias set (stride 0) is not part of the Python surface and not taken."""
    from mlx_amd import _lib
    E, N, K, T = 5, 384, 320, 700
    code = {torch.float16: 1, torch.bfloat16: 2}[dtype]
    ws = _lib.load().mlxrocm_gather_qmm_workspace_size(1, N, K, T, E, gs, bits, code, 0, 0)
    assert ws >= 2 * E * K * (N // gs) * 2, "the grouped path is not taken"
    w = normal_weights((E, K, N), dtype, std=0.5)
    wq, s, b = oracle.quantize(w, gs, bits)
    X = 64
    x = activations((X, 1, K), dtype)
    g = torch.Generator().manual_seed(1)
    rhs = torch.multinomial(torch.tensor([0.6, 0.0, 0.25, 0.1, 0.05]), T,
                            replacement=True, generator=g)
    lhs = torch.randint(0, X, (T,), generator=g)
    assert int((rhs == 0).sum()) > 256 and int((rhs == 1).sum()) == 0
    gx, gwq, gsc, gb, glhs, grhs = _to(gpu, x, wq, s, b, lhs, rhs)
    got = mlx_amd.gather_qmm(gx, gwq, gsc, gb, glhs, grhs, False, gs, bits).cpu()
    assert got.shape == (T, 1, N)
    w_hat = exact_affine_weights(wq, s, b, gs, bits)  # [E, K, N]
    exact = torch.einsum("tk,tkn->tn", x.reshape(X, K).double()[lhs], w_hat[rhs])
    err = float((got.reshape(T, N).double() - exact).abs().max())
    assert err <= exact_tolerance(dtype, K, x, w_hat, exact)
    # against the oracle on a subsample of the pairs (the oracle is scalar and
    # accumulates in the element type: its own distance from exact is discounted)
    sub = torch.arange(0, T, 23)
    ref = oracle.gather_qmm(x, wq, s, b, lhs[sub], rhs[sub], False, gs, bits)
    tol = matmul_tolerance(dtype, K, x, w_hat) + float(
        (ref.reshape(-1, N).double() - exact[sub]).abs().max())
    assert float((got[sub].double() - ref.double()).abs().max()) <= tol
    # two pairs at a time stay on one product per pair: same rows up to rounding
    parts = [
        mlx_amd.gather_qmm(gx, gwq, gsc, gb, glhs[i:i + 2], grhs[i:i + 2], False, gs, bits)
        for i in range(0, 64, 2)
    ]
    single = torch.cat(parts).cpu()
    eps = {torch.float16: 2.0 ** -10, torch.bfloat16: 2.0 ** -7}[dtype]
    assert float((got[:64].double() - single.double()).abs().max()) <= 2 * eps * float(exact.abs().max())
    bad = grhs.clone()
    bad[7] = E + 2
    got_bad = mlx_amd.gather_qmm(gx, gwq, gsc, gb, glhs, bad, False, gs, bits).cpu()
    assert bool((got_bad[7] == 0).all())
    keep = torch.ones(T, dtype=torch.bool)
    keep[7] = False
    assert torch.equal(got_bad[keep], got[keep])


@pytest.mark.parametrize("index_dtype", (torch.int64, torch.int32, torch.uint32, torch.int16))
def test_gather_qmm_many_pairs_and_index_types(oracle, gpu, index_dtype):
    """More than 16384 pairs take the three-kernel grouping (fewer take the
    one-workgroup form); every pair is held to the fp64 product of the exact
    affine weights and to the CPU oracle's loop over the pairs
    (cpu/quantized.cpp:700-747).  Index tensors of every integer width are
    accepted: 32-bit ones are used as they are, others are converted."""
    E, N, K, X = 4, 96, 128, 50
    dtype = torch.bfloat16
    w = normal_weights((E, N, K), dtype, std=0.5)
    wq, s, b = oracle.quantize(w, 64, 4)
    w_hat = exact_affine_weights(wq, s, b, 64, 4)                 # [E, N, K] fp64
    x = activations((X, 1, K), dtype)
    gx, gwq, gs_, gb = _to(gpu, x, wq, s, b)
    for T in (3000, 20000):
        g = torch.Generator().manual_seed(T)
        rhs = torch.randint(0, E, (T,), generator=g)
        lhs = torch.randint(0, X, (T,), generator=g)
        got = mlx_amd.gather_qmm(gx, gwq, gs_, gb, lhs.to(index_dtype).to(gpu),
                                 rhs.to(index_dtype).to(gpu), True, 64, 4).cpu()
        assert got.shape == (T, 1, N)
        exact = torch.einsum("tk,tnk->tn", x.reshape(X, K).double()[lhs], w_hat[rhs])
        err = float((got.reshape(T, N).double() - exact).abs().max())
        assert err <= exact_tolerance(dtype, K, x, w_hat, exact), (T, err)
        ref = oracle.gather_qmm(x, wq, s, b, lhs, rhs, True, 64, 4).reshape(T, N).double()
        tol = matmul_tolerance(dtype, K, x, w_hat) + float((ref - exact).abs().max())
        assert float((got.reshape(T, N).double() - ref).abs().max()) <= tol, T


def test_gather_qmm_grouped_matches_ungrouped(gpu):
    """The grouped launch and the one-GEMV-per-pair launch agree row for row up
    to accumulation order (same fp32 accumulate, one rounding), also with a
    sliced expert stack and an out-of-range expert index (zero row)."""
    E, N, K, T = 6, 448, 512, 96
    dtype = torch.bfloat16
    w = normal_weights((E, N, K), dtype, std=0.5).to(gpu)
    wq, s, b = mlx_amd.quantize(w, 64, 4)
    x = activations((T, 1, K), dtype).to(gpu)
    g = torch.Generator().manual_seed(2)
    rhs = torch.randint(0, 3, (T,), generator=g).to(gpu)
    rhs[5] = 3  # the sliced stack has three experts
    grouped = mlx_amd.gather_qmm(x, wq[::2], s[::2], b[::2], rhs_indices=rhs)
    # the same pairs one small call at a time: below the grouping threshold
    parts = [
        mlx_amd.gather_qmm(x[i:i + 8], wq[::2], s[::2], b[::2], rhs_indices=rhs[i:i + 8])
        for i in range(0, T, 8)
    ]
    single = torch.cat(parts)
    torch.cuda.synchronize()
    assert bool((grouped[5] == 0).all())
    diff = (grouped.float() - single.float()).abs().max()
    scale = single.float().abs().max()
    assert float(diff) <= 2 ** -7 * float(scale)


@pytest.mark.parametrize("bits,gs", ((4, 64), (5, 32), (8, 128)))
def test_gather_qmm_small_groups(oracle, gpu, bits, gs):
    """A few index pairs per expert (at most 64 on average): the pairs are
    grouped into 32-row tiles for the few-row kernel.  One expert gets more than
    one tile, one gets none; ragged N; x rows shared between pairs."""
    E, N, K, T = 8, 200, 384, 100
    dtype = torch.bfloat16
    assert _grouped_ws_bytes(1, N, K, T, E, gs, bits) > 0
    w = normal_weights((E, N, K), dtype, std=0.5)
    wq, s, b = oracle.quantize(w, gs, bits)
    X = 16
    x = activations((X, 1, K), dtype)
    g = torch.Generator().manual_seed(3)
    rhs = torch.multinomial(torch.tensor([0.45, 0.0, 0.1, 0.1, 0.1, 0.1, 0.1, 0.05]), T,
                            replacement=True, generator=g)
    lhs = torch.randint(0, X, (T,), generator=g)
    assert int((rhs == 0).sum()) > 32 and int((rhs == 1).sum()) == 0
    gx, gwq, gsc, gb, glhs, grhs = _to(gpu, x, wq, s, b, lhs, rhs)
    got = mlx_amd.gather_qmm(gx, gwq, gsc, gb, glhs, grhs, True, gs, bits).cpu()
    ref = oracle.gather_qmm(x, wq, s, b, lhs, rhs, True, gs, bits)
    w_hat = exact_affine_weights(wq, s, b, gs, bits)
    exact = torch.einsum("tk,tnk->tn", x.reshape(X, K).double()[lhs], w_hat[rhs])
    assert float((got.reshape(T, N).double() - exact).abs().max()) <= exact_tolerance(
        dtype, K, x, w_hat, exact)
    tol = matmul_tolerance(dtype, K, x, w_hat) + float(
        (ref.reshape(T, N).double() - exact).abs().max())
    assert float((got.double() - ref.double()).abs().max()) <= tol


@pytest.fixture(scope="module")
def mixtral_stack(gpu):
    """8 experts of [14336, 4096], N(0, 0.02), 4-bit group 64, bf16 scales and
    biases, quantized on the GPU (that operator is bit-pinned by its own tests),
    with the fp64 affine weights of every expert beside it."""
    E, N, K = 8, 14336, 4096
    g = torch.Generator().manual_seed(0)
    w = (torch.randn((E, N, K), generator=g) * 0.02).to(torch.bfloat16)
    wq, s, b = mlx_amd.quantize(w.to(gpu), 64, 4)
    del w
    w_hat = exact_affine_weights_on(gpu, wq, s, b, 64, 4)
    yield wq, s, b, w_hat
    del w_hat
    torch.cuda.empty_cache()


@pytest.mark.parametrize("T", (1, 8, 64))
def test_gather_qmm_full_size_moe_few_tokens(oracle, gpu, mixtral_stack, T):
    """The expert-routed decode shapes at full size: T tokens, top-2 of 8 experts
    drawn uniformly (seeded), unsorted and pre-sorted by expert (8 tokens: 16
    pairs, grouped inside the kernel in 16-row tiles; 64: in 32-row tiles).  Every index
    pair against the fp64 product; a subsample of the pairs against the CPU
    oracle; sorted and unsorted runs agree bit for bit after un-permuting."""
    wq, s, b, w_hat = mixtral_stack
    E, N, K = 8, 14336, 4096
    x = activations((T, 1, 1, K), torch.bfloat16, seed=T)
    idx = torch.randint(0, E, (T, 2), generator=torch.Generator().manual_seed(T))
    gx, gidx = x.to(gpu), idx.to(gpu)
    unsorted = mlx_amd.gather_qmm(gx, wq, s, b, rhs_indices=gidx, transpose=True,
                                  group_size=64, bits=4)
    assert unsorted.shape == (T, 2, 1, N)
    flat = gidx.reshape(-1)
    order = torch.argsort(flat, stable=True)
    xs = gx.reshape(T, 1, K)[order // 2].contiguous()
    ys = mlx_amd.gather_qmm(xs, wq, s, b, rhs_indices=flat[order].contiguous(),
                            transpose=True, group_size=64, bits=4, sorted_indices=True)
    torch.cuda.synchronize()
    assert ys.shape == (2 * T, 1, N)
    resorted = ys[torch.argsort(order)].reshape(T, 2, 1, N)
    assert torch.equal(unsorted.view(torch.int16), resorted.view(torch.int16))
    # every pair against fp64, expert by expert
    got = unsorted.reshape(2 * T, N).double()
    xd = gx.reshape(T, K).double()
    tok = torch.arange(2 * T, device=gpu) // 2
    x_absmax = float(x.abs().max())
    for e in range(E):
        pairs = torch.nonzero(flat == e).reshape(-1)
        if pairs.numel() == 0:
            continue
        exact = xd[tok[pairs]] @ w_hat[e].T
        err = float((got[pairs] - exact).abs().max())
        tol = exact_tolerance_from(torch.bfloat16, K, x_absmax, float(w_hat[e].abs().max()),
                                   float(exact.abs().max()))
        assert err <= tol, f"expert {e}: {err} > {tol}"
    # the oracle on a few pairs
    cq = [t.cpu() for t in (wq, s, b)]
    for p in sorted({0, (2 * T) // 3, 2 * T - 1}):
        t, j = p // 2, p % 2
        e = int(idx[t, j])
        xr = x[t].reshape(1, K)
        ref = oracle.qmm(xr, cq[0][e], cq[1][e], cq[2][e], True, 64, 4).double()
        exact = (xr.to(gpu).double() @ w_hat[e].T).cpu()
        tol = 2e-2 * (K ** 0.5) * x_absmax * float(w_hat[e].abs().max()) + float(
            (ref - exact).abs().max())
        assert float((unsorted[t, j].cpu().double() - ref).abs().max()) <= tol


def test_gather_qmm_full_size_moe_prefill(oracle, gpu, mixtral_stack):
    """T = 2048 tokens routed top-2 over the 8 full-size experts (seeded): the
    grouped GEMM.  Every one of the 4096 index pairs against the fp64 product,
    expert by expert; the run on expert-sorted pairs reproduces the unsorted
    run bit for bit after un-permuting (a row depends on its own pair only);
    a few pairs against the CPU oracle."""
    wq, s, b, w_hat = mixtral_stack
    E, N, K, T = 8, 14336, 4096, 2048
    x = activations((T, 1, 1, K), torch.bfloat16, seed=T)
    idx = torch.randint(0, E, (T, 2), generator=torch.Generator().manual_seed(0))
    gx, gidx = x.to(gpu), idx.to(gpu)
    unsorted = mlx_amd.gather_qmm(gx, wq, s, b, rhs_indices=gidx, transpose=True,
                                  group_size=64, bits=4)
    assert unsorted.shape == (T, 2, 1, N)
    flat = gidx.reshape(-1)
    order = torch.argsort(flat, stable=True)
    xs = gx.reshape(T, 1, K)[order // 2].contiguous()
    ys = mlx_amd.gather_qmm(xs, wq, s, b, rhs_indices=flat[order].contiguous(),
                            transpose=True, group_size=64, bits=4, sorted_indices=True)
    torch.cuda.synchronize()
    resorted = ys[torch.argsort(order)].reshape(T, 2, 1, N)
    assert torch.equal(unsorted.view(torch.int16), resorted.view(torch.int16))
    del ys, resorted, xs
    # every pair against fp64, expert by expert
    got = unsorted.reshape(2 * T, N)
    xd = gx.reshape(T, K).double()
    tok = torch.arange(2 * T, device=gpu) // 2
    x_absmax = float(x.abs().max())
    checked = 0
    for e in range(E):
        pairs = torch.nonzero(flat == e).reshape(-1)
        if pairs.numel() == 0:
            continue
        exact = xd[tok[pairs]] @ w_hat[e].T
        err = float((got[pairs].double() - exact).abs().max())
        tol = exact_tolerance_from(torch.bfloat16, K, x_absmax, float(w_hat[e].abs().max()),
                                   float(exact.abs().max()))
        assert err <= tol, f"expert {e}: {err} > {tol}"
        checked += int(pairs.numel())
        del exact
    assert checked == 2 * T
    # the oracle on a few pairs
    cq = [t.cpu() for t in (wq, s, b)]
    for t, j in ((0, 0), (777, 1), (2047, 1)):
        e = int(idx[t, j])
        xr = x[t].reshape(1, K)
        ref = oracle.qmm(xr, cq[0][e], cq[1][e], cq[2][e], True, 64, 4).double()
        exact = (xr.to(gpu).double() @ w_hat[e].T).cpu()
        tol = 2e-2 * (K ** 0.5) * x_absmax * float(w_hat[e].abs().max()) + float(
            (ref - exact).abs().max())
        assert float((unsorted[t, j].cpu().double() - ref).abs().max()) <= tol
