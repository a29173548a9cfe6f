"""GPU parity of the floating-point quantization modes (mxfp4 / mxfp8 / nvfp4)
through the operators of mlx_amd (and so through the C ABI): quantize,
dequantize and the on-the-fly quantize-dequantize bit for bit against the CPU
oracle; quantized_matmul / gather_qmm / qqmm against the oracle (the
reference's translation unit where it was built) within the stated tolerance
and against an fp64 product of the exactly decoded weights.  Cases follow
python/tests/test_quantized.py:41-181 (quantize / dequantize per mode),
:183-237 (qqmm), :300-360 (fp_qmm shapes), :1180-1266 (gather)."""
import itertools
import os

import pytest
import torch

import mlx_amd
from oracle import build as obuild
from oracle import fp_qref, qref

pytestmark = pytest.mark.gpu

MODES = ("mxfp4", "mxfp8", "nvfp4")
DTYPES = (torch.float32, torch.float16, torch.bfloat16)
# fp32 accumulation on the GPU against an fp64 product: relative to the sum of
# absolute products.  The final rounding to the element type adds half an ulp.
ACC_TOL = {torch.float32: 2e-6, torch.float16: 1e-3, torch.bfloat16: 8e-3}
# The CPU reference rounds every product and partial sum to the element type,
# so it is the looser side: bound on |gpu - reference| relative to sum |x w|.
REF_TOL = {torch.float32: 5e-6, torch.float16: 4e-3, torch.bfloat16: 3e-2}


@pytest.fixture(scope="module")
def fp_oracle():
    if not os.path.isfile(qref.QREF_SO):
        obuild.build_qref()
    return fp_qref.FpOracle("reference" if qref.reference_built() else "port")


def _weights(shape, dtype, seed, spread=True):
    """Rows of very different magnitude, exact zeros, whole zero groups and
    values that sit exactly between two codes after scaling."""
    g = torch.Generator().manual_seed(seed)
    w = torch.randn(shape, generator=g)
    if spread:
        rows = w.reshape(-1, shape[-1])
        rows *= torch.exp(torch.randn(rows.shape[0], 1, generator=g) * 2.0)
        rows[0, :64] = 0.0
        rows[1, ::3] = 0.0
        if rows.shape[0] > 2:
            # a group whose maximum is 6: the rest are multiples of 0.25
            rows[2, :32] = torch.randint(-24, 25, (32,), generator=g).float() * 0.25
            rows[2, 0] = 6.0
    return w.to(dtype)


def _equal_bits(a: torch.Tensor, b: torch.Tensor) -> bool:
    """Bit for bit, signed zeros and infinities included; a NaN (0 * inf where a
    scale overflows float16) matches any NaN."""
    nan_a, nan_b = torch.isnan(a), torch.isnan(b)
    if not torch.equal(nan_a, nan_b):
        return False
    a = torch.where(nan_a, torch.zeros_like(a), a)
    b = torch.where(nan_b, torch.zeros_like(b), b)
    view = {4: torch.int32, 2: torch.int16, 1: torch.uint8}[a.element_size()]
    return torch.equal(a.contiguous().view(view), b.contiguous().view(view))


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("mode", MODES)
def test_fp_quantize_matches_oracle_bit_for_bit(fp_oracle, gpu, mode, dtype):
    for shape, seed in (((64, 512), 1), ((3, 17, 64), 2), ((2, 4096), 3)):
        w = _weights(shape, dtype, seed)
        wq, scales = mlx_amd.quantize(w.to(gpu), mode=mode)
        want_q, want_s = fp_oracle.quantize(w, mode)
        assert wq.dtype == torch.uint32 and scales.dtype == torch.uint8
        assert wq.shape == want_q.shape and scales.shape == want_s.shape
        assert torch.equal(scales.cpu(), want_s), (mode, dtype, shape)
        bad = (wq.cpu().view(torch.int32) != want_q.view(torch.int32)).sum().item()
        assert bad == 0, (mode, dtype, shape, bad)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("mode", MODES)
def test_fp_dequantize_matches_oracle_bit_for_bit(fp_oracle, gpu, mode, dtype):
    g = torch.Generator().manual_seed(11)
    bits, gs = fp_qref.BITS[mode], fp_qref.GROUP_SIZE[mode]
    K = 1024
    wq = torch.randint(0, 2 ** 31, (32, K * bits // 32), generator=g, dtype=torch.int64)
    wq = (wq * 2 + torch.randint(0, 2, wq.shape, generator=g)).to(torch.int32).view(torch.uint32)
    if mode == "nvfp4":
        # every e4m3 scale code (the reference's decoder has no NaN codes)
        scales = torch.arange(32 * K // gs, dtype=torch.int64).reshape(32, -1) % 256
    else:
        # every e8m0 exponent but 255, which decodes to NaN
        scales = torch.arange(32 * K // gs, dtype=torch.int64).reshape(32, -1) % 255
    scales = scales.to(torch.uint8)
    got = mlx_amd.dequantize(wq.to(gpu), scales.to(gpu), mode=mode, dtype=dtype)
    want = fp_oracle.dequantize(wq, scales, mode, dtype)
    assert got.dtype == dtype and got.shape == want.shape
    assert _equal_bits(got.cpu(), want), (mode, dtype)
    # default output type of the fp modes is bfloat16 (mlx/ops.cpp:4749-4753)
    assert mlx_amd.dequantize(wq.to(gpu), scales.to(gpu), mode=mode).dtype == torch.bfloat16


@pytest.mark.parametrize("mode", MODES)
def test_fp_values_on_the_code_grid_round_trip(gpu, mode):
    """python/tests/test_quantized.py:41-181: values that are representable
    (code value times a power-of-two scale) come back exactly."""
    g = torch.Generator().manual_seed(5)
    if mode == "mxfp8":
        table = fp_qref._e4m3_values()[:127].float()  # positive codes below 448
        table = table[table <= 448]
    else:
        table = torch.tensor(fp_qref.FP4_VALUES[:8])
    top = table.max()
    gs = fp_qref.GROUP_SIZE[mode]
    idx = torch.randint(0, table.numel(), (16, 256), generator=g)
    w = table[idx] * torch.where(torch.rand(16, 256, generator=g) < 0.5, -1.0, 1.0)
    w.reshape(-1, gs)[:, 0] = top  # every group's maximum is the top code: scale 1
    w = w * torch.exp2(torch.randint(-3, 4, (16, 1), generator=g).float())
    for dtype in DTYPES:
        wq, scales = mlx_amd.quantize(w.to(dtype).to(gpu), mode=mode)
        back = mlx_amd.dequantize(wq, scales, mode=mode, dtype=dtype)
        assert torch.equal(back.cpu().float(), w.to(dtype).float()), (mode, dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("mode", MODES)
def test_fp_quantize_dequantize_matches_oracle_bit_for_bit(fp_oracle, gpu, mode, dtype):
    from mlx_amd import _lib
    from mlx_amd.ops import _DTYPE_CODE, _MODE_CODE

    lib = _lib.load()
    x = _weights((48, 512), dtype, 21)
    xg = x.to(gpu)
    out = torch.empty_like(xg)
    _lib.check(lib.mlxrocm_fp_quantize_dequantize(
        xg.data_ptr(), out.data_ptr(), xg.numel(), _MODE_CODE[mode], _DTYPE_CODE[dtype],
        torch.cuda.current_stream().cuda_stream))
    want = fp_oracle.quantize_dequantize(x, mode)
    assert _equal_bits(out.cpu(), want), (mode, dtype)


def _check_product(got, x, wq, scales, mode, transpose, ref, dtype):
    """got [M, N] against fp64 of the exactly decoded weights and against the
    CPU reference's own result."""
    w = fp_qref.exact_fp_weights(wq, scales, mode)  # [N, K] or [K, N]
    xd = x.double()
    wd = w.T if transpose else w
    exact = xd @ wd
    mag = xd.abs() @ wd.abs() + 1e-30
    err = ((got.double() - exact).abs() / mag).max().item()
    half_ulp = {torch.float32: 2.0 ** -24, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
    assert err <= ACC_TOL[dtype] + half_ulp, (mode, dtype, transpose, err)
    if ref is not None:
        rerr = ((got.double() - ref.double()).abs() / mag).max().item()
        assert rerr <= REF_TOL[dtype], (mode, dtype, transpose, rerr)
        if dtype == torch.float32:
            return
        # 16-bit types: the GPU result is the closer of the two to the exact product
        ours = (got.double() - exact).abs().mean().item()
        theirs = (ref.double() - exact).abs().mean().item()
        assert ours <= theirs * 1.05 + 1e-12, (mode, dtype, ours, theirs)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("transpose", (True, False))
@pytest.mark.parametrize("mode", MODES)
def test_fp_quantized_matmul(fp_oracle, gpu, mode, transpose, dtype):
    # python/tests/test_quantized.py:300-360: M in 8, 32, 33, 64 and gemv rows
    for M, N, K, seed in ((1, 256, 512, 1), (8, 128, 256, 2), (33, 256, 128, 3), (64, 96, 2048, 4),
                          (5, 64, 48 if mode == "nvfp4" else 96, 5)):
        g = torch.Generator().manual_seed(seed)
        w = torch.randn((N, K) if transpose else (K, N), generator=g).to(dtype)
        x = torch.randn((M, K), generator=g).to(dtype)
        wq, scales = mlx_amd.quantize(w.to(gpu), mode=mode)
        got = mlx_amd.quantized_matmul(x.to(gpu), wq, scales, transpose=transpose, mode=mode)
        assert got.dtype == dtype and got.shape == (M, N)
        ref = fp_oracle.qmm(x, wq.cpu(), scales.cpu(), mode, transpose)
        _check_product(got.cpu(), x, wq.cpu(), scales.cpu(), mode, transpose, ref, dtype)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16), ids=str)
@pytest.mark.parametrize("mode", MODES)
def test_fp_quantized_matmul_prefill_tiles(fp_oracle, gpu, mode, dtype):
    """Rows of x from the cut-over to the matrix-core tile kernel on: ragged M
    and N (partial tiles), several tile widths, every output against fp64 and a
    band of rows against the CPU reference."""
    for M, N, K, seed in ((12, 224, 64, 1), (77, 1000, 256, 2), (300, 96, 512, 3), (513, 2240, 1024, 4)):
        g = torch.Generator().manual_seed(seed)
        w = torch.randn((N, K), generator=g).to(dtype)
        w[:, :32] *= 37.0  # groups of very different scale
        x = torch.randn((M, K), generator=g).to(dtype)
        wq, scales = mlx_amd.quantize(w.to(gpu), mode=mode)
        got = mlx_amd.quantized_matmul(x.to(gpu), wq, scales, mode=mode)
        assert got.dtype == dtype and got.shape == (M, N)
        _check_product(got.cpu(), x, wq.cpu(), scales.cpu(), mode, True, None, dtype)
        rows = slice(max(0, M - 5), M)
        ref = fp_oracle.qmm(x[rows], wq.cpu(), scales.cpu(), mode, True)
        _check_product(got[rows].cpu(), x[rows], wq.cpu(), scales.cpu(), mode, True, ref, dtype)
        # the streaming kernel (rows taken four at a time) agrees to fp32 rounding
        few = mlx_amd.quantized_matmul(x[:4].to(gpu), wq, scales, mode=mode)
        assert (few.float() - got[:4].float()).abs().max().item() <= \
            2.0 ** -7 * got[:4].float().abs().max().item()


def test_fp_qmm_workspace_contract(gpu):
    from mlx_amd import _lib

    lib = _lib.load()
    need = lib.mlxrocm_fp_qmm_workspace_size(512, 1024, 256, 1, 0, _lib.MXFP4, _lib.BFLOAT16, 1)
    assert need >= 1024 * (256 // 32) * 4
    assert lib.mlxrocm_fp_qmm_workspace_size(1, 1024, 256, 1, 0, _lib.MXFP4, _lib.BFLOAT16, 1) == 0
    assert lib.mlxrocm_fp_qmm_workspace_size(512, 1024, 256, 1, 0, _lib.MXFP4, _lib.FLOAT32, 1) == 0
    assert lib.mlxrocm_fp_qmm_workspace_size(512, 1024, 256, 1, 0, _lib.MXFP4, _lib.BFLOAT16, 0) == 0
    buf = torch.zeros(1 << 20, dtype=torch.uint8, device=gpu)
    p = buf.data_ptr()
    rc = lib.mlxrocm_fp_qmm(p, p, p, p, 512, 1024, 256, 1, 0, 0, 0, _lib.MXFP4, _lib.BFLOAT16, 1,
                            None, 0, None)
    assert rc == _lib.INVALID_ARGUMENT and "workspace" in _lib.last_error()


@pytest.mark.parametrize("mode", MODES)
def test_fp_quantized_matmul_full_size_decode(gpu, mode):
    """The decode shape of the affine headline, x [1, 4096] @ W [14336, 4096]^T,
    every output against fp64."""
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(7)
    w = torch.randn((14336, 4096), generator=g).to(dtype)
    for M in (1, 4, 6):
        x = torch.randn((M, 4096), generator=g).to(dtype)
        wq, scales = mlx_amd.quantize(w.to(gpu), mode=mode)
        got = mlx_amd.quantized_matmul(x.to(gpu), wq, scales, mode=mode)
        _check_product(got.cpu(), x, wq.cpu(), scales.cpu(), mode, True, None, dtype)


@pytest.mark.parametrize("mode", MODES)
def test_fp_quantized_matmul_batched(fp_oracle, gpu, mode):
    dtype = torch.float16
    g = torch.Generator().manual_seed(9)
    w = torch.randn((3, 64, 128), generator=g).to(dtype)
    x = torch.randn((2, 3, 5, 128), generator=g).to(dtype)
    wq, scales = mlx_amd.quantize(w.to(gpu), mode=mode)
    got = mlx_amd.quantized_matmul(x.to(gpu), wq, scales, mode=mode)
    assert got.shape == (2, 3, 5, 64)
    for b in range(2):
        for e in range(3):
            ref = fp_oracle.qmm(x[b, e], wq[e].cpu(), scales[e].cpu(), mode, True)
            _check_product(got[b, e].cpu(), x[b, e], wq[e].cpu(), scales[e].cpu(), mode, True,
                           ref, dtype)
    # one weight for a batch of x: the batch folds into the rows
    got2 = mlx_amd.quantized_matmul(x.to(gpu), wq[1], scales[1], mode=mode)
    assert got2.shape == (2, 3, 5, 64)
    assert torch.equal(got2[:, 1], got[:, 1])
    # empty reduction and empty outputs
    z = mlx_amd.quantized_matmul(torch.zeros((0, 128), dtype=dtype, device=gpu), wq[0], scales[0],
                                 mode=mode)
    assert z.shape == (0, 64)


@pytest.mark.parametrize("mode", MODES)
def test_fp_quantized_matmul_batched_prefill_and_edges(fp_oracle, gpu, mode):
    """A stack of weights with enough rows of x for the tile kernel (one scale
    image per batch entry), a broadcast weight through the C ABI (stride 0), and
    the empty cases: no rows, no columns, K == 0 (zeros)."""
    from mlx_amd import _lib
    from mlx_amd.ops import _MODE_CODE

    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(17)
    L, M, N, K = 3, 40, 96, 256
    w = torch.randn((L, N, K), generator=g).to(dtype)
    x = torch.randn((L, M, K), generator=g).to(dtype)
    wq, scales = mlx_amd.quantize(w.to(gpu), mode=mode)
    got = mlx_amd.quantized_matmul(x.to(gpu), wq, scales, mode=mode)
    assert got.shape == (L, M, N)
    for l in range(L):
        _check_product(got[l].cpu(), x[l], wq[l].cpu(), scales[l].cpu(), mode, True, None, dtype)
    # one weight for every batch entry, batch kept (stride 0) instead of folded
    lib = _lib.load()
    xg = x.to(gpu).contiguous()
    out = torch.empty((L, M, N), dtype=dtype, device=gpu)
    ws_bytes = lib.mlxrocm_fp_qmm_workspace_size(M, N, K, L, 0, _MODE_CODE[mode], _lib.BFLOAT16, 1)
    ws = torch.empty(max(int(ws_bytes), 16), dtype=torch.uint8, device=gpu)
    _lib.check(lib.mlxrocm_fp_qmm(
        xg.data_ptr(), wq[1].contiguous().data_ptr(), scales[1].contiguous().data_ptr(),
        out.data_ptr(), M, N, K, L, M * K, 0, 0, _MODE_CODE[mode], _lib.BFLOAT16, 1,
        ws.data_ptr(), ws_bytes, torch.cuda.current_stream().cuda_stream))
    for l in range(L):
        _check_product(out[l].cpu(), x[l], wq[1].cpu(), scales[1].cpu(), mode, True, None, dtype)
    # empty shapes
    assert mlx_amd.quantized_matmul(xg[0, :0], wq[0], scales[0], mode=mode).shape == (0, N)
    gs = fp_qref.GROUP_SIZE[mode]
    bits = fp_qref.BITS[mode]
    wq0 = torch.zeros((N, 0), dtype=torch.uint32, device=gpu)
    sc0 = torch.zeros((N, 0), dtype=torch.uint8, device=gpu)
    y0 = mlx_amd.quantized_matmul(torch.zeros((4, 0), dtype=dtype, device=gpu), wq0, sc0, mode=mode)
    assert y0.shape == (4, N) and float(y0.abs().max()) == 0.0
    assert (K * bits) % 32 == 0 and K % gs == 0


@pytest.mark.parametrize("mode", MODES)
def test_fp_gather_qmm_many_pairs_bad_indices_and_no_pairs(fp_oracle, gpu, mode):
    """70,000 pairs (more than one launch's grid depth), a pair whose index is out
    of range (zeros, as the affine path), and an empty index list."""
    dtype = torch.float16
    g = torch.Generator().manual_seed(23)
    E, N, K = 5, 32, 64
    w = torch.randn((E, N, K), generator=g).to(dtype)
    x = torch.randn((7, 1, K), generator=g).to(dtype)
    wq, scales = mlx_amd.quantize(w.to(gpu), mode=mode)
    n_pairs = 70000
    lhs = torch.randint(0, 7, (n_pairs,), generator=g, dtype=torch.int32)
    rhs = torch.randint(0, E, (n_pairs,), generator=g, dtype=torch.int32)
    got = mlx_amd.gather_qmm(x.to(gpu), wq, scales, None, lhs.to(gpu), rhs.to(gpu), mode=mode)
    assert got.shape == (n_pairs, 1, N)
    w_hat = fp_qref.exact_fp_weights(wq.cpu(), scales.cpu(), mode)  # [E, N, K]
    want = torch.einsum("pk,pnk->pn", x[lhs.long(), 0].double(), w_hat[rhs.long()])
    mag = torch.einsum("pk,pnk->pn", x[lhs.long(), 0].double().abs(), w_hat[rhs.long()].abs()) + 1e-30
    err = ((got[:, 0].cpu().double() - want).abs() / mag).max().item()
    assert err <= 1e-3 + 2.0 ** -11, (mode, err)
    # through the C ABI: an out-of-range expert index yields zeros for that pair
    from mlx_amd import _lib
    from mlx_amd.ops import _MODE_CODE

    lib = _lib.load()
    lhs_u = torch.tensor([0, 1, 2], dtype=torch.int32, device=gpu).view(torch.uint32)
    rhs_u = torch.tensor([1, E, 3], dtype=torch.int32, device=gpu).view(torch.uint32)
    out = torch.full((3, 1, N), 7.0, dtype=dtype, device=gpu)
    xg = x.to(gpu).contiguous()
    _lib.check(lib.mlxrocm_fp_gather_qmm(
        xg.data_ptr(), wq.data_ptr(), scales.data_ptr(), lhs_u.data_ptr(), rhs_u.data_ptr(),
        out.data_ptr(), 1, N, K, 3, 7, E, K, wq.stride(0), scales.stride(0), _MODE_CODE[mode],
        _lib.FLOAT16, 1, None, 0, torch.cuda.current_stream().cuda_stream))
    assert float(out[1].abs().max()) == 0.0
    assert float(out[0].abs().max()) > 0.0 and float(out[2].abs().max()) > 0.0
    # no pairs
    empty = torch.zeros((0,), dtype=torch.int32, device=gpu)
    assert mlx_amd.gather_qmm(xg, wq, scales, None, empty, empty, mode=mode).shape == (0, 1, N)


@pytest.mark.parametrize("transpose", (True, False))
@pytest.mark.parametrize("mode", MODES)
def test_fp_gather_qmm(fp_oracle, gpu, mode, transpose):
    # python/tests/test_quantized.py:1180-1266 with mode != "affine"
    dtype = torch.float32
    g = torch.Generator().manual_seed(13)
    E, M, N, K = 6, 3, 64, 128
    w = torch.randn((E, N, K) if transpose else (E, K, N), generator=g).to(dtype)
    x = torch.randn((4, M, K), generator=g).to(dtype)
    wq, scales = mlx_amd.quantize(w.to(gpu), mode=mode)
    lhs = torch.tensor([[0, 3, 1], [2, 2, 0]], dtype=torch.int32)
    rhs = torch.tensor([[5, 0, 2], [1, 1, 4]], dtype=torch.int32)
    got = mlx_amd.gather_qmm(x.to(gpu), wq, scales, None, lhs.to(gpu), rhs.to(gpu),
                             transpose=transpose, mode=mode)
    assert got.shape == (2, 3, M, N)
    for i in range(2):
        for j in range(3):
            e, b = rhs[i, j].item(), lhs[i, j].item()
            ref = fp_oracle.qmm(x[b], wq[e].cpu(), scales[e].cpu(), mode, transpose)
            _check_product(got[i, j].cpu(), x[b], wq[e].cpu(), scales[e].cpu(), mode, transpose,
                           ref, dtype)
    # rhs only: x broadcasts against the index shape
    x1 = x[:1]
    got = mlx_amd.gather_qmm(x1.to(gpu), wq, scales, None, rhs_indices=rhs.reshape(-1).to(gpu),
                             transpose=transpose, mode=mode)
    assert got.shape == (6, M, N)
    for j, e in enumerate(rhs.reshape(-1).tolist()):
        ref = fp_oracle.qmm(x1[0], wq[e].cpu(), scales[e].cpu(), mode, transpose)
        _check_product(got[j].cpu(), x1[0], wq[e].cpu(), scales[e].cpu(), mode, transpose, ref, dtype)


@pytest.mark.parametrize("mode", ("nvfp4", "mxfp8", "mxfp4"))
def test_qqmm(fp_oracle, gpu, mode):
    """python/tests/test_quantized.py:183-290: qqmm(x, w_q, scales) against
    dequantize(quantize(x)) @ dequantize(w_q).T, and -- for one row of x, the
    case the CPU backend implements -- against its result."""
    for M, N, K in ((1, 128, 256), (8, 128, 128), (33, 256, 256), (64, 128, 256)):
        g = torch.Generator().manual_seed(M + N)
        x = torch.randn((M, K), generator=g)
        w = torch.randn((N, K), generator=g)
        wq, scales = mlx_amd.quantize(w.to(gpu), mode=mode)
        got = mlx_amd.qqmm(x.to(gpu), wq, scales, mode=mode)
        assert got.shape == (M, N) and got.dtype == torch.float32
        x_hat = fp_oracle.quantize_dequantize(x, mode)
        w_hat = fp_qref.exact_fp_weights(wq.cpu(), scales.cpu(), mode)
        want = x_hat.double() @ w_hat.T
        assert (got.cpu().double() - want).abs().max().item() < 1e-3
        if M == 1:
            ref = fp_oracle.qqmm(x, wq.cpu(), scales.cpu(), mode)
            assert (got.cpu() - ref).abs().max().item() < 1e-4
        # a floating-point w is quantized inside the call
        got_w = mlx_amd.qqmm(x.to(gpu), w.to(gpu), mode=mode)
        assert torch.equal(got_w, got)
    # gemv input and batched input keep their shapes
    assert mlx_amd.qqmm(x[0].to(gpu), wq, scales, mode=mode).shape == (N,)
    assert mlx_amd.qqmm(x.reshape(8, 8, K).to(gpu), wq, scales, mode=mode).shape == (8, 8, N)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
@pytest.mark.parametrize("mode", ("mxfp8", "mxfp4"))
def test_qqmm_on_the_block_scaled_matrix_instruction(fp_oracle, gpu, mode, dtype):
    """16 rows of x or more in the MX modes: both operands' codes are multiplied
    as they are.  Every output against the fp64 product of the two dequantized
    operands (x by the oracle's quantize-dequantize, w by the definition of the
    format); ragged M and N, one and many K steps, groups of very different
    scale; the first rows also against the route that fewer rows take."""
    half_ulp = {torch.float32: 2.0 ** -24, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
    for M, N, K, seed in ((16, 128, 128, 1), (77, 200, 256, 2), (300, 1000, 1024, 3), (513, 136, 4096, 4)):
        g = torch.Generator().manual_seed(seed)
        x = torch.randn((M, K), generator=g)
        x[:, 32:64] *= 50.0
        x[1, :32] = 0.0
        w = torch.randn((N, K), generator=g)
        w[:, :32] *= 0.01
        x, w = x.to(dtype), w.to(dtype)
        wq, scales = mlx_amd.quantize(w.to(gpu), mode=mode)
        got = mlx_amd.qqmm(x.to(gpu), wq, scales, mode=mode)
        assert got.shape == (M, N) and got.dtype == dtype
        x_hat = fp_oracle.quantize_dequantize(x, mode).double()
        w_hat = fp_qref.exact_fp_weights(wq.cpu(), scales.cpu(), mode)
        want = x_hat @ w_hat.T
        mag = x_hat.abs() @ w_hat.abs().T + 1e-30
        err = ((got.cpu().double() - want).abs() / mag).max().item()
        # e2m1 products are summed exactly by the instruction; for e4m3 it keeps
        # about 17 bits below the largest product of a 128-code step (16-bit
        # results only: float32 problems take the fp32-accumulating kernels)
        acc_tol = 2e-6 if (mode == "mxfp4" or dtype == torch.float32) else 2e-5
        assert err <= acc_tol + half_ulp, (mode, dtype, (M, N, K), err)
        few = mlx_amd.qqmm(x[:8].to(gpu), wq, scales, mode=mode)  # x_hat in dtype, streaming kernel
        ferr = ((few.cpu().double() - got[:8].cpu().double()).abs() / mag[:8]).max().item()
        assert ferr <= 2 * acc_tol + 2 * half_ulp, (mode, dtype, (M, N, K), ferr)


def test_fp_mode_layers(gpu):
    import mlx_amd.nn as qnn

    torch.manual_seed(0)
    lin = torch.nn.Linear(256, 128, bias=True, device=gpu)
    x = torch.randn((5, 256), device=gpu)
    for mode in MODES:
        q = qnn.QuantizedLinear.from_linear(lin, mode=mode)
        assert q.biases is None and q.scales.dtype == torch.uint8
        w_hat = mlx_amd.dequantize(q.weight, q.scales, mode=mode, dtype=torch.float32)
        want = x @ w_hat.T + lin.bias
        assert (q(x) - want).abs().max().item() < 1e-3
        emb = qnn.QuantizedEmbedding.from_embedding(torch.nn.Embedding(16, 64, device=gpu), mode=mode)
        tok = torch.tensor([[1, 5], [0, 15]], device=gpu)
        assert emb(tok).shape == (2, 2, 64)
    plain = torch.nn.Linear(256, 128, bias=False, device=gpu)
    qq = qnn.QQLinear.from_linear(plain)  # training mode: float weight
    assert qq.weight.dtype == torch.float32 and qq.scales is None
    y_train = qq(x)
    qq.eval()
    assert qq.weight.dtype == torch.uint32 and qq.scales.dtype == torch.uint8
    assert torch.equal(qq(x), y_train)
    qq.train()
    assert qq.weight.dtype == torch.float32
    with pytest.raises(NotImplementedError):
        qnn.QQLinear.from_linear(lin)
    model = torch.nn.Sequential(torch.nn.Linear(64, 64, bias=False, device=gpu))
    qnn.quantize(model, mode="mxfp8", quantize_input=True)
    assert isinstance(model[0], qnn.QQLinear)


def test_fp_abi_rejects_bad_arguments(gpu):
    from mlx_amd import _lib

    lib = _lib.load()
    buf = torch.zeros(4096, dtype=torch.uint8, device=gpu)
    p = buf.data_ptr()
    assert lib.mlxrocm_fp_quantize(p, p, p, 64, 3, 0, None) == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_fp_quantize(p, p, p, 48, _lib.MXFP4, 0, None) == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_fp_quantize(p, p, p, 64, _lib.MXFP4, 7, None) == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_fp_dequantize(p, p, p, 40, _lib.NVFP4, 0, None) == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_fp_qmm(p, p, p, p, 1, 8, 40, 1, 0, 0, 0, _lib.MXFP8, 0, 1, None, 0, None) \
        == _lib.INVALID_ARGUMENT
    assert "multiple of group_size" in _lib.last_error()
    assert lib.mlxrocm_fp_qmm(None, p, p, p, 1, 8, 64, 1, 0, 0, 0, _lib.MXFP8, 0, 1, None, 0, None) \
        == _lib.INVALID_ARGUMENT
    # nothing to do
    assert lib.mlxrocm_fp_quantize(None, None, None, 0, _lib.MXFP4, 0, None) == _lib.OK


# ---- nvfp4 with a tensor-wide scale, gather_qqmm ------------------------------
# The reference has these on the GPU only (python/tests/test_quantized.py:183-190,
# 192-300, 1268-1363), so the checker is the numpy restatement of the CUDA
# kernels' fp32 arithmetic in oracle/fp_qref.py: codes, scale bytes and
# dequantized elements bit for bit, products against float64.

def _global_weights(dtype, seed):
    """Rows of very different magnitude, a group of zeros, a group so small that
    its scale underflows to the byte 0, and the tensor's maximum."""
    w = _weights((40, 512), dtype, seed).float()
    w[5, 32:48] = w.abs().max() * 1e-7
    return w.to(dtype)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_nvfp4_global_scale_quantize_and_dequantize_bit_for_bit(gpu, dtype):
    for seed, scale_of_max in ((31, 1.0), (32, 0.37), (33, 4.0)):
        w = _global_weights(dtype, seed)
        gs = float(w.float().abs().max()) * scale_of_max
        gst = torch.tensor(gs, dtype=torch.float32)
        wq, scales = mlx_amd.quantize(w.to(gpu), mode="nvfp4", global_scale=gst.to(gpu))
        want_q, want_s = fp_qref.nvfp4_global_quantize(w, gs)
        assert torch.equal(scales.cpu(), want_s), (dtype, seed)
        bad = (wq.cpu().view(torch.int32) != want_q.view(torch.int32)).sum().item()
        assert bad == 0, (dtype, seed, bad)
        assert (want_s == 0).any() and (want_s == 126).any() == (scale_of_max <= 1.0)
        for out_dtype in DTYPES:
            got = mlx_amd.dequantize(wq, scales, mode="nvfp4", dtype=out_dtype,
                                     global_scale=gst)  # a host scalar is moved to the device
            want = fp_qref.nvfp4_global_dequantize(want_q, want_s, gs, out_dtype)
            assert got.dtype == out_dtype and _equal_bits(got.cpu(), want), (dtype, out_dtype, seed)
    # every scale byte and code
    g = torch.Generator().manual_seed(12)
    wq = torch.randint(-2 ** 31, 2 ** 31, (32, 128), generator=g, dtype=torch.int64).to(torch.int32)
    wq = wq.view(torch.uint32)
    scales = (torch.arange(32 * 64, dtype=torch.int64).reshape(32, 64) % 127).to(torch.uint8)
    got = mlx_amd.dequantize(wq.to(gpu), scales.to(gpu), mode="nvfp4", dtype=dtype,
                             global_scale=torch.tensor(0.731, device=gpu))
    assert _equal_bits(got.cpu(), fp_qref.nvfp4_global_dequantize(wq, scales, 0.731, dtype))


def test_nvfp4_global_scale_round_trip_of_the_reference_test(gpu):
    # python/tests/test_quantized.py:124-190
    g = torch.Generator().manual_seed(1)
    lut = torch.tensor(fp_qref.FP4_VALUES)
    w = lut[torch.randint(0, 16, (128, 512), generator=g)].reshape(-1, 16)
    w[:, 0] = 6
    w = (w + 3e-6).to(torch.bfloat16).reshape(128, 512).to(gpu)
    gs = w.abs().max().float()
    wq, scales = mlx_amd.quantize(w, mode="nvfp4", global_scale=gs)
    w_hat = mlx_amd.dequantize(wq, scales, group_size=16, bits=4, mode="nvfp4", global_scale=gs)
    assert torch.allclose(w.float(), w_hat.float(), rtol=1e-5, atol=1e-5)
    zeros = torch.zeros((256, 512), device=gpu)
    wq, scales = mlx_amd.quantize(zeros, mode="nvfp4", global_scale=torch.ones((), device=gpu))
    assert torch.all(mlx_amd.dequantize(wq, scales, mode="nvfp4",
                                        global_scale=torch.ones((), device=gpu)) == 0)


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_nvfp4_global_scale_quantize_dequantize_bit_for_bit(gpu, dtype):
    from mlx_amd import _lib
    from mlx_amd.ops import _DTYPE_CODE

    lib = _lib.load()
    x = _global_weights(dtype, 41)
    gs = float(x.float().abs().max())
    xg, gst = x.to(gpu), torch.tensor([gs], dtype=torch.float32, device=gpu)
    out = torch.empty_like(xg)
    _lib.check(lib.mlxrocm_nvfp4_quantize_dequantize_global(
        xg.data_ptr(), gst.data_ptr(), out.data_ptr(), xg.numel(), _DTYPE_CODE[dtype],
        torch.cuda.current_stream().cuda_stream))
    assert _equal_bits(out.cpu(), fp_qref.nvfp4_global_quantize_dequantize(x, gs)), dtype


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_qqmm_with_global_scales(gpu, dtype):
    """python/tests/test_quantized.py:192-300 (test_qqmv, test_qqmm): shapes of
    both tests plus shapes that take the tile kernel with and without a split K."""
    half_ulp = {torch.float32: 2.0 ** -24, torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
    shapes = [(1, 256, 64), (1, 67, 512), (8, 128, 128), (32, 256, 256), (33, 128, 256),
              (64, 256, 128), (5, 64, 48), (40, 96, 4096), (300, 520, 1024)]
    for M, N, K in shapes:
        g = torch.Generator().manual_seed(M * 7 + N)
        x = torch.randn((M, K), generator=g).to(dtype)
        w = torch.randn((N, K), generator=g).to(dtype)
        gx, gw = x.float().abs().max(), w.float().abs().max()
        wq, scales = mlx_amd.quantize(w.to(gpu), mode="nvfp4", global_scale=gw.to(gpu))
        got = mlx_amd.qqmm(x.to(gpu), wq, scales, mode="nvfp4",
                           global_scale_x=gx.to(gpu), global_scale_w=gw.to(gpu))
        assert got.shape == (M, N) and got.dtype == dtype
        want, mag = fp_qref.nvfp4_global_qqmm_f64(x, wq.cpu(), scales.cpu(), float(gx), float(gw))
        err = ((got.cpu().double() - want).abs() / (mag + 1e-30)).max().item()
        assert err <= ACC_TOL[dtype] + half_ulp, (dtype, (M, N, K), err)
        if dtype == torch.float32:
            # the reference's own assertion: within 1e-3 of x_hat @ w_hat.T
            x_hat = fp_qref.nvfp4_global_quantize_dequantize(x, float(gx)).double()
            w_hat = fp_qref.nvfp4_global_dequantize(wq.cpu(), scales.cpu(), float(gw)).double()
            assert (got.cpu().double() - x_hat @ w_hat.T).abs().max().item() < 1e-3
        # a floating-point w is quantized inside the call, with its scale
        got_w = mlx_amd.qqmm(x.to(gpu), w.to(gpu), mode="nvfp4",
                             global_scale_x=gx.to(gpu), global_scale_w=gw.to(gpu))
        assert torch.equal(got_w, got)
    with pytest.raises(ValueError, match="either both"):
        mlx_amd.qqmm(x.to(gpu), wq, scales, mode="nvfp4", global_scale_x=gx.to(gpu))


_GATHER_QQMM_BATCHES = (
    # python/tests/test_quantized.py:1275-1306
    ((1,), (0,), (3,), (2, 1)),
    ((1,), None, (3,), (2, 1)),
    ((2,), None, (3,), (2, 1)),
    ((3,), (0, 2), (1,), (0,)),
    ((5,), (0, 2), (3,), (2, 1)),
)


@pytest.mark.parametrize("mode", ("nvfp4", "mxfp8", "mxfp4"))
def test_gather_qqmm(fp_oracle, gpu, mode):
    """python/tests/test_quantized.py:1268-1363: every pair against the float64
    product of x_hat (the oracle's quantize-dequantize of that matrix of x) and
    the exactly decoded expert; nvfp4 with both tensor-wide scales, as there."""
    gsz = fp_qref.GROUP_SIZE[mode]
    for (batch_a, lhs, batch_b, rhs), M, N, K in itertools.product(
            _GATHER_QQMM_BATCHES, (1, 32), (32, 256), (32, 256)):
        if K % gsz:
            continue
        g = torch.Generator().manual_seed(M + N + K + len(batch_a))
        x = torch.randn(batch_a + (M, K), generator=g)
        w = torch.randn(batch_b + (N, K), generator=g)
        use_global = mode == "nvfp4"
        gx = x.abs().max() if use_global else None
        gw = w.abs().max() if use_global else None
        kw = dict(global_scale=gw.to(gpu)) if use_global else {}
        wq, scales = mlx_amd.quantize(w.to(gpu), mode=mode, **kw)
        li = None if lhs is None else torch.tensor(lhs, dtype=torch.int32, device=gpu)
        ri = None if rhs is None else torch.tensor(rhs, dtype=torch.int32, device=gpu)
        kw = dict(global_scale_x=gx.to(gpu), global_scale_w=gw.to(gpu)) if use_global else {}
        got = mlx_amd.gather_qqmm(x.to(gpu), wq, scales, li, ri, mode=mode, **kw)
        lhs_l = list(lhs) if lhs is not None else list(range(batch_a[0]))
        rhs_l = list(rhs)
        n = max(len(lhs_l), len(rhs_l))
        lhs_l = lhs_l * (n // len(lhs_l))
        rhs_l = rhs_l * (n // len(rhs_l))
        assert got.shape == (n, M, N) and got.dtype == torch.float32
        for i in range(n):
            xi, e = x[lhs_l[i]], rhs_l[i]
            if use_global:
                want, mag = fp_qref.nvfp4_global_qqmm_f64(
                    xi, wq[e].cpu(), scales[e].cpu(), float(gx), float(gw))
            else:
                x_hat = fp_oracle.quantize_dequantize(xi, mode).double()
                w_hat = fp_qref.exact_fp_weights(wq[e].cpu(), scales[e].cpu(), mode)
                want, mag = x_hat @ w_hat.T, x_hat.abs() @ w_hat.abs().T
            err = ((got[i].cpu().double() - want).abs() / (mag + 1e-30)).max().item()
            assert err <= ACC_TOL[torch.float32] + 2.0 ** -24, (mode, (M, N, K), i, err)
        # a floating-point w is quantized inside the call
        got_w = mlx_amd.gather_qqmm(x.to(gpu), w.to(gpu), None, li, ri, mode=mode, **kw)
        assert torch.equal(got_w, got)


@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16), ids=str)
def test_gather_qqmm_sixteen_bit_and_bad_indices(fp_oracle, gpu, dtype):
    g = torch.Generator().manual_seed(77)
    x = torch.randn((4, 3, 128), generator=g).to(dtype)
    w = torch.randn((6, 72, 128), generator=g).to(dtype)
    wq, scales = mlx_amd.quantize(w.to(gpu), mode="mxfp4")
    lhs = torch.tensor([0, 3, 1, 2, 9, 0], dtype=torch.int64, device=gpu)   # 9: out of range
    rhs = torch.tensor([5, 0, 2, 2, 1, 6], dtype=torch.int64, device=gpu)   # 6: out of range
    got = mlx_amd.gather_qqmm(x.to(gpu), wq, scales, lhs, rhs, mode="mxfp4")
    assert got.shape == (6, 3, 72) and got.dtype == dtype
    assert torch.all(got[4] == 0) and torch.all(got[5] == 0)
    half_ulp = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
    for i in range(4):
        x_hat = fp_oracle.quantize_dequantize(x[int(lhs[i])], "mxfp4").double()
        w_hat = fp_qref.exact_fp_weights(wq[int(rhs[i])].cpu(), scales[int(rhs[i])].cpu(), "mxfp4")
        err = ((got[i].cpu().double() - x_hat @ w_hat.T).abs() /
               (x_hat.abs() @ w_hat.abs().T + 1e-30)).max().item()
        assert err <= ACC_TOL[dtype] + half_ulp, (dtype, i, err)
    # no pairs
    none = mlx_amd.gather_qqmm(x.to(gpu), wq, scales, lhs[:0], rhs[:0], mode="mxfp4")
    assert none.shape == (0, 3, 72)


def test_global_scale_abi_rejects_bad_arguments(gpu):
    from mlx_amd import _lib

    lib = _lib.load()
    buf = torch.zeros(1 << 16, dtype=torch.uint8, device=gpu)
    p = buf.data_ptr()
    assert lib.mlxrocm_nvfp4_quantize_global(p, None, p, p, 64, 0, None) == _lib.INVALID_ARGUMENT
    assert "global_scale" in _lib.last_error()
    assert lib.mlxrocm_nvfp4_quantize_global(p, p, p, p, 40, 0, None) == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_nvfp4_dequantize_global(p, p, p + 2, p, 64, 0, None) == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_nvfp4_quantize_dequantize_global(p, p, p, 64, 9, None) == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_nvfp4_qqmm_global(p, p, p, p, None, p, 2, 8, 64, 0, p, 1 << 16, None) \
        == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_nvfp4_qqmm_global(p, p, p, p, p, p, 2, 8, 64, 0, p, 16, None) \
        == _lib.INVALID_ARGUMENT
    assert "workspace" in _lib.last_error()
    # gather_qqmm: one scale only; scales outside nvfp4; a workspace that is too small
    args = (2, 8, 64, 1, 1, 1, 128, 0, 0)
    assert lib.mlxrocm_fp_gather_qqmm(p, p, p, p, p, p, None, p, *args, _lib.NVFP4, 0, p, 1 << 16, None) \
        == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_fp_gather_qqmm(p, p, p, p, p, p, p, p, *args, _lib.MXFP4, 0, p, 1 << 16, None) \
        == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_fp_gather_qqmm(p, p, p, p, p, None, None, p, *args, _lib.MXFP4, 0, p, 16, None) \
        == _lib.INVALID_ARGUMENT
    assert lib.mlxrocm_fp_gather_qqmm_workspace_size(2, 8, 64, 1, 3, 1, 0, _lib.MXFP4, 0) \
        == 2 * 64 * 3 * 4
    # nothing to do
    assert lib.mlxrocm_nvfp4_quantize_global(None, p, None, None, 0, 0, None) == _lib.OK


@pytest.mark.parametrize("dtype", DTYPES, ids=str)
def test_to_fp8_and_from_fp8_bit_for_bit(fp_oracle, gpu, dtype):
    """mx.to_fp8 / mx.from_fp8 against the reference's converters (the C port of
    detail::ToFP8 / FromFP8, itself checked value by value against the reference's
    translation unit): every bit pattern of the 16-bit types, sampled and edge
    float32 values; every code back; lengths that are not a multiple of 8."""
    port = fp_oracle.port
    if dtype == torch.float32:
        g = torch.Generator().manual_seed(3)
        x = torch.randn(60001, generator=g) * torch.exp(torch.randn(60001, generator=g) * 4)
        edge = torch.tensor([0.0, -0.0, 448.0, 447.9, 464.0, 465.0, 1e30, -1e30, float("inf"),
                             float("-inf"), float("nan"), 2.0 ** -9, 2.0 ** -10, 1.5 * 2.0 ** -10,
                             0.015625, 0.0009765625, 17.0, 18.0, 19.0])
        x = torch.cat([x, edge, -edge])
    else:
        x = torch.arange(65536, dtype=torch.int32).to(torch.int16).view(dtype)
        x = torch.cat([x, x[:13]])  # a ragged tail
    got = mlx_amd.to_fp8(x.to(gpu))
    assert got.dtype == torch.uint8 and got.shape == x.shape
    want = torch.tensor([port.fpq_to_fp8(float(v)) for v in x.float().tolist()], dtype=torch.uint8)
    assert torch.equal(got.cpu(), want), dtype
    codes = torch.arange(256, dtype=torch.int32).to(torch.uint8)
    for shape in ((256,), (4, 64), (251,)):
        c = codes[: shape[0] * (shape[1] if len(shape) > 1 else 1)].reshape(shape)
        back = mlx_amd.from_fp8(c.to(gpu), dtype)
        vals = torch.tensor([port.fpq_from_fp8(int(v)) for v in c.flatten().tolist()]).reshape(shape)
        assert back.dtype == dtype and torch.equal(back.cpu().float(), vals), (dtype, shape)
    assert mlx_amd.from_fp8(codes.to(gpu)).dtype == torch.bfloat16  # the default
    # python/tests/test_ops.py:4212-4217
    vals = torch.tensor([448, 256, 192, 128, 96, 64, 48, 32, 24, 16, 12, 8, 6, 4, 3, 2, 0.015625])
    for v in (vals, -vals):
        assert torch.equal(mlx_amd.from_fp8(mlx_amd.to_fp8(v.to(dtype).to(gpu)), dtype).cpu().float(), v)
    assert mlx_amd.to_fp8(torch.empty((0, 3), dtype=dtype, device=gpu)).shape == (0, 3)


@pytest.mark.parametrize("mode", ("mxfp4", "mxfp8"))
def test_fp_quantize_dequantize_scales_next_to_a_tie_bit_for_bit(fp_oracle, gpu, mode):
    """round(log2(scale)) flips where the scale's mantissa passes sqrt(2): groups
    whose scale sits a few steps on either side of it (inside and outside the band
    where the kernel evaluates the logarithm), over the whole exponent range,
    subnormal scales and the largest finite values."""
    from mlx_amd import _lib
    from mlx_amd.ops import _DTYPE_CODE, _MODE_CODE

    lib = _lib.load()
    top = 6.0 if mode == "mxfp4" else 448.0
    offs = (-70000, -4200, -4097, -4096, -4095, -300, -2, -1, 0, 1, 2, 300, 4095, 4096, 4097, 4200, 70000)
    rows = []
    g = torch.Generator().manual_seed(8)
    for e in list(range(-126, 120, 5)) + [-126, -125, 118, 119]:
        for off in offs:
            bits = ((e + 127) << 23) | (0x3504F3 + off)
            scale = torch.tensor([bits], dtype=torch.int32).view(torch.float32)
            row = (torch.rand(32, generator=g) * 2 - 1) * scale * top
            row[int(torch.randint(0, 32, (1,), generator=g))] = scale * top
            rows.append(row)
    # subnormal scales, zero, the largest finite elements
    for amax in (1e-44, 3e-39, 1.2e-38 * top, 0.0, 3.4e38, 1.7e38):
        row = (torch.rand(32, generator=g) * 2 - 1) * amax
        row[3] = amax
        rows.append(row)
    x = torch.stack(rows)
    x = torch.nan_to_num(x, nan=0.0, posinf=3.4e38, neginf=-3.4e38).contiguous()
    xg = x.to(gpu)
    out = torch.empty_like(xg)
    _lib.check(lib.mlxrocm_fp_quantize_dequantize(
        xg.data_ptr(), out.data_ptr(), xg.numel(), _MODE_CODE[mode], _DTYPE_CODE[torch.float32],
        torch.cuda.current_stream().cuda_stream))
    want = fp_oracle.quantize_dequantize(x, mode)
    assert _equal_bits(out.cpu(), want), mode
    # the same rule where x goes to codes for the block-scaled matrix instruction
    # (16 rows or more, K a multiple of 128): against a diagonal w every output is
    # one product, exact in float32, so the codes are checked bit for bit too
    keep = (x.abs().amax(-1) < 1e12) & (x.abs().amax(-1) > 1e-12)
    x2 = x[keep]
    x2 = x2[: x2.shape[0] // 4 * 4].reshape(-1, 128)
    assert x2.shape[0] >= 16
    # e4m3 codes take the matrix instruction only for the 16-bit types
    dtype = torch.float32 if mode == "mxfp4" else torch.bfloat16
    x2 = x2.to(dtype)
    wq, scales = mlx_amd.quantize(torch.eye(128, device=gpu, dtype=dtype), mode=mode)
    y = mlx_amd.qqmm(x2.to(gpu), wq, scales, mode=mode)
    w_hat = fp_qref.exact_fp_weights(wq.cpu(), scales.cpu(), mode)
    want = (fp_oracle.quantize_dequantize(x2, mode).double() @ w_hat.T).to(dtype)
    assert _equal_bits(y.cpu(), want), mode



@pytest.mark.parametrize("dtype", (torch.float16, torch.bfloat16), ids=str)
@pytest.mark.parametrize("mode", MODES)
def test_fp_gather_grouped_by_expert(gpu, mode, dtype):
    """One row of x per pair and many pairs per expert: the pairs are sorted by
    expert and every expert multiplied once on the matrix cores.  Every pair
    against float64; an expert with no pair, one with more than a tile of 256,
    pairs with an index out of range (zeros), ragged N, a sliced expert stack;
    and the same call without a workspace (one product per pair)."""
    from mlx_amd import _lib
    from mlx_amd.ops import _DTYPE_CODE, _MODE_CODE

    lib = _lib.load()
    g = torch.Generator().manual_seed(91)
    E, N, K, T = 8, 300, 256, 40
    w = torch.randn((E + 1, N, K), generator=g).to(dtype)
    x = torch.randn((T, 1, K), generator=g).to(dtype)
    wq_all, sc_all = mlx_amd.quantize(w.to(gpu), mode=mode)
    wq, scales = wq_all[1:], sc_all[1:]  # a view that starts at the second expert
    n_pairs = 900
    lhs = torch.randint(0, T, (n_pairs,), generator=g, dtype=torch.int32)
    # expert 3 gets no pair, expert 5 about 400 of them
    rhs = torch.tensor([0, 1, 2, 4, 6, 7], dtype=torch.int32)[
        torch.randint(0, 6, (n_pairs,), generator=g)]
    rhs[::2][:400] = 5
    lhs[17], rhs[18] = T + 3, E  # out of range
    assert lib.mlxrocm_fp_gather_qmm_workspace_size(
        1, N, K, n_pairs, E, 1, _MODE_CODE[mode], _DTYPE_CODE[dtype], 1) > 0
    got = mlx_amd.gather_qmm(x.to(gpu), wq, scales, None, lhs.to(gpu), rhs.to(gpu), mode=mode)
    assert got.shape == (n_pairs, 1, N) and got.dtype == dtype
    assert float(got[17].abs().max()) == 0.0 and float(got[18].abs().max()) == 0.0
    w_hat = fp_qref.exact_fp_weights(wq.cpu(), scales.cpu(), mode)  # [E, N, K]
    ok = torch.ones(n_pairs, dtype=torch.bool)
    ok[17] = ok[18] = False
    li, ri = lhs[ok].long(), rhs[ok].long()
    want = torch.einsum("pk,pnk->pn", x[li, 0].double(), w_hat[ri])
    mag = torch.einsum("pk,pnk->pn", x[li, 0].double().abs(), w_hat[ri].abs()) + 1e-30
    half_ulp = {torch.float16: 2.0 ** -11, torch.bfloat16: 2.0 ** -8}[dtype]
    err = ((got[ok, 0].cpu().double() - want).abs() / mag).max().item()
    assert err <= ACC_TOL[dtype] + half_ulp, (mode, dtype, err)
    # the same pairs without a workspace: one streaming product per pair
    xg, out = x.to(gpu).contiguous(), torch.empty((n_pairs, 1, N), dtype=dtype, device=gpu)
    lhs_u, rhs_u = lhs.to(gpu).view(torch.uint32), rhs.to(gpu).view(torch.uint32)
    _lib.check(lib.mlxrocm_fp_gather_qmm(
        xg.data_ptr(), wq.data_ptr(), scales.data_ptr(), lhs_u.data_ptr(), rhs_u.data_ptr(),
        out.data_ptr(), 1, N, K, n_pairs, T, E, K, wq.stride(0), scales.stride(0),
        _MODE_CODE[mode], _DTYPE_CODE[dtype], 1, None, 0, torch.cuda.current_stream().cuda_stream))
    perr = ((out[ok, 0].cpu().double() - got[ok, 0].cpu().double()).abs() / mag).max().item()
    assert perr <= 2 * (ACC_TOL[dtype] + half_ulp), (mode, dtype, perr)
    assert float(out[17].abs().max()) == 0.0 and float(out[18].abs().max()) == 0.0
    # sorted indices, and fewer pairs than the rule asks for (not grouped): same answers
    order = torch.argsort(rhs.long() * T + lhs.long())
    got_sorted = mlx_amd.gather_qmm(x.to(gpu), wq, scales, None, lhs[order].to(gpu),
                                    rhs[order].to(gpu), mode=mode, sorted_indices=True)
    assert torch.equal(got_sorted, got[order.to(gpu)])
    assert lib.mlxrocm_fp_gather_qmm_workspace_size(
        1, N, K, 24, E, 1, _MODE_CODE[mode], _DTYPE_CODE[dtype], 1) == 0
    few = mlx_amd.gather_qmm(x.to(gpu), wq, scales, None, lhs[:24].to(gpu), rhs[:24].to(gpu), mode=mode)
    ferr = ((few[ok[:24], 0].cpu().double() - got[:24][ok[:24], 0].cpu().double()).abs()
            / mag[: int(ok[:24].sum())]).max().item()
    assert ferr <= 2 * (ACC_TOL[dtype] + half_ulp), (mode, dtype, ferr)


@pytest.mark.parametrize("mode", ("mxfp4", "nvfp4"))
def test_gather_qqmm_grouped_by_expert(fp_oracle, gpu, mode):
    """gather_qqmm with enough pairs for the grouped route (nvfp4 with both
    tensor-wide scales): every pair against float64 of x_hat times the decoded
    expert."""
    dtype = torch.bfloat16
    g = torch.Generator().manual_seed(92)
    E, N, K, T = 4, 96, 128, 64
    w = torch.randn((E, N, K), generator=g).to(dtype)
    x = torch.randn((T, 1, K), generator=g).to(dtype)
    use_global = mode == "nvfp4"
    gx = x.float().abs().max() if use_global else None
    gw = w.float().abs().max() if use_global else None
    wq, scales = mlx_amd.quantize(w.to(gpu), mode=mode,
                                  **(dict(global_scale=gw.to(gpu)) if use_global else {}))
    lhs = torch.arange(T, dtype=torch.int32).repeat_interleave(2)
    rhs = torch.randint(0, E, (2 * T,), generator=g, dtype=torch.int32)
    kw = dict(global_scale_x=gx.to(gpu), global_scale_w=gw.to(gpu)) if use_global else {}
    got = mlx_amd.gather_qqmm(x.to(gpu), wq, scales, lhs.to(gpu), rhs.to(gpu), mode=mode, **kw)
    assert got.shape == (2 * T, 1, N) and got.dtype == dtype
    for i in range(2 * T):
        xi, e = x[int(lhs[i])], int(rhs[i])
        if use_global:
            want, mag = fp_qref.nvfp4_global_qqmm_f64(xi, wq[e].cpu(), scales[e].cpu(),
                                                      float(gx), float(gw))
        else:
            x_hat = fp_oracle.quantize_dequantize(xi, mode).double()
            w_hat = fp_qref.exact_fp_weights(wq[e].cpu(), scales[e].cpu(), mode)
            want, mag = x_hat @ w_hat.T, x_hat.abs() @ w_hat.abs().T
        err = ((got[i].cpu().double() - want).abs() / (mag + 1e-30)).max().item()
        assert err <= ACC_TOL[dtype] + 2.0 ** -8, (mode, i, err)


def test_fp_gather_full_size_moe_prefill(gpu):
    """The expert-routed prefill at full size in mxfp4: 8 experts of
    [14336, 4096], 2048 tokens, top-2 (4096 pairs, grouped by expert).  Every
    pair against float64 on a spread of 384 output columns per expert, and
    invariance under a permutation of the pairs."""
    mode, dtype = "mxfp4", torch.bfloat16
    g = torch.Generator().manual_seed(93)
    E, N, K, T = 8, 14336, 4096, 2048
    wq = torch.empty((E, N, K // 8), dtype=torch.uint32, device=gpu)
    scales = torch.empty((E, N, K // 32), dtype=torch.uint8, device=gpu)
    for e in range(E):  # one expert at a time: the unquantized stack would be 940 MB
        w = (torch.randn((N, K), generator=g) * 0.05).to(dtype).to(gpu)
        wq[e], scales[e] = mlx_amd.quantize(w, mode=mode)
        del w
    x = torch.randn((T, 1, K), generator=g).to(dtype)
    lhs = torch.arange(T, dtype=torch.int32).repeat_interleave(2)
    rhs = torch.stack([torch.randperm(E, generator=g)[:2] for _ in range(T)]).reshape(-1).to(torch.int32)
    got = mlx_amd.gather_qmm(x.to(gpu), wq, scales, None, lhs.to(gpu), rhs.to(gpu), mode=mode)
    assert got.shape == (2 * T, 1, N) and got.dtype == dtype
    cols = torch.cat([torch.arange(0, 128), torch.arange(7000, 7128), torch.arange(N - 128, N)])
    xd = x[:, 0].double()
    for e in range(E):
        wq_e = wq[e].view(torch.int32)[cols.to(gpu)].cpu().view(torch.uint32)
        w_hat = fp_qref.exact_fp_weights(wq_e, scales[e][cols.to(gpu)].cpu(), mode)
        pairs = torch.nonzero(rhs == e).flatten()
        assert pairs.numel() > 256  # more than one tile of the grouped kernel
        xe = xd[lhs[pairs].long()]
        want = xe @ w_hat.T
        mag = xe.abs() @ w_hat.abs().T + 1e-30
        have = got[pairs.to(gpu), 0][:, cols.to(gpu)].cpu().double()
        err = ((have - want).abs() / mag).max().item()
        assert err <= ACC_TOL[dtype] + 2.0 ** -8, (e, err)
    perm = torch.randperm(2 * T, generator=g)
    again = mlx_amd.gather_qmm(x.to(gpu), wq, scales, None, lhs[perm].to(gpu), rhs[perm].to(gpu), mode=mode)
    assert torch.equal(again, got[perm.to(gpu)])
