"""Kernel choice and workspace sizing of mlxrocm_qmm / mlxrocm_gather_qmm,
checked without a GPU: mlxrocm_qmm_plan rehearses a call (same argument checks,
same dispatch table, same workspace claims) and records the launches instead of
issuing them.

* Over a grid of shapes, mlxrocm_qmm_workspace_size is exactly what the call
  claims: the rehearsal succeeds with that many bytes and is refused with one
  byte less (this also covers the rules that run two passes over one region).
* Every benchmark configuration of the path maps to the dispatch rule that the
  design document's table names for it.
"""
import itertools

import pytest

from mlx_amd import _lib

F32, F16, BF16 = _lib.FLOAT32, _lib.FLOAT16, _lib.BFLOAT16

ROWS = (1, 2, 3, 4, 5, 8, 9, 16, 17, 32, 33, 64, 65, 128, 255, 256, 512, 1024, 2048, 8192)
WEIGHTS = ((4096, 4096), (14336, 4096), (4096, 14336), (11008, 4096), (4096, 11008),
           (128256, 4096), (8192, 2048), (96, 384), (67, 512))


def _rules(plan):
    return [part[1:-1] for part in plan.split("+") if part.startswith("[")]


@pytest.mark.parametrize("dtype", (F32, F16, BF16))
@pytest.mark.parametrize("transpose", (True, False))
def test_workspace_size_is_what_the_call_claims(dtype, transpose):
    lib = _lib.load()
    names = {name for name, _ in _lib.dispatch_rules()}
    checked = with_scratch = 0
    for (n, k), M, bits, gs in itertools.product(WEIGHTS, ROWS, (2, 3, 4, 5, 6, 8), (32, 64, 128)):
        if (k if transpose else n) % gs:
            continue
        for L, batched in ((1, False), (3, True)):
            if L > 1 and M > 64:
                continue
            args = (M, n, k, L, int(batched), gs, bits, dtype, int(transpose))
            need = lib.mlxrocm_qmm_workspace_size(*args)
            rc, plan = _lib.qmm_plan(M, n, k, L, batched, gs, bits, dtype, transpose,
                                     workspace_bytes=need)
            assert rc == _lib.OK, (args, need, plan, _lib.last_error())
            rules = _rules(plan)
            assert rules and set(rules) <= names, (args, plan)
            assert plan.split("+")[-1][0] != "[", (args, plan)  # ends in a launch
            if need:
                with_scratch += 1
                rc, short = _lib.qmm_plan(M, n, k, L, batched, gs, bits, dtype, transpose,
                                          workspace_bytes=need - 1)
                assert rc == _lib.INVALID_ARGUMENT, (args, need, short)
            checked += 1
    assert checked > 1500 and with_scratch > 100


# (rule(s) taken, launches) for the benchmark configurations: x bf16 unless stated
BASELINE = (
    # Cfg1: float32 4096 x 4096, 4-bit group 64, one row
    (dict(M=1, N=4096, K=4096, dtype=F32), ["qmv_f32"], "qmv_f32"),
    # Cfg2: decode, gate/up and down projection, B in {1, 4, 8}
    (dict(M=1, N=14336, K=4096), ["qmv_stream"], "qmv_stream(rw=7,kw=1,rm=1)"),
    (dict(M=4, N=14336, K=4096), ["qmv_quad"], "qmv_quad(kw=4,sets=1)"),
    (dict(M=8, N=14336, K=4096), ["qmm_rows8"], "qmm_rows8(kw=4,slots=2)"),
    (dict(M=1, N=4096, K=14336), ["qmv_quad"], None),
    (dict(M=4, N=4096, K=14336), ["qmv_quad"], None),
    (dict(M=8, N=4096, K=14336), ["qmm_slab"], None),
    (dict(M=1, N=14336, K=4096, bits=8, group_size=128), ["qmv_stream"], None),
    (dict(M=4, N=14336, K=4096, bits=8, group_size=128), ["qmv_mfma"], None),
    (dict(M=8, N=14336, K=4096, bits=8, group_size=128), ["qmv_mfma"], None),
    (dict(M=1, N=4096, K=14336, bits=8, group_size=128), ["qmv_stream"], None),
    (dict(M=8, N=4096, K=14336, bits=8, group_size=128), ["qmv_wide"], None),
    # Cfg3: prefill
    (dict(M=2048, N=14336, K=4096), ["qmm_t_tile_sb_transposed"],
     "interleave_sb+qmm_t_tile(nt=7,pairs)"),
    (dict(M=8192, N=14336, K=4096, bits=8, group_size=128), ["qmm_t_tile_sb_transposed"],
     "interleave_sb+qmm_t_tile(nt=7,pairs)"),
    (dict(M=2048, N=4096, K=4096), ["qmm_t_tile_sb_transposed"], "interleave_sb+qmm_t_tile(nt=5,pairs)"),
    (dict(M=512, N=4096, K=14336), ["qmm_t_tile_sb_transposed"], None),
    # Cfg5: odd widths, group 32, both readings of the [4096, 11008] weight
    (dict(M=1, N=11008, K=4096, bits=3, group_size=32), ["qmv_f32"], "qmv_f32"),
    (dict(M=1024, N=11008, K=4096, bits=5, group_size=32), ["qmm_t_tile_sb_transposed"], None),
    (dict(M=1024, N=11008, K=4096, bits=6, group_size=32, dtype=F32), ["qmm_t_split_fp32"],
     None),
    (dict(M=1, N=11008, K=4096, bits=3, group_size=32, transpose=False),
     ["widen_codes", "qmv_n"], None),
    (dict(M=1024, N=11008, K=4096, bits=6, group_size=32, transpose=False),
     ["widen_codes", "qmm_n_tile"], None),
    (dict(M=1024, N=11008, K=4096, bits=2, group_size=32, transpose=False, dtype=F32),
     ["qmm_naive"], "qmm_naive_n"),
)


@pytest.mark.parametrize("shape,rules,launches", BASELINE)
def test_benchmark_shapes_take_the_documented_rule(shape, rules, launches):
    kw = dict(shape)
    rc, plan = _lib.qmm_plan(kw.pop("M"), kw.pop("N"), kw.pop("K"), **kw)
    assert rc == _lib.OK, _lib.last_error()
    assert _rules(plan) == rules, plan
    if launches is not None:
        assert "+".join(p for p in plan.split("+") if not p.startswith("[")) == launches, plan


@pytest.mark.parametrize("tokens,expect", (
    (1, "[qmv_stream]+qmv_stream(rw=7,kw=1,rm=1)"),
    (8, "qmm_slab_grouped(plans,tile=16,ranges=4)"),
    (64, "qmm_slab_grouped(plans,tile=32,ranges=4)"),
    (2048, "gather_group(fused)+qmm_t_tile_grouped"),
))
def test_expert_routed_shapes(tokens, expect):
    """Cfg4: 8 experts of [14336, 4096], top-2."""
    lib = _lib.load()
    pairs = 2 * tokens
    need = lib.mlxrocm_gather_qmm_workspace_size(1, 14336, 4096, pairs, 8, 64, 4, BF16, 1, 0)
    rc, plan = _lib.gather_qmm_plan(1, 14336, 4096, pairs, tokens, 8, workspace_bytes=need)
    assert rc == _lib.OK and plan == expect, (plan, _lib.last_error())


def test_rule_table_is_listed():
    rules = _lib.dispatch_rules()
    assert len(rules) == len({name for name, _ in rules}) >= 20
    assert rules[-1][0] == "qmm_naive"  # the floor matches everything
    assert all(evidence for _, evidence in rules)
    lib = _lib.load()
    assert lib.mlxrocm_qmm_rule_name(len(rules)) is None
    assert lib.mlxrocm_qmm_rule_name(-1) is None


# ---- floating-point modes -------------------------------------------------
FP_MODES = {"mxfp4": _lib.MXFP4, "mxfp8": _lib.MXFP8, "nvfp4": _lib.NVFP4}


def test_fp_qmm_workspace_size_is_exact_and_plans_name_the_kernels():
    """mlxrocm_fp_qmm / mlxrocm_fp_qqmm rehearsed on the CPU: the call goes
    through with exactly the workspace its size function names and is refused
    with one byte fewer; decode, prefill and qqmm shapes take the kernels the
    design notes name."""
    lib = _lib.load()
    for mode in FP_MODES.values():
        for dtype in (_lib.BFLOAT16, _lib.FLOAT16, _lib.FLOAT32):
            for transpose in (True, False):
                for (M, N, K, L, batched) in ((1, 14336, 4096, 1, False), (8, 4096, 14336, 1, False),
                                              (9, 14336, 4096, 1, False), (300, 1000, 256, 1, False),
                                              (2048, 14336, 4096, 1, False), (40, 96, 256, 3, True),
                                              (40, 96, 256, 3, False), (5, 64, 48, 1, False)):
                    if K % (16 if mode == _lib.NVFP4 else 32) or (not transpose and N % 32):
                        continue
                    need = lib.mlxrocm_fp_qmm_workspace_size(M, N, K, L, int(batched), mode, dtype,
                                                             int(transpose))
                    rc, plan = _lib.fp_qmm_plan(M, N, K, L, batched, mode, dtype, transpose, need)
                    assert rc == _lib.OK and plan, (mode, dtype, transpose, M, N, K, L, plan)
                    tiled = "fp_qmm_t_tile" in plan
                    assert tiled == (need > 0), (plan, need)
                    if need:
                        rc, _ = _lib.fp_qmm_plan(M, N, K, L, batched, mode, dtype, transpose, need - 1)
                        assert rc == _lib.INVALID_ARGUMENT
            for (M, N, K) in ((1, 14336, 4096), (15, 128, 256), (16, 128, 256), (8192, 14336, 4096),
                              (64, 128, 96)):
                if K % (16 if mode == _lib.NVFP4 else 32):
                    continue
                need = lib.mlxrocm_fp_qqmm_workspace_size(M, N, K, mode, dtype)
                assert need > 0
                rc, plan = _lib.fp_qqmm_plan(M, N, K, mode, dtype, need)
                assert rc == _lib.OK and plan
                rc, _ = _lib.fp_qqmm_plan(M, N, K, mode, dtype, need - 1)
                assert rc == _lib.INVALID_ARGUMENT

    bf16 = _lib.BFLOAT16
    for mode in FP_MODES.values():
        assert _lib.fp_qmm_plan(1, 14336, 4096, mode=mode)[1] == "fp_qmv16(mb=1)"
        assert _lib.fp_qmm_plan(8, 14336, 4096, mode=mode)[1] == "fp_qmv16(mb=4)"
        assert _lib.fp_qmm_plan(9, 14336, 4096, mode=mode)[1] == \
            "fp_scale_image+fp_qmm_t_tile(ksplit=4)+reduce_k_splits(4)"
        assert _lib.fp_qmm_plan(2048, 14336, 4096, mode=mode)[1] == "fp_scale_image+fp_qmm_t_tile(nt=7)"
        assert _lib.fp_qmm_plan(64, 14336, 4096, mode=mode, dtype=_lib.FLOAT32)[1] == "fp_qmv"
        assert _lib.fp_qmm_plan(64, 14336, 4096, mode=mode, transpose=False)[1] == "fp_qmm_n"
    assert _lib.fp_qmm_plan(5, 64, 48, mode=_lib.NVFP4)[1] == "fp_qmm_naive_t"
    # qqmm: block-scaled matrix instruction from 16 rows on, MX modes, K % 128 == 0
    assert _lib.fp_qqmm_plan(8192, 14336, 4096, _lib.MXFP4, bf16)[1] == \
        "fp_quantize_activations+qq_mfma(e2m1)"
    assert _lib.fp_qqmm_plan(8192, 14336, 4096, _lib.MXFP8, bf16)[1] == \
        "fp_quantize_activations+qq_mfma(e4m3)"
    assert _lib.fp_qqmm_plan(16, 128, 256, _lib.MXFP4, _lib.FLOAT32)[1] == \
        "fp_quantize_activations+qq_mfma(e2m1)"
    # 8-bit codes in float32 stay on the fp32-accumulating kernels
    assert _lib.fp_qqmm_plan(8192, 14336, 4096, _lib.MXFP8, _lib.FLOAT32)[1] == \
        "fp_quantize_dequantize+fp_qmv"
    # fewer than 16 rows: x_hat in the element type, then quantized_matmul's kernels
    assert _lib.fp_qqmm_plan(15, 128, 256, _lib.MXFP4, bf16)[1] == \
        "fp_quantize_dequantize+fp_scale_image+fp_qmm_t_tile(nt=5)"
    assert _lib.fp_qqmm_plan(8, 128, 256, _lib.MXFP4, bf16)[1] == "fp_quantize_dequantize+fp_qmv16(mb=4)"
    assert _lib.fp_qqmm_plan(64, 128, 96, _lib.MXFP4, bf16)[1].startswith("fp_quantize_dequantize+")
    assert _lib.fp_qqmm_plan(8192, 14336, 4096, _lib.NVFP4, bf16)[1] == \
        "fp_quantize_dequantize+fp_scale_image+fp_qmm_t_tile(nt=7)"


def test_no_valid_shape_is_refused():
    """A seeded random walk over valid shapes -- rows of x from 1 to 300,000, N from
    1 to 70,001, ragged K with [K, N] weights, stacks of matrices, every width,
    group size, element type and fp mode -- through the rehearsal of the entry
    points: every call is accepted (shapes the kernels cannot take in one launch
    are cut up on the host, never refused)."""
    import random

    from mlx_amd import _lib

    rnd = random.Random(1)
    rows = (1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 31, 32, 33, 63, 64, 65, 100, 127, 128, 129, 255,
            256, 257, 500, 1000, 2048, 4097, 70000, 300000)
    outer = (1, 2, 3, 5, 7, 8, 9, 31, 32, 33, 64, 67, 100, 127, 128, 255, 256, 1000, 4096, 11008,
             32840, 70001)
    inner = (1, 2, 3, 5, 7, 8, 9, 31, 32, 33, 64, 67, 100, 127, 128, 255, 256, 1000, 4096, 11008)

    def quantized_dim(gs):
        return gs * rnd.randint(1, max(1, rnd.choice((128, 512, 4096, 16384)) // gs))

    refused = []
    for _ in range(6000):
        transpose = rnd.random() < 0.6
        M, L = rnd.choice(rows), rnd.choice((1, 1, 1, 2, 3, 8))
        batched = L > 1 and rnd.random() < 0.5
        dtype = rnd.choice((_lib.FLOAT32, _lib.FLOAT16, _lib.BFLOAT16))
        if rnd.random() < 0.6:
            gs, bits = rnd.choice((32, 64, 128)), rnd.choice((2, 3, 4, 5, 6, 8))
            N, K = (rnd.choice(outer), quantized_dim(gs)) if transpose else \
                (quantized_dim(gs), rnd.choice(inner))
            rc, _ = _lib.qmm_plan(M, N, K, L, batched, gs, bits, dtype, transpose)
            case = ("affine", M, N, K, L, batched, gs, bits, dtype, transpose)
        else:
            mode = rnd.choice((_lib.MXFP4, _lib.MXFP8, _lib.NVFP4))
            gs = 16 if mode == _lib.NVFP4 else 32
            N, K = (rnd.choice(outer), quantized_dim(gs)) if transpose else \
                (quantized_dim(gs), rnd.choice(inner))
            rc, _ = _lib.fp_qmm_plan(M, N, K, L, batched, mode, dtype, transpose)
            case = ("fp", M, N, K, L, batched, mode, dtype, transpose)
            if rc == 0 and transpose and L == 1:
                rc, _ = _lib.fp_qqmm_plan(M, N, K, mode, dtype)
        if rc != 0:
            refused.append((case, _lib.last_error()))
    assert not refused, refused[:5]
