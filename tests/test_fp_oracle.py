"""Pins the CPU oracle of the floating-point quantization modes (oracle/fp_qref.c)
against the reference's own translation unit where that can compute the same
thing through raw pointers, and against the definition of the formats
elsewhere.  CPU only."""
import itertools
import struct

import pytest
import torch

from oracle import build as obuild
from oracle import fp_qref, qref

MODES = ("mxfp4", "mxfp8", "nvfp4")
DTYPES = (torch.float32, torch.float16, torch.bfloat16)


@pytest.fixture(scope="module")
def port():
    obuild.build_qref()
    return fp_qref.FpOracle("port")


@pytest.fixture(scope="module")
def ref():
    if not obuild.reference_available():
        pytest.skip("no reference checkout to compile the translation unit from")
    obuild.build_ref()
    return fp_qref.FpOracle("reference")


def _floats(n, seed):
    g = torch.Generator().manual_seed(seed)
    mag = torch.exp(torch.rand(n, generator=g) * 24.0 - 16.0)
    return (mag * torch.sign(torch.randn(n, generator=g))).tolist()


def test_e4m3_decoding_of_every_code(port, ref):
    table = fp_qref._e4m3_values()
    for c in range(256):
        assert port.port.fpq_from_fp8(c) == ref.ref.ref_from_fp8(c)
        assert port.port.fpq_from_fp8(c) == float(table[c]) or (c & 0x7F) == 0


def test_e4m3_encoding_matches_the_reference(port, ref):
    # every e4m3 value, every midpoint between neighbours, and random floats
    table = sorted(set(abs(float(v)) for v in fp_qref._e4m3_values()))
    probes = list(table) + [(a + b) / 2 for a, b in zip(table, table[1:])]
    probes += [448.0, 464.0, 465.0, 479.9, 480.0, 1e6, 2.0 ** -10, 2.0 ** -11, 0.0]
    probes += _floats(20000, 1)
    for v in probes:
        for x in (v, -v):
            f = struct.unpack("f", struct.pack("f", x))[0]
            assert port.port.fpq_to_fp8(f) == ref.ref.ref_to_fp8(f), f


def test_e8m0_and_e2m1_helpers_match_the_reference(port, ref):
    grid = [0.0, 0.25, 0.5, 0.75, 1.0, 1.25, 1.5, 1.75, 2.0, 2.5, 3.0, 3.5, 4.0, 5.0, 6.0, 7.0]
    eps = [0.0, 1e-6, -1e-6]
    for v, e in itertools.product(grid, eps):
        for x in (v + e, -(v + e)):
            assert port.port.fpq_e2m1(x) == ref.ref.ref_e2m1(x), x
    for x in _floats(5000, 2) + [2.0 ** k for k in range(-130, 130, 7)] + [float("inf"), -1.0]:
        assert port.port.fpq_e8m0(x) == ref.ref.ref_e8m0(x), x
        assert port.port.fpq_e2m1(x) == ref.ref.ref_e2m1(x), x


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("transpose", (True, False))
def test_matmul_matches_the_reference_byte_for_byte(port, ref, mode, dtype, transpose):
    gs = fp_qref.GROUP_SIZE[mode]
    for M, N, K in ((1, 64, 256), (3, 96, 128), (5, 2 * gs, 3 * gs)):
        g = torch.Generator().manual_seed(M * N + K)
        w = (torch.randn((N, K) if transpose else (K, N), generator=g) * 0.3).to(dtype)
        wq, scales = port.quantize(w, mode)
        x = torch.randn((M, K), generator=g).to(dtype)
        mine = port.qmm(x, wq, scales, mode, transpose)
        theirs = ref.qmm(x, wq, scales, mode, transpose)
        assert torch.equal(qref_raw(mine), qref_raw(theirs)), (M, N, K)


def qref_raw(t):
    return t.view(torch.int32 if t.element_size() == 4 else torch.int16)


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_values_on_the_grid_round_trip_exactly(port, mode, dtype):
    # python/tests/test_quantized.py:41-66, 96-122, 124-150: weights drawn from the
    # format's own values, with the group's largest magnitude present, come back
    g = torch.Generator().manual_seed(3)
    if mode == "mxfp8":
        codes = torch.randint(0, 256, (64, 256), generator=g)
        codes = codes[(codes & 0x7F) != 0x7F].reshape(-1)[: 64 * 224].reshape(64, 224)
        w = fp_qref._e4m3_values()[codes].float()
        w = w.reshape(-1, 32)
        w[:, 0] = 448.0
        w = w.reshape(64, 224)
    else:
        w = torch.tensor(fp_qref.FP4_VALUES)[torch.randint(0, 16, (64, 256), generator=g)]
        w = w.reshape(-1, fp_qref.GROUP_SIZE[mode])
        w[:, 0] = 6.0
        w = w.reshape(64, 256)
    w = w.to(dtype)
    wq, scales = port.quantize(w, mode)
    assert wq.shape[-1] == w.shape[-1] * fp_qref.BITS[mode] // 32
    assert scales.shape[-1] == w.shape[-1] // fp_qref.GROUP_SIZE[mode]
    w_hat = port.dequantize(wq, scales, mode, dtype)
    assert torch.equal(w_hat.float(), w.float())
    assert torch.equal(fp_qref.exact_fp_weights(wq, scales, mode), w.double())


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_quantize_picks_the_nearest_value_and_dequantize_is_exact(port, mode, dtype):
    g = torch.Generator().manual_seed(11)
    w = (torch.randn((48, 512), generator=g) * 0.02).to(dtype)
    wq, scales = port.quantize(w, mode)
    exact = fp_qref.exact_fp_weights(wq, scales, mode)
    # dequantize forms exact products in every element type
    assert torch.equal(port.dequantize(wq, scales, mode, dtype).double(), exact)
    assert torch.equal(port.dequantize(wq, scales, mode, torch.float32).double(), exact)
    # every code is a nearest value of its format to w / scale (float32 input:
    # no intermediate of the op graph is rounded beyond float32)
    if dtype == torch.float32:
        gs = fp_qref.GROUP_SIZE[mode]
        if mode == "nvfp4":
            sv = fp_qref._e4m3_values()[scales.to(torch.int64)]
        else:
            sv = torch.pow(torch.tensor(2.0, dtype=torch.float64), scales.double() - 127.0)
        q = w.double() / sv.repeat_interleave(gs, dim=-1)
        chosen = exact / sv.repeat_interleave(gs, dim=-1)
        if fp_qref.BITS[mode] == 4:
            grid = torch.tensor(fp_qref.FP4_VALUES, dtype=torch.float64)
        else:
            grid = fp_qref._e4m3_values()[[c for c in range(256) if (c & 0x7F) < 0x7F]]
        best = (q.unsqueeze(-1) - grid).abs().amin(-1)
        assert bool(((q - chosen).abs() <= best * (1 + 1e-6) + 1e-9).all())
        # the scale is max / maxval to within a factor sqrt(2) (e8m0); e4m3 scales of
        # small groups are subnormal, so only a loose factor holds there
        wmax = w.double().reshape(-1, gs).abs().amax(-1)
        ratio = wmax / (6.0 if fp_qref.BITS[mode] == 4 else 448.0) / sv.reshape(-1)
        lo, hi = (0.6, 1.7) if mode == "nvfp4" else (2 ** -0.5001, 2 ** 0.5001)
        assert bool(((ratio >= lo) & (ratio <= hi)).all())
    # a zero group stays zero
    z = torch.zeros((2, 64), dtype=dtype)
    zq, zs = port.quantize(z, mode)
    assert float(port.dequantize(zq, zs, mode, dtype).abs().max()) == 0.0


@pytest.mark.parametrize("mode", MODES)
def test_quantize_agrees_with_the_fp32_rules_of_the_reference_away_from_ties(port, mode):
    """fp_quantize_dequantize (the translation unit's own fp32 formulation, used
    for qqmm) and dequantize(quantize(w)) (the op graph) give the same values
    for float32 data, where no intermediate is rounded and exact ties have
    measure zero."""
    g = torch.Generator().manual_seed(5)
    w = torch.randn((32, 256), generator=g) * 0.7
    a = port.quantize_dequantize(w, mode)
    wq, scales = port.quantize(w, mode)
    b = port.dequantize(wq, scales, mode, torch.float32)
    mismatch = float((a != b).float().mean())
    assert mismatch < 0.002, mismatch


@pytest.mark.parametrize("mode", MODES)
def test_matmul_equals_the_dense_product(port, mode):
    g = torch.Generator().manual_seed(9)
    for transpose in (True, False):
        N, K, M = 64, 128, 4
        w = torch.randn((N, K) if transpose else (K, N), generator=g) * 0.1
        wq, scales = port.quantize(w, mode)
        x = torch.randn((M, K), generator=g)
        y = port.port_qmm(x, wq, scales, mode, transpose).double()
        w_hat = fp_qref.exact_fp_weights(wq, scales, mode)
        exact = x.double() @ (w_hat.T if transpose else w_hat)
        assert float((y - exact).abs().max()) <= 1e-5 * (K ** 0.5) * float(x.abs().max()) * float(
            w_hat.abs().max())


# ---- golden vectors written by the reference translation unit -------------
# (tests/golden/make_fp_golden.py); these pin the port where the reference
# checkout, and with it oracle/_ref, is absent.
@pytest.fixture(scope="module")
def golden():
    import numpy as np
    import os

    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fp_modes_ref.npz")
    return np.load(path, allow_pickle=False)


def test_converters_match_the_golden_vectors(port, golden):
    import numpy as np

    for c in range(256):
        got = np.array([port.port.fpq_from_fp8(c)], dtype=np.float32).view(np.uint32)[0]
        assert got == golden["from_fp8"][c], c
    probes = golden["probe_bits"]
    assert probes.size > 12000
    for u, want8, want_e, want4 in zip(probes, golden["to_fp8"], golden["e8m0"], golden["e2m1"]):
        f = struct.unpack("f", struct.pack("I", int(u)))[0]
        assert port.port.fpq_to_fp8(f) == want8, f
        assert port.port.fpq_e8m0(f) == want_e, f
        assert port.port.fpq_e2m1(f) == want4, f


@pytest.mark.parametrize("mode", MODES)
@pytest.mark.parametrize("dname", ("f32", "f16", "bf16"))
@pytest.mark.parametrize("transpose", (True, False))
def test_matmul_matches_the_golden_vectors(port, golden, mode, dname, transpose):
    import numpy as np

    dtype = {"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dname]
    tag = f"{mode}_{dname}_{'t' if transpose else 'n'}"

    def tensor(name, dt):
        a = golden[tag + name]
        if dt in (torch.uint32, torch.uint8):
            return torch.from_numpy(a.copy())
        return torch.from_numpy(a.view(np.int32 if dt == torch.float32 else np.int16).copy()).view(dt)

    wq = tensor("_wq", torch.uint32)
    scales = tensor("_scales", torch.uint8)
    x = tensor("_x", dtype)
    want = tensor("_y", dtype)
    got = port.port_qmm(x, wq, scales, mode, transpose)
    assert torch.equal(qref_raw(got), qref_raw(want)), tag


# ---- nvfp4 with a tensor-wide scale (numpy restatement of the CUDA kernels) ----

def test_global_scale_converters_match_the_port_and_the_definition(port):
    """The numpy e4m3 / e2m1 rounding used by the tensor-wide-scale functions
    against the C port (itself checked against the reference's converters) and
    against the formats' definition: no table entry is nearer."""
    import numpy as np

    rs = np.random.RandomState(3)
    vals = np.abs(rs.randn(4000).astype(np.float32)) * np.exp(rs.randn(4000).astype(np.float32) * 3)
    table = fp_qref._e4m3_values()[:127].numpy()
    mid = ((table[:-1] + table[1:]) / 2).astype(np.float32)
    vals = np.concatenate([vals, table.astype(np.float32), mid, np.float32([0, 447.9, 448, 464, 1e9])])
    mine = fp_qref.e4m3_round(vals)
    theirs = np.array([port.port.fpq_to_fp8(float(v)) for v in vals], dtype=np.uint8)
    assert np.array_equal(mine, theirs)
    err = np.abs(table[mine] - np.minimum(vals, 448).astype(np.float64))
    assert np.all(err <= np.abs(table[None, :] - np.minimum(vals, 448)[:, None]).min(axis=1))

    v4 = np.concatenate([
        (rs.randn(4000) * 3).astype(np.float32),
        np.float32([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5, -0.25, -0.75, -5, 7, -7, 0, -0.0,
                    np.inf, -np.inf, np.nan])])
    mine = fp_qref.e2m1_round(v4)
    theirs = np.array([port.port.fpq_e2m1(float(v)) for v in v4], dtype=np.uint8)
    assert np.array_equal(mine, theirs)
    # ties go to the code with an even mantissa bit
    assert list(fp_qref.e2m1_round(np.float32([0.25, 0.75, 1.25, 1.75, 2.5, 3.5, 5]))) == \
        [0, 2, 2, 4, 4, 6, 6]


@pytest.mark.parametrize("dtype", DTYPES)
def test_global_scale_quantize_picks_nearest_codes_and_round_trips(dtype):
    """Every code is a nearest e2m1 value of w * scale_enc / scale (float64 check,
    independent of the rounding routine); the scale byte is the nearest e4m3 of
    amax / 6 * scale_enc; dequantize inverts up to the two fp32 roundings."""
    import numpy as np

    g = torch.Generator().manual_seed(9)
    w = (torch.randn(32, 256, generator=g) * torch.exp(torch.randn(32, 1, generator=g))).to(dtype)
    w[3, :16] = 0
    gs = float(w.float().abs().max())
    wq, scales = fp_qref.nvfp4_global_quantize(w, gs)
    assert wq.shape == (32, 32) and scales.shape == (32, 16)
    scale_enc = np.float32(np.float32(2688.0) / np.float32(gs))
    amax = w.float().reshape(32, 16, 16).abs().amax(-1).numpy()
    want = np.float32(np.float32(amax / np.float32(6)) * scale_enc)
    table = fp_qref._e4m3_values()[:127].numpy()
    sv = table[scales.numpy()]
    assert np.all(np.abs(sv - want) <= np.abs(table[None, None, :] - want[..., None]).min(-1))
    raw = wq.view(torch.uint8).numpy()
    codes = np.stack((raw & 0xF, raw >> 4), -1).reshape(32, 16, 16)
    vals = np.array(fp_qref.FP4_VALUES)[codes]
    live = sv > 0
    scaled = w.float().reshape(32, 16, 16).numpy().astype(np.float64) * \
        np.float32(scale_enc / np.where(live, sv, 1).astype(np.float32))[..., None]
    grid = np.array(fp_qref.FP4_VALUES[:8] + tuple(-v for v in fp_qref.FP4_VALUES[:8]))
    best = np.abs(grid[None, None, None, :] - np.clip(scaled, -6, 6)[..., None]).min(-1)
    # the kernels round the product to float32 before they pick the code: a product
    # within an fp32 ulp of a midpoint may take either neighbour
    slack = 2.0 ** -22 * np.abs(scaled)
    assert np.all((np.abs(vals - np.clip(scaled, -6, 6)) <= best + slack)[live])
    # a group of zeros: scale byte 0, decodes to zeros whatever the codes are
    assert scales[3, 0] == 0
    back = fp_qref.nvfp4_global_dequantize(wq, scales, gs, dtype)
    assert torch.all(back[3, :16] == 0)
    # half a code step at the top of the range (1 of 6) plus the e4m3 rounding of the scale
    err = (back.float() - w.float()).reshape(32, 16, 16).abs().amax(-1)
    assert torch.all(err <= torch.from_numpy(amax) * (1 / 6 + 1 / 16) + 1e-30)


def test_global_scale_round_trip_of_the_reference_test(port):
    """python/tests/test_quantized.py:124-190: table values with a 6 in every
    group, + 3e-6, bfloat16; with global_scale = max |w| the round trip is within
    1e-5 (the assertion of the reference's test)."""
    g = torch.Generator().manual_seed(1)
    lut = torch.tensor(fp_qref.FP4_VALUES)
    w = lut[torch.randint(0, 16, (128, 512), generator=g)].reshape(-1, 16)
    w[:, 0] = 6
    w = (w + 3e-6).to(torch.bfloat16).reshape(128, 512)
    gs = float(w.float().abs().max())
    wq, scales = fp_qref.nvfp4_global_quantize(w, gs)
    back = fp_qref.nvfp4_global_dequantize(wq, scales, gs, torch.bfloat16)
    assert torch.allclose(w.float(), back.float(), rtol=1e-5, atol=1e-5)
    zeros = torch.zeros(8, 64)
    wq, scales = fp_qref.nvfp4_global_quantize(zeros, 1.0)
    assert torch.all(fp_qref.nvfp4_global_dequantize(wq, scales, 1.0) == 0)


@pytest.mark.parametrize("dtype", DTYPES)
def test_global_scale_reduces_to_the_reference_rules_for_power_of_two_scales(port, dtype):
    """With global_scale = 448 * 6 the encode scale is 1, and for groups whose
    maximum is 6 * 2^k every intermediate is exact: quantize-dequantize must then
    equal the reference's CPU fp_quantize_dequantize (same e4m3 scale, same
    ties-to-even codes)."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(64, 128, generator=g).reshape(-1, 16)
    x = x / x.abs().amax(-1, keepdim=True) * 6  # every group's maximum is 6 ...
    x = x * torch.exp2(torch.randint(-4, 5, (x.shape[0], 1), generator=g).float())  # ... times 2^k
    x = x.reshape(64, 128).to(dtype)
    amax = x.float().reshape(-1, 16).abs().amax(-1)
    assert torch.all(torch.log2(amax / 6) == torch.round(torch.log2(amax / 6)))
    got = fp_qref.nvfp4_global_quantize_dequantize(x, 2688.0)
    want = port.quantize_dequantize(x, "nvfp4")
    assert torch.equal(got.float(), want.float())
    # and the codes / scale bytes equal those of dequantize(quantize()) at that scale
    wq, scales = fp_qref.nvfp4_global_quantize(x, 2688.0)
    assert torch.equal(fp_qref.nvfp4_global_dequantize(wq, scales, 2688.0, dtype).float(), got.float())
