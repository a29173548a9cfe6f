"""Shared helpers of the parity tests: seeded synthetic inputs of the benchmark
configurations, raw-bit comparison, and the matmul tolerances."""
from __future__ import annotations

import math

import torch

ALL_BITS = (2, 3, 4, 5, 6, 8)
ALL_GROUPS = (32, 64, 128)
DTYPES = (torch.float32, torch.float16, torch.bfloat16)


def raw(t: torch.Tensor) -> torch.Tensor:
    """Integer view of a tensor's storage, for bit-exact comparisons."""
    t = t.contiguous()
    if t.dtype == torch.uint32:
        return t.view(torch.int32)
    if t.element_size() == 2:
        return t.view(torch.int16)
    if t.element_size() == 4:
        return t.view(torch.int32)
    raise TypeError(t.dtype)


def bits_equal(a: torch.Tensor, b: torch.Tensor) -> bool:
    return a.shape == b.shape and a.dtype == b.dtype and torch.equal(raw(a.cpu()), raw(b.cpu()))


def count_mismatch(a: torch.Tensor, b: torch.Tensor) -> int:
    return int((raw(a.cpu()) != raw(b.cpu())).sum())


def normal_weights(shape, dtype, seed=0, std=0.02):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g, dtype=torch.float32) * std).to(dtype)


def student_t_weights(shape, dtype, seed=0, df=3, scale=0.02):
    """Heavy-tailed weights: Student-t(df) = N(0,1) / sqrt(chi2(df)/df)."""
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(shape, generator=g, dtype=torch.float32)
    chi2 = torch.zeros(shape, dtype=torch.float32)
    for _ in range(df):
        chi2 += torch.randn(shape, generator=g, dtype=torch.float32) ** 2
    return (z / torch.sqrt(chi2 / df) * scale).to(dtype)


def activations(shape, dtype, seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float32).to(dtype)


def matmul_tolerance(dtype, K, x, w_hat):
    """north-star bound: max|err| <= c * sqrt(K) * max|x| * max|w|, c = 1e-5
    for float32 and 2e-2 for the 16-bit types (the CPU reference accumulates
    in the element type, so its own rounding noise grows with sqrt(K))."""
    c = 1e-5 if dtype == torch.float32 else 2e-2
    return c * math.sqrt(K) * float(x.abs().max()) * float(w_hat.abs().max())


def exact_affine_weights(wq, scales, biases, group_size, bits):
    """fp64 s*q+b from the packed words, with no intermediate rounding."""
    from oracle.qref import unpack_codes

    codes = unpack_codes(wq.cpu(), bits).double()
    s = scales.cpu().double().repeat_interleave(group_size, dim=-1)
    b = biases.cpu().double().repeat_interleave(group_size, dim=-1)
    return codes * s + b


def exact_tolerance(dtype, K, x, w_hat, y_exact):
    """Bound against the fp64 product: output rounding of the element type plus
    fp32 accumulation noise."""
    eps_out = {torch.float32: 2.0**-23, torch.float16: 2.0**-10, torch.bfloat16: 2.0**-7}[dtype]
    acc = 2e-6 * math.sqrt(K) * float(x.abs().max()) * float(w_hat.abs().max())
    return eps_out * float(y_exact.abs().max()) + acc


def exact_affine_weights_on(device, wq, scales, biases, group_size, bits, chunk_rows=512):
    """fp64 s*q+b from the packed words by the bit-stream definition, computed
    with plain torch on `device` in chunks of rows (the bit expansion takes
    256 bytes per packed word).  Returns [..., rows, K] float64 on `device`."""
    wq = wq.to(device).contiguous()
    lead, rows, words = tuple(wq.shape[:-2]), wq.shape[-2], wq.shape[-1]
    K = words * 32 // bits
    flat = wq.reshape(-1, words).view(torch.int32)
    s = scales.to(device).reshape(-1, K // group_size)
    b = biases.to(device).reshape(-1, K // group_size)
    shifts = torch.arange(32, dtype=torch.int32, device=device)
    weights = (1 << torch.arange(bits, dtype=torch.int32, device=device))
    out = torch.empty((flat.shape[0], K), dtype=torch.float64, device=device)
    for r0 in range(0, flat.shape[0], chunk_rows):
        w = flat[r0:r0 + chunk_rows]
        stream = (w.unsqueeze(-1) >> shifts) & 1  # [rows, words, 32] bits, LSB first
        codes = (stream.reshape(w.shape[0], K, bits) * weights).sum(-1).double()
        sc = s[r0:r0 + chunk_rows].double().repeat_interleave(group_size, dim=-1)
        bi = b[r0:r0 + chunk_rows].double().repeat_interleave(group_size, dim=-1)
        out[r0:r0 + chunk_rows] = codes * sc + bi
    return out.reshape(lead + (rows, K))


def exact_product_error(got, x, w_hat, transpose=True, block=1024):
    """max |got - x @ w_hat(.T)| over every row, fp64 product with torch on the
    device of `w_hat` in blocks of rows; also returns max |exact|."""
    dev = w_hat.device
    wt = w_hat.T if transpose else w_hat
    err = 0.0
    top = 0.0
    for r0 in range(0, x.shape[0], block):
        exact = x[r0:r0 + block].to(dev).double() @ wt
        err = max(err, float((got[r0:r0 + block].to(dev).double() - exact).abs().max()))
        top = max(top, float(exact.abs().max()))
    return err, top


def exact_tolerance_from(dtype, K, x_absmax, w_absmax, y_absmax):
    eps_out = {torch.float32: 2.0**-23, torch.float16: 2.0**-10, torch.bfloat16: 2.0**-7}[dtype]
    return eps_out * y_absmax + 2e-6 * math.sqrt(K) * x_absmax * w_absmax
