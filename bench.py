#!/usr/bin/env python3
"""Benchmark of the affine quantized-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only qmv|qmm_t] [--sweep]

One "step" is one launch of the decode GEMV (qmv) of the Llama-3-8B gate/up
projection: x bf16 [1, 4096] against W [14336, 4096] quantized to 4 bits,
group 64, bf16 scales/biases.  The launches cycle through a ring of distinct
weight copies (> 512 MB in total) so that the 256 MB Infinity Cache cannot hold
the working set and the figure is HBM bandwidth.  Inputs are resident in HBM
before the timed region starts.  The prefill GEMM (qmm_t, M = 2048, same
weight) is measured in the same run and reported in the "qmm_t" object.

Prints ONE JSON line (see the keys below).  `roofline.achieved` comes from HIP
events recorded on the launch stream around the timed launches.
"""
from __future__ import annotations

import argparse
import ctypes
import json
import os
import sys
import time

HBM_PEAK_GBPS = 8000.0
BF16_PEAK_TFLOPS = 2500.0
FP4_PEAK_TFLOPS = 10100.0
# HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counter passes, scaled by
# a copy of known size (profiles/qmv_stream_4bit_g64_bf16_14336x4096.md and
# profiles/qmm_t_mfma_4bit_g64_bf16_M2048_14336x4096.md).
QMV_TRAFFIC_BYTES = 33225728
QMV_TRAFFIC_SOURCE = "profiles/qmv_stream_4bit_g64_bf16_14336x4096.md"
QMM_T_TRAFFIC_BYTES = 259209114
QMM_T_TRAFFIC_SOURCE = "profiles/qmm_t_mfma_4bit_g64_bf16_M2048_14336x4096.md"

N, K = 14336, 4096
BITS, GS = 4, 64
QMM_M = 2048
RING = 18  # 18 x 33 MB = 595 MB of weights > 2 x the 256 MB Infinity Cache


def qmv_bytes(M: int, n: int, k: int, bits: int, gs: int, esize: int) -> int:
    """Algorithmic bytes of one qmv launch: packed codes + scales + biases + x + out."""
    return n * k * bits // 8 + 2 * n * (k // gs) * esize + M * k * esize + M * n * esize


class Launcher:
    """Issues launches of fn(i, stream) on one stream, either directly or by
    replaying HIP graphs: one graph holds a pass over the weight ring (the
    kernel is a few microseconds long, shorter than a Python-driven launch), a
    second one the remainder, so that any number of launches can be issued
    exactly."""

    def __init__(self, torch, fn, period: int, use_graph: bool):
        self.torch, self.fn, self.period = torch, fn, period
        self.stream = torch.cuda.Stream()
        self.use_graph = use_graph
        self.graphs = {}
        self.stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(self.stream):
            for i in range(period):
                fn(i, self.stream.cuda_stream)
        self.stream.synchronize()
        if use_graph:
            self._graph(period)

    def _graph(self, count: int):
        if count not in self.graphs:
            graph = self.torch.cuda.CUDAGraph()
            with self.torch.cuda.graph(graph, stream=self.stream):
                for i in range(count):
                    self.fn(i, self.torch.cuda.current_stream().cuda_stream)
            self.graphs[count] = graph
        return self.graphs[count]

    def prepare(self, steps: int) -> None:
        """Capture what run(steps) replays, outside any timed region."""
        if self.use_graph and steps % self.period:
            self._graph(steps % self.period)

    def run(self, steps: int) -> int:
        """Enqueue exactly `steps` launches."""
        with self.torch.cuda.stream(self.stream):
            if self.use_graph:
                full, rest = divmod(steps, self.period)
                ring = self._graph(self.period)
                tail = self._graph(rest) if rest else None
                for _ in range(full):
                    ring.replay()
                if tail is not None:
                    tail.replay()
                return steps
            for i in range(steps):
                self.fn(i, self.stream.cuda_stream)
            return steps


def hip_event_ms(lib, launcher: "Launcher", steps: int) -> float:
    """Milliseconds per launch, measured with HIP events recorded on the
    stream the kernels are launched on."""
    stream = launcher.stream.cuda_stream
    launcher.prepare(steps)
    start, stop = ctypes.c_void_p(), ctypes.c_void_p()
    assert lib.mlxrocm_event_create(ctypes.byref(start)) == 0
    assert lib.mlxrocm_event_create(ctypes.byref(stop)) == 0
    assert lib.mlxrocm_event_record(start, stream) == 0
    steps = launcher.run(steps)
    assert lib.mlxrocm_event_record(stop, stream) == 0
    assert lib.mlxrocm_event_synchronize(stop) == 0
    ms = ctypes.c_float()
    assert lib.mlxrocm_event_elapsed_ms(ctypes.byref(ms), start, stop) == 0
    lib.mlxrocm_event_destroy(start)
    lib.mlxrocm_event_destroy(stop)
    return ms.value / steps


# Timing protocol of the headline figures: after at least MIN_WARMUP untimed
# launches, REPEATS timed regions, HIP events around every region; the median
# region is the figure.  A qmv region is max(--steps, QMV_MIN_LAUNCHES) launches
# rounded up to whole passes over the weight ring: a graph replay costs a few
# microseconds of host time, and with only a handful of replays per region (plus
# a shorter tail graph) that cost showed up as 6-8 % on an 8 us kernel.  A
# qmm_t region (200 us per call, launched one by one) is at least MIN_LAUNCHES.
REPEATS = 7
QMV_MIN_LAUNCHES = 1800
MIN_LAUNCHES = 100
MIN_WARMUP = 10


def read_only_floor() -> dict | None:
    """Runs the read-only probe (mlx_amd/lib/read_probe --floor) in a child
    process and returns its figures: what a launch that only loads the decode
    weight's 33 MB costs in the same launch chain, what it costs from the
    cache, and what an empty grid costs.  Called before this process touches
    the GPU.  None when the probe is not built or fails."""
    import subprocess

    exe = os.path.join(os.path.dirname(os.path.abspath(__file__)), "mlx_amd", "lib", "read_probe")
    if not os.path.isfile(exe):
        return None
    try:
        proc = subprocess.run([exe, "--floor"], capture_output=True, text=True, timeout=120)
        if proc.returncode != 0:
            return None
        return json.loads(proc.stdout.strip().splitlines()[-1])
    except (OSError, ValueError, IndexError, subprocess.TimeoutExpired):
        return None


def median_event_ms(lib, launcher: "Launcher", launches: int, repeats: int = REPEATS):
    samples = sorted(hip_event_ms(lib, launcher, launches) for _ in range(repeats))
    return samples[len(samples) // 2], samples


def cpu_baseline(x_cpu, wq_cpu, s_cpu, b_cpu, nbytes: int) -> dict:
    """The CPU backend's qmv on one host core: the reference's own translation
    unit when oracle/_ref is built, else the C restatement.  A bounded sample:
    the first 2048 of the 14336 output rows, repeated for roughly 10 s."""
    from oracle import build as obuild
    from oracle import qref

    if not os.path.isfile(qref.QREF_SO):
        obuild.build_qref()
    kind = "reference" if qref.reference_built() else "port"
    orc = qref.Oracle(kind)
    rows = 2048
    wq_s, s_s, b_s = wq_cpu[:rows].contiguous(), s_cpu[:rows].contiguous(), b_cpu[:rows].contiguous()
    orc.qmm(x_cpu, wq_s, s_s, b_s, True, GS, BITS)  # warm-up
    reps, t0 = 0, time.perf_counter()
    while True:
        orc.qmm(x_cpu, wq_s, s_s, b_s, True, GS, BITS)
        reps += 1
        dt = time.perf_counter() - t0
        if dt > 10.0 or reps >= 200:
            break
    sec_per_full = dt / reps * (N / rows)
    return {
        "value": round(nbytes / sec_per_full / 1e9, 4),
        "unit": "GB/s",
        "cores": 1,
        "kind": kind,
        "sample": f"{rows} of {N} output rows x {reps} repetitions, scaled linearly "
                  f"to the full [{N},{K}] qmv; host has {os.cpu_count()} logical cores",
    }


def sweep(torch, mlx_amd, dev) -> list:
    """The other synthetic configurations of the path (prefill shapes, decode at
    batch 4 and 8, 8-bit, odd code widths, fp32, expert-routed gather, quantize
    and dequantize): one timing each, weights cycled through > 512 MB of copies
    wherever one launch reads less than that, so that figures are HBM figures."""
    rows = []
    g = torch.Generator().manual_seed(0)

    def timed(fn, min_ms=30.0):
        for _ in range(2):
            fn(0)
        torch.cuda.synchronize()
        reps, total = 4, 0.0
        while True:
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            e0.record()
            for i in range(reps):
                fn(i)
            e1.record()
            torch.cuda.synchronize()
            total = e0.elapsed_time(e1)
            if total >= min_ms or reps >= 4096:
                return total / reps
            reps *= 4

    def weights(n, k, dtype, std=0.02):
        return (torch.randn((n, k), generator=g, dtype=torch.float32) * std).to(dtype).to(dev)

    def ring_of(q, nbytes):
        copies = max(1, min(24, int(600e6 // max(nbytes, 1)) + 1))
        return [q] + [tuple(t.clone() for t in q) for _ in range(copies - 1)]

    def add(cfg, name, ms, nbytes=None, flops=None, kernel=None):
        row = {"config": cfg, "case": name, "us": round(ms * 1e3, 2)}
        if nbytes is not None:
            row["GB/s"] = round(nbytes / ms / 1e6, 1)
        if flops is not None:
            row["TFLOP/s"] = round(flops / ms / 1e9, 1)
        if kernel:
            row["kernel"] = kernel
        rows.append(row)
        print(json.dumps(row), file=sys.stderr, flush=True)

    def kname(M, n, k, gs, bits, dtype, transpose=True):
        from mlx_amd import _lib
        code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
        return _lib.load().mlxrocm_qmm_kernel_name(M, n, k, 1, gs, bits, code, int(transpose)).decode()

    def matmul_case(cfg, M, n, k, bits, gs, dtype, transpose=True):
        """One quantized_matmul shape through the C ABI.  Launches that last a few
        microseconds (M <= 64) replay a HIP graph over the weight ring, like the
        headline figure; the others are launched one by one.  transpose=False: the
        weight is [k, n] and quantized along n."""
        from mlx_amd import _lib
        lib = _lib.load()
        esz = 4 if dtype == torch.float32 else 2
        code = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}[dtype]
        q = mlx_amd.quantize(weights(n, k, dtype) if transpose else weights(k, n, dtype), gs, bits)
        wbytes = n * k * bits // 8 + 2 * n * (k // gs) * esz
        small = M <= 64
        ring = ring_of(q, wbytes) if small else [q]
        x = torch.randn((M, k), generator=g, dtype=torch.float32).to(dtype).to(dev)
        out = torch.empty((M, n), dtype=dtype, device=dev)
        ws_bytes = lib.mlxrocm_qmm_workspace_size(M, n, k, 1, 0, gs, bits, code, int(transpose))
        ws = torch.empty(max(int(ws_bytes), 16), dtype=torch.uint8, device=dev)

        def step(i, stream):
            wq_, s_, b_ = ring[i % len(ring)]
            rc = lib.mlxrocm_qmm(x.data_ptr(), wq_.data_ptr(), s_.data_ptr(), b_.data_ptr(),
                                 out.data_ptr(), M, n, k, 1, M * k, 0, 0, gs, bits, code,
                                 int(transpose), ws.data_ptr(), ws_bytes, stream)
            if rc != 0:
                raise RuntimeError(_lib.last_error())

        launcher = Launcher(torch, step, len(ring), small)
        launcher.run(len(ring))
        torch.cuda.synchronize()
        if small:
            ms = hip_event_ms(lib, launcher, max(len(ring) * 20, 10))
        else:
            # launches of 40 us to 1 ms: warm up until the clocks have settled, then
            # the median of five regions of at least 5 ms each (a single region of
            # ten cold launches read 15-20 % slow at 8192 rows)
            launcher.run(10)
            torch.cuda.synchronize()
            first = hip_event_ms(lib, launcher, 10)
            per_region = max(10, int(5.0 / max(first, 1e-3)))
            ms, _ = median_event_ms(lib, launcher, per_region, repeats=5)
        wshape = f"[{n},{k}]" if transpose else f"[{k},{n}] transpose=False"
        name = f"x {str(dtype)[6:]} [{M},{k}] W {wshape} b{bits} g{gs}"
        if small:
            add(cfg, name, ms, nbytes=qmv_bytes(M, n, k, bits, gs, esz),
                kernel=kname(M, n, k, gs, bits, dtype, transpose))
        else:
            add(cfg, name, ms, flops=2.0 * M * n * k,
                kernel=kname(M, n, k, gs, bits, dtype, transpose))

    bf16, f32 = torch.bfloat16, torch.float32
    # Cfg1: fp32 4096 x 4096, 4-bit group 64
    w = weights(4096, 4096, f32)
    ms = timed(lambda i: mlx_amd.quantize(w, 64, 4))
    qbytes = 4096 * 4096 * 4 + 4096 * 4096 // 2 + 2 * 4096 * 64 * 4
    add("cfg1", "quantize f32 [4096,4096] b4 g64", ms, nbytes=qbytes)
    q = mlx_amd.quantize(w, 64, 4)
    ms = timed(lambda i: mlx_amd.dequantize(*q, 64, 4))
    add("cfg1", "dequantize f32 [4096,4096] b4 g64", ms, nbytes=qbytes)
    matmul_case("cfg1", 1, 4096, 4096, 4, 64, f32)
    # Cfg2: decode, Llama-3-8B MLP shapes
    for (n, k) in ((14336, 4096), (4096, 14336)):
        for (bits, gs) in ((4, 64), (8, 128)):
            for B in (1, 2, 4, 8) + ((16, 32) if bits == 4 else ()):
                matmul_case("cfg2", B, n, k, bits, gs, bf16)
    # Cfg3: prefill
    for (n, k) in ((4096, 4096), (14336, 4096), (4096, 14336)):
        for (bits, gs) in ((4, 64), (8, 128)):
            for M in (512, 2048, 8192):
                matmul_case("cfg3", M, n, k, bits, gs, bf16)
    # gated MLP decode (nn callers): silu(gate(x)) * up(x), fused entry point against
    # two quantized_matmul launches and the elementwise arithmetic
    def swiglu_case(M, n, k, bits, gs):
        from mlx_amd import _lib
        lib = _lib.load()
        qg = mlx_amd.quantize(weights(n, k, bf16), gs, bits)
        wbytes = n * k * bits // 8 + 2 * n * (k // gs) * 2
        ring = ring_of(qg, wbytes)  # entries 2i, 2i+1: gate and up
        x = torch.randn((M, k), generator=g, dtype=torch.float32).to(bf16).to(dev)
        out = torch.empty((M, n), dtype=bf16, device=dev)
        gate = torch.empty((M, n), dtype=bf16, device=dev)
        up = torch.empty((M, n), dtype=bf16, device=dev)
        ws = torch.empty(lib.mlxrocm_qmm_swiglu_workspace_size(M, n, 2), dtype=torch.uint8, device=dev)
        R = len(ring) // 2

        def fused(i, stream):
            a, b = ring[2 * (i % R)], ring[2 * (i % R) + 1]
            rc = lib.mlxrocm_qmm_swiglu(x.data_ptr(), a[0].data_ptr(), a[1].data_ptr(), a[2].data_ptr(),
                                        b[0].data_ptr(), b[1].data_ptr(), b[2].data_ptr(),
                                        out.data_ptr(), ws.data_ptr(), M, n, k, gs, bits, 2, stream)
            if rc != 0:
                raise RuntimeError(_lib.last_error())

        def unfused(i, stream):
            a, b = ring[2 * (i % R)], ring[2 * (i % R) + 1]
            for q_, o_ in ((a, gate), (b, up)):
                rc = lib.mlxrocm_qmm(x.data_ptr(), q_[0].data_ptr(), q_[1].data_ptr(), q_[2].data_ptr(),
                                     o_.data_ptr(), M, n, k, 1, M * k, 0, 0, gs, bits, 2, 1,
                                     None, 0, stream)
                if rc != 0:
                    raise RuntimeError(_lib.last_error())
            torch.mul(torch.nn.functional.silu(gate), up, out=out)

        nb = 2 * qmv_bytes(M, n, k, bits, gs, 2) - M * k * 2
        for label, fn in (("fused entry point", fused), ("two launches + elementwise", unfused)):
            launcher = Launcher(torch, fn, R, True)
            launcher.run(R)
            torch.cuda.synchronize()
            ms = hip_event_ms(lib, launcher, R * 20)
            add("f1", f"silu(gate(x))*up(x), x bfloat16 [{M},{k}] W 2x[{n},{k}] b{bits} g{gs}, {label}",
                ms, nbytes=nb)

    for B in (1, 4):
        swiglu_case(B, 14336, 4096, 4, 64)
    # transpose=False (the vjp of a quantized linear layer): w [k, n] quantized along n
    for M in (1, 512, 2048):
        matmul_case("f3", M, 14336, 4096, 4, 64, bf16, transpose=False)
        matmul_case("f3", M, 4096, 14336, 8, 128, bf16, transpose=False)
    # ... at an odd width (codes repacked at 4 bits first)
    for M in (1, 512):
        matmul_case("f3", M, 11008, 4096, 3, 32, bf16, transpose=False)
    # Cfg4: 8 experts, top-2 routing
    E, n, k = 8, 14336, 4096
    wq, sc, bi = mlx_amd.quantize(
        (torch.randn((E, n, k), generator=g, dtype=torch.float32) * 0.02).to(bf16).to(dev), 64, 4)
    for T in (1, 8, 64, 2048):
        x = torch.randn((T, 1, 1, k), generator=g, dtype=torch.float32).to(bf16).to(dev)
        idx = torch.randint(0, E, (T, 2), generator=torch.Generator().manual_seed(0)).to(dev)
        ms = timed(lambda i: mlx_amd.gather_qmm(x, wq, sc, bi, rhs_indices=idx, transpose=True,
                                                group_size=64, bits=4))
        add("cfg4", f"gather T={T} top-2 of 8, unsorted", ms, flops=4.0 * T * n * k)
        flat = idx.reshape(-1)
        order = torch.argsort(flat, stable=True)
        xs = x.reshape(T, 1, k)[order // 2].contiguous()
        fs = flat[order].contiguous()
        ms = timed(lambda i: mlx_amd.gather_qmm(xs, wq, sc, bi, rhs_indices=fs, transpose=True,
                                                group_size=64, bits=4, sorted_indices=True))
        add("cfg4", f"gather T={T} top-2 of 8, sorted", ms, flops=4.0 * T * n * k)
        # the same unsorted call through the C ABI (no Python operator in the loop)
        from mlx_amd import _lib
        lib = _lib.load()
        n_idx = 2 * T
        lhs_u = torch.arange(T, device=dev).repeat_interleave(2).to(torch.uint32).contiguous()
        rhs_u = idx.reshape(-1).to(torch.uint32).contiguous()
        xb = x.reshape(T, 1, k).contiguous()
        out = torch.empty((n_idx, 1, n), dtype=bf16, device=dev)
        ws_bytes = lib.mlxrocm_gather_qmm_workspace_size(1, n, k, n_idx, E, 64, 4, 2, 1, 0)
        ws = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)

        def gstep(i, stream):
            rc = lib.mlxrocm_gather_qmm(
                xb.data_ptr(), wq.data_ptr(), sc.data_ptr(), bi.data_ptr(), lhs_u.data_ptr(),
                rhs_u.data_ptr(), out.data_ptr(), 1, n, k, n_idx, T, E, k, wq.stride(0),
                sc.stride(0), 64, 4, 2, 1, 0, ws.data_ptr() if ws_bytes else None, ws_bytes, stream)
            if rc != 0:
                raise RuntimeError(_lib.last_error())

        small = T <= 64
        launcher = Launcher(torch, gstep, 4, small)
        launcher.run(4)
        torch.cuda.synchronize()
        ms = hip_event_ms(lib, launcher, 40 if small else 10)
        add("cfg4", f"gather T={T} top-2 of 8, unsorted, C ABI" + (" (2 experts, cache-resident)" if T == 1 else ""), ms, flops=4.0 * T * n * k)
        if T in (8, 64):
            # the same launch over three expert stacks in rotation (792 MB): the rows
            # above re-read one 264 MB stack, about the size of the Infinity Cache
            stacks = [(wq, sc, bi)] + [tuple(t.clone() for t in (wq, sc, bi)) for _ in range(2)]

            def gstep3(i, stream):
                wq_, sc_, bi_ = stacks[i % 3]
                rc = lib.mlxrocm_gather_qmm(
                    xb.data_ptr(), wq_.data_ptr(), sc_.data_ptr(), bi_.data_ptr(), lhs_u.data_ptr(),
                    rhs_u.data_ptr(), out.data_ptr(), 1, n, k, n_idx, T, E, k, wq_.stride(0),
                    sc_.stride(0), 64, 4, 2, 1, 0, ws.data_ptr() if ws_bytes else None, ws_bytes,
                    stream)
                if rc != 0:
                    raise RuntimeError(_lib.last_error())

            launcher = Launcher(torch, gstep3, 6, True)
            launcher.run(6)
            torch.cuda.synchronize()
            ms = hip_event_ms(lib, launcher, 42)
            add("cfg4", f"gather T={T} top-2 of 8, unsorted, C ABI, three expert stacks in rotation",
                ms, flops=4.0 * T * n * k)
            del stacks
    # transpose=False over the same stack (the input gradient of the expert layer,
    # GatherQMM::vjp): cotangent rows [1, 14336] x W as [14336, 4096]
    for T in (64, 2048):
        cot = torch.randn((T, 2, 1, n), generator=g, dtype=torch.float32).to(bf16).to(dev)
        idx = torch.randint(0, E, (T, 2), generator=torch.Generator().manual_seed(0)).to(dev)
        lhs = torch.arange(2 * T, device=dev).reshape(T, 2)
        ms = timed(lambda i: mlx_amd.gather_qmm(cot, wq, sc, bi, lhs_indices=lhs,
                                                rhs_indices=idx, transpose=False,
                                                group_size=64, bits=4))
        add("f3", f"gather transpose=False T={T} top-2 of 8 (x [1,{n}] per pair, W [{n},{k}])", ms,
            flops=4.0 * T * n * k)
    del wq, sc, bi
    # Cfg5: odd code widths, group 32, Llama-2-7B MLP shapes
    for dtype in (bf16, f32):
        esz = 4 if dtype == f32 else 2
        for bits in (2, 3, 5, 6):
            w = weights(11008, 4096, dtype)
            ms = timed(lambda i: mlx_amd.quantize(w, 32, bits))
            nb = 11008 * 4096 * esz + 11008 * 4096 * bits // 8 + 2 * 11008 * 128 * esz
            add("cfg5", f"quantize {str(dtype)[6:]} [11008,4096] b{bits} g32", ms, nbytes=nb)
            matmul_case("cfg5", 1, 11008, 4096, bits, 32, dtype)
            matmul_case("cfg5", 1024, 11008, 4096, bits, 32, dtype)
            matmul_case("cfg5", 1, 4096, 11008, bits, 32, dtype)

    # floating-point modes: quantize / dequantize and the matmul at the headline shape
    def fp_case(mode, M, n, k):
        from mlx_amd import _lib
        lib = _lib.load()
        mcode = {"mxfp4": _lib.MXFP4, "mxfp8": _lib.MXFP8, "nvfp4": _lib.NVFP4}[mode]
        bits = 8 if mode == "mxfp8" else 4
        gs = 16 if mode == "nvfp4" else 32
        q = mlx_amd.quantize(weights(n, k, bf16, std=1.0), mode=mode)
        wbytes = n * k * bits // 8 + n * (k // gs)
        small = M <= 64
        ring = ring_of(q, wbytes) if small else [q]
        x = torch.randn((M, k), generator=g, dtype=torch.float32).to(bf16).to(dev)
        out = torch.empty((M, n), dtype=bf16, device=dev)
        ws_bytes = lib.mlxrocm_fp_qmm_workspace_size(M, n, k, 1, 0, mcode, 2, 1)
        ws = torch.empty(max(int(ws_bytes), 16), dtype=torch.uint8, device=dev)

        def step(i, stream):
            wq_, s_ = ring[i % len(ring)]
            rc = lib.mlxrocm_fp_qmm(x.data_ptr(), wq_.data_ptr(), s_.data_ptr(), out.data_ptr(),
                                    M, n, k, 1, M * k, 0, 0, mcode, 2, 1, ws.data_ptr(), ws_bytes,
                                    stream)
            if rc != 0:
                raise RuntimeError(_lib.last_error())

        launcher = Launcher(torch, step, len(ring), small)
        launcher.run(len(ring))
        torch.cuda.synchronize()
        if small:
            ms = hip_event_ms(lib, launcher, max(len(ring) * 20, 10))
        else:
            launcher.run(10)
            torch.cuda.synchronize()
            first = hip_event_ms(lib, launcher, 10)
            per_region = max(10, int(5.0 / max(first, 1e-3)))
            ms, _ = median_event_ms(lib, launcher, per_region, repeats=5)
        name = f"{mode}: x bfloat16 [{M},{k}] W [{n},{k}]"
        if small:
            add("f4", name, ms, nbytes=wbytes + M * k * 2 + M * n * 2)
        else:
            add("f4", name, ms, flops=2.0 * M * n * k)

    def qq_case(mode, M, n, k):
        """qqmm: x quantized inside the call, then the product (MX modes from 16
        rows on: both operands' codes on the block-scaled matrix instruction)."""
        from mlx_amd import _lib
        lib = _lib.load()
        mcode = {"mxfp4": _lib.MXFP4, "mxfp8": _lib.MXFP8, "nvfp4": _lib.NVFP4}[mode]
        q = mlx_amd.quantize(weights(n, k, bf16, std=1.0), mode=mode)
        x = torch.randn((M, k), generator=g, dtype=torch.float32).to(bf16).to(dev)
        out = torch.empty((M, n), dtype=bf16, device=dev)
        ws_bytes = lib.mlxrocm_fp_qqmm_workspace_size(M, n, k, mcode, 2)
        ws = torch.empty(max(int(ws_bytes), 256), dtype=torch.uint8, device=dev)

        def step(i, stream):
            rc = lib.mlxrocm_fp_qqmm(x.data_ptr(), q[0].data_ptr(), q[1].data_ptr(), out.data_ptr(),
                                     M, n, k, mcode, 2, ws.data_ptr(), ws_bytes, stream)
            if rc != 0:
                raise RuntimeError(_lib.last_error())

        launcher = Launcher(torch, step, 1, False)
        launcher.run(10)
        torch.cuda.synchronize()
        first = hip_event_ms(lib, launcher, 10)
        per_region = max(10, int(5.0 / max(first, 1e-3)))
        ms, _ = median_event_ms(lib, launcher, per_region, repeats=5)
        add("f4", f"qqmm {mode}: x bfloat16 [{M},{k}] W [{n},{k}] (x quantized in the call)", ms,
            flops=2.0 * M * n * k)

    for mode in ("mxfp8", "mxfp4", "nvfp4"):
        for M in (512, 2048, 8192):
            qq_case(mode, M, 14336, 4096)

    # nvfp4 with the tensor-wide scales, and gather_qqmm (operator calls)
    for M in (1, 512, 2048):
        w = weights(14336, 4096, bf16, std=1.0)
        x = torch.randn((M, 4096), generator=g, dtype=torch.float32).to(bf16).to(dev)
        gx, gw = x.float().abs().max(), w.float().abs().max()
        q = mlx_amd.quantize(w, mode="nvfp4", global_scale=gw)
        ms = timed(lambda i: mlx_amd.qqmm(x, *q, mode="nvfp4", global_scale_x=gx, global_scale_w=gw))
        add("f4", f"qqmm nvfp4 with global scales: x bfloat16 [{M},4096] W [14336,4096]", ms,
            flops=2.0 * M * 14336 * 4096)
    for mode in ("mxfp4", "nvfp4"):
        E, topk = 8, 2
        w = (torch.randn((E, 14336, 4096), generator=g, dtype=torch.float32)).to(bf16).to(dev)
        q = mlx_amd.quantize(w, mode=mode)
        del w
        for T in (8, 64, 2048):
            x = torch.randn((T, 1, 4096), generator=g, dtype=torch.float32).to(bf16).to(dev)
            lhs = torch.arange(T, dtype=torch.int32, device=dev).repeat_interleave(topk)
            rhs = torch.randint(0, E, (T * topk,), generator=g, dtype=torch.int32).to(dev)
            ms = timed(lambda i: mlx_amd.gather_qmm(x, *q, None, lhs, rhs, mode=mode))
            add("f4", f"gather_qmm {mode}: T={T} top-{topk} of {E}, x bfloat16 [{T},1,4096] "
                f"W [{E},14336,4096]", ms, flops=2.0 * T * topk * 14336 * 4096)
            ms = timed(lambda i: mlx_amd.gather_qqmm(x, *q, lhs, rhs, mode=mode))
            add("f4", f"gather_qqmm {mode}: T={T} top-{topk} of {E}, x bfloat16 [{T},1,4096] "
                f"W [{E},14336,4096]", ms, flops=2.0 * T * topk * 14336 * 4096)
        del q

    for mode in ("mxfp4", "mxfp8", "nvfp4"):
        bits = 8 if mode == "mxfp8" else 4
        gs = 16 if mode == "nvfp4" else 32
        w = weights(14336, 4096, bf16, std=1.0)
        nb = 14336 * 4096 * 2 + 14336 * 4096 * bits // 8 + 14336 * 4096 // gs
        ms = timed(lambda i: mlx_amd.quantize(w, mode=mode))
        add("f4", f"quantize bfloat16 [14336,4096] {mode}", ms, nbytes=nb)
        q = mlx_amd.quantize(w, mode=mode)
        ms = timed(lambda i: mlx_amd.dequantize(*q, mode=mode))
        add("f4", f"dequantize bfloat16 [14336,4096] {mode}", ms, nbytes=nb)
        for M in (1, 4, 512, 2048):
            fp_case(mode, M, 14336, 4096)

    # GGUF blocks -> affine triplet (load-time conversion of a [14336, 4096] tensor)
    from mlx_amd import gguf
    for name, type_id, block_bytes, out_bytes in (("Q4_0", 2, 18, 20), ("Q4_1", 3, 20, 20), ("Q8_0", 8, 34, 36)):
        n_blocks = 14336 * 4096 // 32
        blocks = torch.randint(0, 256, (n_blocks * block_bytes,), generator=g, dtype=torch.uint8).to(dev)
        ms = timed(lambda i: gguf.repack(blocks, type_id, (14336, 4096)))
        add("gguf", f"repack {name} [14336,4096] -> affine g32", ms, nbytes=n_blocks * (block_bytes + out_bytes))

    # element copies around the matmuls (C-ABI launches into a preallocated output)
    from mlx_amd import _copy, _lib
    import ctypes
    lib = _lib.load()
    stream = torch.cuda.current_stream(dev).cuda_stream
    n = 64 << 20
    src = torch.randn(n, generator=torch.Generator(device=dev).manual_seed(1), device=dev,
                      dtype=torch.float32).to(torch.bfloat16)
    dst = torch.empty(n, dtype=torch.float32, device=dev)
    code = _copy.DTYPE_CODE
    ms = timed(lambda i: _lib.check(lib.mlxrocm_copy_contiguous(
        src.data_ptr(), code[torch.bfloat16], dst.data_ptr(), code[torch.float32], n, 0, stream)))
    add("copy", "contiguous bfloat16 -> float32, 64 Mi elements", ms, nbytes=n * 6)
    back = torch.empty(n, dtype=torch.bfloat16, device=dev)
    ms = timed(lambda i: _lib.check(lib.mlxrocm_copy_contiguous(
        dst.data_ptr(), code[torch.float32], back.data_ptr(), code[torch.bfloat16], n, 0, stream)))
    add("copy", "contiguous float32 -> bfloat16, 64 Mi elements", ms, nbytes=n * 6)
    arr = lambda v: (ctypes.c_int64 * len(v))(*v)
    ms = timed(lambda i: _lib.check(lib.mlxrocm_copy_strided(
        src.data_ptr(), code[torch.bfloat16], arr((1, 8192)), back.data_ptr(), code[torch.bfloat16],
        None, 2, arr((8192, 8192)), stream)))
    add("copy", "transpose of bfloat16 [8192,8192] into rows (strided source)", ms, nbytes=n * 4)
    ms = timed(lambda i: _lib.check(lib.mlxrocm_copy_strided(
        src.data_ptr(), code[torch.bfloat16], arr((2 * 4096, 1)), back.data_ptr(), code[torch.bfloat16],
        None, 2, arr((8192, 4096)), stream)))
    add("copy", "left half of bfloat16 [8192,8192] rows into [8192,4096] (row-strided source)", ms,
        nbytes=8192 * 4096 * 4)
    one = torch.ones(1, dtype=torch.float32, device=dev)
    ms = timed(lambda i: _lib.check(lib.mlxrocm_copy_contiguous(
        one.data_ptr(), code[torch.float32], back.data_ptr(), code[torch.bfloat16], n, 1, stream)))
    add("copy", "fill bfloat16, 64 Mi elements", ms, nbytes=n * 2)
    return rows


def fp_mode_figures(torch, mlx_amd, lib, dev) -> dict:
    """The same shapes in the mxfp4 mode (floating-point codes, one e8m0 scale
    byte per 32): decode GEMV over a ring of 18 weight copies (graph replays, HIP
    events, median of 3 regions of 1800 launches), the prefill GEMM at 2048 rows
    and qqmm -- x quantized inside the call, both operands' codes on the
    block-scaled matrix instruction -- at 2048 and 8192 rows.  Extra figures
    beside the headline ones, each with the peak it is priced against."""
    from mlx_amd import _lib

    g = torch.Generator().manual_seed(7)
    bf16 = torch.bfloat16
    mode, mcode = "mxfp4", _lib.MXFP4
    w = torch.randn((N, K), generator=g, dtype=torch.float32).to(bf16).to(dev)
    q = mlx_amd.quantize(w, mode=mode)
    del w
    ring = [q] + [tuple(t.clone() for t in q) for _ in range(RING - 1)]
    out = {"mode": mode}

    x1 = torch.randn((1, K), generator=g, dtype=torch.float32).to(bf16).to(dev)
    y1 = torch.empty((1, N), dtype=bf16, device=dev)

    def decode_step(i, stream):
        wq_, s_ = ring[i % RING]
        rc = lib.mlxrocm_fp_qmm(x1.data_ptr(), wq_.data_ptr(), s_.data_ptr(), y1.data_ptr(),
                                1, N, K, 1, K, 0, 0, mcode, _lib.BFLOAT16, 1, None, 0, stream)
        if rc != 0:
            raise RuntimeError(_lib.last_error())

    launcher = Launcher(torch, decode_step, RING, True)
    launcher.run(2 * RING)
    torch.cuda.synchronize()
    launches = -(-QMV_MIN_LAUNCHES // RING) * RING
    ms, samples = median_event_ms(lib, launcher, launches, repeats=3)
    nbytes = N * K // 2 + N * (K // 32) + K * 2 + N * 2
    gbps = nbytes / (ms * 1e-3) / 1e9
    out["qmv"] = {
        "workload": f"x bf16 [1,{K}], W [{N},{K}] mxfp4",
        "bytes_per_launch": nbytes, "us_per_launch": round(ms * 1e3, 3),
        "value": round(gbps, 2), "unit": "GB/s", "bound": "hbm", "peak": HBM_PEAK_GBPS,
        "frac": round(gbps / HBM_PEAK_GBPS, 4), "launches_timed": launches, "repeats": len(samples),
    }

    def big(name, M, entry, peak, what):
        x = torch.randn((M, K), generator=g, dtype=torch.float32).to(bf16).to(dev)
        y = torch.empty((M, N), dtype=bf16, device=dev)
        if entry == "qmm":
            ws_bytes = lib.mlxrocm_fp_qmm_workspace_size(M, N, K, 1, 0, mcode, _lib.BFLOAT16, 1)
        else:
            ws_bytes = lib.mlxrocm_fp_qqmm_workspace_size(M, N, K, mcode, _lib.BFLOAT16)
        ws = torch.empty(max(int(ws_bytes), 256), dtype=torch.uint8, device=dev)

        def step(i, stream):
            wq_, s_ = ring[i % RING]
            if entry == "qmm":
                rc = lib.mlxrocm_fp_qmm(x.data_ptr(), wq_.data_ptr(), s_.data_ptr(), y.data_ptr(),
                                        M, N, K, 1, M * K, 0, 0, mcode, _lib.BFLOAT16, 1,
                                        ws.data_ptr(), ws_bytes, stream)
            else:
                rc = lib.mlxrocm_fp_qqmm(x.data_ptr(), wq_.data_ptr(), s_.data_ptr(), y.data_ptr(),
                                         M, N, K, mcode, _lib.BFLOAT16, ws.data_ptr(), ws_bytes, stream)
            if rc != 0:
                raise RuntimeError(_lib.last_error())

        launcher = Launcher(torch, step, RING, False)
        launcher.run(10)
        torch.cuda.synchronize()
        first = hip_event_ms(lib, launcher, 10)
        per_region = max(50, int(10.0 / max(first, 1e-3)))
        ms, samples = median_event_ms(lib, launcher, per_region, repeats=3)
        tflops = 2.0 * M * N * K / (ms * 1e-3) / 1e12
        out[name] = {
            "workload": f"x bf16 [{M},{K}], W [{N},{K}] mxfp4; {what}",
            "us_per_launch": round(ms * 1e3, 2), "value": round(tflops, 2), "unit": "TFLOP/s",
            "bound": "mfma", "peak": peak, "frac": round(tflops / peak, 4),
            "launches_timed": per_region, "repeats": len(samples),
        }

    big("qmm_t", QMM_M, "qmm", BF16_PEAK_TFLOPS,
        "weights widened to bf16 in the tile kernel (bf16 MFMA peak)")
    big("qqmm_2048", QMM_M, "qqmm", FP4_PEAK_TFLOPS,
        "x quantized inside the call, block-scaled fp4 MFMA (fp4 peak)")
    big("qqmm_8192", 8192, "qqmm", FP4_PEAK_TFLOPS,
        "x quantized inside the call, block-scaled fp4 MFMA (fp4 peak)")
    return out


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--only", choices=("qmv", "qmm_t"), default=None)
    ap.add_argument("--no-graph", action="store_true",
                    help="launch every kernel from Python instead of replaying a HIP graph")
    ap.add_argument("--no-fp", action="store_true",
                    help="skip the extra figures of the mxfp4 mode (fp_modes)")
    ap.add_argument("--no-floor", action="store_true",
                    help="skip the read-only probe (roofline.read_only_floor_us)")
    ap.add_argument("--sweep", action="store_true",
                    help="time the other synthetic configurations of the path instead of "
                         "the headline pair; prints one JSON line {\"sweep\": [...]}")
    ap.add_argument("--copy-probe", action="store_true",
                    help="only run 20 device-to-device copies of 256 MiB: the known-size "
                         "kernel that FETCH_SIZE / WRITE_SIZE readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU; this build has no multi-GPU path "
              "(run with --gpus 1)", file=sys.stderr)
        return 2

    # the load-only floor of a 33 MB launch, measured by a child process before
    # this one initialises the GPU
    floor = None
    if not (args.copy_probe or args.sweep or args.no_floor) and args.only in (None, "qmv"):
        floor = read_only_floor()

    import torch

    import mlx_amd
    from mlx_amd import _lib

    lib = _lib.load()
    if not torch.cuda.is_available():
        print("no GPU visible", file=sys.stderr)
        return 1
    dev = torch.device("cuda:0")
    dt = torch.bfloat16

    if args.copy_probe:
        nbytes = 256 << 20
        src = torch.empty(nbytes, dtype=torch.uint8, device=dev).fill_(1)
        dst = torch.empty_like(src)
        stream = torch.cuda.current_stream(dev).cuda_stream
        for _ in range(20):
            _lib.check(lib.mlxrocm_memcpy_d2d(dst.data_ptr(), src.data_ptr(), nbytes, stream))
        torch.cuda.synchronize()
        print(json.dumps({"copy_probe_bytes": nbytes, "copies": 20}))
        return 0

    if args.sweep:
        print(json.dumps({"sweep": sweep(torch, mlx_amd, dev)}))
        return 0

    g = torch.Generator().manual_seed(0)
    x_cpu = torch.randn((1, K), generator=g, dtype=torch.float32).to(dt)
    x = x_cpu.to(dev)
    # The ring lives in one allocation made before anything else, each weight at
    # a 2 MiB boundary: how the driver backs many separate allocations (page
    # sizes, placement) differs from box to box and showed up as a spread in the
    # streaming rate.
    w_words, sb_elems = N * K * BITS // 32, N * K // GS
    slot = -(-(w_words * 4 + 2 * sb_elems * 2) // (2 << 20)) * (2 << 20)
    pool = torch.empty(RING * slot + (2 << 20), dtype=torch.uint8, device=dev)
    pool = pool[(-pool.data_ptr()) % (2 << 20):]
    ring = []
    for i in range(RING):
        w = (torch.randn((N, K), generator=g, dtype=torch.float32) * 0.02).to(dt).to(dev)
        wq, s, b = mlx_amd.quantize(w, GS, BITS)
        base = pool[i * slot:(i + 1) * slot]
        wq_v = base[:w_words * 4].view(torch.uint32).view(N, -1)
        s_v = base[w_words * 4:w_words * 4 + sb_elems * 2].view(dt).view(N, -1)
        b_v = base[w_words * 4 + sb_elems * 2:w_words * 4 + sb_elems * 4].view(dt).view(N, -1)
        wq_v.copy_(wq)
        s_v.copy_(s)
        b_v.copy_(b)
        ring.append((wq_v, s_v, b_v))
        del w, wq, s, b
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    out = torch.empty((1, N), dtype=dt, device=dev)
    code = _lib.BFLOAT16
    result = {}

    # ------------------------------------------------------------------ qmv
    nbytes = qmv_bytes(1, N, K, BITS, GS, 2)
    ptrs = [(wq.data_ptr(), s.data_ptr(), b.data_ptr()) for wq, s, b in ring]

    def qmv_step(i, stream):
        wq_p, s_p, b_p = ptrs[i % RING]
        rc = lib.mlxrocm_qmm(x.data_ptr(), wq_p, s_p, b_p, out.data_ptr(),
                             1, N, K, 1, K, 0, 0, GS, BITS, code, 1, None, 0, stream)
        if rc != 0:
            raise RuntimeError(_lib.last_error())

    if args.only in (None, "qmv"):
        launcher = Launcher(torch, qmv_step, RING, not args.no_graph)
        warmup = max(args.warmup, MIN_WARMUP)
        launches = -(-max(args.steps, QMV_MIN_LAUNCHES) // RING) * RING
        launcher.prepare(warmup)
        launcher.prepare(launches)
        launcher.run(warmup)
        torch.cuda.synchronize()
        ev_ms, samples = median_event_ms(lib, launcher, launches)
        # single hot buffer: served from the Infinity Cache, reported separately
        hot = Launcher(torch, lambda i, st: qmv_step(0, st), RING, not args.no_graph)
        hot.run(warmup)
        llc_ms, _ = median_event_ms(lib, hot, launches)
        gbps = nbytes / (ev_ms * 1e-3) / 1e9
        result.update({
            "metric": "4-bit qmv HBM GB/s (%peak) at 14336x4096; qmm_t TFLOP/s (%peak) at M=2048",
            "value": round(gbps, 2),
            "unit": "GB/s",
            "n_gpus": 1,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": round(ev_ms, 6),
            "higher_is_better": True,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": "bf16",
            "data": "synthetic",
            "config": {
                "workload": "qmv decode GEMV, Llama-3-8B gate/up: x bf16 [1,4096], "
                            "W [14336,4096] 4-bit group 64, bf16 scales/biases, transpose=True",
                "weight_ring": RING,
                "launch": "direct" if args.no_graph else f"hip graph of {RING} launches",
                "kernel": lib.mlxrocm_qmm_kernel_name(1, N, K, 1, GS, BITS, code, 1).decode(),
            },
            "timing": {
                "method": "HIP events on the launch stream; median of the timed regions",
                "launches_timed": launches,
                "repeats": len(samples),
                "warmup_launches": warmup,
                "us_per_launch_min_median_max": [round(samples[0] * 1e3, 3), round(ev_ms * 1e3, 3),
                                                 round(samples[-1] * 1e3, 3)],
            },
            "roofline": {
                "bound": "hbm",
                "achieved": round(gbps, 2),
                "peak": HBM_PEAK_GBPS,
                "unit": "GB/s",
                "frac": round(gbps / HBM_PEAK_GBPS, 4),
                "traffic": QMV_TRAFFIC_BYTES,
                "traffic_source": QMV_TRAFFIC_SOURCE,
                "kernel_us": round(ev_ms * 1e3, 3),
                "bytes_per_launch": nbytes,
                "llc_resident_gbps": round(nbytes / (llc_ms * 1e-3) / 1e9, 2),
            },
        })
        if floor is not None:
            # the same bytes through a kernel that only loads, same launch chain
            result["roofline"].update({
                "read_only_floor_us": floor["read_only_floor_us"],
                "read_only_floor_frac": round(
                    floor["bytes"] / (floor["read_only_floor_us"] * 1e-6) / 1e9 / HBM_PEAK_GBPS, 4),
                "read_only_cache_resident_us": floor["read_only_cache_resident_us"],
                "empty_launch_us": floor["empty_launch_us"],
                "floor_source": "mlx_amd/lib/read_probe --floor (child process, before this "
                                "process initialised the GPU)",
            })

    # ---------------------------------------------------------------- qmm_t
    if args.only in (None, "qmm_t"):
        xm = torch.randn((QMM_M, K), generator=g, dtype=torch.float32).to(dt).to(dev)
        outm = torch.empty((QMM_M, N), dtype=dt, device=dev)
        flops = 2.0 * QMM_M * N * K
        ws_bytes = lib.mlxrocm_qmm_workspace_size(QMM_M, N, K, 1, 0, GS, BITS, code, 1)
        ws = torch.empty(max(int(ws_bytes), 16), dtype=torch.uint8, device=dev)

        def qmm_step(i, stream):
            wq_p, s_p, b_p = ptrs[i % RING]
            rc = lib.mlxrocm_qmm(xm.data_ptr(), wq_p, s_p, b_p, outm.data_ptr(),
                                 QMM_M, N, K, 1, QMM_M * K, 0, 0, GS, BITS, code, 1,
                                 ws.data_ptr(), ws_bytes, stream)
            if rc != 0:
                raise RuntimeError(_lib.last_error())

        launches = max(args.steps // 20, MIN_LAUNCHES)
        mm = Launcher(torch, qmm_step, RING, False)
        mm.run(max(args.warmup // 20, MIN_WARMUP))
        torch.cuda.synchronize()
        ms, samples = median_event_ms(lib, mm, launches, repeats=5)
        tflops = flops / (ms * 1e-3) / 1e12
        result["qmm_t"] = {
            "workload": f"qmm_t prefill GEMM: x bf16 [{QMM_M},{K}], W [{N},{K}] 4-bit group 64",
            "kernel": lib.mlxrocm_qmm_kernel_name(QMM_M, N, K, 1, GS, BITS, code, 1).decode(),
            "value": round(tflops, 2),
            "unit": "TFLOP/s",
            "launches_timed": launches,
            "repeats": len(samples),
            "ms_per_step": round(ms, 5),
            "us_per_launch_min_median_max": [round(samples[0] * 1e3, 2), round(ms * 1e3, 2),
                                             round(samples[-1] * 1e3, 2)],
            "roofline": {
                "bound": "mfma",
                "achieved": round(tflops, 2),
                "peak": BF16_PEAK_TFLOPS,
                "unit": "TFLOP/s",
                "frac": round(tflops / BF16_PEAK_TFLOPS, 4),
                "traffic": QMM_T_TRAFFIC_BYTES,
                "traffic_source": QMM_T_TRAFFIC_SOURCE,
            },
        }

        # The same call with the transposed scale / bias image of every weight
        # built beforehand (mlxrocm_qmm_sb_image: weights do not change between
        # calls, so a caller can keep it) -- a second figure beside the plain call,
        # never the headline.
        img_bytes = lib.mlxrocm_qmm_sb_image_size(N, K, 1, GS, code)
        images = [torch.empty(img_bytes, dtype=torch.uint8, device=dev) for _ in range(RING)]
        stream0 = torch.cuda.current_stream(dev).cuda_stream
        for (wq_p, s_p, b_p), img in zip(ptrs, images):
            rc = lib.mlxrocm_qmm_sb_image(s_p, b_p, img.data_ptr(), N, K, 1, 0, GS, code, stream0)
            if rc != 0:
                raise RuntimeError(_lib.last_error())
        torch.cuda.synchronize()

        def qmm_pre_step(i, stream):
            wq_p, s_p, b_p = ptrs[i % RING]
            rc = lib.mlxrocm_qmm_prepacked(xm.data_ptr(), wq_p, s_p, b_p,
                                           images[i % RING].data_ptr(), outm.data_ptr(),
                                           QMM_M, N, K, 1, QMM_M * K, 0, 0, GS, BITS, code, 1,
                                           ws.data_ptr(), ws_bytes, stream)
            if rc != 0:
                raise RuntimeError(_lib.last_error())

        mp = Launcher(torch, qmm_pre_step, RING, False)
        mp.run(max(args.warmup // 20, MIN_WARMUP))
        torch.cuda.synchronize()
        ms_p, samples_p = median_event_ms(lib, mp, launches, repeats=5)
        tflops_p = flops / (ms_p * 1e-3) / 1e12
        result["qmm_t"]["with_cached_scale_image"] = {
            "what": "mlxrocm_qmm_prepacked: the scale / bias transposition done once per weight, "
                    "outside the timed region",
            "value": round(tflops_p, 2),
            "unit": "TFLOP/s",
            "frac": round(tflops_p / BF16_PEAK_TFLOPS, 4),
            "us_per_launch_min_median_max": [round(samples_p[0] * 1e3, 2), round(ms_p * 1e3, 2),
                                             round(samples_p[-1] * 1e3, 2)],
        }

    if args.only is None and not args.no_fp:
        try:
            result["fp_modes"] = fp_mode_figures(torch, mlx_amd, lib, dev)
        except Exception as exc:  # extra figures: the headline line is printed regardless
            result["fp_modes"] = {"error": f"{type(exc).__name__}: {exc}"}

    if not args.no_cpu and args.only in (None, "qmv"):
        wq0, s0, b0 = ring[0]
        result["cpu_baseline"] = cpu_baseline(x_cpu, wq0.cpu(), s0.cpu(), b0.cpu(), nbytes)

    name = ctypes.create_string_buffer(256)
    cus, clk = ctypes.c_int(), ctypes.c_int()
    lib.mlxrocm_device_info(0, name, ctypes.byref(cus), None, ctypes.byref(clk))
    result["device"] = {"name": name.value.decode(), "compute_units": cus.value,
                        "clock_mhz": clk.value // 1000}
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
