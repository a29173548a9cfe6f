#!/usr/bin/env python3
"""Benchmark of the affine quantized-matmul hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only qmv|qmm_t]

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
# HBM bytes per launch from the FETCH_SIZE / WRITE_SIZE counter passes, scaled by
# a copy of known size (profiles/qmv_stream_4bit_g64_bf16_14336x4096.md and
# profiles/qmm_t_mfma_4bit_g64_bf16_M2048_14336x4096.md).
QMV_TRAFFIC_BYTES = 33224900
QMM_T_TRAFFIC_BYTES = 276972000

N, K = 14336, 4096
BITS, GS = 4, 64
QMM_M = 2048
RING = 18  # 18 x 33 MB = 595 MB of weights > 2 x the 256 MB Infinity Cache


def qmv_bytes(M: int, n: int, k: int, bits: int, gs: int, esize: int) -> int:
    """Algorithmic bytes of one qmv launch: packed codes + scales + biases + x + out."""
    return n * k * bits // 8 + 2 * n * (k // gs) * esize + M * k * esize + M * n * esize


class Launcher:
    """Issues `steps` launches of fn(i, stream) on one stream, either directly
    or by replaying a HIP graph that holds one pass over the weight ring (the
    kernel is a few microseconds long, shorter than a Python-driven launch)."""

    def __init__(self, torch, fn, period: int, use_graph: bool):
        self.torch, self.fn, self.period = torch, fn, period
        self.stream = torch.cuda.Stream()
        self.graph = None
        self.stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(self.stream):
            for i in range(period):
                fn(i, self.stream.cuda_stream)
        self.stream.synchronize()
        if use_graph:
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph, stream=self.stream):
                for i in range(period):
                    fn(i, torch.cuda.current_stream().cuda_stream)

    def run(self, steps: int) -> int:
        """Enqueue at least `steps` launches; returns how many were issued."""
        with self.torch.cuda.stream(self.stream):
            if self.graph is not None:
                replays = (steps + self.period - 1) // self.period
                for _ in range(replays):
                    self.graph.replay()
                return replays * self.period
            for i in range(steps):
                self.fn(i, self.stream.cuda_stream)
            return steps


def hip_event_ms(lib, launcher: "Launcher", steps: int) -> float:
    """Milliseconds per launch, measured with HIP events recorded on the
    stream the kernels are launched on."""
    stream = launcher.stream.cuda_stream
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


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=200)
    ap.add_argument("--no-cpu", action="store_true", help="skip the cpu_baseline leg")
    ap.add_argument("--only", choices=("qmv", "qmm_t"), default=None)
    ap.add_argument("--no-graph", action="store_true",
                    help="launch every kernel from Python instead of replaying a HIP graph")
    ap.add_argument("--copy-probe", action="store_true",
                    help="only run 20 device-to-device copies of 256 MiB: the known-size "
                         "kernel that FETCH_SIZE / WRITE_SIZE readings are scaled by")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU; this build has no multi-GPU path "
              "(run with --gpus 1)", file=sys.stderr)
        return 2

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

    g = torch.Generator().manual_seed(0)
    x_cpu = torch.randn((1, K), generator=g, dtype=torch.float32).to(dt)
    x = x_cpu.to(dev)
    ring = []
    for i in range(RING):
        w = (torch.randn((N, K), generator=g, dtype=torch.float32) * 0.02).to(dt).to(dev)
        ring.append(mlx_amd.quantize(w, GS, BITS))
        del w
    out = torch.empty((1, N), dtype=dt, device=dev)
    code = _lib.BFLOAT16
    result = {}

    # ------------------------------------------------------------------ qmv
    nbytes = qmv_bytes(1, N, K, BITS, GS, 2)
    ptrs = [(wq.data_ptr(), s.data_ptr(), b.data_ptr()) for wq, s, b in ring]

    def qmv_step(i, stream):
        wq_p, s_p, b_p = ptrs[i % RING]
        rc = lib.mlxrocm_qmm(x.data_ptr(), wq_p, s_p, b_p, out.data_ptr(),
                             1, N, K, 1, K, 0, 0, GS, BITS, code, 1, stream)
        if rc != 0:
            raise RuntimeError(_lib.last_error())

    if args.only in (None, "qmv"):
        launcher = Launcher(torch, qmv_step, RING, not args.no_graph)
        launcher.run(args.warmup)
        torch.cuda.synchronize()
        steps = (args.steps + RING - 1) // RING * RING if not args.no_graph else args.steps
        t0 = time.perf_counter()
        ev_ms = hip_event_ms(lib, launcher, steps)
        torch.cuda.synchronize()
        wall_ms = (time.perf_counter() - t0) * 1e3 / steps
        args.steps = steps
        # single hot buffer: served from the Infinity Cache, reported separately
        hot = Launcher(torch, lambda i, st: qmv_step(0, st), RING, not args.no_graph)
        llc_ms = hip_event_ms(lib, hot, steps)
        gbps = nbytes / (ev_ms * 1e-3) / 1e9
        result.update({
            "metric": "4-bit qmv HBM GB/s (%peak) at 14336x4096; qmm_t TFLOP/s (%peak) at M=2048",
            "value": round(nbytes / (wall_ms * 1e-3) / 1e9, 2),
            "unit": "GB/s",
            "n_gpus": 1,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": round(wall_ms, 6),
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
            "roofline": {
                "bound": "hbm",
                "achieved": round(gbps, 2),
                "peak": HBM_PEAK_GBPS,
                "unit": "GB/s",
                "frac": round(gbps / HBM_PEAK_GBPS, 4),
                "traffic": QMV_TRAFFIC_BYTES,
                "kernel_us": round(ev_ms * 1e3, 3),
                "bytes_per_launch": nbytes,
                "llc_resident_gbps": round(nbytes / (llc_ms * 1e-3) / 1e9, 2),
            },
        })

    # ---------------------------------------------------------------- qmm_t
    if args.only in (None, "qmm_t"):
        xm = torch.randn((QMM_M, K), generator=g, dtype=torch.float32).to(dt).to(dev)
        outm = torch.empty((QMM_M, N), dtype=dt, device=dev)
        flops = 2.0 * QMM_M * N * K

        def qmm_step(i, stream):
            wq_p, s_p, b_p = ptrs[i % RING]
            rc = lib.mlxrocm_qmm(xm.data_ptr(), wq_p, s_p, b_p, outm.data_ptr(),
                                 QMM_M, N, K, 1, QMM_M * K, 0, 0, GS, BITS, code, 1, stream)
            if rc != 0:
                raise RuntimeError(_lib.last_error())

        steps = max(RING, args.steps // 20)
        mm = Launcher(torch, qmm_step, RING, False)
        mm.run(max(3, args.warmup // 20))
        torch.cuda.synchronize()
        ms = hip_event_ms(lib, mm, steps)
        tflops = flops / (ms * 1e-3) / 1e12
        result["qmm_t"] = {
            "workload": f"qmm_t prefill GEMM: x bf16 [{QMM_M},{K}], W [{N},{K}] 4-bit group 64",
            "kernel": lib.mlxrocm_qmm_kernel_name(QMM_M, N, K, 1, GS, BITS, code, 1).decode(),
            "value": round(tflops, 2),
            "unit": "TFLOP/s",
            "steps": steps,
            "ms_per_step": round(ms, 5),
            "roofline": {
                "bound": "mfma",
                "achieved": round(tflops, 2),
                "peak": BF16_PEAK_TFLOPS,
                "unit": "TFLOP/s",
                "frac": round(tflops / BF16_PEAK_TFLOPS, 4),
                "traffic": QMM_T_TRAFFIC_BYTES,
            },
        }

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
