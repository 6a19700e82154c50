#!/usr/bin/env python3
"""Benchmark of the cooperative-vector hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c2]

A "step" is one pass of the hot path over one batch of synthetic, seeded input that already
lives in HBM.  The default workload is the configuration the headline metric is quoted on:
a single fp16 coopVecMatMulAdd layer 64x64 (fp32 accumulate, fp16 output) over 2^22 vectors,
weights in InferencingOptimal layout (the layout conversion is timed separately and reported
as `layout_conversion_us`).  Prints ONE JSON line.

`roofline.achieved` = algorithmic bytes per launch / average kernel duration, the duration
measured with HIP events on the launch stream around the timed launches.  `cpu_baseline` times
the CPU oracle's restatement of Slang's CPU-target fallback (oracle/, test infrastructure) on a
bounded sample of the same workload on the host cores.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

REPO = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, REPO)
sys.path.insert(0, os.path.join(REPO, "tests"))

METRIC = "CoopVec MLP samples/sec (fp16/fp8/int8 fwd, fp16 train step); % MFMA peak"
HBM_PEAK_GBS = 8000.0
MFMA_PEAK_TFLOPS = {"f16": 2500.0, "fp8": 5000.0, "int8": 5000.0}

# HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE / WRITE_SIZE, scaled by a copy
# kernel of known size); the summaries are in profiles/.  None where not measured.
MEASURED_TRAFFIC_BYTES = {}


def ensure_built():
    from slang_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from slang_amd import build
        build.build_library()
    return _lib.load()


def workload_c2(torch, cv, steps, warmup):
    """fp16 64x64 matMulAdd, batch 2^22, InferencingOptimal weights."""
    import numpy as np
    from slang_amd.coopvec import CoopVecComponentType as CT, CoopVecMatrixLayout as ML, CooperativeVectorMatrixDesc as D
    dev = "cuda"
    B, M, K = 1 << 22, 64, 64
    g = torch.Generator(device=dev); g.manual_seed(20251)
    x = torch.randn(B, K, device=dev, generator=g).half()
    W = (torch.randn(M, K, device=dev, generator=g) / 8.0).half()
    b = (torch.rand(M, device=dev, generator=g) * 0.2 - 0.1).half()
    wrow = W.contiguous().view(torch.uint8).flatten()
    size = cv.getCooperativeVectorMatrixSize(M, K, CT.Float16, ML.InferencingOptimal)
    wopt = torch.empty(size, dtype=torch.uint8, device=dev)
    dst = [D(M, K, CT.Float16, ML.InferencingOptimal, size, 0, 0)]
    src = [D(M, K, CT.Float16, ML.RowMajor, M * K * 2, 0, K * 2)]
    cv.convertCooperativeVectorMatrix(wopt, dst, wrow, src)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        cv.convertCooperativeVectorMatrix(wopt, dst, wrow, src)
    e1.record(); torch.cuda.synchronize()
    conv_us = e0.elapsed_time(e1) / 20 * 1e3
    bb = b.view(torch.uint8)
    out = torch.empty(B, M, dtype=torch.float16, device=dev)

    def step():
        cv.coopVecMatMulAdd(x, CT.Float16, wopt, 0, CT.Float16, bb, 0, CT.Float16, ML.InferencingOptimal,
                            False, 0, M=M, out=out)

    def cpu_baseline():
        import ctypes
        import concurrent.futures as cf
        import oracle_binding as ob
        L = ob.lib()
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")), 16)
        per_core = 1 << 13
        n = per_core * cores
        xs = x[:n].cpu().numpy(); Wn = W.cpu().numpy(); bn = b.cpu().numpy()
        outn = np.zeros((n, M), np.float16)
        groups = (n + 255) // 256

        def run(g0, g1, mode):
            rc = L.cvo_slang_dispatch_matmul_add(g0, g1, n, ob.ptr(xs), K * 2, ob.F16, K, ob.F16, K, ob.ptr(outn),
                                                 M * 2, ob.F16, M, ob.ptr(Wn), 0, ob.F16, ob.ROW, 0, K * 2,
                                                 ob.ptr(bn), 0, ob.F16, mode)
            assert rc == 0
        # one core, the faithful shape: Slang's CPU target runs work-items serially
        t0 = time.perf_counter(); run(0, per_core // 256, ob.HALF_SLANG); t1 = time.perf_counter()
        one_core = per_core / (t1 - t0)
        # all cores: the group range split the way the CPU ABI intends (startGroupID..endGroupID)
        chunk = groups // cores
        t0 = time.perf_counter()
        with cf.ThreadPoolExecutor(cores) as pool:
            list(pool.map(lambda c: run(c * chunk, (c + 1) * chunk, ob.HALF_SLANG), range(cores)))
        t1 = time.perf_counter()
        return {"value": n / (t1 - t0), "unit": "samples/s", "cores": cores, "kind": "port",
                "value_1core": one_core,
                "sample": "first %d of the 2^22 vectors (%d per core); C restatement of the Slang CPU-target "
                          "fallback (fp16 accumulate, software half as gcc<12 selects), -O2" % (n, per_core)}

    return dict(step=step, samples=B, alg_bytes=B * (K * 2 + M * 2), alg_flops=B * 2 * M * K,
                bound="hbm", dtype="f16", kernel="matmulKernel<F16Mma,4,2,4,half>",
                config={"workload": "c2: fp16 coopVecMatMulAdd 64x64, batch 2^22, InferencingOptimal weights, "
                                    "fp32 accumulate, fp16 out", "batch": B, "m": M, "k": K,
                        "layout": "InferencingOptimal"},
                extra={"layout_conversion_us": conv_us}, cpu_baseline=cpu_baseline, key="c2")


WORKLOADS = {"c2": workload_c2}


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default="c2", choices=sorted(WORKLOADS))
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU leg (profiling runs)")
    args = ap.parse_args(argv)
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path is data-parallel over samples; "
              "see DESIGN.md for how it would shard); use --gpus 1", file=sys.stderr)
        return 2
    ensure_built()
    import torch
    from slang_amd import coopvec as cv
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    torch.cuda.set_device(0)
    w = WORKLOADS[args.workload](torch, cv, args.steps, args.warmup)
    step = w["step"]
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(args.steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    wall_ms = (t1 - t0) * 1e3 / args.steps
    kern_ms = ev0.elapsed_time(ev1) / args.steps          # HIP events on the launch stream
    value = w["samples"] / (wall_ms * 1e-3)
    if w["bound"] == "hbm":
        achieved = w["alg_bytes"] / (kern_ms * 1e-3) / 1e9
        peak, unit = HBM_PEAK_GBS, "GB/s"
    else:
        achieved = w["alg_flops"] / (kern_ms * 1e-3) / 1e12
        peak, unit = MFMA_PEAK_TFLOPS[w["mfma"]], "TFLOP/s"
    line = {
        "metric": METRIC, "value": value, "unit": "samples/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": w["dtype"], "data": "synthetic", "config": w["config"],
        "roofline": {"bound": w["bound"], "achieved": achieved, "peak": peak, "unit": unit,
                     "frac": achieved / peak, "traffic": MEASURED_TRAFFIC_BYTES.get(w["key"]),
                     "kernel": w["kernel"], "kernel_ms": kern_ms,
                     "alg_bytes_per_launch": w["alg_bytes"], "alg_flops_per_launch": w["alg_flops"]},
        "cpu_baseline": None if args.no_cpu_baseline else w["cpu_baseline"](),
    }
    line.update(w.get("extra", {}))
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
