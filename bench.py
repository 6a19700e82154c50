#!/usr/bin/env python3
"""Benchmark of the cooperative-vector hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A "step" is one pass of the hot path over one batch of synthetic, seeded input that already
lives in HBM.  The headline workload (top-level fields of the JSON line) is the configuration the
metric is quoted on: a single fp16 coopVecMatMulAdd layer 64x64 (fp32 accumulate, fp16 output) over
2^22 vectors, weights in InferencingOptimal layout (the layout conversion is timed separately and
reported as `layout_conversion_us`).  Without --workload every other configuration is timed the same
way in the same run (W warm-up steps, K timed steps, HIP events on the launch stream) and reported
under "workloads": c1 (RowMajor weights, as the configuration names them), c2r (c2 with RowMajor weights), c2b (c2 in
bfloat16), c3, c3c (c3 with ColumnMajor weights), c4 (e4m3 decoded to the fp16 matrix pipeline), c4n (fp8 matrix pipeline),
c4h (c4 fed with fp16 vectors), c5f (forward pass of config 5's network at batch 2^22: the fp16 inference workload that the
matrix pipeline bounds), c5 (training step), c5l (c5 with the example's leaky ReLU behind every layer), c5r (c5 on the kernel whose waves share a tile by kind of work: opt-in, slower),
t32 / t128 (training steps of a 32-wide and of a 128-wide network), ex (one whole iteration of the example at its own shape: training step +
Adam update, two kernels in a HIP graph), op / rs (stand-alone outer-product / reduce-sum accumulate), pe / peb / ped
(permutohedral encoder: the reference test's configuration forward and reverse, and a decoder-shaped one in half), pef / peu
(that encoder and its decoder network in one kernel / as two calls), ew (an element-wise operator), ad (the Adam update
over 2^24 parameters), cm (the example's per-iteration layout conversion), nf (the neural module's FFLayer chain over a
parameter block), f32 / f32t (forward pass / training step of an fp32 network).  With --workload only that one runs and becomes the headline (profiling runs; also
c5g = c5 on the layer-by-layer step, copy = a plain device copy of
known size for scaling the traffic counters).  Prints ONE JSON line.

Before the W warm-up steps of a workload its step runs untimed for --clock-ramp-ms (default 100 ms,
reported as `clock_ramp_ms`): a fresh process finds the GPU in a low-power state whose clocks need
tens of milliseconds of continuous work to come up, far more than a handful of 0.2 ms steps; the
timed region is still exactly K steps and what it reports is the sustained rate.

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
MFMA_PEAK_TFLOPS = {"f16": 2500.0, "fp8": 5000.0, "int8": 5000.0, "f32": 157.3}

def profiled_traffic():
    """HBM bytes per step (all kernels of the step) as measured with rocprofv3 --pmc (FETCH_SIZE / WRITE_SIZE, scaled by a
    copy of known size): not measured by this script, read from the committed profile summaries, whose lines
    `traffic[<workload>] = <bytes> B per step` carry them.  {workload: (bytes, file)}"""
    import glob
    import re
    found = {}
    for path in sorted(glob.glob(os.path.join(REPO, "profiles", "*.md"))):
        with open(path) as f:
            for m in re.finditer(r"^traffic\[(\w+)\] = (\d+) B per step", f.read(), re.M):
                found[m.group(1)] = (int(m.group(2)), "profiles/" + os.path.basename(path))
    return found


def ensure_built():
    from slang_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from slang_amd import build
        build.build_library()
    return _lib.load()


def workload_c2(torch, cv, steps, warmup, bf16=False, row_major=False):
    """fp16 (or bfloat16) 64x64 matMulAdd, batch 2^22, InferencingOptimal (or RowMajor) weights."""
    import numpy as np
    from slang_amd.coopvec import CoopVecComponentType as CT, CoopVecMatrixLayout as ML, CooperativeVectorMatrixDesc as D
    dev = "cuda"
    B, M, K = 1 << 22, 64, 64
    ct, tdt = (CT.BFloat16, torch.bfloat16) if bf16 else (CT.Float16, torch.float16)
    g = torch.Generator(device=dev); g.manual_seed(20251)
    x = torch.randn(B, K, device=dev, generator=g).to(tdt)
    W = (torch.randn(M, K, device=dev, generator=g) / 8.0).to(tdt)
    b = (torch.rand(M, device=dev, generator=g) * 0.2 - 0.1).to(tdt)
    wrow = W.contiguous().view(torch.uint8).flatten()
    size = cv.getCooperativeVectorMatrixSize(M, K, ct, ML.InferencingOptimal)
    wopt = torch.empty(size, dtype=torch.uint8, device=dev)
    dst = [D(M, K, ct, ML.InferencingOptimal, size, 0, 0)]
    src = [D(M, K, ct, ML.RowMajor, M * K * 2, 0, K * 2)]
    cv.convertCooperativeVectorMatrix(wopt, dst, wrow, src)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        cv.convertCooperativeVectorMatrix(wopt, dst, wrow, src)
    e1.record(); torch.cuda.synchronize()
    conv_us = e0.elapsed_time(e1) / 20 * 1e3
    bb = b.view(torch.uint8)
    out = torch.empty(B, M, dtype=tdt, device=dev)

    def step():
        if row_major:
            cv.coopVecMatMulAdd(x, ct, wrow, 0, ct, bb, 0, ct, ML.RowMajor, False, K * 2, M=M, out=out)
        else:
            cv.coopVecMatMulAdd(x, ct, wopt, 0, ct, bb, 0, ct, ML.InferencingOptimal, False, 0, M=M, out=out)

    def cpu_baseline_bf16():
        import oracle_binding as ob
        n = 1 << 14
        xs = x[:n].view(torch.int16).cpu().numpy().view(np.uint16)
        Wn = W.view(torch.int16).cpu().numpy().view(np.uint8).ravel()
        bn = b.view(torch.int16).cpu().numpy().view(np.uint16)
        t0 = time.perf_counter()
        ob.ref_matmul_f32(xs, ob.BF16, Wn, ob.BF16, ob.ROW, 2 * K, M, K, bn, ob.BF16)
        t1 = time.perf_counter()
        return {"value": n / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": "first %d vectors, one core; the fp32-accumulate parity oracle (the reference has no bfloat16 "
                          "CoopVec component type, so there is no reference CPU form of this configuration)" % n}

    def cpu_baseline():
        import ctypes
        import concurrent.futures as cf
        import oracle_binding as ob
        L = ob.lib()
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")), 16)
        per_core = 1 << 17          # about 6 s on one core, then about 9 s on all of them
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

    name = "bf16" if bf16 else "fp16"
    key = "c2b" if bf16 else ("c2r" if row_major else "c2")
    layout = "RowMajor" if row_major else "InferencingOptimal"
    return dict(step=step, samples=B, alg_bytes=B * (K * 2 + M * 2), alg_flops=B * 2 * M * K,
                bound="hbm", mfma="f16", dtype="bf16" if bf16 else "f16",
                config={"workload": "%s: %s coopVecMatMulAdd 64x64, batch 2^22, %s weights, "
                                    "fp32 accumulate, %s out" % (key, name, layout, name), "batch": B, "m": M, "k": K,
                        "layout": layout},
                extra={} if row_major else {"layout_conversion_us": conv_us},
                cpu_baseline=cpu_baseline_bf16 if bf16 else cpu_baseline, key=key)


def workload_c2b(torch, cv, steps, warmup):
    return workload_c2(torch, cv, steps, warmup, bf16=True)


def workload_c2r(torch, cv, steps, warmup):
    return workload_c2(torch, cv, steps, warmup, row_major=True)


def workload_copy(torch, cv, steps, warmup):
    """A plain device-to-device copy of 2^29 bytes (torch's copy kernel): the known-size transfer that
    the FETCH_SIZE / WRITE_SIZE counters of the profiles are scaled by, and the box's copy ceiling."""
    n = 1 << 29
    src = torch.empty(n, dtype=torch.uint8, device="cuda").fill_(1)
    dst = torch.empty_like(src)

    def step():
        dst.copy_(src)

    return dict(step=step, samples=n, alg_bytes=2 * n, alg_flops=0, bound="hbm", mfma="f16", dtype="u8",
                config={"workload": "copy: plain device copy of 2^29 bytes (counter calibration, copy ceiling)", "bytes": n},
                cpu_baseline=lambda: None, key="copy", kernel="torch copy kernel")


def workload_c3(torch, cv, steps, warmup, column_major=False):
    """int8 128x128 -> int32 + int32 bias, batch 2^22, InferencingOptimal (or ColumnMajor) weights (bit-exact path)."""
    import numpy as np
    from slang_amd.coopvec import CoopVecComponentType as CT, CoopVecMatrixLayout as ML, CooperativeVectorMatrixDesc as D
    dev = "cuda"
    B, M, K = 1 << 22, 128, 128
    g = torch.Generator(device=dev); g.manual_seed(20253)
    x = torch.randint(-128, 128, (B, K), device=dev, dtype=torch.int8, generator=g)
    W = torch.randint(-127, 128, (M, K), device=dev, dtype=torch.int8, generator=g)
    b = torch.randint(-65536, 65537, (M,), device=dev, dtype=torch.int32, generator=g)
    wcol = W.t().contiguous().view(torch.uint8).flatten()          # ColumnMajor storage of the M x K matrix
    size = cv.getCooperativeVectorMatrixSize(M, K, CT.SignedInt8, ML.InferencingOptimal)
    wopt = torch.empty(size, dtype=torch.uint8, device=dev)
    dst, src = [D(M, K, CT.SignedInt8, ML.InferencingOptimal, size, 0, 0)], [D(M, K, CT.SignedInt8, ML.ColumnMajor, M * K, 0, M)]
    cv.convertCooperativeVectorMatrix(wopt, dst, wcol, src)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(20):
        cv.convertCooperativeVectorMatrix(wopt, dst, wcol, src)
    e1.record(); torch.cuda.synchronize()
    conv_us = e0.elapsed_time(e1) / 20 * 1e3
    bb = b.view(torch.uint8)
    out = torch.empty(B, M, dtype=torch.int32, device=dev)

    def step():
        if column_major:
            cv.coopVecMatMulAdd(x, CT.SignedInt8, wcol, 0, CT.SignedInt8, bb, 0, CT.SignedInt32, ML.ColumnMajor,
                                False, M, M=M, out=out)
        else:
            cv.coopVecMatMulAdd(x, CT.SignedInt8, wopt, 0, CT.SignedInt8, bb, 0, CT.SignedInt32, ML.InferencingOptimal,
                                False, 0, M=M, out=out)

    def cpu_baseline():
        import concurrent.futures as cf
        import oracle_binding as ob
        L = ob.lib()
        cores = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")), 16)
        per_core = 1 << 12
        n = per_core * cores
        xs = x[:n].cpu().numpy().view(np.uint32); Wn = wcol.cpu().numpy(); bn = b.cpu().numpy()
        outn = np.zeros((n, M), np.int32)

        def run(g0, g1):
            rc = L.cvo_slang_dispatch_matmul_add(g0, g1, n, ob.ptr(xs), K, ob.U32, K // 4, ob.S8P, K, ob.ptr(outn),
                                                 M * 4, ob.S32, M, ob.ptr(Wn), 0, ob.S8, ob.COL, 0, M,
                                                 ob.ptr(bn), 0, ob.S32, ob.HALF_RNE)
            assert rc == 0
        t0 = time.perf_counter(); run(0, per_core // 256); t1 = time.perf_counter()
        one_core = per_core / (t1 - t0)
        chunk = (n // 256) // cores
        t0 = time.perf_counter()
        with cf.ThreadPoolExecutor(cores) as pool:
            list(pool.map(lambda c: run(c * chunk, (c + 1) * chunk), range(cores)))
        t1 = time.perf_counter()
        return {"value": n / (t1 - t0), "unit": "samples/s", "cores": cores, "kind": "port", "value_1core": one_core,
                "sample": "first %d of the 2^22 vectors; C restatement of the Slang CPU-target fallback "
                          "(packed int8, ColumnMajor, int32 accumulate), -O2" % n}

    layout = "ColumnMajor" if column_major else "InferencingOptimal"
    return dict(step=step, samples=B, alg_bytes=B * (K + M * 4), alg_flops=B * 2 * M * K, bound="hbm", mfma="int8", dtype="int8",
                config={"workload": "%s: int8 coopVecMatMulAdd 128x128 -> int32 + int32 bias, batch 2^22, "
                                    "%s weights" % ("c3c" if column_major else "c3", layout), "batch": B, "m": M, "k": K, "layout": layout},
                extra={} if column_major else {"layout_conversion_us": conv_us},
                cpu_baseline=cpu_baseline, key="c3c" if column_major else "c3")


def workload_c3c(torch, cv, steps, warmup):
    return workload_c3(torch, cv, steps, warmup, column_major=True)


def _mlp_workload(torch, cv, dims, B, wtype_name, flags, key, desc, x_maker, init_std, with_bias=True, row_major=False,
                  bias_range=0.0, bound="hbm"):
    import numpy as np
    from slang_amd.coopvec import (Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML,
                                   CooperativeVectorMatrixDesc as D, FeedForwardLayer)
    dev = "cuda"
    g = torch.Generator(device=dev); g.manual_seed(20250 + len(dims))
    wtype = CT.Float16 if wtype_name == "f16" else CT.FloatE4M3
    layers, host = [], []
    for i in range(len(dims) - 1):
        fi, fo = dims[i], dims[i + 1]
        Wf = torch.randn(fo, fi, device=dev, generator=g) * init_std(fi)
        Wt = Wf.half() if wtype == CT.Float16 else Wf.clamp(-448, 448).to(torch.float8_e4m3fn)
        esz = Wt.element_size()
        wrow = Wt.contiguous().view(torch.uint8).flatten()
        if row_major:
            wmem, wlayout, wstride = wrow, ML.RowMajor, fi * esz
        else:
            size = cv.getCooperativeVectorMatrixSize(fo, fi, wtype, ML.InferencingOptimal)
            wmem, wlayout, wstride = torch.empty(size, dtype=torch.uint8, device=dev), ML.InferencingOptimal, 0
            cv.convertCooperativeVectorMatrix(wmem, [D(fo, fi, wtype, ML.InferencingOptimal, size, 0, 0)],
                                              wrow, [D(fo, fi, wtype, ML.RowMajor, fo * fi * esz, 0, fi * esz)])
        # the configurations have zero / no biases unless a range is given
        bias = ((torch.rand(fo, device=dev, generator=g) * 2 - 1) * bias_range).half()
        last = i == len(dims) - 2
        layers.append(FeedForwardLayer(fi, fo, wmem, bias.view(torch.uint8) if with_bias else None, wlayout, wstride,
                                       Activation.NoActivation if last else Activation.ReLU, 0.0))
        host.append((Wt, bias))
    x = x_maker(torch, g, B, dims[0], dev)
    out = torch.empty(B, dims[-1], dtype=torch.float16, device=dev)

    # the network description is marshalled once, as a C caller fills its CvMlpDesc once: a step is the
    # C-ABI call with the vectors (for the small configuration the Python marshalling would otherwise
    # cost more than the kernel)
    plan = cv.MlpForwardPlan(layers, weightType=wtype, flags=flags)

    def step():
        plan(x, out)

    macs = sum(dims[i] * dims[i + 1] for i in range(len(dims) - 1))
    in_bytes = dims[0] * x.element_size()

    def cpu_baseline():
        import oracle_binding as ob
        if wtype != CT.Float16:
            # the reference's CPU target cannot compile e4m3 CoopVec (no case in
            # __coopVecComponentTypeStride, hlsl.meta.slang:32636-32668): time the fp32 oracle instead
            n = 1 << 14
            specs = [dict(W=W.view(torch.uint8).cpu().numpy(), b=None, act=1 if i < len(host) - 1 else 0)
                     for i, (W, _) in enumerate(host)]
            xs = x[:n].view(torch.uint8).cpu().numpy()
            t0 = time.perf_counter(); ob.ref_mlp_forward(specs, xs, ob.E4M3); t1 = time.perf_counter()
            return {"value": n / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                    "sample": "first %d vectors; fp32-accumulate parity oracle (the Slang CPU target has no "
                              "e4m3 CoopVec, so there is no reference CPU build of this configuration)" % n}
        L = ob.lib()
        n = 1 << 13
        cur = x[:n].cpu().numpy()
        t0 = time.perf_counter()
        for i, (W, bias) in enumerate(host):
            fo, fi = W.shape
            Wn = W.cpu().numpy(); bn = bias.cpu().numpy()
            nxt = np.zeros((n, fo), np.float16)
            rc = L.cvo_slang_dispatch_matmul_add(0, (n + 255) // 256, n, ob.ptr(cur), fi * 2, ob.F16, fi, ob.F16, fi,
                                                 ob.ptr(nxt), fo * 2, ob.F16, fo, ob.ptr(Wn), 0, ob.F16, ob.ROW, 0,
                                                 fi * 2, ob.ptr(bn), 0, ob.F16, ob.HALF_SLANG)
            assert rc == 0
            cur = np.maximum(nxt, np.float16(0)) if i < len(host) - 1 else nxt
        t1 = time.perf_counter()
        return {"value": n / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": "first %d vectors, one core; C restatement of the Slang CPU-target fallback layer by "
                          "layer (fp16 accumulate, software half), -O2" % n}

    return dict(step=step, samples=B, alg_bytes=B * (in_bytes + dims[-1] * 2), alg_flops=B * 2 * macs,
                bound=bound, mfma="fp8" if flags == 1 else "f16", dtype=wtype_name,
                config={"workload": desc, "batch": B, "layers": dims}, cpu_baseline=cpu_baseline, key=key)


def workload_c1(torch, cv, steps, warmup):
    """fp16 2->16->16->16->1 ReLU MLP, batch 65536 (the CPU-runnable configuration)."""
    w = _mlp_workload(torch, cv, [2, 16, 16, 16, 1], 65536, "f16", 0, "c1",
                      "c1: fp16 MLP 2->16->16->16->1, ReLU, zero biases, RowMajor weights, batch 65536, fused forward",
                      lambda torch, g, B, k, dev: torch.rand(B, k, device=dev, generator=g).half(),
                      lambda fi: (1.0 / fi) ** 0.5, row_major=True)
    w["graph"] = True       # a few microseconds of kernel per step: launch-bound
    return w


def workload_c5f(torch, cv, steps, warmup, flags=0):
    """Forward pass of config 5's network: fp16 8->64->64->64->64->1, ReLU, biases, RowMajor weights, batch 2^22.
    25 728 flop against 18 bytes per sample: the fp16 inference workload that the matrix pipeline bounds."""
    return _mlp_workload(torch, cv, [8, 64, 64, 64, 64, 1], 1 << 22, "f16", flags, "c5f" if not flags else "c5f16",
                         "c5f: fp16 MLP 8->64->64->64->64->1 forward, ReLU, biases, RowMajor weights, batch 2^22, fused forward"
                         + (", kernels on 16-sample tiles" if flags else ""),
                         lambda torch, g, B, k, dev: (torch.rand(B, k, device=dev, generator=g) * 2 - 1).half(),
                         lambda fi: (2.0 / fi) ** 0.5, row_major=True, bias_range=0.1, bound="mfma")


def workload_c5f16(torch, cv, steps, warmup):
    return workload_c5f(torch, cv, steps, warmup, flags=cv.FLAG_FORWARD_TILE16)


def workload_c4(torch, cv, steps, warmup, flags=0):
    """e4m3 32->64->64->8 decoder MLP, batch 2^24."""
    w = _mlp_workload(torch, cv, [32, 64, 64, 8], 1 << 24, "fp8", flags, "c4" if not flags else "c4n",
                         "c4: e4m3 MLP 32->64->64->8, ReLU, fp16 out, batch 2^24, fused forward, "
                         + ("fp8 matrix pipeline" if flags else "e4m3 decoded to the fp16 matrix pipeline"),
                         lambda torch, g, B, k, dev: (torch.randn(B, k, device=dev, generator=g) * 0.5).to(torch.float8_e4m3fn),
                         lambda fi: 0.5, with_bias=False)
    if not flags:
        # What bounds this kernel is issue on the vector-ALU port, not HBM or the matrix pipeline: per 32-sample tile
        # 32 conversions to e4m3 (8.3 cycles each), 16 matrix instructions (7.3) and 127 other vector instructions (4.3),
        # 512 tiles per SIMD, at the 1.945 GHz the shader clock settles at under this load.
        w["issue_bound"] = {"ms": 929 * 512 / 1.945e9 * 1e3,
                            "model": "929 vector-ALU port cycles per 32-sample tile (32 x 8.3 + 16 x 7.3 + 127 x 4.3), "
                                     "512 tiles per SIMD, 1.945 GHz"}
    return w


def workload_c4n(torch, cv, steps, warmup):
    return workload_c4(torch, cv, steps, warmup, flags=1)


def workload_c4h(torch, cv, steps, warmup):
    """c4 in the form the Slang API takes: fp16 vectors with inputInterpretation FloatE4M3 (quantised on load)."""
    return _mlp_workload(torch, cv, [32, 64, 64, 8], 1 << 24, "fp8", 0, "c4h",
                         "c4h: e4m3 MLP 32->64->64->8 fed with fp16 vectors (inputInterpretation FloatE4M3, quantised "
                         "on load), ReLU, fp16 out, batch 2^24, e4m3 decoded to the fp16 matrix pipeline",
                         lambda torch, g, B, k, dev: (torch.randn(B, k, device=dev, generator=g) * 0.5).half(),
                         lambda fi: 0.5, with_bias=False)


def workload_f32(torch, cv, steps, warmup):
    """Forward pass of a network of float (the neural module's FFLayer<float> chain), 32->64->64->8, batch 2^22."""
    import numpy as np
    from slang_amd.coopvec import Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML, FeedForwardLayer
    dev = "cuda"
    dims = [32, 64, 64, 8]
    B = 1 << 22
    g = torch.Generator(device=dev); g.manual_seed(20259)
    layers, host = [], []
    for i in range(len(dims) - 1):
        fi, fo = dims[i], dims[i + 1]
        W = torch.randn(fo, fi, device=dev, generator=g) * (2.0 / fi) ** 0.5
        bias = torch.randn(fo, device=dev, generator=g) * 0.1
        last = i == len(dims) - 2
        layers.append(FeedForwardLayer(fi, fo, W.contiguous().view(torch.uint8).flatten(), bias.view(torch.uint8), ML.RowMajor, fi * 4,
                                       Activation.NoActivation if last else Activation.ReLU, 0.0))
        host.append((W, bias))
    x = torch.rand(B, dims[0], device=dev, generator=g) * 2 - 1
    out = torch.empty(B, dims[-1], dtype=torch.float32, device=dev)
    plan = cv.MlpForwardPlan(layers, weightType=CT.Float32)

    def step():
        plan(x, out)

    macs = sum(dims[i] * dims[i + 1] for i in range(len(dims) - 1))

    def cpu_baseline():
        n = 1 << 17
        h = x[:n].cpu().numpy()
        t0 = time.perf_counter()
        for i, (W, b) in enumerate(host):
            h = h @ W.cpu().numpy().T + b.cpu().numpy()
            if i < len(host) - 1:
                h = np.maximum(h, 0)
        t1 = time.perf_counter()
        return {"value": n / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": "first %d vectors; numpy fp32 (the fallback's arithmetic for T = float is plain fp32 products and sums)" % n}

    return dict(step=step, samples=B, alg_bytes=B * (dims[0] + dims[-1]) * 4, alg_flops=B * 2 * macs, bound="hbm", mfma="f32",
                dtype="f32", config={"workload": "f32: fp32 MLP 32->64->64->8, ReLU, fp32 in and out, batch 2^22, fused forward "
                                                 "(v_mfma_f32_16x16x4_f32)", "batch": B, "layers": dims},
                cpu_baseline=cpu_baseline, key="f32")


def workload_c5(torch, cv, steps, warmup, flags=0, dims=None, key=None, leaky=False):
    """fp16 training step 8->64->64->64->64->1, ReLU, MSE vs sin(sum x), batch 2^20, fp32 TrainingOptimal grads."""
    import numpy as np
    from slang_amd.coopvec import (Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML,
                                   FeedForwardLayer)
    dev = "cuda"
    dims = dims or [8, 64, 64, 64, 64, 1]
    B = 1 << 20
    g = torch.Generator(device=dev); g.manual_seed(20255)
    layers, host = [], []
    for i in range(len(dims) - 1):
        fi, fo = dims[i], dims[i + 1]
        W = (torch.randn(fo, fi, device=dev, generator=g) * (2.0 / fi) ** 0.5).half()        # He init
        bias = torch.zeros(fo, dtype=torch.float16, device=dev)
        gsize = cv.getCooperativeVectorMatrixSize(fo, fi, CT.Float32, ML.TrainingOptimal)
        wg = torch.zeros(gsize, dtype=torch.uint8, device=dev)
        bg = torch.zeros(fo, dtype=torch.float32, device=dev)
        last = i == len(dims) - 2
        # (leaky: the example's FeedForwardLayer, max(z, 0.001 z) behind every layer, the last one too: fflayer.slang:60-66)
        act = Activation.LeakyReLU if leaky else (Activation.NoActivation if last else Activation.ReLU)
        layers.append(FeedForwardLayer(fi, fo, W.contiguous().view(torch.uint8).flatten(), bias.view(torch.uint8),
                                       ML.RowMajor, fi * 2, act, 0.001 if leaky else 0.0,
                                       wg, bg.view(torch.uint8), ML.TrainingOptimal, 0))
        host.append((W, bias))
    x = (torch.rand(B, dims[0], device=dev, generator=g) * 2 - 1).half()
    ws = torch.empty(cv.mlpTrainStepWorkspaceSize(layers, B, flags=flags), dtype=torch.uint8, device=dev)
    loss = torch.zeros(1, dtype=torch.float32, device=dev)

    def step():
        cv.mlpTrainStep(layers, x, None, workspace=ws, lossSum=loss, flags=flags)

    macs = sum(dims[i] * dims[i + 1] for i in range(len(dims) - 1))
    macs_dx = sum(dims[i] * dims[i + 1] for i in range(1, len(dims) - 1))

    def cpu_baseline():
        import oracle_binding as ob
        n = 1 << 11
        specs = [dict(W=W.cpu().numpy(), b=b.cpu().numpy(), act=(2 if leaky else 1) if (leaky or i < len(host) - 1) else 0,
                      slope=float(np.float16(0.001)) if leaky else 0.0)
                 for i, (W, b) in enumerate(host)]
        xs = x[:n].cpu().numpy()
        t0 = time.perf_counter(); ob.ref_mlp_train(specs, xs, None, 1.0, True); t1 = time.perf_counter()
        return {"value": n / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": "first %d samples, one core; the parity oracle's training step (fp16 carriers, fp32 forward "
                          "sums, fp64 gradient sums). The Slang CPU target cannot run the example's learnGradient "
                          "(wave intrinsics and atomics, docs/cpu-target.md:15-21)" % n}

    return dict(step=step, samples=B, alg_bytes=B * dims[0] * 2, alg_flops=B * 2 * (2 * macs + macs_dx),
                bound="mfma", mfma="f16", dtype="f16",
                config={"workload": "%s: fp16 train step %s, %s, MSE vs sin(sum x), batch 2^20, "
                                    "fp32 TrainingOptimal gradients, deterministic reduction%s"
                                    % (key or ("c5g" if flags else "c5"), "->".join(str(d) for d in dims),
                                       "leaky ReLU (slope 0.001) behind every layer, as the example's layers have it" if leaky else "ReLU",
                                       ", layer-by-layer step (the one for arbitrary layer sizes)" if flags == cv.FLAG_LAYERWISE_TRAINING
                                       else ", waves split by kind of work (CV_FLAG_TRAIN_SPLIT_BY_ROLE)" if flags else ""),
                        "batch": B, "layers": dims},
                cpu_baseline=cpu_baseline, key=key or ("c5g" if flags else "c5"))


def workload_f32t(torch, cv, steps, warmup):
    """fp32 training step 32->64->64->8 (FFLayer<float> chain), ReLU, MSE against given targets, batch 2^20, fp32 TrainingOptimal
    gradients: the layer-by-layer step on the fp32 matMul, element-wise and outer-product kernels."""
    import numpy as np
    from slang_amd.coopvec import (Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML,
                                   FeedForwardLayer)
    dev = "cuda"
    dims = [32, 64, 64, 8]
    B = 1 << 20
    g = torch.Generator(device=dev); g.manual_seed(20256)
    layers, host = [], []
    for i in range(len(dims) - 1):
        fi, fo = dims[i], dims[i + 1]
        W = torch.randn(fo, fi, device=dev, generator=g) * (2.0 / fi) ** 0.5
        bias = torch.randn(fo, device=dev, generator=g) * 0.1
        gsize = cv.getCooperativeVectorMatrixSize(fo, fi, CT.Float32, ML.TrainingOptimal)
        wg = torch.zeros(gsize, dtype=torch.uint8, device=dev)
        bg = torch.zeros(fo, dtype=torch.float32, device=dev)
        last = i == len(dims) - 2
        layers.append(FeedForwardLayer(fi, fo, W.contiguous().view(torch.uint8).flatten(), bias.view(torch.uint8),
                                       ML.RowMajor, fi * 4, Activation.NoActivation if last else Activation.ReLU, 0.0,
                                       wg, bg.view(torch.uint8), ML.TrainingOptimal, 0))
        host.append((W, bias))
    x = torch.rand(B, dims[0], device=dev, generator=g) * 2 - 1
    t = torch.rand(B, dims[-1], device=dev, generator=g) * 2 - 1
    ws = torch.empty(cv.mlpTrainStepWorkspaceSize(layers, B, weightType=CT.Float32), dtype=torch.uint8, device=dev)
    loss = torch.zeros(1, dtype=torch.float32, device=dev)

    def step():
        cv.mlpTrainStep(layers, x, t, workspace=ws, lossSum=loss, lossScale=1.0 / B, weightType=CT.Float32)

    macs = sum(dims[i] * dims[i + 1] for i in range(len(dims) - 1))
    macs_dx = sum(dims[i] * dims[i + 1] for i in range(1, len(dims) - 1))

    def cpu_baseline():
        n = 1 << 15
        xs, ts = x[:n].cpu().numpy(), t[:n].cpu().numpy()
        Ws = [(W.cpu().numpy(), b.cpu().numpy()) for W, b in host]
        t0 = time.perf_counter()
        acts, zs, h = [xs], [], xs
        for i, (W, b) in enumerate(Ws):
            z = h @ W.T + b
            zs.append(z)
            h = np.maximum(z, 0) if i < len(Ws) - 1 else z
            acts.append(h)
        gz = (h - ts) * (2.0 / B)
        for i in range(len(Ws) - 1, -1, -1):
            dW = gz.T @ acts[i]; db = gz.sum(axis=0)
            if i:
                gz = (gz @ Ws[i][0]) * (zs[i - 1] > 0)
        t1 = time.perf_counter()
        return {"value": n / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": "first %d samples; numpy fp32 backpropagation (for T = float the fallback's arithmetic is plain fp32 "
                          "products and sums)" % n}

    # (the bytes a layer-by-layer step moves: every per-layer vector of the batch is written once and read by its consumers)
    widths = dims[1:]
    moved = B * 4 * (dims[0] * 2 + dims[-1] + sum(w * (2 + 3) for w in widths[:-1]) + widths[-1] * 4 + sum(w * 4 for w in widths[:-1]))
    return dict(step=step, samples=B, alg_bytes=moved, alg_flops=B * 2 * (2 * macs + macs_dx),
                bound="hbm", mfma="f32", dtype="f32",
                config={"workload": "f32t: fp32 train step 32->64->64->8, ReLU, MSE against targets, batch 2^20, fp32 "
                                    "TrainingOptimal gradients, layer-by-layer step (fp32 networks have no fused one)",
                        "batch": B, "layers": dims},
                cpu_baseline=cpu_baseline, key="f32t")


def workload_c5l(torch, cv, steps, warmup):
    """config 5's network built from the example's layer: leaky ReLU behind every layer (the paired kernel's leaky instantiation)"""
    return workload_c5(torch, cv, steps, warmup, key="c5l", leaky=True)


def workload_t32(torch, cv, steps, warmup):
    """the training step of a 32-wide decoder-sized network, 8->32->32->32->4 (the one-wave fused kernel)"""
    return workload_c5(torch, cv, steps, warmup, dims=[8, 32, 32, 32, 4], key="t32")


def workload_t128(torch, cv, steps, warmup):
    """the training step of a 128-wide network, 16->128->128->8 (the fused kernel in which four waves share the dW accumulators)"""
    return workload_c5(torch, cv, steps, warmup, dims=[16, 128, 128, 8], key="t128")


def workload_c5g(torch, cv, steps, warmup):
    return workload_c5(torch, cv, steps, warmup, flags=cv.FLAG_LAYERWISE_TRAINING)


def workload_c5r(torch, cv, steps, warmup):
    """c5 on the kernel whose waves share a tile of samples by kind of work (weights in registers); not the default"""
    return workload_c5(torch, cv, steps, warmup, flags=cv.FLAG_TRAIN_SPLIT_BY_ROLE, key="c5r")


def workload_ex(torch, cv, steps, warmup):
    """One whole iteration of examples/mlp-training-coopvec at its own shape (mlp-training-coopvec.cpp:164-250):
    4 -> 16 -> 4, leaky ReLU, 16 float2 samples encoded (x, y, x^2, y^2), fp16 TrainingOptimal gradients; learnGradient
    (cvMlpTrainStep: one kernel, the single workgroup of such a small batch adds its sums to the gradients itself) + the
    parameter update read straight from those gradients (cvMlpAdamStep: one kernel, which also leaves them cleared).
    Launch-bound: the figure to hold it against is the cost of two graph nodes."""
    import numpy as np
    from slang_amd.coopvec import Activation, CoopVecComponentType as CT, CoopVecMatrixLayout as ML, FeedForwardLayer
    dev = "cuda"
    dims = [4, 16, 4]
    n = 16
    g = torch.Generator(device=dev); g.manual_seed(1072)
    layers, wst, bst, host = [], [], [], []
    slope = float(np.float16(0.001))
    for i in range(len(dims) - 1):
        fi, fo = dims[i], dims[i + 1]
        W = (torch.rand(fo, fi, device=dev, generator=g) * 2 - 1).half()
        b = (torch.rand(fo, device=dev, generator=g) * 2 - 1).half()
        gsize = cv.getCooperativeVectorMatrixSize(fo, fi, CT.Float16, ML.TrainingOptimal)
        wg = torch.zeros(gsize, dtype=torch.uint8, device=dev)
        bg = torch.zeros(fo, dtype=torch.float16, device=dev)
        layers.append(FeedForwardLayer(fi, fo, W.view(torch.uint8).flatten(), b.view(torch.uint8), ML.RowMajor, fi * 2,
                                       Activation.LeakyReLU, slope, wg, bg.view(torch.uint8), ML.TrainingOptimal, 0))
        wst.append(torch.zeros(fo * fi * 8, dtype=torch.uint8, device=dev))
        bst.append(torch.zeros(fo * 8, dtype=torch.uint8, device=dev))
        host.append((W.clone(), b.clone()))
    xy = torch.rand(n, 2, device=dev, generator=g)
    ws = torch.empty(cv.mlpTrainStepWorkspaceSize(layers, n, gradType=CT.Float16, inputEncoding=1), dtype=torch.uint8, device=dev)
    loss = torch.zeros(1, dtype=torch.float32, device=dev)
    lmax = torch.zeros(1, dtype=torch.float32, device=dev)

    def step():
        cv.mlpTrainStep(layers, xy, None, gradType=CT.Float16, workspace=ws, lossSum=loss, lossMax=lmax, inputEncoding=1)
        cv.mlpAdjustParameters(layers, wst, bst, gradType=CT.Float16)

    macs = sum(dims[i] * dims[i + 1] for i in range(len(dims) - 1))
    nparams = sum(dims[i] * dims[i + 1] + dims[i + 1] for i in range(len(dims) - 1))

    def cpu_baseline():
        import oracle_binding as ob
        specs = [dict(W=W.cpu().numpy(), b=b.cpu().numpy(), act=2, slope=slope) for W, b in host]
        xs = xy.cpu().numpy().astype(np.float16)
        enc = np.concatenate([xs, (xs.astype(np.float32) ** 2).astype(np.float16)], axis=1)
        tgt = np.zeros((n, 4), np.float16)
        p = np.zeros(nparams, np.float16); st = np.zeros(nparams, ob.ADAM_STATE_DTYPE); gr = np.zeros(nparams, np.float16)
        reps = 200
        t0 = time.perf_counter()
        for _ in range(reps):
            ob.ref_mlp_train(specs, enc, tgt, 1.0, True)
            ob.slang_adam_step(st, p, gr)
        t1 = time.perf_counter()
        return {"value": reps * n / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": "%d iterations of 16 samples, one core; the parity oracle's training step plus the C restatement "
                          "of AdamOptimizer::step, called from Python" % reps}

    w = dict(step=step, samples=n, alg_bytes=n * 8 + nparams * 12, alg_flops=n * 2 * (3 * macs), bound="hbm", mfma="f16",
             dtype="f16", cpu_baseline=cpu_baseline, key="ex",
             config={"workload": "ex: one iteration of the example (4->16->4, leaky ReLU, 16 float2 samples, fp16 TrainingOptimal "
                                 "gradients): learnGradient + Adam update read from those gradients, two kernels", "batch": n,
                     "layers": dims, "launches_per_step": 2})
    w["graph"] = True
    w["launch_floor_us"] = 2 * 1.6      # two graph nodes; an empty kernel costs 1.6 us per node of a HIP graph on MI355X
    return w


def workload_pe(torch, cv, steps, warmup, backward=False, decoder=False):
    """PermutoEncoder.encode (or its reverse mode) over 2^22 positions.  `pe` / `peb`: the configuration of the
    reference's own test (tests/neural/permuto-encoder-test.slang: 2 dimensions, 2 features per entry, 2^8 entries per
    level, 4 levels, fp32) scaled to 2^22 positions.  `ped`: a neural-texture shaped encoder in half (3 dimensions, 2
    features, 2^12 entries, 8 levels: 16 features per position), the input of a 16-wide decoder MLP.  What a position
    costs in memory: its coordinates in, levels x features out, and (D+1) gathered table entries per level, which
    these tables serve from the caches."""
    import numpy as np
    dev = "cuda"
    B = 1 << 22
    if decoder:
        D, F, log2, levels, dt = 3, 2, 12, 8, torch.float16
        enc = cv.PermutoEncoder(D, F, log2, levels, baseScale=4.0, log2PerLevelScale=1.0, dtype=dt)
    else:
        D, F, log2, levels, dt = 2, 2, 8, 4, torch.float32
        enc = cv.PermutoEncoder(D, F, log2, levels, baseScale=1.0, log2PerLevelScale=1.0, maxLevelRatio=1.1, seed=1337, dtype=dt)
    g = torch.Generator(device=dev); g.manual_seed(20260)
    pos = torch.rand(B, D, device=dev, generator=g).to(dt)
    table = (torch.randn(enc.featureTableElements, device=dev, generator=g) * 0.5).to(dt)
    out = torch.empty(B, enc.outputSize, dtype=dt, device=dev)
    esz = pos.element_size()
    if backward:
        dout = torch.randn(B, enc.outputSize, device=dev, generator=g)
        dtab = torch.zeros_like(table)

        def step():
            enc.backward(pos, table, dout, dFeatureTable=dtab)
        alg = B * (D * esz + enc.outputSize * esz + D * esz)
    else:
        def step():
            enc.encode(pos, table, out=out)
        alg = B * (D * esz + enc.outputSize * esz)
    gathered = B * (D + 1) * levels * F * esz

    def cpu_baseline():
        import oracle_binding as ob
        n = 1 << 15
        lv = ob.permuto_levels(D, log2, levels, 4.0 if decoder else 1.0, 1.0, 1337)
        pn = pos[:n].cpu().numpy(); tn = table.cpu().numpy()
        t0 = time.perf_counter(); ob.permuto_encode(lv, F, 1.1 * levels, pn, tn); t1 = time.perf_counter()
        return {"value": n / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": "first %d positions, one core; C restatement of PermutoEncoder.encode (forward)" % n}

    key = "ped" if decoder else ("peb" if backward else "pe")
    return dict(step=step, samples=B, alg_bytes=alg, alg_flops=0, bound="hbm", mfma="f32", dtype="f16" if decoder else "f32",
                cpu_baseline=cpu_baseline, key=key, extra={"gathered_table_bytes_per_step": gathered},
                config={"workload": "%s: PermutoEncoder %s, %d dimensions, %d features per entry, 2^%d entries per level, %d levels, %s, "
                                    "2^22 positions" % (key, "reverse mode (atomic adds into the table gradient)" if backward else "encode",
                                                        D, F, log2, levels, "fp16" if decoder else "fp32"),
                        "batch": B})


def workload_pef(torch, cv, steps, warmup, fused=True):
    """The neural-texture pipeline: encoder of `ped` (3 dimensions, 2 features, 2^12 entries, 8 levels, half) and its
    decoder 16 -> 64 -> 64 -> 3 (ReLU) over 2^22 positions.  `pef`: one kernel (cvPermutoMlpForward), the encoded vectors
    never reach memory; `peu`: cvPermutoEncode then cvMlpForward, which write and re-read 32 bytes per position."""
    import numpy as np
    from slang_amd.coopvec import Activation, CoopVecMatrixLayout as ML, FeedForwardLayer
    dev = "cuda"
    B = 1 << 22
    D, F, log2, levels = 3, 2, 12, 8
    enc = cv.PermutoEncoder(D, F, log2, levels, baseScale=4.0, log2PerLevelScale=1.0, dtype=torch.float16)
    g = torch.Generator(device=dev); g.manual_seed(20263)
    pos = torch.rand(B, D, device=dev, generator=g).half()
    table = (torch.randn(enc.featureTableElements, device=dev, generator=g) * 0.5).half()
    dims = [16, 64, 64, 3]
    layers, host = [], []
    for i in range(len(dims) - 1):
        fi, fo = dims[i], dims[i + 1]
        W = (torch.randn(fo, fi, device=dev, generator=g) * (2.0 / fi) ** 0.5).half()
        b = (torch.rand(fo, device=dev, generator=g) * 0.2 - 0.1).half()
        layers.append(FeedForwardLayer(fi, fo, W.view(torch.uint8).flatten(), b.view(torch.uint8), ML.RowMajor, fi * 2,
                                       Activation.ReLU if i < len(dims) - 2 else Activation.NoActivation, 0.0))
        host.append((W, b))
    out = torch.empty(B, dims[-1], dtype=torch.float16, device=dev)
    feats = torch.empty(B, dims[0], dtype=torch.float16, device=dev)
    plan = cv.MlpForwardPlan(layers)

    if fused:
        def step():
            enc.encodeAndEval(pos, table, layers, out=out)
    else:
        def step():
            enc.encode(pos, table, out=feats)
            plan(feats, out=out)

    macs = sum(dims[i] * dims[i + 1] for i in range(len(dims) - 1))

    def cpu_baseline():
        import oracle_binding as ob
        n = 1 << 14
        lv = ob.permuto_levels(D, log2, levels, 4.0, 1.0, 1337)
        pn = pos[:n].cpu().numpy(); tn = table.cpu().numpy()
        specs = [dict(W=W.cpu().numpy(), b=b.cpu().numpy(), act=1 if i < len(host) - 1 else 0, slope=0.0) for i, (W, b) in enumerate(host)]
        t0 = time.perf_counter()
        f = ob.permuto_encode(lv, F, 1.1 * levels, pn, tn)
        ob.ref_mlp_forward(specs, f, ob.F16)
        t1 = time.perf_counter()
        return {"value": n / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": "first %d positions, one core; C restatements of PermutoEncoder.encode and of the layer chain" % n}

    key = "pef" if fused else "peu"
    return dict(step=step, samples=B, alg_bytes=B * (D * 2 + dims[-1] * 2), alg_flops=B * 2 * macs, bound="hbm", mfma="f16", dtype="f16",
                cpu_baseline=cpu_baseline, key=key,
                config={"workload": "%s: PermutoEncoder (3 dimensions, 2 features per entry, 2^12 entries per level, 8 levels, fp16) + decoder "
                                    "16->64->64->3 (ReLU), 2^22 positions, %s" % (key, "one kernel" if fused else "two calls, features through memory"),
                        "batch": B, "layers": dims})


def workload_peu(torch, cv, steps, warmup):
    return workload_pef(torch, cv, steps, warmup, fused=False)


def workload_peb(torch, cv, steps, warmup):
    return workload_pe(torch, cv, steps, warmup, backward=True)


def workload_ped(torch, cv, steps, warmup):
    return workload_pe(torch, cv, steps, warmup, decoder=True)


def workload_cm(torch, cv, steps, warmup):
    """convertCooperativeVectorMatrix as the example calls it once per iteration (mlp-training-coopvec.cpp:203-236): the
    weight gradients of every layer from TrainingOptimal to RowMajor, fp16, one call; here for config 5's five layers
    (12.9 K elements).  Launch-bound."""
    from slang_amd.coopvec import CoopVecComponentType as CT, CoopVecMatrixLayout as ML, CooperativeVectorMatrixDesc as D
    dev = "cuda"
    dims = [8, 64, 64, 64, 64, 1]
    src, dst, so, do = [], [], 0, 0
    for i in range(len(dims) - 1):
        fi, fo = dims[i], dims[i + 1]
        ssz = cv.getCooperativeVectorMatrixSize(fo, fi, CT.Float16, ML.TrainingOptimal)
        dsz = cv.getCooperativeVectorMatrixSize(fo, fi, CT.Float16, ML.RowMajor, fi * 2)
        src.append(D(fo, fi, CT.Float16, ML.TrainingOptimal, ssz, so, 0)); so += (ssz + 63) // 64 * 64
        dst.append(D(fo, fi, CT.Float16, ML.RowMajor, dsz, do, fi * 2)); do += (dsz + 63) // 64 * 64
    g = torch.Generator(device=dev); g.manual_seed(20264)
    sbuf = torch.randint(0, 255, (so,), dtype=torch.uint8, device=dev, generator=g)
    dbuf = torch.zeros(do, dtype=torch.uint8, device=dev)
    elems = sum(dims[i] * dims[i + 1] for i in range(len(dims) - 1))

    def step():
        cv.convertCooperativeVectorMatrix(dbuf, dst, sbuf, src)

    w = dict(step=step, samples=elems, alg_bytes=elems * 4, alg_flops=0, bound="hbm", mfma="f16", dtype="f16", cpu_baseline=lambda: None,
             key="cm", config={"workload": "cm: convertCooperativeVectorMatrix, the five weight-gradient matrices of 8->64x4->1 from "
                                           "TrainingOptimal to RowMajor (fp16) in one call, as once per iteration of the example",
                               "elements": elems, "launches_per_step": 1})
    w["graph"] = True
    w["launch_floor_us"] = 1.6
    return w


def workload_nf(torch, cv, steps, warmup):
    """The neural module's front: FFLayer chain 32 -> 64 -> 64 -> 8 (ReLU) of halfs evaluated from one parameter block in
    the optimal layout (cvNeuralMlpForward after cvNeuralToOptimalLayout; layers.slang:34-110), 2^22 samples."""
    import numpy as np
    from slang_amd.coopvec import Activation
    dev = "cuda"
    B = 1 << 22
    dims = [32, 64, 64, 8]
    conv = cv.NetworkParameterLayoutConverter(torch.float16, 0b111, *dims)
    g = torch.Generator(device=dev); g.manual_seed(20265)
    portable = (torch.randn(conv.ElementCountLogical, device=dev, generator=g) * 0.15).half()
    optimal = conv.toOptimalLayout(portable)
    x = torch.randn(B, dims[0], device=dev, generator=g).half()
    out = torch.empty(B, dims[-1], dtype=torch.float16, device=dev)
    acts = [Activation.ReLU, Activation.ReLU, Activation.NoActivation]

    def step():
        conv.eval(optimal, x, optimalLayout=True, activations=acts, out=out)

    macs = sum(dims[i] * dims[i + 1] for i in range(len(dims) - 1))
    return dict(step=step, samples=B, alg_bytes=B * (dims[0] + dims[-1]) * 2, alg_flops=B * 2 * macs, bound="hbm", mfma="f16", dtype="f16",
                cpu_baseline=lambda: None, key="nf",
                config={"workload": "nf: cvNeuralMlpForward, FFLayer chain 32->64->64->8 (ReLU) of halfs from one parameter block in the "
                                    "optimal layout, 2^22 samples", "batch": B, "layers": dims})


def workload_ew(torch, cv, steps, warmup):
    """An element-wise operator of CoopVec<half, 64> over 2^22 vectors: tanh (hlsl.meta.slang:32383-32401), 2 bytes in and
    2 bytes out per element."""
    import numpy as np
    from slang_amd.coopvec import ElementwiseOp
    dev = "cuda"
    B, N = 1 << 22, 64
    g = torch.Generator(device=dev); g.manual_seed(20261)
    x = (torch.rand(B, N, device=dev, generator=g) * 4 - 2).half()
    out = torch.empty_like(x)

    def step():
        cv.elementwise(ElementwiseOp.Tanh, x, out=out)

    def cpu_baseline():
        import oracle_binding as ob
        n = 1 << 14
        xn = x[:n].cpu().numpy()
        t0 = time.perf_counter(); ob.elementwise(int(ElementwiseOp.Tanh), xn); t1 = time.perf_counter()
        return {"value": n / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": "first %d vectors, one core; the oracle's element loop (double tanh, one rounding to half)" % n}

    return dict(step=step, samples=B, alg_bytes=B * N * 4, alg_flops=0, bound="hbm", mfma="f16", dtype="f16", cpu_baseline=cpu_baseline,
                key="ew", config={"workload": "ew: element-wise tanh of CoopVec<half,64> over 2^22 vectors", "batch": B, "n": N})


def workload_ad(torch, cv, steps, warmup):
    """adjustParameters (AdamOptimizer::step in half) over 2^24 parameters: per parameter 2 + 2 + 8 bytes read and as
    many written (parameter, gradient, AdamState)."""
    import numpy as np
    dev = "cuda"
    n = 1 << 24
    g = torch.Generator(device=dev); g.manual_seed(20262)
    params = (torch.rand(n, device=dev, generator=g) * 2 - 1).half()
    grads = (torch.randn(n, device=dev, generator=g) * 0.1).half()
    states = torch.zeros(n * 8, dtype=torch.uint8, device=dev)

    def step():
        cv.adjustParameters(states, params, grads)     # the gradients read are zero from the second step on: same traffic

    def cpu_baseline():
        import oracle_binding as ob
        m = 1 << 18
        p = params[:m].cpu().numpy(); gr = (np.random.default_rng(0).standard_normal(m) * 0.1).astype(np.float16)
        st = np.zeros(m, ob.ADAM_STATE_DTYPE)
        t0 = time.perf_counter(); ob.slang_adam_step(st, p, gr); t1 = time.perf_counter()
        return {"value": m / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": "%d parameters, one core; C restatement of adjustParameters + AdamOptimizer::step (software half)" % m}

    return dict(step=step, samples=n, alg_bytes=n * 24, alg_flops=0, bound="hbm", mfma="f16", dtype="f16", cpu_baseline=cpu_baseline,
                key="ad", config={"workload": "ad: adjustParameters (Adam step in half) over 2^24 fp16 parameters", "parameters": n})


def workload_op(torch, cv, steps, warmup):
    """stand-alone coopVecOuterProductAccumulate 64x64 over 2^20 vector pairs, fp32 TrainingOptimal destination."""
    from slang_amd.coopvec import CoopVecComponentType as CT, CoopVecMatrixLayout as ML
    dev = "cuda"
    B, M, N = 1 << 20, 64, 64
    g = torch.Generator(device=dev); g.manual_seed(20256)
    a = (torch.randn(B, M, device=dev, generator=g) * 0.25).half()
    b = (torch.rand(B, N, device=dev, generator=g) * 2 - 1).half()
    size = cv.getCooperativeVectorMatrixSize(M, N, CT.Float32, ML.TrainingOptimal)
    mat = torch.zeros(size, dtype=torch.uint8, device=dev)
    import ctypes
    from slang_amd import _lib
    need = ctypes.c_size_t(0)
    _lib.load().cvOuterProductAccumulateWorkspaceSize(M, N, B, ctypes.byref(need))
    ws = torch.empty(max(need.value, 16), dtype=torch.uint8, device=dev)

    def step():
        cv.coopVecOuterProductAccumulate(a, b, mat, 0, 0, ML.TrainingOptimal, CT.Float32, workspace=ws)

    def cpu_baseline():
        import numpy as np
        import oracle_binding as ob
        n = 1 << 12
        an, bn = a[:n].cpu().numpy(), b[:n].cpu().numpy()
        dst = np.zeros((M, N), np.float16)
        L = ob.lib()
        t0 = time.perf_counter()
        for s_ in range(n):
            rc = L.cvo_slang_outer_product_accumulate(ob.ptr(an[s_]), M, ob.ptr(bn[s_]), N, ob.F16, ob.ptr(dst), 0,
                                                      N * 2, ob.ROW, ob.F16, ob.HALF_SLANG)
            assert rc == 0
        t1 = time.perf_counter()
        return {"value": n / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": "first %d vector pairs, one core; C restatement of the Slang CPU-target fallback "
                          "(per-thread load-add-store in half, RowMajor), -O2, called per thread from Python" % n}

    return dict(step=step, samples=B, alg_bytes=B * (M + N) * 2, alg_flops=B * 2 * M * N, bound="hbm", mfma="f16",
                dtype="f16", config={"workload": "op: coopVecOuterProductAccumulate 64x64 over 2^20 fp16 vector pairs, "
                                                 "fp32 TrainingOptimal destination, deterministic reduction",
                                     "batch": B, "m": M, "n": N}, cpu_baseline=cpu_baseline, key="op")


def workload_rs(torch, cv, steps, warmup):
    """stand-alone coopVecReduceSumAccumulate of 64-vectors over a batch of 2^22, fp32 destination."""
    from slang_amd.coopvec import CoopVecComponentType as CT
    dev = "cuda"
    B, N = 1 << 22, 64
    g = torch.Generator(device=dev); g.manual_seed(20257)
    v = (torch.rand(B, N, device=dev, generator=g) * 2 - 1).half()
    buf = torch.zeros(N, dtype=torch.float32, device=dev)
    import ctypes
    from slang_amd import _lib
    need = ctypes.c_size_t(0)
    _lib.load().cvReduceSumAccumulateWorkspaceSize(N, B, ctypes.byref(need))
    ws = torch.empty(max(need.value, 16), dtype=torch.uint8, device=dev)

    def step():
        cv.coopVecReduceSumAccumulate(v, buf.view(torch.uint8), 0, bufferType=CT.Float32, workspace=ws)

    def cpu_baseline():
        import numpy as np
        import oracle_binding as ob
        n = 1 << 14
        vn = v[:n].cpu().numpy()
        dst = np.zeros(N, np.float16)
        L = ob.lib()
        t0 = time.perf_counter()
        for s_ in range(n):
            assert L.cvo_slang_reduce_sum_accumulate(ob.ptr(vn[s_]), N, ob.F16, ob.ptr(dst), 0, ob.HALF_SLANG) == 0
        t1 = time.perf_counter()
        return {"value": n / (t1 - t0), "unit": "samples/s", "cores": 1, "kind": "port",
                "sample": "first %d vectors, one core; C restatement of the Slang CPU-target fallback (per-thread "
                          "load-add-store in half), -O2, called per thread from Python" % n}

    return dict(step=step, samples=B, alg_bytes=B * N * 2, alg_flops=B * N, bound="hbm", mfma="f16", dtype="f16",
                config={"workload": "rs: coopVecReduceSumAccumulate of 64-vectors over 2^22 fp16 vectors, fp32 destination",
                        "batch": B, "n": N}, cpu_baseline=cpu_baseline, key="rs")


WORKLOADS = {"c1": workload_c1, "c2": workload_c2, "c2r": workload_c2r, "c2b": workload_c2b, "c3": workload_c3, "c3c": workload_c3c, "c4": workload_c4,
             "c4n": workload_c4n, "c5": workload_c5, "t32": workload_t32, "c5f": workload_c5f, "ex": workload_ex, "op": workload_op, "rs": workload_rs,
             "cm": workload_cm, "nf": workload_nf, "pe": workload_pe, "pef": workload_pef, "peu": workload_peu, "peb": workload_peb, "ped": workload_ped, "ew": workload_ew, "ad": workload_ad,
             # only with --workload: variants and the counter-calibration copy
             "c4h": workload_c4h, "c5g": workload_c5g, "c5r": workload_c5r, "t128": workload_t128, "c5l": workload_c5l, "c5f16": workload_c5f16, "f32": workload_f32, "f32t": workload_f32t, "copy": workload_copy}
DEFAULT_RUN = ("c1", "c2r", "c2b", "c3", "c3c", "c4", "c4h", "c4n", "c5f", "c5", "c5l", "c5r", "t32", "t128", "ex", "op", "rs", "pe", "peb", "ped", "pef", "peu", "ew", "ad", "cm", "nf", "f32", "f32t")
HEADLINE = "c2"


def measure(torch, w, steps, warmup, with_cpu, ramp_ms=0.0):
    """W untimed warm-up steps, then exactly K timed steps between synchronisations; kernel time from
    HIP events recorded on the launch stream (torch's current stream is the one handed to the library).

    Clock ramp: a fresh process finds the GPU in a low-power state, and its clocks take tens of
    milliseconds of continuous work to come up (measured: the e4m3 forward pass takes 323 us per step
    averaged over the first 50 launches and 272 us from then on, for as long as launches follow each
    other).  Five warm-up steps of 0.2 ms end long before that, so the same step is first run, untimed,
    for `ramp_ms` of wall time; the W warm-up steps and the K timed steps follow without a pause.  The
    figure reported is therefore the sustained rate."""
    from slang_amd import _lib
    step = w["step"]
    if ramp_ms > 0:
        t_end = time.perf_counter() + ramp_ms * 1e-3
        while time.perf_counter() < t_end:
            for _ in range(20):
                step()
            torch.cuda.synchronize()
    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    ev0.record()
    for _ in range(steps):
        step()
    ev1.record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    kernel = w.get("kernel") or _lib.load().cvGetLastKernelName().decode()
    wall_ms = (t1 - t0) * 1e3 / steps
    kern_ms = ev0.elapsed_time(ev1) / steps
    extra = dict(w.get("extra", {}))
    if w.get("graph"):
        # A launch-bound step (microseconds of kernel behind a host call of the same order): the K steps are
        # recorded once into a HIP graph and the timed region is one replay of it.  The figure from K separate
        # launches stays in `extra`.
        extra["ms_per_step_separate_launches"] = wall_ms
        extra["kernel_ms_separate_launches"] = kern_ms
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            for _ in range(steps):
                step()
        g.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        ev0.record()
        g.replay()
        ev1.record()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        wall_ms = (t1 - t0) * 1e3 / steps
        kern_ms = ev0.elapsed_time(ev1) / steps
        extra["launch"] = "one HIP graph of the %d steps" % steps
    hbm = w["alg_bytes"] / (kern_ms * 1e-3) / 1e9
    tflops = w["alg_flops"] / (kern_ms * 1e-3) / 1e12
    mfma_peak = MFMA_PEAK_TFLOPS[w["mfma"]]
    if w["bound"] == "hbm":
        achieved, peak, unit = hbm, HBM_PEAK_GBS, "GB/s"
    else:
        achieved, peak, unit = tflops, mfma_peak, "TFLOP/s"
    traffic = profiled_traffic().get(w["key"])
    roofline = {"bound": w["bound"], "achieved": achieved, "peak": peak, "unit": unit, "frac": achieved / peak,
                "traffic": traffic[0] if traffic else None,
                "traffic_source": (traffic[1] + " (rocprofv3 --pmc, not measured by this run)") if traffic else None,
                "kernel": kernel, "kernel_ms": kern_ms,
                "alg_bytes_per_launch": w["alg_bytes"], "alg_flops_per_launch": w["alg_flops"],
                "hbm_GBps": hbm, "hbm_frac": hbm / HBM_PEAK_GBS,
                "mfma_TFLOPs": tflops, "mfma_peak_TFLOPs": mfma_peak, "mfma_frac": tflops / mfma_peak}
    if w.get("launch_floor_us"):
        # launch-bound workloads: the time of a step against what its graph nodes cost when they are empty kernels
        roofline["launch_floor_us"] = w["launch_floor_us"]
        roofline["launch_floor_frac"] = w["launch_floor_us"] / (kern_ms * 1e3)
    if w.get("issue_bound"):
        roofline["issue_bound_ms"] = w["issue_bound"]["ms"]
        roofline["issue_bound_model"] = w["issue_bound"]["model"]
        roofline["issue_bound_frac"] = w["issue_bound"]["ms"] / kern_ms
    return {"value": w["samples"] / (wall_ms * 1e-3), "unit": "samples/s", "ms_per_step": wall_ms, "dtype": w["dtype"],
            "config": w["config"], "roofline": roofline,
            "cpu_baseline": w["cpu_baseline"]() if with_cpu else None, "extra": extra}


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default=None, choices=sorted(WORKLOADS),
                    help="run only this workload (default: the headline c2 plus all others under 'workloads')")
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU leg (profiling runs)")
    ap.add_argument("--clock-ramp-ms", type=float, default=100.0,
                    help="untimed run of the same step before the warm-up steps, until the GPU clocks are up (0: none)")
    args = ap.parse_args(argv)
    if args.gpus != 1:
        print("bench.py: this build runs on one GPU only (the path is data-parallel over samples: a batch "
              "shards with replicated weights and one all-reduce of the gradients); use --gpus 1", file=sys.stderr)
        return 2
    ensure_built()
    import torch
    from slang_amd import coopvec as cv
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    torch.cuda.set_device(0)
    head_key = args.workload or HEADLINE
    others = [] if args.workload else list(DEFAULT_RUN)

    def run(key):
        w = WORKLOADS[key](torch, cv, args.steps, args.warmup)
        r = measure(torch, w, args.steps, args.warmup, not args.no_cpu_baseline, args.clock_ramp_ms)
        del w
        torch.cuda.empty_cache()
        return r

    h = run(head_key)
    line = {
        "metric": METRIC, "value": h["value"], "unit": "samples/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "clock_ramp_ms": args.clock_ramp_ms, "ms_per_step": h["ms_per_step"], "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": h["dtype"], "data": "synthetic", "config": h["config"],
        "roofline": h["roofline"], "cpu_baseline": h["cpu_baseline"],
    }
    line.update(h["extra"])
    if others:
        line["workloads"] = {}
        for k in others:
            r = run(k)
            r.update(r.pop("extra"))
            line["workloads"][k] = r
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
