#!/usr/bin/env python3
"""Benchmark of the Kronecker-matrix multiplication hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config c1|c2|c3|c4|c5|c1d] [--only] [--tune] [--no-cpu]

One "step" is one call of the C-ABI entry point (sgemkm / dgemkm / sgekmm / sgemkmStridedBatched) on a
synthetic problem whose operands are already resident in HBM.  The default workload is c2, the
configuration the headline metric is quoted on: sgemkm, X 1024 x 65536, four 16x16 factors.
Prints ONE JSON line: GFLOP/s with FastKron's FLOP count (2*M*sum_i Kin_i*Q_i), the roofline of the
dominant kernel measured with HIP events on the library's stream, a CPU baseline (the oracle's
vectorised OpenMP port) timed on the host cores in the same run, and under "configs" the same GPU figures
(ms, GFLOP/s, roofline fraction, launches, kernels) for the other four configurations, timed the same way, under
"cpu_baselines" the CPU figure of each of those, and under "published_shapes" the fp32 GeMKM shapes of the reference's
published table (plus c1 / c2 transposed and as sgekmm) timed through the same handle.
"""
import argparse
import ctypes
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0            # MI355X HBM3E
FP64_PEAK_TFLOPS = 78.6          # MI355X fp64 (vector = matrix)
FP32_PEAK_TFLOPS = 157.3         # MI355X fp32 (vector = matrix)

# name: (call, M, Ps, Qs, dtype, alpha, beta, batch, bound)
CONFIGS = {
    "c1": ("sgemkm", 1024, [8] * 5, [8] * 5, "f32", 1.0, 0.0, 1, "hbm"),
    "c2": ("sgemkm", 1024, [16] * 4, [16] * 4, "f32", 1.0, 0.0, 1, "hbm"),
    "c3": ("dgemkm", 256, [64] * 3, [64] * 3, "f64", 1.0, 0.0, 1, "mfma"),
    "c4": ("sgekmm", 2048, [4] * 6, [4] * 6, "f32", 1.5, 0.5, 1, "hbm"),
    "c5": ("sgemkmStridedBatched", 512, [32] * 3, [16] * 3, "f32", 1.0, 1.0, 8, "hbm"),
    # c1's shape in fp64 (reference documents/performance.md:49, the double GeMKM row of 1024 x 8^5): the fp64 whole-row kernel
    "c1d": ("dgemkm", 1024, [8] * 5, [8] * 5, "f64", 1.0, 0.0, 1, "hbm"),
}


def flop_count(M, Ps, Qs, batch):
    kk, ops = int(np.prod(Ps)), 0
    for p, q in zip(reversed(Ps), reversed(Qs)):
        kk = kk // p * q
        ops += kk * p
    return 2 * M * ops * batch


def compulsory_bytes(M, Ps, Qs, batch, esize, beta):
    """Read X once, write Z once, read Y once when beta != 0, read the factors."""
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    b = M * K + M * L + (M * L if beta != 0 else 0)
    return (b * batch + batch * sum(p * q for p, q in zip(Ps, Qs))) * esize


class HipEvents:
    """hipEvent timing on an explicit stream (the one handed to fastKronInitHIP)."""

    def __init__(self):
        self.hip = ctypes.CDLL("libamdhip64.so.7")
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [ctypes.c_void_p]

    def create(self):
        e = ctypes.c_void_p()
        assert self.hip.hipEventCreate(ctypes.byref(e)) == 0
        return e

    def record(self, e, stream):
        assert self.hip.hipEventRecord(e, stream) == 0

    def elapsed_ms(self, e0, e1):
        assert self.hip.hipEventSynchronize(e1) == 0
        ms = ctypes.c_float()
        assert self.hip.hipEventElapsedTime(ctypes.byref(ms), e0, e1) == 0
        return ms.value


def cpu_baseline(M, Ps, Qs, dt, alpha, beta, batch, budget_s):
    """The oracle's OpenMP port on a bounded sample of the same workload: at most 256 rows of one
    batch, repeated until about `budget_s` seconds of CPU work have been spent."""
    from oracle import kron_oracle as ko
    rows = min(M, 256)
    rng = np.random.default_rng(0)
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    X = rng.uniform(-1, 1, size=(rows, K)).astype(dt)
    Fs = [rng.uniform(-1, 1, size=(p, q)).astype(dt) for p, q in zip(Ps, Qs)]
    Y = rng.uniform(-1, 1, size=(rows, L)).astype(dt) if beta != 0 else None
    out = np.empty(rows * L, dtype=dt)
    ko.sliced_multiply_fast(rows, Ps, Qs, X, Fs, alpha, beta, Y, out=out)       # warm-up, page in
    best, spent, reps = float("inf"), 0.0, 0
    while spent < budget_s and reps < 100000:
        t0 = time.perf_counter()
        ko.sliced_multiply_fast(rows, Ps, Qs, X, Fs, alpha, beta, Y, out=out)
        dtm = time.perf_counter() - t0
        best = min(best, dtm)
        spent += dtm
        reps += 1
    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    gflops = flop_count(rows, Ps, Qs, 1) / best / 1e9
    return {"value": round(gflops, 2), "unit": "GFLOP/s", "cores": cores, "kind": "port",
            "sample": f"{rows} of {M * batch} rows, MKM form of the same factors, best of {reps} runs "
                      f"({spent:.1f} s of CPU work)"}


def measure(fk, name, steps, warmup, ramp_seconds, nsets, ev, stream, calibrate_copy=False):
    """Times `steps` calls of configuration `name` (operands resident in HBM, `nsets` operand sets rotated) and
    returns its figures: wall-clock and hipEvent time per step, GFLOP/s, and the roofline of its launches."""
    import torch
    from fastkron_amd import capi

    call, M, Ps, Qs, dts, alpha, beta, batch, bound = CONFIGS[name]
    tdt = torch.float32 if dts == "f32" else torch.float64
    esize = 4 if dts == "f32" else 8
    K, L = int(np.prod(Ps)), int(np.prod(Qs))
    dev = torch.device("cuda:0")
    ye, te = fk.sizes(M, Ps, Qs)

    gen = torch.Generator(device=dev)
    gen.manual_seed(0xFA57C0DE)

    def uniform(n):
        return torch.rand(n, generator=gen, device=dev, dtype=tdt) * 2 - 1

    # enough operand sets that one pass over all of them moves well over twice the 256 MB of the memory-side cache:
    # a smaller rotation (three sets of c4's 96 MB) is partly served from that cache and flatters the figure
    set_bytes = batch * (M * K + ye + (M * L if beta != 0 else 0)) * esize
    nsets = max(nsets, -(-640 * 1024 * 1024 // set_bytes))
    sets = []
    for _ in range(nsets):
        X = uniform(batch * M * K)
        Fs = [uniform(batch * p * q) for p, q in zip(Ps, Qs)]
        Y = uniform(batch * M * L) if beta != 0 else None
        Z = torch.empty(batch * ye, device=dev, dtype=tdt)
        sets.append((X, Fs, Y, Z))
    t1 = torch.empty(batch * te, device=dev, dtype=tdt)
    t2 = torch.empty(batch * te, device=dev, dtype=tdt)

    # the ctypes arguments of every operand set are marshalled once; a step is then one C call
    calls = []
    for X, Fs, Y, Z in sets:
        if call == "sgemkmStridedBatched":
            calls.append(fk.prepared("xgemkm_strided_batched", M, Ps, Qs, X, M * K, Fs, [p * q for p, q in zip(Ps, Qs)],
                                     Z, M * L, batch, alpha, beta, Y, M * L, t1, t2))
        elif call == "sgekmm":
            calls.append(fk.prepared("xgekmm", M, Ps, Qs, X, Fs, Z, alpha, beta, Y, t1, t2))
        else:
            calls.append(fk.prepared("xgemkm", M, Ps, Qs, X, Fs, Z, alpha, beta, Y, t1, t2))

    def step(i):
        e = calls[i % len(calls)]()
        if e != capi.SUCCESS:
            raise RuntimeError(f"{call} failed with fastKronError {e}")

    if calibrate_copy:
        src = torch.empty(64 * 1024 * 1024, device=dev, dtype=torch.float32).normal_()
        dst = torch.empty_like(src)
        for _ in range(4):
            dst.copy_(src)                    # reads 256 MiB, writes 256 MiB
        torch.cuda.synchronize()

    t_ramp = time.perf_counter()
    while time.perf_counter() - t_ramp < ramp_seconds:
        for i in range(20):
            step(i)
        torch.cuda.synchronize()
    for i in range(max(warmup, 1)):
        step(i)
    torch.cuda.synchronize()

    e0, e1 = ev.create(), ev.create()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ev.record(e0, stream)
    for i in range(steps):
        step(i)
    ev.record(e1, stream)
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    gpu_ms = ev.elapsed_ms(e0, e1)

    flop = flop_count(M, Ps, Qs, batch)
    # Roofline of the dominant kernel.  The unit of work is "one factor applied to one row"; the
    # algorithmic bytes of a unit are the call's compulsory bytes / (rows * factors), so the launches
    # of one call add up to exactly the compulsory bytes.  Average launch duration = event time / launches,
    # bytes (or FLOPs) per launch = the call's / launches.
    plan = fk.last_plan()
    launches = len(plan)
    kernel_ms = gpu_ms / steps / launches
    cbytes = compulsory_bytes(M, Ps, Qs, batch, esize, beta)
    if bound == "hbm":
        achieved = cbytes / launches / (kernel_ms * 1e-3) / 1e9
        roof = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4)}
    else:
        achieved = flop / launches / (kernel_ms * 1e-3) / 1e12
        roof = {"bound": "mfma", "achieved": round(achieved, 2), "peak": FP64_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": round(achieved / FP64_PEAK_TFLOPS, 4)}
    # HBM bytes per launch as rocprofv3 --pmc measured them in separate runs of this command (FETCH_SIZE, then
    # WRITE_SIZE, scaled by a device copy of known size): read from the committed summary, not measured in this run
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    traffic = None
    if os.path.exists(tpath):
        traffic = json.load(open(tpath)).get(name, {}).get("traffic_bytes_per_launch")
    roof["traffic"] = traffic
    roof["traffic_source"] = "profiles/traffic.json (rocprofv3 --pmc runs of this command, not this run)" if traffic else None
    # the other roof of the same run, for reference: the fraction of the matrix peak of the element type
    # and the fraction of the HBM peak that the compulsory bytes of the whole call correspond to
    step_s = gpu_ms / steps * 1e-3
    roof["matrix_frac"] = round(flop / step_s / 1e12 / (FP32_PEAK_TFLOPS if dts == "f32" else FP64_PEAK_TFLOPS), 4)
    roof["compulsory_hbm_frac"] = round(cbytes / step_s / 1e9 / HBM_PEAK_GBS, 4)
    roof["kernel"] = sorted(set(k for _, _, k in plan))
    roof["launches_per_step"] = launches
    roof["kernel_ms"] = round(kernel_ms, 5)
    workload = (f"{name}: {call} M={M} factors={len(Ps)}x({Ps[0]}x{Qs[0]}) K={K} L={L} alpha={alpha} beta={beta} "
                f"batch={batch}, uniform[-1,1], seed 0xFA57C0DE")
    del sets, calls, t1, t2
    torch.cuda.empty_cache()
    return {"workload": workload, "dtype": dts, "sets": nsets, "ms_per_step": wall * 1e3 / steps, "gpu_ms_per_step": gpu_ms / steps,
            "gflops": flop / (wall / steps) / 1e9, "roofline": roof, "dims": (M, Ps, Qs, alpha, beta, batch)}


# reference documents/performance.md:5-137, the shapes of its A100 tables, "M_PxP^N"
PUBLISHED_GPU_SHAPES = [(1024, 8, 5), (1024, 8, 6), (1024, 16, 4), (1024, 16, 5), (1024, 32, 3), (1024, 32, 4), (1024, 64, 2),
                        (1024, 64, 3), (1024, 128, 2), (320, 128, 3), (16, 8, 8), (16, 16, 6), (16, 32, 5), (16, 64, 4),
                        (16, 128, 3)]


def shape_table(fk):
    """Times every shape of the reference's published GPU table through the handle as a user gets it (online rules
    plus the tuned plans that ship), operands rotated so that no cache holds them; wall clock around batches of
    calls with a device synchronisation on both sides."""
    import torch
    from fastkron_amd.capi import OP_N, OP_T
    from fastkron_amd.tune import _Case
    for mm in ("mkm", "kmm"):
        for dtype, dn in ((torch.float32, "float"), (torch.float64, "double")):
            for ops, on in (((OP_N, OP_N), "NN"), ((OP_T, OP_T), "TT")):
                for M, P, N in PUBLISHED_GPU_SHAPES:
                    try:
                        case = _Case(fk, mm, M, [P] * N, [P] * N, dtype)
                    except torch.cuda.OutOfMemoryError:
                        continue
                    ms = case.time(fk, *ops, runs=20, samples=4)
                    print(json.dumps({"mmtype": mm, "type": dn, "ops": on, "shape": f"{M}_{P}x{P}^{N}", "ms": round(ms, 5),
                                      "gflops": round(case.gflops(ms), 1),
                                      "launches": [k for _, _, k in fk.last_plan()]}), flush=True)
                    del case
                    torch.cuda.empty_cache()


def pattern_ceilings(fk, steps, warmup, ev, stream):
    """c4's bytes (X, Y read, Z written, 4096 x 2048 fp32 each) moved by copy kernels that have the access pattern of a
    4x4^6 GeKMM kernel and none of its arithmetic (include/fastkron_ext.h, fastKronProbeCopyPattern), timed like the
    configurations: 7 operand sets rotated (672 MB per rotation), hipEvents on the library's stream."""
    import torch
    from fastkron_amd import capi
    M, n = 2048, 4096 * 2048
    dev = torch.device("cuda:0")
    gen = torch.Generator(device=dev)
    gen.manual_seed(0xFA57C0DE)
    sets = [tuple(torch.rand(n, generator=gen, device=dev) * 2 - 1 for _ in range(2)) + (torch.empty(n, device=dev),)
            for _ in range(7)]
    T = torch.empty(n, device=dev)
    names = {0: "contiguous 16-byte accesses", 1: "32-byte strips of 8 columns x 4096 rows per workgroup",
             2: "256-byte pieces, two phases, intermediate through the L2"}
    out = {}
    for pattern, label in names.items():
        def step(i):
            X, Y, Z = sets[i % len(sets)]
            e = fk.lib.fastKronProbeCopyPattern(fk.h, pattern, X.data_ptr(), Y.data_ptr(), Z.data_ptr(), T.data_ptr(), M)
            if e != capi.SUCCESS:
                raise RuntimeError(f"fastKronProbeCopyPattern failed with fastKronError {e}")
        t_ramp = time.perf_counter()
        while time.perf_counter() - t_ramp < 0.25:
            for i in range(20):
                step(i)
            torch.cuda.synchronize()
        for i in range(max(warmup, 1)):
            step(i)
        torch.cuda.synchronize()
        e0, e1 = ev.create(), ev.create()
        ev.record(e0, stream)
        for i in range(steps):
            step(i)
        ev.record(e1, stream)
        torch.cuda.synchronize()
        ms = ev.elapsed_ms(e0, e1) / steps
        X, Y, Z = sets[(steps - 1) % len(sets)]
        # (the strips are read in the order of the kernel's first phase and written in that of its second: a permuted copy)
        ok = bool(torch.allclose(Z, 1.5 * X + 0.5 * Y, rtol=0, atol=1e-5)) if pattern != 1 else None
        gbs = 3 * n * 4 / (ms * 1e-3) / 1e9
        out[str(pattern)] = {"pattern": label, "ms": round(ms, 5), "gbs": round(gbs, 1), "frac_of_hbm_peak": round(gbs / HBM_PEAK_GBS, 4),
                             "copy_is_exact": ok}
    out["sync_error"] = fk.sync_error()
    return out


def published_shapes(fk, budget_s):
    """The 15 fp32 GeMKM shapes of the reference's published table (documents/performance.md:9-23), plus c1 and c2's
    shapes with both operands transposed, as sgekmm (the rows nearest to them there: :29-31, :89-91) and in fp64, through the
    same handle, operands rotated so that the memory-side cache holds none, wall clock around batches of calls with
    a device synchronisation on both sides.  Stops adding shapes once `budget_s` seconds are spent."""
    import torch
    from fastkron_amd.capi import OP_N, OP_T
    from fastkron_amd.tune import _Case
    # (the four extra fp32 rows and the two fp64 rows come first: they are the ones this leg is for, and the largest of
    # the 15 table shapes use most of the budget)
    f32, f64 = torch.float32, torch.float64
    todo = [("mkm", 1024, 8, 5, OP_T, "TT", f32), ("mkm", 1024, 16, 4, OP_T, "TT", f32),
            ("kmm", 1024, 8, 5, OP_N, "NN", f32), ("kmm", 1024, 16, 4, OP_N, "NN", f32),
            ("mkm", 1024, 8, 5, OP_N, "NN", f64), ("mkm", 1024, 16, 4, OP_N, "NN", f64)]     # reference :49-51 (double)
    todo += [("mkm", M, P, N, OP_N, "NN", f32) for M, P, N in PUBLISHED_GPU_SHAPES]
    out, t_start = {}, time.perf_counter()
    for mm, M, P, N, op, on, dt in todo:
        if time.perf_counter() - t_start > budget_s:
            break
        try:
            case = _Case(fk, mm, M, [P] * N, [P] * N, dt)
        except torch.cuda.OutOfMemoryError:
            continue
        ms = case.time(fk, op, op, runs=10, samples=3)
        out[f"{'s' if dt == f32 else 'd'}{'gemkm' if mm == 'mkm' else 'gekmm'}_{M}_{P}x{P}^{N}_{on}"] = {
            "ms": round(ms, 5), "gflops": round(case.gflops(ms), 1), "launches": len(fk.last_plan())}
        del case
        torch.cuda.empty_cache()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--ramp-seconds", type=float, default=0.25,
                    help="untimed steps run for this long before the warm-up steps (the GPU raises its clocks over "
                         "the first tens of milliseconds of load; steady-state throughput is what is reported)")
    ap.add_argument("--config", default="c2", choices=sorted(CONFIGS), help="the workload of the headline figures")
    ap.add_argument("--only", action="store_true", help="time the --config workload alone (profiling runs)")
    ap.add_argument("--tune", action="store_true", help="time candidate launch plans first (excluded from timing)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=10.0,
                    help="CPU work spent on the headline workload's baseline (the other four get 3 s each)")
    ap.add_argument("--published-seconds", type=float, default=45.0,
                    help="time budget of the published-shapes leg (0 skips it)")
    ap.add_argument("--sets", type=int, default=3,
                    help="least number of operand sets rotated between steps; raised per workload until the sets add up "
                         "to 640 MB, so that the 256 MB Infinity Cache serves none of the traffic")
    ap.add_argument("--shape-table", action="store_true",
                    help="instead of the benchmark line: time the shapes of the reference's published GPU table "
                         "(reference documents/performance.md:5-137: M_PxP^N for MKM and KMM, float and double, operands "
                         "untransposed and transposed) with cold operands and print one JSON line per shape")
    ap.add_argument("--pattern-ceilings", action="store_true",
                    help="instead of the benchmark line: time copy kernels with the access patterns of the 4x4^6 GeKMM "
                         "kernels on c4's operands (what the memory system gives each pattern) and print one JSON line")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run 4 plain device copies of 256 MiB (a known-size kernel for scaling rocprof counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs on ONE GPU only (no multi-GPU path exists); use --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    import fastkron_amd

    torch.cuda.set_device(torch.device("cuda:0"))
    stream = torch.cuda.current_stream()
    fk = fastkron_amd.FastKron(stream=stream, tune=args.tune)
    ev = HipEvents()
    sp = ctypes.c_void_p(stream.cuda_stream)

    if args.shape_table:
        shape_table(fk)
        return
    if args.pattern_ceilings:
        out = pattern_ceilings(fk, args.steps, args.warmup, ev, sp)
        out["c4"] = {k: v for k, v in measure(fk, "c4", args.steps, args.warmup, args.ramp_seconds, args.sets, ev, sp).items()
                     if k in ("gpu_ms_per_step", "roofline")}
        print(json.dumps(out))
        return
    head = measure(fk, args.config, args.steps, args.warmup, args.ramp_seconds, args.sets, ev, sp, args.calibrate_copy)
    out = {
        "metric": "GeMKM/GeKMM GFLOP/s on 1 MI355X (FastKron FLOP count 2*M*sum Kin_i*Q_i)",
        "value": round(head["gflops"], 1), "unit": "GFLOP/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(head["ms_per_step"], 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": head["dtype"], "data": "synthetic",
        "config": {"workload": head["workload"], "operand_sets_rotated": head["sets"], "tuned": bool(args.tune)},
        "roofline": head["roofline"],
        "gpu_ms_per_step_events": round(head["gpu_ms_per_step"], 5),
    }
    # the other configurations, timed the same way in the same process (the CPU leg stays with the headline workload)
    if not args.only:
        others = {}
        for name in sorted(CONFIGS):
            if name == args.config:
                continue
            r = measure(fk, name, args.steps, args.warmup, args.ramp_seconds, args.sets, ev, sp)
            rf = r["roofline"]
            others[name] = {"workload": r["workload"], "dtype": r["dtype"], "operand_sets_rotated": r["sets"], "ms": round(r["gpu_ms_per_step"], 5),
                            "ms_wall": round(r["ms_per_step"], 5), "gflops": round(r["gflops"], 1),
                            "roofline": {k: rf[k] for k in ("bound", "achieved", "peak", "unit", "frac")},
                            "launches": rf["launches_per_step"], "kernel": rf["kernel"]}
        out["configs"] = others
        if args.published_seconds > 0:
            out["published_shapes"] = published_shapes(fk, args.published_seconds)
    if not args.no_cpu:
        M, Ps, Qs, alpha, beta, batch = head["dims"]
        dt = np.float32 if head["dtype"] == "f32" else np.float64
        out["cpu_baseline"] = cpu_baseline(M, Ps, Qs, dt, alpha, beta, batch, args.cpu_seconds)
        # the same port on the other configurations (c1 is the one the reference's own x86 case is stated on), so
        # that every GPU figure of this line has its CPU figure from the same host beside it
        if not args.only:
            out["cpu_baselines"] = {}
            for name in sorted(CONFIGS):
                if name == args.config:
                    continue
                _, M, Ps, Qs, dts, alpha, beta, batch, _ = CONFIGS[name]
                out["cpu_baselines"][name] = cpu_baseline(M, Ps, Qs, np.float32 if dts == "f32" else np.float64, alpha, beta,
                                                          batch, 6.0 if name == "c1" else 3.0)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
