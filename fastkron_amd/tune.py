"""Tune launch plans for given problem shapes on this GPU and keep them in a tuned-plan file.

    python -m fastkron_amd.tune --db plans.txt --mmtype mkm --type float -m 1024 --same-factors 4 16,16
    python -m fastkron_amd.tune --db plans.txt --mmtype kmm --type double -m 64 256 --distinct-factors 8,8 16,16
    python -m fastkron_amd.tune --db fastkron_amd/gfx950_plans.txt --table --keep-if-faster 0.03

For every shape the library times each of its kernels on each sub-chain of the factors, for the chain as given, with
small factors merged, and as every two-part plan; it keeps the fastest alternative in the file
(`fastKronSetTunedDB`); later handles that are given the same file (or the environment variable FASTKRON_TUNED_DB)
use the stored plan without tuning.  Prints the plan and the measured rate per shape.  Counterpart of the
reference's src/print_best_kernel_for_shapes.py:13-21,72-83, which drives its benchmark binary with --tune and greps
the log; here the tuner is called through the C API.

`--table` tunes the shapes of the reference's published performance table (reference documents/performance.md:9-480:
M_PxP^N for both layouts, both types, untransposed and transposed operands), chains with odd, rectangular and differing
factors of the kinds its tests run, and the five benchmark configurations;
with `--keep-if-faster F` a record is only kept when the tuned plan beats the online selection by that fraction,
which is how fastkron_amd/gfx950_plans.txt, the file the library loads by default, was made.
"""
import argparse
import math
import os
import sys
import tempfile
import time

from .capi import OP_N, OP_T

# reference documents/performance.md: the shapes of its tables, "M_PxP^N"
TABLE = [(1024, 8, 5), (1024, 8, 6), (1024, 16, 4), (1024, 16, 5), (1024, 32, 3), (1024, 32, 4), (1024, 64, 2),
         (1024, 64, 3), (1024, 128, 2), (320, 128, 3), (16, 8, 8), (16, 16, 6), (16, 32, 5), (16, 64, 4), (16, 128, 3),
         (256, 8, 5), (256, 8, 6), (256, 16, 4), (256, 16, 5), (256, 32, 3), (256, 32, 4), (256, 64, 2), (256, 64, 3),
         (256, 128, 2), (128, 128, 3)]

# chains of the kinds the reference's tests run (reference tests/src/general-tests-NN.cpp:53-100: odd sizes, rectangular
# factors; :102-160: factors that differ), here with 1024 rows (MKM) or columns (KMM) of X
IRREGULAR = [([3] * 7, [3] * 7), ([5] * 6, [5] * 6), ([6] * 6, [6] * 6), ([12] * 4, [12] * 4), ([24] * 3, [24] * 3),
             ([31] * 3, [31] * 3), ([50] * 3, [50] * 3), ([62] * 2, [62] * 2), ([127] * 2, [127] * 2), ([129] * 2, [129] * 2),
             ([2] * 7, [4] * 7), ([31] * 3, [63] * 3), ([63] * 3, [31] * 3), ([16] * 5, [8] * 5), ([8] * 4, [32] * 4),
             ([12] * 5, [16] * 5), ([32] * 3, [64] * 3), ([2, 3, 4, 5, 6, 7, 8], [2, 3, 4, 5, 6, 7, 8]),
             ([8, 16, 32], [8, 16, 32]), ([64, 32, 16, 8], [64, 32, 16, 8])]


def _shapes(args):
    out = []
    for case in args.same_factors or []:
        n, pq = int(case[0]), case[1].split(",")
        out.append(([int(pq[0])] * n, [int(pq[1])] * n))
    for case in args.distinct_factors or []:
        pqs = [c.split(",") for c in case]
        out.append(([int(p) for p, _ in pqs], [int(q) for _, q in pqs]))
    return out


class _Case:
    """Operands of one shape in HBM (several sets, so that timed calls do not run from the memory-side cache)."""

    def __init__(self, handle, mmtype, M, Ps, Qs, dtype, alpha=1.0, beta=0.0, batch=1):
        import torch
        self.mmtype, self.M, self.Ps, self.Qs, self.alpha, self.beta, self.batch = mmtype, M, Ps, Qs, alpha, beta, batch
        K, L = math.prod(Ps), math.prod(Qs)
        self.K, self.L = K, L
        ye, te = handle.sizes(M, Ps, Qs)
        esize = 4 if dtype == torch.float32 else 8
        set_bytes = batch * (M * K + ye) * esize
        free = torch.cuda.mem_get_info()[0]
        nsets = max(1, min(4, (640 << 20) // set_bytes + 1, int(free * 0.35) // max(set_bytes, 1)))
        dev = "cuda"
        self.sets = []
        for _ in range(nsets):
            X = torch.rand(batch * M * K, dtype=dtype, device=dev) * 2 - 1
            Z = torch.empty(batch * ye, dtype=dtype, device=dev)
            Y = (torch.rand(batch * M * L, dtype=dtype, device=dev) * 2 - 1) if beta != 0 else None
            self.sets.append((X, Y, Z))
        self.Fs = [torch.rand(batch * p * q, dtype=dtype, device=dev) * 2 - 1 for p, q in zip(Ps, Qs)]
        self.t1 = torch.empty(batch * te, dtype=dtype, device=dev)
        self.t2 = torch.empty(batch * te, dtype=dtype, device=dev)

    def call(self, handle, i, opX=OP_N, opF=OP_N):
        X, Y, Z = self.sets[i % len(self.sets)]
        M, Ps, Qs = self.M, self.Ps, self.Qs
        if self.batch > 1:
            fn = handle.xgemkm_strided_batched if self.mmtype == "mkm" else handle.xgekmm_strided_batched
            return fn(M, Ps, Qs, X, M * self.K, self.Fs, [p * q for p, q in zip(Ps, Qs)], Z, M * self.L, self.batch,
                      self.alpha, self.beta, Y, M * self.L, self.t1, self.t2, opX, opF)
        fn = handle.xgemkm if self.mmtype == "mkm" else handle.xgekmm
        return fn(M, Ps, Qs, X, self.Fs, Z, self.alpha, self.beta, Y, self.t1, self.t2, opX, opF)

    def time(self, handle, opX=OP_N, opF=OP_N, runs=12, samples=3):
        import torch
        for i in range(3):
            e = self.call(handle, i, opX, opF)
            if e != 0:
                raise RuntimeError(f"fastKronError {e} for M={self.M} Ps={self.Ps} Qs={self.Qs}")
        torch.cuda.synchronize()
        best = float("inf")
        for _ in range(samples):
            t0 = time.perf_counter()
            for i in range(runs):
                self.call(handle, i, opX, opF)
            torch.cuda.synchronize()
            best = min(best, (time.perf_counter() - t0) / runs * 1e3)
        return best

    def gflops(self, ms):
        flop, k = 0, self.K
        for p, q in zip(reversed(self.Ps), reversed(self.Qs)):     # FastKron's count: 2 * M * sum Kin_i * Q_i
            k = k // p * q
            flop += k * p
        return 2.0 * self.M * self.batch * flop / ms / 1e6


def tune_shape(handle, mmtype, M, Ps, Qs, dtype, runs=10, opX=OP_N, opF=OP_N, alpha=1.0, beta=0.0, batch=1):
    """Tunes one shape (first call) and times the stored plan; returns (plan, ms, gflops)."""
    case = _Case(handle, mmtype, M, Ps, Qs, dtype, alpha, beta, batch)
    ms = case.time(handle, opX, opF, runs=runs)          # the first call tunes, stores and saves the plan
    return handle.last_plan(), ms, case.gflops(ms)


def _record_lines(path):
    if not os.path.exists(path):
        return []
    return [l for l in open(path).read().splitlines() if l and not l.startswith("#")]


def tune_table(db, keep_if_faster, only=None, verbose=True):
    """Tunes the reference's shape table and the benchmark configurations; appends the records worth keeping to `db`."""
    import torch
    import fastkron_amd
    os.environ["FASTKRON_SHIPPED_PLANS"] = "0"          # the comparison is against the online rules alone
    problems = []
    for mm in ("mkm", "kmm"):
        for dtype in (torch.float32, torch.float64):
            for ops in ((OP_N, OP_N), (OP_T, OP_T)):
                for M, P, N in TABLE:
                    problems.append((mm, dtype, ops, M, [P] * N, [P] * N, 1.0, 0.0, 1))
    for mm in ("mkm", "kmm"):
        for dtype in (torch.float32, torch.float64):
            for Ps, Qs in IRREGULAR:
                problems.append((mm, dtype, (OP_N, OP_N), 1024, Ps, Qs, 1.0, 0.0, 1))
    problems += [("mkm", torch.float32, (OP_N, OP_N), 1024, [8] * 5, [8] * 5, 1.0, 0.0, 1),
                 ("kmm", torch.float32, (OP_N, OP_N), 2048, [4] * 6, [4] * 6, 1.5, 0.5, 1),
                 ("mkm", torch.float32, (OP_N, OP_N), 512, [32] * 3, [16] * 3, 1.0, 1.0, 8)]
    kept = _record_lines(db)
    have = {l.split()[0] for l in kept}
    online = fastkron_amd.FastKron(tune=False)
    for idx, (mm, dtype, ops, M, Ps, Qs, alpha, beta, batch) in enumerate(problems):
        if only is not None and idx % only[1] != only[0]:
            continue
        tag = f"{mm} {'f' if dtype == torch.float32 else 'd'} {'NN' if ops[0] == OP_N else 'TT'} {M}_" + \
              (f"{Ps[0]}x{Qs[0]}^{len(Ps)}" if len(set(zip(Ps, Qs))) == 1 else ",".join(f"{p}x{q}" for p, q in zip(Ps, Qs)))
        try:
            case = _Case(online, mm, M, Ps, Qs, dtype, alpha, beta, batch)
        except torch.cuda.OutOfMemoryError:
            print(f"{tag}: skipped (operands do not fit)", flush=True)
            continue
        with tempfile.TemporaryDirectory() as tmp:
            one = os.path.join(tmp, "one.txt")
            tuner = fastkron_amd.FastKron(tune=True)
            tuner.set_tuned_db(one)
            try:
                t_tuned = case.time(tuner, *ops)
                t_online = case.time(online, *ops)
                t_tuned = min(t_tuned, case.time(tuner, *ops))
                plan_t, plan_o = tuner.last_plan(), online.last_plan()
            finally:
                tuner.close()
            lines = _record_lines(one)
        gain = t_online / t_tuned - 1.0
        keep = gain >= keep_if_faster and plan_t != plan_o and len(lines) == 1 and lines[0].split()[0] not in have
        if verbose:
            print(f"{tag}: online {t_online:.4f} ms ({case.gflops(t_online):.0f} GFLOP/s), tuned {t_tuned:.4f} ms "
                  f"({case.gflops(t_tuned):.0f} GFLOP/s), {gain * 100:+.1f}% {'KEPT' if keep else ''}\n"
                  f"    online {[(lo, hi, k) for lo, hi, k in plan_o]}\n    tuned  {[(lo, hi, k) for lo, hi, k in plan_t]}",
                  flush=True)
        if keep:
            kept.append(lines[0])
            have.add(lines[0].split()[0])
            with open(db, "w") as f:
                f.write("# fastkron gfx950 launch plans tuned on one MI355X (python -m fastkron_amd.tune --table): only shapes whose\n"
                        "# tuned plan beat the online selection; format: problem ms M<merge> S<split> nsteps {lo hi kernel}\n")
                f.write("\n".join(kept) + "\n")
        del case
        torch.cuda.empty_cache()
    online.close()
    return 0


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--db", required=True, help="tuned-plan file to load and extend")
    ap.add_argument("--mmtype", choices=["mkm", "kmm"])
    ap.add_argument("--type", choices=["float", "double"], default="float")
    ap.add_argument("-m", type=int, nargs="+", help="rows of X (MKM) / columns of X (KMM)")
    ap.add_argument("--same-factors", nargs=2, action="append", metavar=("N", "P,Q"))
    ap.add_argument("--distinct-factors", nargs="+", action="append", metavar="P,Q")
    ap.add_argument("--table", action="store_true", help="tune the reference's published shape table")
    ap.add_argument("--keep-if-faster", type=float, default=0.0,
                    help="with --table: keep a record only when the tuned plan is this fraction faster than the online one")
    ap.add_argument("--part", type=int, nargs=2, metavar=("I", "N"), help="with --table: only every N-th problem, starting at I")
    args = ap.parse_args(argv)
    if args.table:
        return tune_table(args.db, args.keep_if_faster, tuple(args.part) if args.part else None)
    shapes = _shapes(args)
    if not shapes or not args.mmtype or not args.m:
        ap.error("give --table, or --mmtype, -m and --same-factors N P,Q and/or --distinct-factors P,Q ...")
    import torch
    import fastkron_amd
    h = fastkron_amd.FastKron(tune=True)
    h.set_tuned_db(args.db)
    dtype = torch.float32 if args.type == "float" else torch.float64
    try:
        for Ps, Qs in shapes:
            for M in args.m:
                plan, ms, gflops = tune_shape(h, args.mmtype, M, Ps, Qs, dtype)
                names = ", ".join(f"[{lo},{hi}] {k}" for lo, hi, k in plan)
                print(f"{args.mmtype} M={M} P={Ps} Q={Qs} {args.type}: {ms:.4f} ms {gflops:.0f} GFLOP/s  {names}", flush=True)
    finally:
        h.close()
    return 0


if __name__ == "__main__":
    sys.exit(main())
