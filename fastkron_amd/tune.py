"""Tune launch plans for given problem shapes on this GPU and keep them in a tuned-plan file.

    python -m fastkron_amd.tune --db plans.txt --mmtype mkm --type float -m 1024 --same-factors 4 16,16
    python -m fastkron_amd.tune --db plans.txt --mmtype kmm --type double -m 64 256 --distinct-factors 8,8 16,16

For every shape the library times each of its kernels on each sub-chain of the factors, picks the fastest
series of launches and stores it in the file (`fastKronSetTunedDB`); later handles that are given the same
file (or the environment variable FASTKRON_TUNED_DB) use the stored plan without tuning.  Prints the plan and
the measured rate per shape.  Counterpart of the reference's src/print_best_kernel_for_shapes.py:13-21,72-83,
which drives its benchmark binary with --tune and greps the log; here the tuner is called through the C API.
"""
import argparse
import sys
import time


def _shapes(args):
    out = []
    for case in args.same_factors or []:
        n, pq = int(case[0]), case[1].split(",")
        out.append(([int(pq[0])] * n, [int(pq[1])] * n))
    for case in args.distinct_factors or []:
        pqs = [c.split(",") for c in case]
        out.append(([int(p) for p, _ in pqs], [int(q) for _, q in pqs]))
    return out


def tune_shape(handle, mmtype, M, Ps, Qs, dtype, runs=10):
    """Tunes one shape (first call) and times the stored plan; returns (plan, ms, gflops)."""
    import math
    import torch
    K, L = math.prod(Ps), math.prod(Qs)
    ye, te = handle.sizes(M, Ps, Qs)
    dev = "cuda"
    X = torch.rand(M * K, dtype=dtype, device=dev)
    Fs = [torch.rand(p * q, dtype=dtype, device=dev) for p, q in zip(Ps, Qs)]
    Z = torch.empty(ye, dtype=dtype, device=dev)
    t1, t2 = torch.empty(te, dtype=dtype, device=dev), torch.empty(te, dtype=dtype, device=dev)
    call = handle.xgemkm if mmtype == "mkm" else handle.xgekmm
    run = lambda: call(M, Ps, Qs, X, Fs, Z, 1.0, 0.0, None, t1, t2)
    e = run()                                         # tunes, stores and saves the plan
    if e != 0:
        raise RuntimeError(f"fastKronError {e} for M={M} Ps={Ps} Qs={Qs}")
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(runs):
        run()
    torch.cuda.synchronize()
    ms = (time.perf_counter() - t0) / runs * 1e3
    flop, k = 0, K
    for p, q in zip(reversed(Ps), reversed(Qs)):     # FastKron's count: 2 * M * sum Kin_i * Q_i
        k = k // p * q
        flop += k * p
    return handle.last_plan(), ms, 2.0 * M * flop / ms / 1e6


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--db", required=True, help="tuned-plan file to load and extend")
    ap.add_argument("--mmtype", choices=["mkm", "kmm"], required=True)
    ap.add_argument("--type", choices=["float", "double"], default="float")
    ap.add_argument("-m", type=int, nargs="+", required=True, help="rows of X (MKM) / columns of X (KMM)")
    ap.add_argument("--same-factors", nargs=2, action="append", metavar=("N", "P,Q"))
    ap.add_argument("--distinct-factors", nargs="+", action="append", metavar="P,Q")
    args = ap.parse_args(argv)
    shapes = _shapes(args)
    if not shapes:
        ap.error("give --same-factors N P,Q and/or --distinct-factors P,Q ...")
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
