"""The tuner (fastKronOptionsTune): what it searches, what it stores, and that a stored plan is what a later handle
runs.  Counterpart of the reference's fast tuning (reference src/autotuner/autotuner.cpp:24-150,158-328), which times
every kernel on every sub-chain and keeps the result in memory; here the search also covers merged / unmerged chains
and two-part plans, and the result is kept in a file."""
import re
import time

import numpy as np
import pytest

from oracle import kron_oracle as ko
from tests.gpu_util import TOL, make_case, normwise, oracle_answer, run_gpu

pytestmark = pytest.mark.gpu


def run_and_check(h, mm, M, Ps, dt, alpha, beta, seed, **run_kw):
    X, Fs, Y = make_case(mm, M, Ps, Ps, dt, seed=seed, with_y=(beta != 0))
    want = oracle_answer(mm, M, Ps, Ps, X, Fs, Y, alpha, beta)
    got, e = run_gpu(h, mm, M, Ps, Ps, X, Fs, Y, alpha, beta, **run_kw)
    assert e == 0
    assert normwise(got, want) <= TOL[dt]


def record_of(text, key):
    for line in text.splitlines():
        if line.startswith(key + " "):
            return line
    return None


@pytest.mark.parametrize("M,Ps,dt", [(8, [16] * 5, np.float32), (4, [4] * 8, np.float32), (2, [64] * 3, np.float64),
                                     (16, [2, 3, 4, 5, 6, 7, 8], np.float32), (4, [8] * 5, np.float64)])
def test_tuned_record_names_merging_and_split_and_is_reused(tmp_path, M, Ps, dt):
    import fastkron_amd
    db = str(tmp_path / "plans.txt")
    h = fastkron_amd.FastKron(tune=True)
    h.set_tuned_db(db)
    try:
        run_and_check(h, ko.MKM, M, Ps, dt, 1.5, 0.5, seed=301)
        tuned_plan = h.last_plan()
    finally:
        h.close()
    K = int(np.prod(Ps))
    facs = f"{Ps[0]}x{Ps[0]}^{len(Ps)}" if len(set(Ps)) == 1 else "(x)".join(f"{p}x{p}" for p in Ps)
    key = f"{M}x{K}*({facs})_NN_{'f' if dt == np.float32 else 'd'}"
    rec = record_of(open(db).read(), key)
    assert rec is not None, open(db).read()
    assert re.match(re.escape(key) + r" [0-9.e+-]+ M[01] S\d+ \d+ ", rec), rec
    # a handle that does not tune runs the stored plan, on other data
    h2 = fastkron_amd.FastKron(tune=False)
    h2.set_tuned_db(db)
    try:
        run_and_check(h2, ko.MKM, M, Ps, dt, 1.0, 0.0, seed=302)
        assert h2.last_plan() == tuned_plan
        # ... and falls back to the online selection when the call's buffers do not allow the stored plan
        run_and_check(h2, ko.MKM, M, Ps, dt, 1.0, 0.0, seed=303, use_temp2=False)
    finally:
        h2.close()


def _time_calls(h, M, Ps, X, Fs, Z, t1, t2, reps=30):
    import torch
    for _ in range(5):
        assert h.xgemkm(M, Ps, Ps, X, Fs, Z, 1.0, 0.0, None, t1, t2) == 0
    torch.cuda.synchronize()
    best = float("inf")
    for _ in range(5):
        t0 = time.perf_counter()
        for _ in range(reps):
            h.xgemkm(M, Ps, Ps, X, Fs, Z, 1.0, 0.0, None, t1, t2)
        torch.cuda.synchronize()
        best = min(best, (time.perf_counter() - t0) / reps)
    return best


def test_tuned_plan_of_a_mixed_chain_is_not_slower_than_the_online_one(tmp_path):
    """2x2 (x) 3x3 (x) ... (x) 8x8: the online rules group the factors greedily from the last one; the tuner times the
    groupings and stores its choice; the plan that runs afterwards is that record."""
    import torch
    import fastkron_amd
    M, Ps = 1024, [2, 3, 4, 5, 6, 7, 8]
    K = int(np.prod(Ps))
    dev = "cuda:0"
    X = torch.rand(M * K, device=dev) * 2 - 1
    Fs = [torch.rand(p * p, device=dev) * 2 - 1 for p in Ps]
    Z = torch.empty(M * K, device=dev)
    t1, t2 = torch.empty(M * K, device=dev), torch.empty(M * K, device=dev)
    online = fastkron_amd.FastKron(tune=False)
    tuned = fastkron_amd.FastKron(tune=True)
    tuned.set_tuned_db(str(tmp_path / "plans.txt"))
    try:
        t_online = _time_calls(online, M, Ps, X, Fs, Z, t1, t2)
        z_online = Z.clone()
        t_tuned = _time_calls(tuned, M, Ps, X, Fs, Z, t1, t2)
        assert normwise(Z.cpu().numpy(), z_online.cpu().numpy()) <= 1e-5
        print(f"online {t_online * 1e3:.4f} ms {online.last_plan()}\ntuned  {t_tuned * 1e3:.4f} ms {tuned.last_plan()}")
        # What is deterministic is asserted: the tuner stored a record for the problem, it names kernels the library
        # has, and the plan that ran is that record.  The two times are reported; only a tuned plan far slower than
        # the online one (which would mean the search measured something else than what runs) fails the test.
        rec = record_of(open(str(tmp_path / "plans.txt")).read(), f"{M}x{K}*(" + "(x)".join(f"{p}x{p}" for p in Ps) + ")_NN_f")
        assert rec is not None
        for _, _, k in tuned.last_plan():
            assert k in rec, (k, rec)
        assert t_tuned <= 2.0 * t_online, (t_tuned, t_online, tuned.last_plan(), online.last_plan())
    finally:
        online.close()
        tuned.close()


@pytest.mark.parametrize("mm,M,Ps,dt,opX,opF", [
    (ko.MKM, 256, [64, 64], np.float64, ko.OP_T, ko.OP_T), (ko.KMM, 256, [64, 64], np.float64, ko.OP_N, ko.OP_N),
    (ko.MKM, 256, [128, 128], np.float64, ko.OP_N, ko.OP_N), (ko.KMM, 256, [128, 128], np.float32, ko.OP_T, ko.OP_T),
    (ko.MKM, 256, [128, 128], np.float32, ko.OP_T, ko.OP_T), (ko.MKM, 256, [16] * 4, np.float64, ko.OP_T, ko.OP_T),
    (ko.KMM, 256, [16] * 4, np.float32, ko.OP_T, ko.OP_T), (ko.KMM, 256, [16] * 4, np.float64, ko.OP_T, ko.OP_T)])
def test_shapes_with_a_shipped_plan_match_the_oracle(mm, M, Ps, dt, opX, opF):
    """Shapes of the reference's performance table for which fastkron_amd/gfx950_plans.txt holds a tuned plan, or held
    one until the online rules took it over: a default handle runs the shipped plan where there is one (checked on the
    host in tests/test_planner_cpu.py) and the result is the oracle's."""
    import fastkron_amd
    h = fastkron_amd.FastKron()
    try:
        X, Fs, Y = make_case(mm, M, Ps, Ps, dt, seed=311, opX=opX, opFs=opF)
        want = oracle_answer(mm, M, Ps, Ps, X, Fs, Y, 1.5, 0.5, opX=opX, opFs=opF)
        got, e = run_gpu(h, mm, M, Ps, Ps, X, Fs, Y, 1.5, 0.5, opX=opX, opFs=opF)
        assert e == 0
        assert normwise(got, want) <= TOL[dt], h.last_plan()
    finally:
        h.close()


VARIANTS = [
    # problem string, factor range, kernel variant, (mm, M, Ps, dtype, kwargs)
    ("64x32768*(8x8^5)_NN_f", 4, "mkm_hip_gfx950_512_f_8x8_8x8_5_1x32768wg1_mfma4x4x1_NN_strided_0_3", (ko.MKM, 64, [8] * 5, np.float32)),
    ("64x32768*(8x8^5)_NN_f", 4, "mkm_hip_gfx950_512_f_8x8_8x8_5_1x32768wg2nd_mfma4x4x1_NN_strided_0_3", (ko.MKM, 64, [8] * 5, np.float32)),
    ("600x65536*(16x16^4)_NN_f", 3, "mkm_hip_gfx950_1024_f_16x16_16x16_4_1x65536ns_mfma16x16x4_NN_strided_0_3", (ko.MKM, 600, [16] * 4, np.float32)),
    ("96x16384*(128x128^2)_NN_f", -2, "mkm_hip_gfx950_256_f_128x128_128x128_1_1x4096wg1_mfma16x16x4lds_NN_strided_0_3", (ko.MKM, 96, [128] * 2, np.float32)),
    ("128x4096*(64x64^2)_NN_d", -2, "mkm_hip_gfx950_256_d_64x64_64x64_1_1x2048wg2_mfma16x16x4lds_NN_strided_0_3", (ko.MKM, 128, [64] * 2, np.float64)),
    ("(32x32^1)*32x256_NN_f", 0, "kmm_hip_gfx950_256_f_32x32_32x32_1_128x32wg1_mfma16x16x4lds_NN_strided_0_3", (ko.KMM, 256, [32], np.float32)),
    ("(4x4^6)*4096x512_NN_f", 5, "kmm_hip_gfx950_256_f_4x4_4x4_6_256x4096_mfma4x4x1_NN_strided_0_3", (ko.KMM, 512, [4] * 6, np.float32)),
]


@pytest.mark.parametrize("key,hi,kernel,case", VARIANTS, ids=[v[2].split("_NN_")[0][16:] for v in VARIANTS])
def test_tile_and_schedule_variants_that_only_the_tuner_chooses(tmp_path, key, hi, kernel, case):
    """Kernels registered for the tuner alone (another tile, workgroups per CU or start schedule than the online rules
    take; the variant is named in the tile field of the kernel string): a tuned-plan file naming one makes a handle run
    it, and the result is the oracle's.  Counterpart of the tile sizes the reference's generator enumerates
    (reference src/gen_tuner_kernels.py:396-469)."""
    import fastkron_amd
    mm, M, Ps, dt = case
    db = tmp_path / "plans.txt"
    # hi >= 0: one launch on factors 0..hi; hi = -n: n launches of one factor each
    steps = [(0, hi, kernel)] if hi >= 0 else [(i, i, kernel) for i in range(-hi - 1, -1, -1)]
    db.write_text(f"{key} 0.1 M0 S0 {len(steps)} " + " ".join(f"{lo} {h_} {k}" for lo, h_, k in steps) + "\n")
    h = fastkron_amd.FastKron()
    h.set_tuned_db(str(db))
    try:
        for alpha, beta, seed in [(1.5, 0.5, 701), (1.0, 0.0, 702)]:
            run_and_check(h, mm, M, Ps, dt, alpha, beta, seed=seed)
            assert h.last_plan() == steps, h.last_plan()
    finally:
        h.close()
