"""Randomised GPU parity: a fixed-seed stream of small problems over both layouts, both types, square and
rectangular factors of many sizes, transposed operands, batches with shared or per-batch factors, alpha / beta / Y
and one or two temporaries, each compared with the oracle through the C ABI.  The shapes are drawn so that every
kernel family and planner path (merged factors, two-part plans, LDS-fused groups, padded matrix-core steps, plain
kernel) is hit many times."""
import numpy as np
import pytest

from tests.gpu_util import TOL, make_case, normwise, oracle_answer, run_gpu
from oracle import kron_oracle as ko

pytestmark = pytest.mark.gpu

SIZES = [1, 2, 2, 3, 4, 4, 5, 6, 7, 8, 8, 10, 12, 16, 16, 16, 17, 24, 31, 32, 32, 33, 64, 64]


def draw(rng):
    mm = ko.MKM if rng.random() < 0.6 else ko.KMM
    dt = np.float32 if rng.random() < 0.5 else np.float64
    n = int(rng.integers(1, 7))
    square = rng.random() < 0.7
    same = rng.random() < 0.5
    Ps, Qs = [], []
    base = int(rng.choice(SIZES))
    for _ in range(n):
        p = base if same else int(rng.choice(SIZES))
        q = p if square else int(rng.choice(SIZES))
        Ps.append(p); Qs.append(q)
    # keep every intermediate small enough for the oracle
    while True:
        w, widths = int(np.prod(Ps)), []
        for p, q in zip(reversed(Ps), reversed(Qs)):
            w = w // p * q
            widths.append(w)
        if max(widths + [int(np.prod(Ps))]) <= 1 << 16 or len(Ps) == 1:
            break
        Ps.pop(0); Qs.pop(0)
    if max(Ps) * max(Qs) > 64 * 64 and len(Ps) > 2:
        Ps, Qs = Ps[-2:], Qs[-2:]
    M = int(rng.choice([1, 2, 3, 5, 8, 16, 17, 32, 48, 64, 70]))
    batch = int(rng.choice([1, 1, 1, 2, 3]))
    kw = dict(opX=ko.OP_T if rng.random() < 0.15 else ko.OP_N, opFs=ko.OP_T if rng.random() < 0.3 else ko.OP_N)
    if batch > 1:
        kw.update(batch=batch, share_f=bool(rng.random() < 0.5), share_y=bool(rng.random() < 0.3))
    alpha = float(rng.choice([1.0, 1.0, -0.5, 2.0]))
    beta = float(rng.choice([0.0, 0.0, 1.0, 0.5]))
    run_kw = {"use_temp2": False} if (Ps == Qs and rng.random() < 0.2) else {}      # Z doubles as the second temporary
    return mm, M, Ps, Qs, dt, alpha, beta, kw, run_kw


@pytest.fixture(scope="module")
def fk():
    import fastkron_amd
    h = fastkron_amd.FastKron()
    yield h
    h.close()


@pytest.mark.parametrize("chunk", range(8))
def test_random_problems(fk, chunk):
    rng = np.random.default_rng(1000 + chunk)
    for i in range(120):
        mm, M, Ps, Qs, dt, alpha, beta, kw, run_kw = draw(rng)
        X, Fs, Y = make_case(mm, M, Ps, Qs, dt, seed=chunk * 100 + i, with_y=(beta != 0), **kw)
        want = oracle_answer(mm, M, Ps, Qs, X, Fs, Y, alpha, beta, **kw)
        got, e = run_gpu(fk, mm, M, Ps, Qs, X, Fs, Y, alpha, beta, **kw, **run_kw)
        what = (f"case {chunk}/{i}: mm={mm} M={M} Ps={Ps} Qs={Qs} {dt.__name__} alpha={alpha} beta={beta} {kw} {run_kw} "
                f"plan={fk.last_plan()}")
        assert e == 0, what
        assert not np.isnan(got).any(), what
        err = normwise(got, want)
        assert err <= TOL[dt], f"{what}: normwise error {err:.3e}"
