"""Every tuned plan that ships with the library (fastkron_amd/gfx950_plans.txt), run at its own shape on a default
handle: the plan that runs must be the record, and the result must be the oracle's (sampled chains and the checksum
over all chains, tests/gpu_util.py:sampled_check).  A default handle runs these plans for every user of the shapes."""
import numpy as np
import pytest

from oracle import kron_oracle as ko
from tests.gpu_util import TOL, sampled_check
from tests.test_planner_cpu import _parse_key, _shipped_records
from fastkron_amd import capi

pytestmark = pytest.mark.gpu

RECORDS = [r for r in _shipped_records() if "stridedBatched" not in r[0]]


@pytest.fixture(scope="module")
def fk():
    import fastkron_amd
    h = fastkron_amd.FastKron()
    yield h
    h.close()


@pytest.mark.parametrize("key,flags,steps", RECORDS, ids=[r[0] for r in RECORDS])
def test_shipped_record_runs_and_matches_the_oracle(fk, key, flags, steps):
    mm, dt, M, Ps, Qs, opX, opF = _parse_key(key)
    mm = ko.MKM if mm == "mkm" else ko.KMM
    dt = np.float32 if dt == "s" else np.float64
    opX = ko.OP_T if opX == capi.OP_T else ko.OP_N
    opF = ko.OP_T if opF == capi.OP_T else ko.OP_N
    for alpha, beta in [(1.5, 0.5), (1.0, 0.0)]:
        err_rows, err_sum = sampled_check(fk, mm, M, Ps, Qs, dt, alpha=alpha, beta=beta, opX=opX, opFs=opF, seed=411)
        plan = fk.last_plan()
        ran = [(lo, hi, k) for lo, hi, k in plan if not k.startswith("transpose_")]
        assert ran == list(steps), (key, plan)
        assert any(k.startswith("transpose_") for _, _, k in plan) == bool(flags.get("X", 0)), (key, plan)
        assert err_rows <= TOL[dt], f"{key}: sampled chains off by {err_rows:.3e}"
        assert err_sum <= TOL[dt], f"{key}: checksum over all chains off by {err_sum:.3e}"
