"""sgemkmStaticScratch (include/fastkron_ext.h): the variant of sgemkm that takes its temporaries and the
merged-factor workspace from the library's static device array and allocates nothing.  Called through the C ABI and
compared with the oracle (normwise 1e-5, the fp32 bound of every parity test here) and with sgemkm on the same
operands: the two run the same launches, so their results agree bit for bit.  Two calls in a row share the array, the
second on a smaller problem, so stale contents of the first must not leak into it."""
import ctypes

import numpy as np
import pytest

from fastkron_amd import capi
from oracle import kron_oracle as ko
from tests.gpu_util import normwise, seeded

pytestmark = pytest.mark.gpu

TOL = 1e-5


def both(fk, M, Ps, alpha, beta, seed):
    import torch
    dev = "cuda:0"
    K = int(np.prod(Ps))
    X = torch.from_numpy(seeded(seed, (M * K,), np.float32)).to(dev)
    Fs = [torch.from_numpy(seeded(seed + 1 + i, (p * p,), np.float32)).to(dev) for i, p in enumerate(Ps)]
    Y = torch.from_numpy(seeded(seed + 50, (M * K,), np.float32)).to(dev)
    ye, te = fk.sizes(M, Ps, Ps)
    want = torch.full((ye,), float("nan"), dtype=torch.float32, device=dev)
    t1 = torch.full((te,), float("nan"), dtype=torch.float32, device=dev)
    t2 = torch.full((te,), float("nan"), dtype=torch.float32, device=dev)
    assert fk.xgemkm(M, Ps, Ps, X, Fs, want, alpha, beta, Y, t1, t2) == capi.SUCCESS
    plan = fk.last_plan()
    got = torch.full((ye,), float("nan"), dtype=torch.float32, device=dev)
    # one call ahead of the measured one, so that code objects and function attributes are set up
    assert fk.xgemkm_static_scratch(M, Ps, Ps, X, Fs, got, alpha, beta, Y) == capi.SUCCESS
    got.fill_(float("nan"))
    torch.cuda.synchronize()
    # free device memory as the driver sees it (the library's own hipMalloc / hipFree would show here, which
    # torch's allocator statistics would not), and torch's own allocations
    free_before, before = torch.cuda.mem_get_info()[0], torch.cuda.memory_allocated()
    e = fk.xgemkm_static_scratch(M, Ps, Ps, X, Fs, got, alpha, beta, Y)
    torch.cuda.synchronize()
    assert e == capi.SUCCESS, e
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    assert fk.last_plan() == plan
    oracle = ko.sliced_multiply(ko.MKM, M, Ps, Ps, X.cpu().numpy().reshape(1, -1), [f.cpu().numpy().reshape(1, -1) for f in Fs],
                                alpha=alpha, beta=beta, Y=Y.cpu().numpy().reshape(1, -1), batch=1, strideX=M * K,
                                strideF=[p * p for p in Ps], strideZ=M * K, strideY=M * K).reshape(-1)
    got, want = got.cpu().numpy(), want.cpu().numpy()
    assert not np.isnan(got).any()
    assert normwise(got, oracle) <= TOL, normwise(got, oracle)
    return got, want, plan


@pytest.mark.parametrize("tune", [False, True])
def test_static_scratch_entry_point_matches_sgemkm_on_two_calls_in_a_row(tune):
    """(tune=True: a handle with tuning switched on must not tune, i.e. allocate, in this entry point either)"""
    import fastkron_amd
    fk = fastkron_amd.FastKron(tune=tune)
    try:
        # first call: two-part plan (whole-block kernel into temp1, leading factor across the blocks), 8 MiB temporaries
        got, want, plan = both(fk, 2, [16] * 5, 1.5, 0.5, seed=901)
        assert tune or len(plan) >= 2, plan
        assert normwise(got, want) <= TOL
        assert np.array_equal(got, want)
        # second call, smaller, and through the merged-factor part of the array: 4x4^8 runs as 16x16^4
        got, want, plan = both(fk, 3, [4] * 8, 1.0, 1.0, seed=902)
        assert tune or any("16x16" in k for _, _, k in plan), plan
        assert normwise(got, want) <= TOL
        assert np.array_equal(got, want)
        # a third, smaller still, with three launches ping-ponging between the two temporaries
        got, want, plan = both(fk, 1, [8] * 7, 2.0, 0.0, seed=903)
        assert normwise(got, want) <= TOL
        assert np.array_equal(got, want)
    finally:
        fk.close()


def test_static_scratch_entry_point_refuses_problems_beyond_its_array():
    import torch
    import fastkron_amd
    fk = fastkron_amd.FastKron()
    try:
        M, Ps = 64, [16] * 5                      # temporaries of 256 MiB each
        ye, te = fk.sizes(M, Ps, Ps)
        assert te * 4 > capi.STATIC_SCRATCH_TEMP_BYTES
        fake = torch.empty(16, dtype=torch.float32, device="cuda:0")     # never touched: the size check comes first
        e = fk.xgemkm_static_scratch(M, Ps, Ps, fake, [fake] * 5, fake, 1.0, 0.0, None)
        assert e == capi.INVALID_ARGUMENT
        # the largest problem of this shape that fits is accepted
        M = capi.STATIC_SCRATCH_TEMP_BYTES // 4 // 16 ** 5
        assert M == 4
        got, want, _ = both(fk, M, Ps, 1.0, 0.0, seed=904)
        assert np.array_equal(got, want)
    finally:
        fk.close()
