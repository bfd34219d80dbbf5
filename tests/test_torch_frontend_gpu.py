"""GPU tests of the PyTorch front end (`fastkron_amd.gemkm` / `gekmm` / `MKM` / `KMM`): the case matrix of the
reference's own Python tests (reference tests/python/test_torch.py:118-152: batch broadcasting, transposed views,
fp32 / fp64, gradcheck), with integer-valued operands as there.  Expected values come from the oracle, one batch
element at a time; the library call underneath goes through the C ABI."""
import numpy as np
import pytest

from tests.gpu_util import TOL, normwise, oracle_answer
from oracle import kron_oracle as ko

pytestmark = pytest.mark.gpu


def expected(mm, x, fs, y, alpha, beta):
    """numpy result for logical operands: x (.., M, K) / (.., K, M), fs (.., P, Q) / (.., Q, P), y broadcastable."""
    if mm == "mkm":
        M, K = x.shape[-2:]
        Ps, Qs = [f.shape[-2] for f in fs], [f.shape[-1] for f in fs]
    else:
        K, M = x.shape[-2:]
        Ps, Qs = [f.shape[-1] for f in fs], [f.shape[-2] for f in fs]
    L = int(np.prod(Qs))
    zb = np.broadcast_shapes(x.shape[:-2], fs[0].shape[:-2])
    zshape = zb + ((M, L) if mm == "mkm" else (L, M))
    xs = np.broadcast_to(x, zb + x.shape[-2:])
    fbs = [np.broadcast_to(f, zb + f.shape[-2:]) for f in fs]
    ys = np.broadcast_to(y, zshape) if y is not None else None
    z = np.empty(zshape, dtype=x.dtype)
    for idx in np.ndindex(*zb):
        X = np.ascontiguousarray(xs[idx]).reshape(1, -1)
        Fs = [np.ascontiguousarray(f[idx]).reshape(1, -1) for f in fbs]
        Y = np.ascontiguousarray(ys[idx]).reshape(1, -1) if ys is not None else None
        z[idx] = oracle_answer(ko.MKM if mm == "mkm" else ko.KMM, M, Ps, Qs, X, Fs, Y, alpha, beta).reshape(zshape[-2:])
    return z


def make(mm, m, n, p, q, dtype, trX, trF, bx=(), bf=(), by=(), seed=0, high=5):
    import torch
    g = torch.Generator().manual_seed(seed)
    ps, qs = [p] * n, [q] * n
    K, L = int(np.prod(ps)), int(np.prod(qs))
    xshape = ([m, K] if mm == "mkm" else [K, m])
    if trX:
        xshape = xshape[::-1]
    fshape = [[ps[i], qs[i]] if mm == "mkm" else [qs[i], ps[i]] for i in range(n)]
    if trF:
        fshape = [s[::-1] for s in fshape]
    x = torch.randint(0, high, list(bx) + xshape, generator=g).to(dtype).cuda()
    fs = [torch.randint(0, high, list(bf) + s, generator=g).to(dtype).cuda() for s in fshape]
    y = torch.randint(0, high, list(by) + ([m, L] if mm == "mkm" else [L, m]), generator=g).to(dtype).cuda()
    if trX:
        x = x.mT                     # a transposed view of a row-major buffer
    if trF:
        fs = [f.mT for f in fs]
    return x, fs, y


CASES = [
    # m, n, p, q, dtype, trX, trF, batch dims of x, of fs, of y     (reference tests/python/test_torch.py:121-143)
    (16, 5, 8, 8, "float32", False, False, (), (), ()),
    (10, 5, 6, 6, "float32", True, False, (), (), ()),
    (16, 5, 8, 8, "float32", False, False, (2,), (), (2,)),
    (32, 5, 8, 8, "float32", False, False, (2, 3), (2, 3), ()),
    (8, 5, 8, 8, "float32", False, False, (2, 1), (3,), ()),
    (2, 5, 8, 8, "float32", False, False, (2, 1), (2, 4), ()),
    (32, 4, 8, 8, "float32", False, False, (3, 3, 1), (3, 1, 4), ()),
    (24, 4, 8, 8, "float32", False, False, (2,), (3, 2), ()),
    (16, 4, 8, 8, "float32", False, False, (2,), (3, 2), (3, 1)),
    (16, 4, 16, 8, "float32", True, True, (2,), (), ()),
    (32, 5, 8, 8, "float32", True, True, (2, 1), (3,), ()),
    (13, 5, 8, 8, "float32", True, True, (2, 1), (2, 4), ()),
    (19, 3, 8, 32, "float32", True, True, (2,), (3, 2), ()),
    (11, 10, 3, 3, "float64", False, True, (), (), ()),
    (200, 2, 32, 32, "float64", True, True, (), (), ()),
    (128, 5, 8, 8, "float64", True, True, (2, 1), (2, 4), ()),
]


@pytest.mark.parametrize("mm", ["mkm", "kmm"])
@pytest.mark.parametrize("case", CASES, ids=[f"{c[0]}x{c[2]}x{c[3]}^{c[1]}_{c[4]}_{'T' if c[5] else 'N'}{'T' if c[6] else 'N'}_{c[7]}_{c[8]}_{c[9]}" for c in CASES])
def test_reference_case_matrix(mm, case):
    import torch
    import fastkron_amd as fk
    m, n, p, q, dt, trX, trF, bx, bf, by = case
    dtype = getattr(torch, dt)
    x, fs, y = make(mm, m, n, p, q, dtype, trX, trF, bx, bf, by, seed=m + n)
    alpha, beta = 3.0, 1.0
    with torch.no_grad():
        z = fk.gemkm(x, fs, alpha, beta, y) if mm == "mkm" else fk.gekmm(fs, x, alpha, beta, y)
    torch.cuda.synchronize()
    want = expected(mm, x.cpu().numpy(), [f.cpu().numpy() for f in fs], y.cpu().numpy(), alpha, beta)
    assert tuple(z.shape) == want.shape
    err = normwise(z.cpu().numpy(), want)
    assert err <= TOL[np.float32 if dt == "float32" else np.float64], err


@pytest.mark.parametrize("mm", ["mkm", "kmm"])
def test_vector_operand(mm):
    import torch
    import fastkron_amd as fk
    g = torch.Generator().manual_seed(7)
    x = torch.randint(0, 5, (8 ** 3,), generator=g).double().cuda()
    fs = [torch.randint(0, 5, (8, 8), generator=g).double().cuda() for _ in range(3)]
    z = fk.gemkm(x, fs) if mm == "mkm" else fk.gekmm(fs, x)
    assert z.shape == (512,)
    kron = np.kron(np.kron(fs[0].cpu().numpy(), fs[1].cpu().numpy()), fs[2].cpu().numpy())
    want = x.cpu().numpy() @ kron if mm == "mkm" else kron @ x.cpu().numpy()
    assert normwise(z.cpu().numpy(), want) <= TOL[np.float64]


@pytest.mark.parametrize("mm", ["mkm", "kmm"])
@pytest.mark.parametrize("m,n,p,q,trX,trF", [(5, 4, 6, 6, False, True), (5, 4, 4, 6, True, True)])
def test_gradcheck(mm, m, n, p, q, trX, trF):
    """reference tests/python/test_torch.py:145-147: gradients of X and of every factor, batched factors."""
    import torch
    import fastkron_amd as fk
    x, fs, _ = make(mm, m, n, p, q, torch.float64, trX, trF, (1,), (2,), (), seed=11)
    x = x.detach().requires_grad_(True)
    fs = [f.detach().requires_grad_(True) for f in fs]
    fn = fk.MKM.apply if mm == "mkm" else fk.KMM.apply
    assert torch.autograd.gradcheck(fn, (x, *fs), eps=1e-5, atol=1e-4)


@pytest.mark.parametrize("mm", ["mkm", "kmm"])
def test_gradient_of_x_only_is_one_fused_call(mm):
    import torch
    import fastkron_amd as fk
    x, fs, _ = make(mm, 96, 4, 16, 16, torch.float32, False, False, seed=3, high=3)
    x = x.detach().requires_grad_(True)
    z = fk.gemkm(x, fs) if mm == "mkm" else fk.gekmm(fs, x)
    w = torch.randint(0, 3, z.shape, generator=torch.Generator().manual_seed(5)).float().cuda()
    (z * w).sum().backward()
    plan = fk.default_handle().last_plan()
    if mm == "mkm":
        assert all("generic" not in k for _, _, k in plan), plan
        assert len(plan) == 1, plan                                    # the backward call: four fused 16x16 factors
    kron = fs[0]
    for f in fs[1:]:
        kron = torch.kron(kron, f)
    want = (w.double() @ kron.double().mT) if mm == "mkm" else (kron.double().mT @ w.double())
    assert normwise(x.grad.cpu().numpy(), want.cpu().numpy()) <= TOL[np.float32]


def test_argument_errors():
    import torch
    import fastkron_amd as fk
    x = torch.zeros(4, 16, device="cuda")
    fs = [torch.zeros(4, 4, device="cuda")] * 2
    with pytest.raises(ValueError):
        fk.gemkm(x, [torch.zeros(4, 4, device="cuda"), torch.zeros(5, 4, device="cuda")])     # K mismatch
    with pytest.raises(ValueError):
        fk.gemkm(x, fs, 1.0, 1.0, None)                                                       # beta without y
    with pytest.raises(ValueError):
        fk.gemkm(x, [f.double() for f in fs])                                                 # mixed dtypes
    with pytest.raises(TypeError):
        fk.gemkm(x.half(), [f.half() for f in fs])                                            # unsupported dtype
    with pytest.raises(RuntimeError):
        fk.gemkm(x.cpu(), [f.cpu() for f in fs])                                              # no CPU path
    with pytest.raises(ValueError):
        fk.gemkm(x.requires_grad_(True), fs, alpha=2.0)                                       # epilogue with autograd


@pytest.mark.parametrize("mm,m,n,p", [("mkm", 32, 4, 16), ("kmm", 64, 6, 4), ("mkm", 8, 8, 4), ("mkm", 6, 3, 24)])
def test_calls_can_be_captured_in_a_hip_graph(mm, m, n, p):
    """The library calls allocate nothing and never synchronise, so a call recorded into a HIP graph replays
    correctly: every replay (with eager work and synchronisation in between, new operand values each time) is
    compared with the eager result.  The third shape goes through the factor merging launch, the last one
    through the zero-padded matrix-core step."""
    import torch
    import fastkron_amd as fk
    x, fs, _ = make(mm, m, n, p, p, torch.float32, False, False, seed=21)
    call = (lambda: fk.gemkm(x, fs)) if mm == "mkm" else (lambda: fk.gekmm(fs, x))
    with torch.no_grad():
        call()                                        # plan selection and one-time kernel attributes, outside the capture
        torch.cuda.synchronize()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            call()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            z = call()
        gen = torch.Generator().manual_seed(33)
        for rep in range(3):
            x.copy_(torch.randint(0, 5, x.shape, generator=gen).float())
            for f in fs:
                f.copy_(torch.randint(0, 5, f.shape, generator=gen).float())
            graph.replay()
            torch.cuda.synchronize()
            got = z.clone()
            want = call()                             # eager, after the replay
            torch.cuda.synchronize()
            assert torch.equal(got, want), f"replay {rep} differs from the eager call"
