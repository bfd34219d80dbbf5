"""Host-side checks of the C-ABI library that need no GPU: every symbol declared in
include/fastkron.h is exported, sizes agree with the oracle, and the argument checks return the
codes the reference returns (reference src/handle/handle.cpp:94-95,116-122,378-379; src/fastkron.cpp:78-90)."""
import ctypes
import os
import re

import pytest

from fastkron_amd import capi
from oracle import kron_oracle as ko

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    src = open(os.path.join(ROOT, "include", "fastkron.h")).read()
    src = re.sub(r"/\*.*?\*/", "", src, flags=re.S)
    body = src[src.index('extern "C"'):]
    names = re.findall(r"\b(?:fastKronError|const char\*|uint32_t|void)\s+(\w+)\s*\(", body)
    return sorted(set(names))


def test_library_exports_every_declared_symbol():
    lib = capi.load()
    names = declared_functions()
    assert len(names) == 30, names
    assert sorted(capi.EXPORTS) == names
    for n in names:
        assert hasattr(lib, n), n


def test_version_backends_and_error_strings():
    lib = capi.load()
    assert lib.fastKronVersion().decode().startswith("1.1.0+")
    assert lib.fastKronGetBackends() == capi.BACKEND_HIP
    assert lib.fastKronCUDAArchs() is None
    assert lib.fastKronGetErrorString(0) == b"Operation successfull"
    assert lib.fastKronGetErrorString(4) == b"An argument to the function is invalid"
    assert lib.fastKronGetErrorString(5) is None          # as in the reference: no string for this code


@pytest.fixture
def handle():
    lib = capi.load()
    h = ctypes.c_void_p()
    assert lib.fastKronInit(ctypes.byref(h), capi.BACKEND_HIP) == capi.SUCCESS
    yield lib, h
    lib.fastKronDestroy(h)


def test_init_with_a_backend_that_is_not_built():
    lib = capi.load()
    h = ctypes.c_void_p()
    assert lib.fastKronInit(ctypes.byref(h), capi.BACKEND_X86) == capi.INVALID_ARGUMENT
    assert h.value                                          # the handle is allocated all the same
    assert lib.fastKronInitX86(h) == capi.BACKEND_NOT_AVAILABLE
    assert lib.fastKronInitCUDA(h, None) == capi.BACKEND_NOT_AVAILABLE
    assert lib.fastKronInitHIP(h, None) == capi.BACKEND_NOT_AVAILABLE   # HIP is not in this handle
    lib.fastKronDestroy(h)


def test_set_stream_argument_checks(handle):
    lib, h = handle
    assert lib.fastKronSetStream(h, capi.BACKEND_HIP, None) == capi.INVALID_ARGUMENT
    s = ctypes.c_void_p(0)
    assert lib.fastKronSetStream(h, capi.BACKEND_CUDA, ctypes.byref(s)) == capi.BACKEND_NOT_AVAILABLE
    assert lib.fastKronSetStream(h, capi.BACKEND_HIP, ctypes.byref(s)) == capi.SUCCESS


@pytest.mark.parametrize("M,Ps,Qs", [
    (1024, [8] * 5, [8] * 5), (1024, [16] * 4, [16] * 4), (256, [64] * 3, [64] * 3),
    (2048, [4] * 6, [4] * 6), (512, [32] * 3, [16] * 3), (4, [8, 8], [32, 32]), (4, [8], [32]),
    (7, [2, 3, 5], [5, 1, 3]), (3, [31, 63], [63, 31]),
])
def test_sizes_agree_with_oracle(handle, M, Ps, Qs):
    lib, h = handle
    y, t = ctypes.c_size_t(), ctypes.c_size_t()
    e = lib.gekmmSizes(h, M, len(Ps), capi.arr_u32(Ps), capi.arr_u32(Qs), ctypes.byref(y), ctypes.byref(t))
    assert e == capi.SUCCESS
    assert (y.value, t.value) == ko.gekmm_sizes(M, Ps, Qs)
    inter = (ctypes.c_size_t * len(Ps))()
    e = lib.gekmmSizesForward(h, M, len(Ps), capi.arr_u32(Ps), capi.arr_u32(Qs), ctypes.byref(y), inter)
    assert e == capi.SUCCESS
    yo, io = ko.gekmm_sizes_forward(M, Ps, Qs)
    assert y.value == yo and [inter[i] for i in range(len(Ps) - 1)] == io


def test_sizes_null_outputs(handle):
    lib, h = handle
    y = ctypes.c_size_t()
    assert lib.gekmmSizes(h, 4, 1, capi.arr_u32([2]), capi.arr_u32([2]), None, ctypes.byref(y)) == capi.INVALID_ARGUMENT
    assert lib.gekmmSizes(h, 4, 1, capi.arr_u32([2]), capi.arr_u32([2]), ctypes.byref(y), None) == capi.INVALID_ARGUMENT


def test_gemm_argument_checks_return_before_touching_a_device(handle):
    """Null Z, null temp1, a backend the handle lacks, and Z == Y without temp2 are all
    fastKronInvalidArgument (4), decided on the host."""
    lib, h = handle
    Ps, Qs = capi.arr_u32([2, 2]), capi.arr_u32([2, 2])
    fake = ctypes.c_void_p(0x1000)                # never dereferenced: the checks come first
    fs = capi.arr_ptr([0x2000, 0x3000])
    f32 = ctypes.c_float
    call = lambda backend, Z, Y, t1, t2: lib.sgemkm(h, backend, 4, 2, Ps, Qs, fake, capi.OP_N, fs, capi.OP_N,
                                                    Z, f32(1), f32(0), Y, t1, t2)
    assert call(capi.BACKEND_HIP, None, None, fake, None) == capi.INVALID_ARGUMENT
    assert call(capi.BACKEND_HIP, fake, None, None, None) == capi.INVALID_ARGUMENT
    assert call(capi.BACKEND_X86, fake, None, fake, None) == capi.INVALID_ARGUMENT
    assert call(capi.BACKEND_HIP, fake, fake, ctypes.c_void_p(0x4000), None) == capi.INVALID_ARGUMENT
    callk = lambda Z: lib.dgekmm(h, capi.BACKEND_HIP, 2, Qs, Ps, 4, fs, capi.OP_N, fake, capi.OP_N, Z,
                                 ctypes.c_double(1), ctypes.c_double(0), None, fake, None)
    assert callk(None) == capi.INVALID_ARGUMENT


def test_extension_symbols_and_last_plan_before_any_call(handle):
    lib, h = handle
    for n in capi.EXT_EXPORTS:                      # include/fastkron_ext.h
        assert hasattr(lib, n), n
    buf = ctypes.create_string_buffer(64)
    assert lib.fastKronGetLastPlan(h, buf, 64) == 0
    assert lib.fastKronSetTunedDB(h, None) == capi.SUCCESS


def test_tuned_plan_file_round_trip(tmp_path, handle):
    """A tuned-plan file written by hand is accepted; unknown kernel names are ignored at lookup time."""
    lib, h = handle
    f = tmp_path / "tuned.db"
    f.write_text("# comment\n8x64*(8x8^2)_NN_f 0.01 1 0 1 no_such_kernel\n")
    assert lib.fastKronSetTunedDB(h, str(f).encode()) == capi.SUCCESS
