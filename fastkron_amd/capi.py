"""ctypes declarations of libFastKron.so, the C-ABI library declared in include/fastkron.h.

This is the binding a host program uses: plain pointers and sizes, no torch types.  `load()` fails
loudly when the library has not been built; there is no CPU fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.environ.get("FASTKRON_LIB", os.path.join(_HERE, "lib", "libFastKron.so"))

# enum values of include/fastkron.h
OP_N, OP_T = 1, 2
BACKEND_NONE, BACKEND_X86, BACKEND_ARM, BACKEND_CUDA, BACKEND_HIP = 1, 2, 4, 8, 16
OPT_NONE, OPT_USE_FUSION, OPT_TUNE = 1, 2, 4
SUCCESS, BACKEND_NOT_AVAILABLE, INVALID_MEMORY_ACCESS, KERNEL_NOT_FOUND, INVALID_ARGUMENT, \
    INVALID_KMM_PROBLEM, OTHER_ERROR = range(7)
STATIC_SCRATCH_TEMP_BYTES = 16 << 20        # FASTKRON_STATIC_SCRATCH_TEMP_BYTES of include/fastkron_ext.h

EXPORTS = [
    "fastKronVersion", "fastKronCUDAArchs", "fastKronGetErrorString", "fastKronGetBackends",
    "fastKronInit", "fastKronInitAllBackends", "fastKronSetOptions", "fastKronDestroy",
    "fastKronInitCUDA", "fastKronInitHIP", "fastKronInitX86", "fastKronSetStream",
    "gekmmSizes", "sgemkm", "dgemkm", "sgekmm", "dgekmm",
    "sgemkmStridedBatched", "dgemkmStridedBatched", "sgekmmStridedBatched", "dgekmmStridedBatched",
    "gekmmSizesForward", "smkmForward", "dmkmForward", "skmmForward", "dkmmForward",
    "smkmForwardStridedBatched", "dmkmForwardStridedBatched",
    "skmmForwardStridedBatched", "dkmmForwardStridedBatched",
]

EXT_EXPORTS = ["fastKronGetLastPlan", "fastKronSetTunedDB", "fastKronSetPlanOnly", "fastKronGetLastLaunches",
               "sgemkmStaticScratch", "fastKronGetSyncError", "fastKronSetSyncHelpAfter",
               "fastKronProbeCopyPattern"]     # include/fastkron_ext.h

_lib = None

u32, u64, vp, cint = ctypes.c_uint32, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_int
u32p, u64p, szp = ctypes.POINTER(u32), ctypes.POINTER(u64), ctypes.POINTER(ctypes.c_size_t)
vpp = ctypes.POINTER(vp)


def load():
    global _lib
    if _lib is not None:
        return _lib
    try:
        # PyTorch bundles its own libamdhip64.so.7; importing it first makes the dynamic loader bind
        # libFastKron.so to that same runtime, so the process holds exactly one HIP runtime and
        # torch's allocations and streams are valid inside the library.
        import torch  # noqa: F401
    except ImportError:
        pass
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with fastkron_amd/csrc/build.sh (or __graft_entry__.build())")
    lib = ctypes.CDLL(LIB_PATH)
    lib.fastKronVersion.restype = ctypes.c_char_p
    lib.fastKronCUDAArchs.restype = ctypes.c_char_p
    lib.fastKronGetErrorString.restype = ctypes.c_char_p
    lib.fastKronGetErrorString.argtypes = [cint]
    lib.fastKronGetBackends.restype = u32
    lib.fastKronInit.argtypes = [vpp, u32]
    lib.fastKronInitAllBackends.argtypes = [vpp]
    lib.fastKronSetOptions.argtypes = [vp, u32]
    lib.fastKronDestroy.argtypes = [vp]
    lib.fastKronDestroy.restype = None
    lib.fastKronInitCUDA.argtypes = [vp, vp]
    lib.fastKronInitHIP.argtypes = [vp, vp]
    lib.fastKronInitX86.argtypes = [vp]
    lib.fastKronSetStream.argtypes = [vp, cint, vp]
    lib.gekmmSizes.argtypes = [vp, u32, u32, u32p, u32p, szp, szp]
    lib.gekmmSizesForward.argtypes = [vp, u32, u32, u32p, u32p, szp, szp]
    for name, sc in (("s", ctypes.c_float), ("d", ctypes.c_double)):
        getattr(lib, name + "gemkm").argtypes = [vp, cint, u32, u32, u32p, u32p, vp, cint, vpp, cint,
                                                 vp, sc, sc, vp, vp, vp]
        getattr(lib, name + "gekmm").argtypes = [vp, cint, u32, u32p, u32p, u32, vpp, cint, vp, cint,
                                                 vp, sc, sc, vp, vp, vp]
        getattr(lib, name + "gemkmStridedBatched").argtypes = [
            vp, cint, u32, u32, u32p, u32p, vp, cint, u64, vpp, cint, u64p,
            vp, u64, sc, sc, u32, vp, u64, vp, vp]
        getattr(lib, name + "gekmmStridedBatched").argtypes = [
            vp, cint, u32, u32p, u32p, u32, vpp, cint, u64p, vp, cint, u64,
            vp, u64, sc, sc, u32, vp, u64, vp, vp]
        getattr(lib, name + "mkmForward").argtypes = [vp, cint, u32, u32, u32p, u32p, vp, cint, vpp, cint, vp, vpp]
        getattr(lib, name + "kmmForward").argtypes = [vp, cint, u32, u32p, u32p, u32, vpp, cint, vp, cint, vp, vpp]
        getattr(lib, name + "mkmForwardStridedBatched").argtypes = [
            vp, cint, u32, u32, u32p, u32p, vp, cint, u64, vpp, cint, u64p, vp, u64, u32, vpp, u64p]
        getattr(lib, name + "kmmForwardStridedBatched").argtypes = [
            vp, cint, u32, u32p, u32p, u32, vpp, cint, u64p, vp, cint, u64, vp, u64, u32, vpp, u64p]
    lib.fastKronGetLastPlan.argtypes = [vp, ctypes.c_char_p, ctypes.c_size_t]
    lib.fastKronGetLastPlan.restype = ctypes.c_size_t
    lib.fastKronSetTunedDB.argtypes = [vp, ctypes.c_char_p]
    lib.sgemkmStaticScratch.argtypes = [vp, cint, u32, u32, u32p, u32p, vp, cint, vpp, cint, vp, ctypes.c_float,
                                        ctypes.c_float, vp]
    lib.sgemkmStaticScratch.restype = cint
    lib.fastKronGetSyncError.argtypes = [vp, u32p]
    lib.fastKronSetSyncHelpAfter.argtypes = [u32]
    lib.fastKronProbeCopyPattern.argtypes = [vp, cint, vp, vp, vp, vp, u32]
    lib.fastKronSetPlanOnly.argtypes = [vp, cint]
    lib.fastKronGetLastLaunches.argtypes = [vp, ctypes.c_char_p, ctypes.c_size_t]
    lib.fastKronGetLastLaunches.restype = ctypes.c_size_t
    for n in EXPORTS:
        f = getattr(lib, n)
        if f.restype is ctypes.c_int and n not in ("fastKronGetBackends",):
            f.restype = cint
    _lib = lib
    return lib


def arr_u32(v):
    return (u32 * len(v))(*[int(x) for x in v])


def arr_u64(v):
    return (u64 * len(v))(*[int(x) for x in v])


def arr_ptr(v):
    return (vp * len(v))(*[int(x) if x is not None else None for x in v])
