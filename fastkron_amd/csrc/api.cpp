// extern "C" entry points of include/fastkron.h: argument marshalling only.
// Role of reference src/fastkron.cpp:19-386.
#include <cstdlib>
#include <cstring>

#include "../../include/fastkron.h"
#include "../../include/fastkron_ext.h"
#include "handle.h"
#include "kernels/launch.h"

using namespace fk;

#ifndef FASTKRON_VERSION
#define FASTKRON_VERSION "1.1.0"
#endif

static inline Handle* H(fastKronHandle h) { return (Handle*)h; }

extern "C" {

const char* fastKronVersion(void) { return FASTKRON_VERSION "+gfx950"; }

const char* fastKronCUDAArchs(void) { return nullptr; }             // reference fastkron.cpp:33-42

const char* fastKronGetErrorString(fastKronError err) {             // strings of reference fastkron.cpp:44-61
  switch (err) {
    case fastKronSuccess:             return "Operation successfull";
    case fastKronBackendNotAvailable: return "Requested backend is not available";
    case fastKronInvalidMemoryAccess: return "Illegal memory access";
    case fastKronKernelNotFound:      return "Kernel to execute the problem not found";
    case fastKronInvalidArgument:     return "An argument to the function is invalid";
    case fastKronOtherError:          return "Unknown error occurred";
    default:                          return nullptr;               // InvalidKMMProblem has no string there
  }
}

uint32_t fastKronGetBackends(void) { return fastKronBackend_HIP; }

fastKronError fastKronInit(fastKronHandle* handle, uint32_t backends) {
  if (!handle) return fastKronInvalidArgument;
  Handle* h = new Handle(backends);
  *handle = (fastKronHandle)h;
  uint32_t opts = fastKronOptionsUseFusion;                         // reference fastkron.cpp:81-84
  const char* t = getenv("FASTKRON_TUNE");
  if (t && strcmp(t, "0") != 0 && t[0] != '\0') opts |= fastKronOptionsTune;
  h->setOptions(opts);
  // the handle exists even when an unavailable backend was asked for (reference fastkron.cpp:86-87)
  if ((backends & fastKronGetBackends()) != backends) return fastKronInvalidArgument;
  return fastKronSuccess;
}

fastKronError fastKronInitAllBackends(fastKronHandle* handle) { return fastKronInit(handle, fastKronGetBackends()); }

fastKronError fastKronSetOptions(fastKronHandle handle, uint32_t options) {
  if (!handle) return fastKronInvalidArgument;
  H(handle)->setOptions(options);
  return fastKronSuccess;
}

void fastKronDestroy(fastKronHandle handle) { delete H(handle); }

fastKronError fastKronInitCUDA(fastKronHandle, void*) { return fastKronBackendNotAvailable; }
fastKronError fastKronInitX86(fastKronHandle) { return fastKronBackendNotAvailable; }

fastKronError fastKronInitHIP(fastKronHandle handle, void* ptrToStream) {
  if (!handle) return fastKronInvalidArgument;
  return H(handle)->initHIP(ptrToStream);
}

fastKronError fastKronSetStream(fastKronHandle handle, fastKronBackend backend, void* ptrToStream) {
  if (!handle) return fastKronInvalidArgument;
  return H(handle)->setStream(backend, ptrToStream);
}

size_t fastKronGetLastPlan(fastKronHandle handle, char* buf, size_t bufLen) {
  if (!handle) return 0;
  const std::string& s = H(handle)->lastPlan();
  if (buf && bufLen) {
    const size_t n = s.size() < bufLen - 1 ? s.size() : bufLen - 1;
    memcpy(buf, s.data(), n);
    buf[n] = 0;
  }
  return s.size();
}

fastKronError fastKronSetPlanOnly(fastKronHandle handle, int on) {
  if (!handle) return fastKronInvalidArgument;
  H(handle)->setPlanOnly(on != 0);
  return fastKronSuccess;
}

size_t fastKronGetLastLaunches(fastKronHandle handle, char* buf, size_t bufLen) {
  if (!handle) return 0;
  const std::string& s = H(handle)->lastLaunches();
  if (buf && bufLen) {
    const size_t n = s.size() < bufLen - 1 ? s.size() : bufLen - 1;
    memcpy(buf, s.data(), n);
    buf[n] = 0;
  }
  return s.size();
}

fastKronError fastKronGetSyncError(fastKronHandle handle, uint32_t* word) {
  if (!handle || !word) return fastKronInvalidArgument;
  return H(handle)->syncError(word);
}

fastKronError fastKronProbeCopyPattern(fastKronHandle handle, int pattern, const float* X, const float* Y, float* Z,
                                       float* T, uint32_t M) {
  if (!handle) return fastKronInvalidArgument;
  return fk::launchPatternProbe(pattern, X, Y, Z, T, H(handle)->syncArea(), M, H(handle)->stream()) == hipSuccess
             ? fastKronSuccess : fastKronInvalidArgument;
}

fastKronError fastKronSetSyncHelpAfter(uint32_t polls) {
  fk::setKmm4x6TwoPhaseHelpAfter(polls);
  return fastKronSuccess;
}

fastKronError fastKronSetTunedDB(fastKronHandle handle, const char* path) {
  if (!handle) return fastKronInvalidArgument;
  H(handle)->setTunedDB(path);
  return fastKronSuccess;
}

fastKronError gekmmSizes(fastKronHandle handle, uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
                         size_t* yElems, size_t* tmpElems) {
  (void)handle;
  return Handle::sizes(M, N, Ps, Qs, yElems, tmpElems);
}

fastKronError gekmmSizesForward(fastKronHandle handle, uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
                                size_t* yElems, size_t* intermediateElems) {
  (void)handle;
  return Handle::sizesForward(M, N, Ps, Qs, yElems, intermediateElems);
}

}  // extern "C"

namespace {

struct Call {
  MMType mm; DType dt;
  uint32_t M, N; const uint32_t *Ps, *Qs;
  const void* X; fastKronOp opX; uint64_t strideX;
  const void* const* Fs; fastKronOp opFs; const uint64_t* strideF;
  void* Z; uint64_t strideZ; double alpha, beta;
  uint32_t batch; const void* Y; uint64_t strideY;
  bool strided;
  void* const* inter; const uint64_t* strideInter; bool forward;
};

fastKronError run(fastKronHandle handle, fastKronBackend backend, const Call& c, void* t1, void* t2) {
  if (!handle) return fastKronInvalidArgument;
  if (c.N == 0 || c.N > kMaxFactors || !c.Ps || !c.Qs || !c.Fs) return fastKronInvalidKMMProblem;
  KronProblem p{};
  p.mm = c.mm; p.dt = c.dt; p.M = c.M; p.N = c.N;
  for (uint32_t i = 0; i < c.N; i++) {
    p.P[i] = c.Ps[i]; p.Q[i] = c.Qs[i]; p.F[i] = c.Fs[i];
    p.strideF[i] = (c.strided && c.strideF) ? c.strideF[i] : 0;
  }
  p.X = c.X; p.opX = c.opX; p.strideX = c.strided ? c.strideX : 0;
  p.opF = c.opFs;
  p.Z = c.Z; p.strideZ = c.strided ? c.strideZ : 0;
  p.Y = c.Y; p.strideY = c.strided ? c.strideY : 0;
  p.alpha = c.alpha; p.beta = c.beta;
  p.batch = c.strided ? c.batch : 1;
  p.strided = c.strided;
  p.forward = c.forward;
  p.haveStrideInter = false;
  if (c.forward) {
    for (uint32_t i = 0; i + 1 < c.N; i++) {
      p.inter[i] = c.inter ? c.inter[i] : nullptr;
      if (c.strideInter) { p.strideInter[i] = c.strideInter[i]; p.haveStrideInter = true; }
    }
  }
  // A strided-batched call with a single batch entry never uses its strides: they are cleared here so that no
  // plan that re-views the rows of one problem as batch entries of another (the two-part plan does) can carry a
  // caller's stride into a batch index of its own.
  if (p.batch == 1) {
    p.strideX = p.strideZ = p.strideY = 0;
    for (uint32_t i = 0; i < c.N; i++) { p.strideF[i] = 0; p.strideInter[i] = 0; }
    p.haveStrideInter = false;
  }
  return H(handle)->xgemm(p, backend, t1, t2);
}

}  // namespace

extern "C" {

#define FK_GEMM(NAME, T, DT, MM, ARGS_DECL, MVAL, NVAL, PSV, QSV)                                         \
  fastKronError NAME ARGS_DECL {                                                                          \
    Call c{MM, DT, MVAL, NVAL, PSV, QSV, X, opX, 0, (const void* const*)Fs, opFs, nullptr, Z, 0,          \
           (double)alpha, (double)beta, 1, Y, 0, false, nullptr, nullptr, false};                         \
    return run(handle, backend, c, temp1, temp2);                                                         \
  }

FK_GEMM(sgemkm, float, DType::F32, MMType::MKM,
        (fastKronHandle handle, fastKronBackend backend, uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
         const float* X, fastKronOp opX, const float* const Fs[], fastKronOp opFs, float* Z, float alpha,
         float beta, const float* Y, float* temp1, float* temp2), M, N, Ps, Qs)
FK_GEMM(dgemkm, double, DType::F64, MMType::MKM,
        (fastKronHandle handle, fastKronBackend backend, uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
         const double* X, fastKronOp opX, const double* const Fs[], fastKronOp opFs, double* Z, double alpha,
         double beta, const double* Y, double* temp1, double* temp2), M, N, Ps, Qs)
FK_GEMM(sgekmm, float, DType::F32, MMType::KMM,
        (fastKronHandle handle, fastKronBackend backend, uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
         const float* const Fs[], fastKronOp opFs, const float* X, fastKronOp opX, float* Z, float alpha,
         float beta, const float* Y, float* temp1, float* temp2), M, N, Ps, Qs)
FK_GEMM(dgekmm, double, DType::F64, MMType::KMM,
        (fastKronHandle handle, fastKronBackend backend, uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
         const double* const Fs[], fastKronOp opFs, const double* X, fastKronOp opX, double* Z, double alpha,
         double beta, const double* Y, double* temp1, double* temp2), M, N, Ps, Qs)

#define FK_GEMM_SB(NAME, T, DT, MM, ARGS_DECL)                                                            \
  fastKronError NAME ARGS_DECL {                                                                          \
    Call c{MM, DT, M, N, Ps, Qs, X, opX, strideX, (const void* const*)Fs, opFs, strideF, Z, strideZ,      \
           (double)alpha, (double)beta, batchCount, Y, strideY, true, nullptr, nullptr, false};           \
    return run(handle, backend, c, temp1, temp2);                                                         \
  }

FK_GEMM_SB(sgemkmStridedBatched, float, DType::F32, MMType::MKM,
           (fastKronHandle handle, fastKronBackend backend, uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
            const float* X, fastKronOp opX, uint64_t strideX, const float* const Fs[], fastKronOp opFs,
            uint64_t strideF[], float* Z, uint64_t strideZ, float alpha, float beta, uint32_t batchCount,
            const float* Y, uint64_t strideY, float* temp1, float* temp2))
FK_GEMM_SB(dgemkmStridedBatched, double, DType::F64, MMType::MKM,
           (fastKronHandle handle, fastKronBackend backend, uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
            const double* X, fastKronOp opX, uint64_t strideX, const double* const Fs[], fastKronOp opFs,
            uint64_t strideF[], double* Z, uint64_t strideZ, double alpha, double beta, uint32_t batchCount,
            const double* Y, uint64_t strideY, double* temp1, double* temp2))
FK_GEMM_SB(sgekmmStridedBatched, float, DType::F32, MMType::KMM,
           (fastKronHandle handle, fastKronBackend backend, uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
            const float* const Fs[], fastKronOp opFs, uint64_t strideF[], const float* X, fastKronOp opX,
            uint64_t strideX, float* Z, uint64_t strideZ, float alpha, float beta, uint32_t batchCount,
            const float* Y, uint64_t strideY, float* temp1, float* temp2))
FK_GEMM_SB(dgekmmStridedBatched, double, DType::F64, MMType::KMM,
           (fastKronHandle handle, fastKronBackend backend, uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
            const double* const Fs[], fastKronOp opFs, uint64_t strideF[], const double* X, fastKronOp opX,
            uint64_t strideX, double* Z, uint64_t strideZ, double alpha, double beta, uint32_t batchCount,
            const double* Y, uint64_t strideY, double* temp1, double* temp2))

// Forward family: alpha = 1, beta = 0, no Y (reference fastkron.cpp:279-386).
#define FK_FWD(NAME, T, DT, MM, ARGS_DECL)                                                                \
  fastKronError NAME ARGS_DECL {                                                                          \
    Call c{MM, DT, M, N, Ps, Qs, X, opX, 0, (const void* const*)Fs, opFs, nullptr, Z, 0, 1.0, 0.0, 1,     \
           nullptr, 0, false, (void* const*)Intermediates, nullptr, true};                                \
    return run(handle, backend, c, nullptr, nullptr);                                                     \
  }

FK_FWD(smkmForward, float, DType::F32, MMType::MKM,
       (fastKronHandle handle, fastKronBackend backend, uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
        const float* X, fastKronOp opX, const float* const Fs[], fastKronOp opFs, float* Z, float* Intermediates[]))
FK_FWD(dmkmForward, double, DType::F64, MMType::MKM,
       (fastKronHandle handle, fastKronBackend backend, uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
        const double* X, fastKronOp opX, const double* const Fs[], fastKronOp opFs, double* Z, double* Intermediates[]))
FK_FWD(skmmForward, float, DType::F32, MMType::KMM,
       (fastKronHandle handle, fastKronBackend backend, uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
        const float* const Fs[], fastKronOp opFs, const float* X, fastKronOp opX, float* Z, float* Intermediates[]))
FK_FWD(dkmmForward, double, DType::F64, MMType::KMM,
       (fastKronHandle handle, fastKronBackend backend, uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
        const double* const Fs[], fastKronOp opFs, const double* X, fastKronOp opX, double* Z, double* Intermediates[]))

#define FK_FWD_SB(NAME, T, DT, MM, ARGS_DECL)                                                             \
  fastKronError NAME ARGS_DECL {                                                                          \
    Call c{MM, DT, M, N, Ps, Qs, X, opX, strideX, (const void* const*)Fs, opFs, strideF, Z, strideZ, 1.0, \
           0.0, batchCount, nullptr, 0, true, (void* const*)Intermediates, strideIntermediates, true};    \
    return run(handle, backend, c, nullptr, nullptr);                                                     \
  }

FK_FWD_SB(smkmForwardStridedBatched, float, DType::F32, MMType::MKM,
          (fastKronHandle handle, fastKronBackend backend, uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
           const float* X, fastKronOp opX, uint64_t strideX, const float* const Fs[], fastKronOp opFs,
           uint64_t strideF[], float* Z, uint64_t strideZ, uint32_t batchCount, float* Intermediates[],
           uint64_t strideIntermediates[]))
FK_FWD_SB(dmkmForwardStridedBatched, double, DType::F64, MMType::MKM,
          (fastKronHandle handle, fastKronBackend backend, uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
           const double* X, fastKronOp opX, uint64_t strideX, const double* const Fs[], fastKronOp opFs,
           uint64_t strideF[], double* Z, uint64_t strideZ, uint32_t batchCount, double* Intermediates[],
           uint64_t strideIntermediates[]))
FK_FWD_SB(skmmForwardStridedBatched, float, DType::F32, MMType::KMM,
          (fastKronHandle handle, fastKronBackend backend, uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
           const float* const Fs[], fastKronOp opFs, uint64_t strideF[], const float* X, fastKronOp opX,
           uint64_t strideX, float* Z, uint64_t strideZ, uint32_t batchCount, float* Intermediates[],
           uint64_t strideIntermediates[]))
FK_FWD_SB(dkmmForwardStridedBatched, double, DType::F64, MMType::KMM,
          (fastKronHandle handle, fastKronBackend backend, uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
           const double* const Fs[], fastKronOp opFs, uint64_t strideF[], const double* X, fastKronOp opX,
           uint64_t strideX, double* Z, uint64_t strideZ, uint32_t batchCount, double* Intermediates[],
           uint64_t strideIntermediates[]))

}  // extern "C"
