// sgemkmStaticScratch: sgemkm for callers that cannot allocate device memory (code under HIP graph capture, tight
// serving loops, harnesses that forbid hipMalloc).  sgemkm takes two temporaries from its caller and the
// merged-factor workspace from the handle; here all three live in one file-scope device array that every GPU holds
// from the moment the library is loaded until the process ends.  The call allocates nothing and frees nothing.
//
// Layout of the array: [temp1 | temp2 | merged factors], each part 256-byte aligned.  The array keeps whatever the
// previous call left in it; nothing in it has to start at zero (a temporary is written in full by the launch that
// precedes its first reader, the merged factors by the merge launch).  All calls on one GPU share the array:
// two calls that overlap on one GPU (different streams, different handles) race.
#include <hip/hip_runtime.h>

#include <atomic>
#include <cstdio>

#include "../../include/fastkron.h"
#include "../../include/fastkron_ext.h"
#include "handle.h"
#include "kernels/launch.h"

namespace fk {

constexpr size_t kStaticTempBytes = FASTKRON_STATIC_SCRATCH_TEMP_BYTES;           // each of the two temporaries
constexpr size_t kStaticMergeBytes = (size_t)kMaxMergeGroups * 64 * 64 * sizeof(double);
constexpr size_t kStaticScratchBytes = 2 * kStaticTempBytes + kStaticMergeBytes;

static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

// In host code `scratch` is only a handle for the symbol; the array's address on a GPU comes from
// hipGetSymbolAddress with that GPU current, and every GPU has its own copy at its own address.
static std::atomic<void*> scratchOnDevice[kMaxDevices];

hipError_t staticScratchForCurrentDevice(void** out) {
  int d = 0;
  hipError_t e = hipGetDevice(&d);
  if (e != hipSuccess) return e;
  if (d < 0 || d >= kMaxDevices) return hipErrorInvalidDevice;
  void* p = scratchOnDevice[d].load(std::memory_order_acquire);
  if (!p) {
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    if (!p) return hipErrorInvalidSymbol;
    scratchOnDevice[d].store(p, std::memory_order_release);
  }
  *out = p;
  return hipSuccess;
}

}  // namespace fk

using namespace fk;

extern "C" fastKronError sgemkmStaticScratch(fastKronHandle handle, fastKronBackend backend, uint32_t M, uint32_t N,
                                             uint32_t Ps[], uint32_t Qs[], const float* X, fastKronOp opX,
                                             const float* const Fs[], fastKronOp opFs, float* Z, float alpha,
                                             float beta, const float* Y) {
  if (!handle) return fastKronInvalidArgument;
  if (N == 0 || N > kMaxFactors || !Ps || !Qs || !Fs) return fastKronInvalidKMMProblem;
  Handle* h = (Handle*)handle;
  size_t yElems = 0, tmpElems = 0;
  fastKronError e = Handle::sizes(M, N, Ps, Qs, &yElems, &tmpElems);
  if (e != fastKronSuccess) return e;
  if (tmpElems > kStaticTempBytes / sizeof(float)) {
    fprintf(stderr, "[fastkron] sgemkmStaticScratch: this problem needs temporaries of %zu bytes each, the static scratch "
                    "holds %zu; use sgemkm with temporaries of the caller's own\n",
            tmpElems * sizeof(float), kStaticTempBytes);
    return fastKronInvalidArgument;
  }
  void* base = nullptr;
  if (h->planOnly()) base = (void*)(uintptr_t)0x7e0000000000ull;              // nothing is launched in that mode
  else if (staticScratchForCurrentDevice(&base) != hipSuccess) return fastKronBackendNotAvailable;

  KronProblem p{};
  p.mm = MMType::MKM; p.dt = DType::F32; p.M = M; p.N = N;
  for (uint32_t i = 0; i < N; i++) { p.P[i] = Ps[i]; p.Q[i] = Qs[i]; p.F[i] = Fs[i]; }
  p.X = X; p.opX = opX; p.opF = opFs; p.Z = Z; p.Y = Y;
  p.alpha = alpha; p.beta = beta; p.batch = 1;
  Handle::CallWorkspace ws{(char*)base + 2 * kStaticTempBytes, kStaticMergeBytes};
  return h->xgemm(p, backend, base, (char*)base + kStaticTempBytes, &ws);
}
