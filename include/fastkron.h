/*
 * fastkron.h -- C ABI of the MI355X (gfx950) Kronecker-matrix multiplication library.
 *
 * Every declaration below is binary compatible with the FastKron public header
 * (reference include/fastkron.h): same enum values, same opaque handle type, same
 * symbol names, argument order and argument types.  A program or binding compiled
 * against the reference header links against this library unchanged.  The reference
 * line each declaration replaces is cited next to it.
 *
 * Conventions (reference include/fastkron.h:206-231):
 *   GeMKM   Z = alpha * op(X) * (op(F1) (x) ... (x) op(FN)) + beta * Y
 *           op(X) is M x K row-major, K = prod(Ps); op(Fi) is Ps[i] x Qs[i]; Y, Z are M x L, L = prod(Qs).
 *   GeKMM   Z = alpha * (op(F1) (x) ... (x) op(FN)) * op(X) + beta * Y
 *           op(X) is K x M row-major; op(Fi) is Qs[i] x Ps[i]; Y, Z are L x M.
 *   fastKronOp_T means the buffer holds the transpose of the operand (a column-major view).
 *   All device pointers are HBM addresses of the current HIP device; calls are asynchronous on
 *   the stream given to fastKronInitHIP / fastKronSetStream and never synchronise.
 */
#pragma once

#include <stdint.h>
#include <stddef.h>
#ifdef __cplusplus
#include <cstdio>
#include <cstdlib>
#else
#include <stdio.h>
#include <stdlib.h>
#endif

/* reference include/fastkron.h:6-13 */
#define FastKronCHECK(cmd) do {                                          \
  fastKronError e_ = (cmd);                                              \
  if (e_ != fastKronSuccess) {                                           \
    printf("Failed: FastKron error %s:%d at %s:%d \n",                   \
           fastKronGetErrorString(e_), (int)e_, __FILE__, __LINE__);     \
    exit(EXIT_FAILURE);                                                  \
  }                                                                      \
} while (0)

/* reference include/fastkron.h:27-30 */
enum fastKronOp {
  fastKronOp_N = 1,   /* buffer is the row-major operand */
  fastKronOp_T = 2    /* buffer is the row-major transpose of the operand */
};

/* reference include/fastkron.h:41-47 */
enum fastKronBackend {
  fastKronBackend_NONE = 1 << 0,
  fastKronBackend_X86  = 1 << 1,
  fastKronBackend_ARM  = 1 << 2,
  fastKronBackend_CUDA = 1 << 3,
  fastKronBackend_HIP  = 1 << 4   /* the only backend this library is built with */
};

/* reference include/fastkron.h:57-61 */
enum fastKronOptions {
  fastKronOptionsNone      = 1 << 0,
  fastKronOptionsUseFusion = 1 << 1,  /* allow several factors per launch (always set at init) */
  fastKronOptionsTune      = 1 << 2   /* time candidate launch plans on first use of a problem */
};

/* reference include/fastkron.h:74-82 */
enum fastKronError {
  fastKronSuccess             = 0,
  fastKronBackendNotAvailable = 1,
  fastKronInvalidMemoryAccess = 2,
  fastKronKernelNotFound      = 3,
  fastKronInvalidArgument     = 4,
  fastKronInvalidKMMProblem   = 5,
  fastKronOtherError          = 6
};

#ifdef __cplusplus
extern "C" {
#else
typedef enum fastKronOp fastKronOp;
typedef enum fastKronBackend fastKronBackend;
typedef enum fastKronError fastKronError;
#endif

typedef void* fastKronHandle;                                   /* reference :85 */

/* ---- library information (reference :95-116) ---- */
const char* fastKronVersion(void);                              /* :95  "1.1.0+gfx950" style string */
const char* fastKronCUDAArchs(void);                            /* :101 always NULL, as in the reference */
const char* fastKronGetErrorString(fastKronError err);          /* :109 */
uint32_t    fastKronGetBackends(void);                          /* :116 == fastKronBackend_HIP */

/* ---- handle life cycle (reference :126-204) ---- */
fastKronError fastKronInit(fastKronHandle* handle, uint32_t backends);           /* :126 */
fastKronError fastKronInitAllBackends(fastKronHandle* handle);                   /* :137 */
fastKronError fastKronSetOptions(fastKronHandle handle, uint32_t options);       /* :146 */
void          fastKronDestroy(fastKronHandle handle);                            /* :158 */
fastKronError fastKronInitCUDA(fastKronHandle handle, void* ptrToStream);        /* :170 BackendNotAvailable here */
fastKronError fastKronInitHIP(fastKronHandle handle, void* ptrToStream);         /* :183 ptr to a hipStream_t, NULL = default stream */
fastKronError fastKronInitX86(fastKronHandle handle);                            /* :194 BackendNotAvailable here */
fastKronError fastKronSetStream(fastKronHandle handle, fastKronBackend backend,
                                void* ptrToStream);                              /* :204 */

/* ---- buffer sizes, in elements (reference :249) ---- */
fastKronError gekmmSizes(fastKronHandle handle, uint32_t M, uint32_t N,
                         uint32_t Ps[], uint32_t Qs[],
                         size_t* yElems, size_t* tmpElems);

/* ---- GeMKM (reference :284-296) ---- */
fastKronError sgemkm(fastKronHandle handle, fastKronBackend backend,
                     uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
                     const float* X, fastKronOp opX,
                     const float* const Fs[], fastKronOp opFs,
                     float* Z, float alpha, float beta,
                     const float* Y, float* temp1, float* temp2);

fastKronError dgemkm(fastKronHandle handle, fastKronBackend backend,
                     uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
                     const double* X, fastKronOp opX,
                     const double* const Fs[], fastKronOp opFs,
                     double* Z, double alpha, double beta,
                     const double* Y, double* temp1, double* temp2);

/* ---- GeKMM (reference :329-341); note the Qs-before-Ps and factors-before-X order ---- */
fastKronError sgekmm(fastKronHandle handle, fastKronBackend backend,
                     uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
                     const float* const Fs[], fastKronOp opFs,
                     const float* X, fastKronOp opX,
                     float* Z, float alpha, float beta,
                     const float* Y, float* temp1, float* temp2);

fastKronError dgekmm(fastKronHandle handle, fastKronBackend backend,
                     uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
                     const double* const Fs[], fastKronOp opFs,
                     const double* X, fastKronOp opX,
                     double* Z, double alpha, double beta,
                     const double* Y, double* temp1, double* temp2);

/* ---- strided-batched GeMKM (reference :384-398); strides in elements, 0 = shared by all batches ---- */
fastKronError sgemkmStridedBatched(fastKronHandle handle, fastKronBackend backend,
                                   uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
                                   const float* X, fastKronOp opX, uint64_t strideX,
                                   const float* const Fs[], fastKronOp opFs, uint64_t strideF[],
                                   float* Z, uint64_t strideZ, float alpha, float beta,
                                   uint32_t batchCount, const float* Y, uint64_t strideY,
                                   float* temp1, float* temp2);

fastKronError dgemkmStridedBatched(fastKronHandle handle, fastKronBackend backend,
                                   uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
                                   const double* X, fastKronOp opX, uint64_t strideX,
                                   const double* const Fs[], fastKronOp opFs, uint64_t strideF[],
                                   double* Z, uint64_t strideZ, double alpha, double beta,
                                   uint32_t batchCount, const double* Y, uint64_t strideY,
                                   double* temp1, double* temp2);

/* ---- strided-batched GeKMM (reference :435-449) ---- */
fastKronError sgekmmStridedBatched(fastKronHandle handle, fastKronBackend backend,
                                   uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
                                   const float* const Fs[], fastKronOp opFs, uint64_t strideF[],
                                   const float* X, fastKronOp opX, uint64_t strideX,
                                   float* Z, uint64_t strideZ, float alpha, float beta,
                                   uint32_t batchCount, const float* Y, uint64_t strideY,
                                   float* temp1, float* temp2);

fastKronError dgekmmStridedBatched(fastKronHandle handle, fastKronBackend backend,
                                   uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
                                   const double* const Fs[], fastKronOp opFs, uint64_t strideF[],
                                   const double* X, fastKronOp opX, uint64_t strideX,
                                   double* Z, uint64_t strideZ, double alpha, double beta,
                                   uint32_t batchCount, const double* Y, uint64_t strideY,
                                   double* temp1, double* temp2);

/* ---- forward family: alpha = 1, beta = 0, every step's output is kept (reference :470-628).
 *      Intermediates[j], j = 0..N-2, receives the output of the step that multiplies factor j+1,
 *      an M x (K * prod_{i>j} Qs[i] / prod_{i>j} Ps[i]) matrix (transposed for KMM). ---- */
fastKronError gekmmSizesForward(fastKronHandle handle, uint32_t M, uint32_t N,
                                uint32_t Ps[], uint32_t Qs[],
                                size_t* yElems, size_t* intermediateElems);                /* :470 */

fastKronError smkmForward(fastKronHandle handle, fastKronBackend backend,
                          uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
                          const float* X, fastKronOp opX,
                          const float* const Fs[], fastKronOp opFs,
                          float* Z, float* Intermediates[]);                               /* :497 */

fastKronError dmkmForward(fastKronHandle handle, fastKronBackend backend,
                          uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
                          const double* X, fastKronOp opX,
                          const double* const Fs[], fastKronOp opFs,
                          double* Z, double* Intermediates[]);                             /* :503 */

fastKronError skmmForward(fastKronHandle handle, fastKronBackend backend,
                          uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
                          const float* const Fs[], fastKronOp opFs,
                          const float* X, fastKronOp opX,
                          float* Z, float* Intermediates[]);                               /* :533 */

fastKronError dkmmForward(fastKronHandle handle, fastKronBackend backend,
                          uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
                          const double* const Fs[], fastKronOp opFs,
                          const double* X, fastKronOp opX,
                          double* Z, double* Intermediates[]);                             /* :539 */

fastKronError smkmForwardStridedBatched(fastKronHandle handle, fastKronBackend backend,
                                        uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
                                        const float* X, fastKronOp opX, uint64_t strideX,
                                        const float* const Fs[], fastKronOp opFs, uint64_t strideF[],
                                        float* Z, uint64_t strideZ, uint32_t batchCount,
                                        float* Intermediates[], uint64_t strideIntermediates[]);   /* :574 */

fastKronError dmkmForwardStridedBatched(fastKronHandle handle, fastKronBackend backend,
                                        uint32_t M, uint32_t N, uint32_t Ps[], uint32_t Qs[],
                                        const double* X, fastKronOp opX, uint64_t strideX,
                                        const double* const Fs[], fastKronOp opFs, uint64_t strideF[],
                                        double* Z, uint64_t strideZ, uint32_t batchCount,
                                        double* Intermediates[], uint64_t strideIntermediates[]);  /* :581 */

fastKronError skmmForwardStridedBatched(fastKronHandle handle, fastKronBackend backend,
                                        uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
                                        const float* const Fs[], fastKronOp opFs, uint64_t strideF[],
                                        const float* X, fastKronOp opX, uint64_t strideX,
                                        float* Z, uint64_t strideZ, uint32_t batchCount,
                                        float* Intermediates[], uint64_t strideIntermediates[]);   /* :616 */

fastKronError dkmmForwardStridedBatched(fastKronHandle handle, fastKronBackend backend,
                                        uint32_t N, uint32_t Qs[], uint32_t Ps[], uint32_t M,
                                        const double* const Fs[], fastKronOp opFs, uint64_t strideF[],
                                        const double* X, fastKronOp opX, uint64_t strideX,
                                        double* Z, uint64_t strideZ, uint32_t batchCount,
                                        double* Intermediates[], uint64_t strideIntermediates[]);  /* :623 */

#ifdef __cplusplus
}
#endif
