// Problem and launch descriptors shared by the planner, the kernel database and the kernels.
//
// A Kronecker-matrix product is run as a series of launches, each applying a contiguous group of
// factors (last factor first, as reference src/kmm/kmmalgo.cpp:172-214 does).  Both GeMKM and GeKMM
// are expressed on one canonical view: an operand is a set of M independent "rows" of `cols`
// elements, element (m, c) living at base + m*ldm + c*ldc.  MKM row-major has ldm = cols, ldc = 1;
// KMM (a cols x M row-major buffer) has ldm = 1, ldc = M; opX = T swaps the two for the first launch.
#pragma once
#include <cstdint>
#include <cstddef>
#include <string>
#include <vector>

namespace fk {

constexpr uint32_t kMaxFactors = 64;   // reference src/kmm/kmmalgo.h:336
constexpr uint32_t kMaxFused   = 8;

enum class MMType : int { MKM = 0, KMM = 1 };
enum class DType  : int { F32 = 0, F64 = 1 };

inline size_t dtypeSize(DType t) { return t == DType::F32 ? 4 : 8; }

struct KronProblem {
  MMType   mm;
  DType    dt;
  uint32_t M, N;
  uint32_t P[kMaxFactors], Q[kMaxFactors];
  const void* X;  int opX;  uint64_t strideX;
  const void* F[kMaxFactors]; int opF; uint64_t strideF[kMaxFactors];
  void* Z;        uint64_t strideZ;
  const void* Y;  uint64_t strideY;
  double alpha, beta;
  uint32_t batch;
  bool strided;                       // came in through a *StridedBatched entry point
  bool forward;                       // keep every step's output (forward family)
  void* inter[kMaxFactors];           // forward only: inter[j] = output of the step of factor j+1
  uint64_t strideInter[kMaxFactors];
  bool haveStrideInter;
  // Set for the parts of a call that the library runs as problems of their own: X was written by a launch of this
  // call just before (a transposed copy, the first part of a two-part plan) / Z is read by the next launch.
  bool xJustWritten, zReadNext;

  uint64_t K() const { uint64_t k = 1; for (uint32_t i = 0; i < N; i++) k *= P[i]; return k; }
  uint64_t L() const { uint64_t l = 1; for (uint32_t i = 0; i < N; i++) l *= Q[i]; return l; }
  // columns of the matrix that enters the step of factor i (i = N-1 is X itself)
  uint64_t colsBefore(uint32_t i) const {
    uint64_t w = K();
    for (uint32_t j = N - 1; j > i; j--) w = (w / P[j]) * Q[j];
    return w;
  }
  uint64_t colsAfter(uint32_t i) const { return (colsBefore(i) / P[i]) * Q[i]; }
  uint64_t flop() const {             // reference src/kmm/kmmalgo.h:174-184 (x batch, :479-481)
    uint64_t ops = 0, kk = K();
    for (int i = (int)N - 1; i >= 0; i--) { kk = (kk / P[i]) * Q[i]; ops += kk * P[i]; }
    return 2ull * M * ops * batch;
  }
  bool sameShapes(uint32_t lo, uint32_t hi) const {
    for (uint32_t i = lo + 1; i <= hi; i++) if (P[i] != P[lo] || Q[i] != Q[lo]) return false;
    return true;
  }
  std::string str() const;            // reference problem-string grammar, src/kmm/kmmalgo.h:304-328
};

// Arguments of one launch.  f[0] is the factor applied first (the highest-numbered one of the group).
struct StepArgs {
  const void* in;  void* out;  const void* y;
  const void* f[kMaxFused];
  uint64_t f_batch[kMaxFused];
  int64_t  f_sp[kMaxFused], f_sq[kMaxFused];   // element (p, q) of factor i at f[i] + p*f_sp + q*f_sq
  uint32_t p[kMaxFused], q[kMaxFused];
  uint32_t nf;
  uint32_t M, batch;
  uint64_t Kin, Kout;
  int64_t  in_ldm, in_ldc, out_ldm, out_ldc, y_ldm, y_ldc;
  uint64_t in_batch, out_batch, y_batch;
  double   alpha, beta;
  uint32_t epilogue;                   // 1: out = alpha*acc + beta*y (beta term skipped when y is null)
  // Hints for the kernels that have non-temporal variants: the input is large and was not written just before by
  // a launch of this call / the output is large and no launch of this call reads it back (or it is larger than
  // the memory-side cache anyway).  Such data gains nothing from being kept in the caches.
  uint32_t stream_in, stream_out;
  // A temporary of the call that this launch neither reads nor writes (null when there is none), for kernels that
  // pass an intermediate through memory inside one launch, and a small zero-initialised counter area of the handle
  // (null for calls that must not touch the handle's device memory).
  void*    scratch;
  uint64_t scratch_elems;
  void*    sync;
};

// Merging of adjacent small factors into their Kronecker product (kernels/merge_factors.hip).
constexpr uint32_t kMaxMergeGroups = 16;   // merged factors per call
constexpr uint32_t kMaxMergeSources = 6;   // factors per merged factor (six 2x2 make a 64x64)

struct MergeGroup {
  const void* src[kMaxMergeSources];
  int64_t  sp[kMaxMergeSources], sq[kMaxMergeSources];   // element (p, q) of source j at src[j] + p*sp + q*sq
  uint32_t p[kMaxMergeSources], q[kMaxMergeSources];
  uint32_t count;
  void*    dst;
  int64_t  dsp, dsq;                                     // element (p, q) of the product at dst + p*dsp + q*dsq
};

struct MergeArgs {
  MergeGroup g[kMaxMergeGroups];
  uint32_t groups;
};

}  // namespace fk
