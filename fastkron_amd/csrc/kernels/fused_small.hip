// Several small factors of any shape (P <= 8, any Q) in one launch: the fused sliced multiply for the shapes the
// matrix-core kernels do not take (3x3, 5x5, 6x6, 7x5 ..., 2x2 where merging does not apply), MKM or KMM layout,
// fp32 or fp64.
//
// A group of nf adjacent factors acts on the matrix like one sliced multiply with their Kronecker product G
// (Pg x Qg, Pg = prod P_j, Qg = prod Q_j):
//
//   out[m, qd*U + u] = sum_kd in[m, u*Pg + kd] * G[kd, qd],   U = Kin / Pg
//
// A workgroup takes TM rows x TU consecutive u: a contiguous piece of TU*Pg input columns per row (MKM) or TM
// consecutive rows of the same columns (KMM).  The piece goes to LDS once, the nf factors are applied to it one
// after the other between two LDS buffers, each as the small sliced multiply
//
//   dst[q*A + a] = sum_p src[a*P + p] * F[p, q]
//
// and the result is written with runs of TU (MKM) or TM (KMM) contiguous elements: HBM is read once and written
// once for nf factors.  The factor values are the same for every lane, so they are fetched through the scalar
// data path into SGPRs (read only) and enter the FMAs as scalar operands: the inner loop reads P values from
// LDS, does P*Q FMAs and writes Q values.
//
// This is the reference's central idea, fusing factors in shared memory (reference src/kernels/cuda/kernel.cuh:
// 165-219, tile choice in src/kernel_db/kernel_db.cpp:152-290); tile shapes, the two layouts in one kernel, the
// scalar factor operands and the power-of-two tiles with ragged edges are this kernel's own.
// Algorithmic traffic per launch: read M*Kin, write M*Kout elements (+ M*Kout for Y when it writes Z).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

constexpr int kFsThreads = 512;
constexpr uint32_t kFsMaxP = 8;             // larger factors run faster one at a time on the matrix cores
constexpr size_t kFsBufBytes = 32768;        // per LDS buffer; two buffers: two workgroups fit a CU (measured best)

struct FusedTile {
  uint32_t TM, TU, tmShift, tuShift;         // rows and slices per workgroup, both powers of two
  uint32_t U, uTiles, mTiles;
  uint32_t Pg, Qg;
  uint32_t E0, Ef, magicE0, magicEf;         // per-row piece lengths before / after the group: TU*Pg, TU*Qg
  uint32_t A[kMaxFused], magicA[kMaxFused];  // per-row slice count of step j: (piece length before step j) / P_j
  uint32_t bufElems;
};

// floor(x / d) = mulhi(x, magic) for x < 65536 * d, d < 65536
static uint32_t fsMagic(uint32_t d) { return d <= 1 ? 0u : (uint32_t)((1ull << 32) / d) + 1u; }
__device__ __forceinline__ uint32_t fsDiv(uint32_t x, uint32_t d, uint32_t magic) {
  return d == 1 ? x : __umulhi(x, magic);
}

// How a tile is laid out in LDS: [piece] of one row (MKM, TM = 1), [row][piece] (MKM, TM > 1: slices are numbered
// through the rows and the row of a slice is found by division), or [piece][row] (KMM, TM rows innermost).
enum FsMode : int { kFsOneRow = 0, kFsRows = 1, kFsKmm = 2 };

// UNR slices of one thread (sl, sl + threads, ...): NQ output columns each.  All LDS reads are issued before the
// first FMA.  Integer multiplies are slow on this hardware; the addresses are kept as running sums instead.
template <typename T, int P, int NQ, int UNR, int MODE, bool PRED>
__device__ __forceinline__ void fsPass(const T* __restrict__ src, T* __restrict__ dst, const T (&Fr)[P][NQ],
                                       const uint32_t sl, const uint32_t inb, const uint32_t outb,
                                       const uint32_t strideP, const uint32_t strideQ, const uint32_t rowExtra,
                                       const uint32_t A, const uint32_t magicA, const uint32_t nsl) {
  T x[UNR][P];
#pragma unroll
  for (int u = 0; u < UNR; u++) {
    if (PRED && sl + u * kFsThreads >= nsl) continue;
#pragma unroll
    for (int pp = 0; pp < P; pp++) x[u][pp] = src[inb + u * (kFsThreads * P) + pp * strideP];
  }
#pragma unroll
  for (int u = 0; u < UNR; u++) {
    if (PRED && sl + u * kFsThreads >= nsl) continue;
    uint32_t ob = outb + u * kFsThreads;
    if (MODE == kFsRows) ob += fsDiv(sl + u * kFsThreads, A, magicA) * rowExtra;
#pragma unroll
    for (int tq = 0; tq < NQ; tq++) {
      T acc = x[u][0] * Fr[0][tq];
#pragma unroll
      for (int pp = 1; pp < P; pp++) acc += x[u][pp] * Fr[pp][tq];
      dst[ob + tq * strideQ] = acc;
    }
  }
}

// NQ output columns (q0 .. q0+NQ-1) of one local step on the whole tile: dst[q*A + a] = sum_p src[a*P + p] F[p][q]
// per row (MKM) or the same with every element standing for TM rows (KMM).
template <typename T, int P, int NQ, int MODE>
__device__ __forceinline__ void fsColumns(const T* __restrict__ src, T* __restrict__ dst, const T* F, const int64_t sp,
                                          const int64_t sq, const uint32_t q0, const uint32_t Q, const uint32_t A,
                                          const uint32_t magicA, const uint32_t nsl, const uint32_t ishift,
                                          const uint32_t tid) {
  // the factor is read-only for the whole launch and its address is the same in every lane: the constant
  // address space makes these scalar loads, and the values enter the FMAs as scalar operands
  typedef const __attribute__((address_space(4))) T* ConstPtr;
  const ConstPtr Fc = (ConstPtr)(uintptr_t)F;
  T Fr[P][NQ];
#pragma unroll
  for (int pp = 0; pp < P; pp++)
#pragma unroll
    for (int tq = 0; tq < NQ; tq++) Fr[pp][tq] = Fc[(int64_t)pp * sp + (int64_t)(q0 + tq) * sq];
  const uint32_t strideP = MODE == kFsKmm ? (1u << ishift) : 1u;
  const uint32_t strideQ = MODE == kFsKmm ? (A << ishift) : A;
  const uint32_t rowExtra = (Q - 1) * A;           // kFsRows: output rows are Q*A apart, slice numbers only A
  constexpr int UNR = (P * (int)sizeof(T) <= 32) ? 4 : 2;
  // slice sl = tid + k*threads: the input offset of slice sl is sl*P (MKM) or, with the TM rows innermost and
  // threads a multiple of TM, (sl / TM)*P*TM + sl % TM (KMM); both advance by threads*P per k
  uint32_t inb = MODE == kFsKmm ? (tid >> ishift) * ((uint32_t)P << ishift) + (tid & (strideP - 1)) : tid * P;
  uint32_t outb = tid + q0 * strideQ;
  uint32_t sl = tid;
  // passes of UNR slices per thread while every one of them exists, then single slices, the last pass predicated
  uint32_t done = 0;                                // slices below `done` are finished (same in all threads)
  for (; done + UNR * kFsThreads <= nsl; done += UNR * kFsThreads) {
    fsPass<T, P, NQ, UNR, MODE, false>(src, dst, Fr, sl, inb, outb, strideP, strideQ, rowExtra, A, magicA, nsl);
    sl += UNR * kFsThreads; inb += UNR * kFsThreads * P; outb += UNR * kFsThreads;
  }
  for (; done + kFsThreads <= nsl; done += kFsThreads) {
    fsPass<T, P, NQ, 1, MODE, false>(src, dst, Fr, sl, inb, outb, strideP, strideQ, rowExtra, A, magicA, nsl);
    sl += kFsThreads; inb += kFsThreads * P; outb += kFsThreads;
  }
  if (done < nsl)
    fsPass<T, P, NQ, 1, MODE, true>(src, dst, Fr, sl, inb, outb, strideP, strideQ, rowExtra, A, magicA, nsl);
}

// One local step: the Q output columns in passes of at most TQ, P * TQ factor values in scalar registers per pass.
template <typename T, int P, int MODE>
__device__ __forceinline__ void fsLocalStep(const T* __restrict__ src, T* __restrict__ dst, const T* F, const int64_t sp,
                                            const int64_t sq, const uint32_t Q, const uint32_t A,
                                            const uint32_t magicA, const uint32_t nsl, const uint32_t ishift,
                                            const uint32_t tid) {
  constexpr int TQ0 = (sizeof(T) == 4 ? 32 : 16) / P;
  constexpr int TQ = TQ0 > 8 ? 8 : TQ0;
  for (uint32_t q0 = 0; q0 < Q; q0 += TQ) {
    const uint32_t nq = Q - q0 < (uint32_t)TQ ? Q - q0 : (uint32_t)TQ;
#define FS_NQ(N) case N: if constexpr (N <= TQ) fsColumns<T, P, N, MODE>(src, dst, F, sp, sq, q0, Q, A, magicA, nsl, ishift, tid); break;
    switch (nq) {
      FS_NQ(1) FS_NQ(2) FS_NQ(3) FS_NQ(4) FS_NQ(5) FS_NQ(6) FS_NQ(7) FS_NQ(8)
      default: break;
    }
#undef FS_NQ
  }
}

template <typename T, int MODE, bool HAS_Y>
__global__ __launch_bounds__(kFsThreads, 4) void kron_fused_small_kernel(const StepArgs a, const FusedTile t) {
  extern __shared__ __align__(16) unsigned char fsLds[];
  T* const lds = (T*)fsLds;                  // two buffers of t.bufElems elements
  const uint32_t tid = threadIdx.x;
  const uint32_t b = blockIdx.y;
  // workgroups go round-robin over the 8 XCDs: neighbouring tiles, whose output runs share cache lines, are
  // numbered onto the same XCD so that the partial lines meet in its L2
  const uint32_t perXcd = (t.uTiles * t.mTiles + 7) / 8;
  const uint32_t tile = (blockIdx.x & 7) * perXcd + (blockIdx.x >> 3);
  if (tile >= t.uTiles * t.mTiles) return;
  const uint32_t mt = tile / t.uTiles, ut = tile % t.uTiles;
  const uint32_t m0 = mt << t.tmShift, u0 = ut << t.tuShift;
  const T* in = (const T*)a.in + (size_t)b * a.in_batch;
  T* out = (T*)a.out + (size_t)b * a.out_batch;
  const T* y = HAS_Y ? (const T*)a.y + (size_t)b * a.y_batch : nullptr;
  const T alpha = a.epilogue ? (T)a.alpha : T(1), beta = (T)a.beta;
  constexpr int LU = 8;                         // memory operations in flight per thread

  // ---- load: per row the TU*Pg contiguous columns from u0*Pg on.  Elements beyond the matrix are left as they
  //      are: every slice only feeds its own outputs, and those of such slices are not stored. ----
  const uint64_t c0 = (uint64_t)u0 * t.Pg;
  const uint32_t len = (uint32_t)(a.Kin - c0 < t.E0 ? a.Kin - c0 : t.E0);      // columns of the piece inside the matrix
  if (MODE == kFsOneRow) {
    const T* row = in + (int64_t)m0 * a.in_ldm + c0;
    for (uint32_t j0 = tid; j0 < len; j0 += LU * kFsThreads) {
      T v[LU];
#pragma unroll
      for (int k = 0; k < LU; k++) if (j0 + k * kFsThreads < len) v[k] = row[j0 + k * kFsThreads];
#pragma unroll
      for (int k = 0; k < LU; k++) if (j0 + k * kFsThreads < len) lds[j0 + k * kFsThreads] = v[k];
    }
  } else if (MODE == kFsKmm) {
    // e = j*TM + mm with threads a multiple of TM: mm is fixed per thread, j advances by threads/TM
    const uint32_t mm = tid & (t.TM - 1), jStep = kFsThreads >> t.tmShift;
    const bool rowOk = m0 + mm < a.M;
    const T* ptr = in + (m0 + mm) + (int64_t)(c0 + (tid >> t.tmShift)) * a.in_ldc;
    const int64_t pStep = (int64_t)jStep * a.in_ldc;
    for (uint32_t j0 = tid >> t.tmShift; j0 < len; j0 += LU * jStep) {
      T v[LU];
#pragma unroll
      for (int k = 0; k < LU; k++) { if (rowOk && j0 + k * jStep < len) v[k] = *ptr; ptr += pStep; }
#pragma unroll
      for (int k = 0; k < LU; k++)
        if (rowOk && j0 + k * jStep < len) lds[((j0 + k * jStep) << t.tmShift) + mm] = v[k];
    }
  } else {
    const uint32_t nIn = t.E0 << t.tmShift;
    for (uint32_t e0 = tid; e0 < nIn; e0 += LU * kFsThreads) {
      T v[LU];
#pragma unroll
      for (int k = 0; k < LU; k++) {
        const uint32_t e = e0 + k * kFsThreads;
        const uint32_t mm = fsDiv(e, t.E0, t.magicE0), j = e - mm * t.E0;
        v[k] = T(0);
        if (e < nIn && m0 + mm < a.M && j < len) v[k] = in[(int64_t)(m0 + mm) * a.in_ldm + (int64_t)(c0 + j)];
      }
#pragma unroll
      for (int k = 0; k < LU; k++) if (e0 + k * kFsThreads < nIn) lds[e0 + k * kFsThreads] = v[k];
    }
  }
  __syncthreads();

  // ---- the factors, one after the other ----
  for (uint32_t j = 0; j < a.nf; j++) {
    const T* F = (const T*)a.f[j] + (size_t)b * a.f_batch[j];
    const T* src = lds + ((j & 1) ? t.bufElems : 0u);
    T* dst = lds + ((j & 1) ? 0u : t.bufElems);
    const uint32_t nsl = t.A[j] << t.tmShift;
#define FS_CASE(PV) case PV: fsLocalStep<T, PV, MODE>(src, dst, F, a.f_sp[j], a.f_sq[j], a.q[j], t.A[j], t.magicA[j], nsl, t.tmShift, tid); break;
    switch (a.p[j]) {
      FS_CASE(1) FS_CASE(2) FS_CASE(3) FS_CASE(4) FS_CASE(5) FS_CASE(6) FS_CASE(7) FS_CASE(8)
      default: break;
    }
#undef FS_CASE
    __syncthreads();
  }

  // ---- store: the tile holds [qd][uu] per row (MKM) / [qd][uu][row] (KMM); column of (qd, uu) = qd*U + u0 + uu ----
  const T* res = lds + ((a.nf & 1) ? t.bufElems : 0u);
  if (MODE == kFsOneRow) {
    // r = qd*TU + uu with threads a multiple of TU: uu is fixed per thread, qd advances by threads/TU
    const uint32_t uu = tid & (t.TU - 1), qStep = kFsThreads >> t.tuShift;
    const bool ok = u0 + uu < t.U;
    const uint64_t col0 = (uint64_t)(tid >> t.tuShift) * t.U + u0 + uu;
    T* op = out + (int64_t)m0 * a.out_ldm + col0;
    const T* yp = HAS_Y ? y + (int64_t)m0 * a.y_ldm + col0 : nullptr;
    const uint64_t cStep = (uint64_t)qStep * t.U;
    for (uint32_t r0 = tid; r0 < t.Ef; r0 += LU * kFsThreads) {
      T yv[HAS_Y ? LU : 1];
      if (HAS_Y) {
#pragma unroll
        for (int k = 0; k < LU; k++) if (ok && r0 + k * kFsThreads < t.Ef) yv[k] = yp[k * cStep];
      }
#pragma unroll
      for (int k = 0; k < LU; k++) {
        if (!(ok && r0 + k * kFsThreads < t.Ef)) continue;
        T v = res[r0 + k * kFsThreads] * alpha;
        if (HAS_Y) v += beta * yv[k];
        op[k * cStep] = v;
      }
      op += LU * cStep;
      if (HAS_Y) yp += LU * cStep;
    }
  } else {
    const uint32_t nOut = t.Ef << t.tmShift;
    for (uint32_t e0 = tid; e0 < nOut; e0 += LU * kFsThreads) {
      T yv[HAS_Y ? LU : 1];
      int64_t off[LU];
#pragma unroll
      for (int k = 0; k < LU; k++) {
        const uint32_t e = e0 + k * kFsThreads;
        uint32_t mm, r;
        if (MODE == kFsKmm) { mm = e & (t.TM - 1); r = e >> t.tmShift; }
        else                { mm = fsDiv(e, t.Ef, t.magicEf); r = e - mm * t.Ef; }
        const uint32_t uu = r & (t.TU - 1), qd = r >> t.tuShift;
        const uint64_t col = (uint64_t)qd * t.U + u0 + uu;
        const bool ok = e < nOut && m0 + mm < a.M && u0 + uu < t.U;
        off[k] = ok ? (int64_t)(m0 + mm) * a.out_ldm + (int64_t)col * a.out_ldc : -1;
        if (HAS_Y) yv[k] = ok ? y[(int64_t)(m0 + mm) * a.y_ldm + (int64_t)col * a.y_ldc] : T(0);
      }
#pragma unroll
      for (int k = 0; k < LU; k++) {
        if (off[k] < 0) continue;
        T v = res[e0 + k * kFsThreads] * alpha;
        if (HAS_Y) v += beta * yv[k];
        out[off[k]] = v;
      }
    }
  }
}

static uint32_t fsPow2Ceil(uint64_t v) { uint32_t r = 1; while (r < v && r < (1u << 30)) r <<= 1; return r; }
static uint32_t fsLog2(uint32_t v) { uint32_t s = 0; while ((1u << s) < v) s++; return s; }

// Tile for a group of factors (p[0], q[0] is the one applied first); false when the group does not fit the LDS
// buffers with runs long enough to use the memory system well.
static bool fusedSmallTile(uint32_t nf, const uint32_t* p, const uint32_t* q, uint64_t Kin, uint32_t M, bool kmm, DType dt,
                    FusedTile* t) {
  if (nf < 1 || nf > kMaxFused) return false;
  uint64_t Pg = 1, Qg = 1, e = 1, emax = 1;
  for (uint32_t j = 0; j < nf; j++) {
    if (p[j] == 0 || p[j] > kFsMaxP || q[j] == 0) return false;
    Pg *= p[j]; Qg *= q[j];
    if (Pg > 65536 || Qg > 65536) return false;
  }
  if (Kin % Pg) return false;
  const uint64_t U = Kin / Pg;
  if (U >= (1ull << 31)) return false;
  e = emax = Pg;
  for (uint32_t j = 0; j < nf; j++) { e = e / p[j] * q[j]; if (e > emax) emax = e; }
  const uint64_t cap = kFsBufBytes / dtypeSize(dt);
  if (emax > cap) return false;
  uint32_t TM, TU;
  if (kmm) {
    // rows are the contiguous dimension: 32 of them (128 bytes in fp32) per run, fewer only for a narrow matrix
    TM = M >= 32 ? 32 : fsPow2Ceil(M);
    while (TM > 8 && (uint64_t)TM * emax > cap) TM >>= 1;
    if ((uint64_t)TM * emax > cap) return false;
    if (TM < 16 && TM < fsPow2Ceil(M)) return false;
    TU = 1;
    while ((uint64_t)TM * (TU * 2) * emax <= cap && TU * 2 <= fsPow2Ceil(U) && TU < 64) TU <<= 1;
  } else {
    TU = U >= 32 ? 32 : fsPow2Ceil(U);
    while (TU > 1 && (uint64_t)TU * emax > cap) TU >>= 1;
    // runs of fewer than 16 elements waste most of every memory transaction
    if (TU < 16 && TU < fsPow2Ceil(U)) return false;
    // longer runs first (one row per workgroup keeps the addressing simple), then more rows
    while ((uint64_t)(TU * 2) * emax <= cap && TU * 2 <= fsPow2Ceil(U) && TU < 256) TU <<= 1;
    TM = 1;
    while ((uint64_t)(TM * 2) * TU * emax <= cap && TM * 2 <= fsPow2Ceil(M) && TM < 64) TM <<= 1;
  }
  if ((uint64_t)TM * TU * emax >= 65536) return false;        // 16-bit slice numbers for the division by multiplication
  t->TM = TM; t->TU = TU; t->tmShift = fsLog2(TM); t->tuShift = fsLog2(TU);
  t->U = (uint32_t)U; t->uTiles = (uint32_t)((U + TU - 1) / TU); t->mTiles = (M + TM - 1) / TM;
  t->Pg = (uint32_t)Pg; t->Qg = (uint32_t)Qg;
  t->E0 = (uint32_t)(TU * Pg); t->Ef = (uint32_t)(TU * Qg);
  t->magicE0 = fsMagic(t->E0); t->magicEf = fsMagic(t->Ef);
  e = (uint64_t)TU * Pg;
  for (uint32_t j = 0; j < nf; j++) {
    t->A[j] = (uint32_t)(e / p[j]);
    t->magicA[j] = fsMagic(t->A[j]);
    e = e / p[j] * q[j];
  }
  t->bufElems = (uint32_t)((uint64_t)TM * TU * emax);
  return (uint64_t)t->uTiles * t->mTiles < (1ull << 31);
}

bool fusedSmallFits(uint32_t nf, const uint32_t* p, const uint32_t* q, uint64_t Kin, uint32_t M, bool kmm, DType dt) {
  FusedTile t;
  return fusedSmallTile(nf, p, q, Kin, M, kmm, dt, &t);
}

static bool fsIsKmm(const StepArgs& a) { return a.in_ldm == 1 && a.in_ldc != 1; }

bool fusedSmallSupported(const StepArgs& a, DType dt) {
  if (a.batch > 65535 || a.M == 0) return false;
  const bool kmm = fsIsKmm(a);
  // one layout for the input, the output and Y: rows contiguous (KMM) or columns contiguous (MKM)
  if (kmm) { if (a.out_ldm != 1 || (a.y && a.y_ldm != 1)) return false; }
  else     { if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false; }
  FusedTile t;
  return fusedSmallTile(a.nf, a.p, a.q, a.Kin, a.M, kmm, dt, &t);
}

template <typename T>
static hipError_t launchFusedSmallT(const StepArgs& a, const FusedTile& t, bool kmm, hipStream_t stream) {
  dim3 grid((t.uTiles * t.mTiles + 7) / 8 * 8, a.batch), block(kFsThreads);
  const size_t lds = 2 * (size_t)t.bufElems * sizeof(T);
  const bool y = a.y && a.epilogue;
  const int mode = kmm ? kFsKmm : (t.TM == 1 ? kFsOneRow : kFsRows);
#define FS_LAUNCH(MODE) \
  if (y) hipLaunchKernelGGL((kron_fused_small_kernel<T, MODE, true>), grid, block, lds, stream, a, t); \
  else   hipLaunchKernelGGL((kron_fused_small_kernel<T, MODE, false>), grid, block, lds, stream, a, t);
  if (mode == kFsKmm) { FS_LAUNCH(kFsKmm) }
  else if (mode == kFsOneRow) { FS_LAUNCH(kFsOneRow) }
  else { FS_LAUNCH(kFsRows) }
#undef FS_LAUNCH
  return hipGetLastError();
}

hipError_t launchFusedSmall(const StepArgs& a, DType dt, hipStream_t stream) {
  if (!fusedSmallSupported(a, dt)) return hipErrorInvalidValue;
  const bool kmm = fsIsKmm(a);
  FusedTile t;
  if (!fusedSmallTile(a.nf, a.p, a.q, a.Kin, a.M, kmm, dt, &t)) return hipErrorInvalidValue;
  return dt == DType::F32 ? launchFusedSmallT<float>(a, t, kmm, stream) : launchFusedSmallT<double>(a, t, kmm, stream);
}

}  // namespace fk
