// One sliced-multiply step with a factor of any shape up to 256 x 512 on the matrix cores, fp32 or fp64, MKM or
// KMM layout, opX = T included: the sizes between the specialised kernels (24x24, 31x63, 50x50, 8x32, 100x100,
// 200x200 ...).
//
//   out[m, q*S + s] = sum_p in[m, s*P + p] * F[p, q],   S = Kin / P
//
// The factor is padded with zeros to 4*pc rows (pc = ceil(P/4)) and 16*qb columns (qb = ceil(Q/16)) and staged in
// LDS once per workgroup.  A tile is 16 lanes wide along the dimension that is contiguous in the output (slices of
// one row in the MKM layout, rows of one slice in the KMM layout) and is computed transposed,
// D[q][j] = sum_p F^T[q][p] * X^T[p][j], with V_MFMA_*_16X16X4:
//   * B operand (lane = 16*k + j): lane group k covers the contraction indices p = k*pc + c, c < pc, so a lane
//     reads pc elements that are consecutive in memory in the MKM layout; indices beyond P read as zero;
//   * A operand (lane = 16*k + q): F[k*pc + c][16*ib + q] from LDS, one read per product (the k groups are offset
//     by 16 elements so that the four groups hit different banks);
//   * the accumulator rows are output columns q: every quarter wave stores 16 consecutive elements.
// Waves are persistent and load the next tile before computing the current one.  pc is a runtime value below
// the template bound PCMAX (4 ... 64): the product loops are unrolled to PCMAX with wave-uniform guards.  A factor
// whose padded copy does not fit 64 KB of LDS is split into slabs of output columns, one slab per workgroup
// (grid z); the slabs of a tile re-read its input through the caches.
//
// Plays the role of the reference's generated kernels for arbitrary factor shapes (reference
// src/kernels/cuda/kernel.cuh:53-224, which computes on CUDA cores, and src/gen_tuner_kernels.py which instantiates
// one kernel per shape); one kernel with zero padding is this library's way.
// Algorithmic traffic per launch: read M*Kin, write M*Kout elements (+ M*Kout for Y on the launch that writes Z).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef double sad4 __attribute__((ext_vector_type(4)));
typedef float saf4 __attribute__((ext_vector_type(4)));

template <typename T> struct SaMfma;
template <> struct SaMfma<double> {
  using Acc = sad4;
  static __device__ __forceinline__ Acc mma(double a, double b, Acc c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  // row index (0..15) of accumulator register r in the lane group hi = lane >> 4
  static __device__ __forceinline__ int row(int r, int hi) { return 4 * r + hi; }
};
template <> struct SaMfma<float> {
  using Acc = saf4;
  static __device__ __forceinline__ Acc mma(float a, float b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int row(int r, int hi) { return 4 * hi + r; }
};

constexpr int kSaWaves = 8;              // per workgroup; they share the LDS copy of the factor (4 waves: 5 to 10 % slower on 128x128)
constexpr int kSaThreads = 64 * kSaWaves;
constexpr uint32_t kSaMaxP = 256, kSaMaxQ = 512;
constexpr size_t kSaLdsTarget = 65536;     // per workgroup: two workgroups per CU

// A "line" is what a tile's 16 lanes run along: the slices of one row (MKM) or the rows of one slice (KMM).
// Element (line, j, p) of the input lives at line*inLine + j*inJ + p*inP, element (line, q, j) of the output at
// line*outLine + q*outQ + j*outJ, likewise for Y.
struct StepAnyGeom {
  uint32_t P, Q, pc, pcPad, qb, kStride;   // pcPad: pc rounded up to 4; kStride: LDS elements between lane groups
  uint32_t qbSlab, nSlabs;             // 16-column blocks per slab of output columns, slabs per factor
  uint32_t vecLoad;                    // elements per vector load of the input (0: element by element)
  uint32_t nJ, jBlocks, totalTiles;
  int64_t inLine, inJ, inP, outLine, outJ, outQ, yLine, yJ, yQ;
};

// NBT > 0: every slab has exactly NBT full 16-column blocks (Q a multiple of 16) and P is a multiple of 4; the tile loop
// then has no conditional memory operation (see there).  NBT = 0: anything.
template <typename T, int PCMAX, bool HAS_Y, bool PREFETCH, int NBT>
__global__ __launch_bounds__(kSaThreads, 2) void kron_step_any_kernel(const StepArgs a, const StepAnyGeom g) {
  using MF = SaMfma<T>;
  using Acc = typename MF::Acc;
  extern __shared__ __align__(16) unsigned char saLds[];
  T* fl = (T*)saLds;
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lo = l & 15, hi = l >> 4;
  const uint32_t bt = blockIdx.y;
  const uint32_t pc = g.pc, Qp = g.qbSlab * 16;          // columns of this workgroup's slab of the factor
  const uint32_t ib0 = blockIdx.z * g.qbSlab;
  const uint32_t nb = g.qb - ib0 < g.qbSlab ? g.qb - ib0 : g.qbSlab;

  const T* inB = (const T*)a.in + (size_t)bt * a.in_batch;
  T* outB = (T*)a.out + (size_t)bt * a.out_batch;
  const T* YB = HAS_Y ? (const T*)a.y + (size_t)bt * a.y_batch : nullptr;
  const T alpha = a.epilogue ? (T)a.alpha : (T)1, beta = (T)a.beta;

  // the zero-padded slab of the factor: fl[k*kStride + c*Qp + q] = F[k*pc + c][16*ib0 + q]
  {
    const T* F = (const T*)a.f[0] + (size_t)bt * a.f_batch[0];
    const uint32_t perK = g.pcPad * Qp;                // rows pc .. pcPad-1 of a lane group are zero
    // eight loads of a thread go out before the first LDS write waits for one: a loop of load, wait, write would
    // put one memory round trip per element of a thread in front of the first product
    constexpr int kBatch = 8;
    for (uint32_t base = tid; base < 4 * perK; base += kBatch * kSaThreads) {
      T v[kBatch];
      uint32_t dst[kBatch];
#pragma unroll
      for (int u = 0; u < kBatch; u++) {
        const uint32_t idx = base + u * kSaThreads;
        const uint32_t k = idx / perK, rem = idx - k * perK, c = rem / Qp, q = rem - c * Qp;
        const uint32_t p = k * pc + c, qq = 16 * ib0 + q;
        v[u] = (T)0;
        if (idx < 4 * perK && c < pc && p < g.P && qq < g.Q) v[u] = F[(int64_t)p * a.f_sp[0] + (int64_t)qq * a.f_sq[0]];
        dst[u] = k * g.kStride + c * Qp + q;
      }
#pragma unroll
      for (int u = 0; u < kBatch; u++)
        if (base + u * kSaThreads < 4 * perK) fl[dst[u]] = v[u];
    }
  }
  __syncthreads();

  const uint32_t nWaves = gridDim.x * kSaWaves;
  const uint32_t wave = blockIdx.x * kSaWaves + w;
  const uint32_t p0 = hi * pc;                        // first contraction index of this lane group
  const T* fa = fl + hi * g.kStride + lo;

  auto loadTile = [&](uint32_t t, T (&x)[PCMAX]) {
    const uint32_t line = t / g.jBlocks, j0 = (t - line * g.jBlocks) * 16;
    const uint32_t j = (j0 + lo < g.nJ) ? j0 + lo : j0;                 // clamped: computed, not stored
    const T* xp = inB + (int64_t)line * g.inLine + (int64_t)j * g.inJ + (int64_t)p0 * g.inP;
    uint32_t nvalid = p0 < g.P ? g.P - p0 : 0u;                         // contraction indices of this lane group below P
    nvalid = nvalid < pc ? nvalid : pc;
    if (g.vecLoad) {
      // P is a multiple of 4 (no ragged lane group), the pc elements of a lane are contiguous and aligned:
      // 16- or 8-byte loads
      constexpr int VE = 16 / sizeof(T);
      typedef T VT __attribute__((ext_vector_type(VE)));
      typedef T V2 __attribute__((ext_vector_type(2)));
      if (g.vecLoad >= (uint32_t)VE) {
#pragma unroll
        for (int c = 0; c < PCMAX; c += VE) {
          if (c < (int)pc) {
            const VT v = *(const VT*)(xp + c);
#pragma unroll
            for (int e = 0; e < VE; e++) x[c + e] = v[e];
          } else if (c < (int)g.pcPad) {
#pragma unroll
            for (int e = 0; e < VE; e++) x[c + e] = (T)0;
          }
        }
      } else {
#pragma unroll
        for (int c = 0; c < PCMAX; c += 2) {
          if (c < (int)pc) {
            const V2 v = *(const V2*)(xp + c);
            x[c] = v[0]; x[c + 1] = v[1];
          } else if (c < (int)g.pcPad) {
            x[c] = (T)0; x[c + 1] = (T)0;
          }
        }
      }
      return;
    }
#pragma unroll
    for (int c = 0; c < PCMAX; c++) {
      if (c < (int)g.pcPad) {
        x[c] = (T)0;                                                    // indices beyond P count as zero and are not read
        if ((uint32_t)c < nvalid) x[c] = xp[(int64_t)c * g.inP];
      }
    }
  };

  if constexpr (NBT > 0) {
    // Loads and stores retire through one in-order counter, and the wait for the prefetched tile is counted in
    // younger operations: with the number of stores behind the prefetch the same on every path the compiler waits
    // for the tile alone, otherwise it drains the stores of the tile just computed first.  So nothing here is
    // conditional: lanes beyond the end of a ragged tile work on a copy of the tile's first slice (column) and store
    // the same values to the same places as its first lane, the last tile of a wave prefetches itself again, and the
    // first tile is peeled off the loop.
    static_assert(PREFETCH, "the unguarded loop prefetches");
    T xn[PCMAX];
    auto nextOf = [&](uint32_t t) { return t + nWaves < g.totalTiles ? t + nWaves : t; };
    auto computeTile = [&](uint32_t t) {
      T x[PCMAX];
#pragma unroll
      for (int c = 0; c < PCMAX; c++) x[c] = xn[c];
      loadTile(nextOf(t), xn);
      const uint32_t line = t / g.jBlocks, j0 = (t - line * g.jBlocks) * 16;
      const uint32_t j = (j0 + lo < g.nJ) ? j0 + lo : j0;
      T* out = outB + (int64_t)line * g.outLine + (int64_t)j * g.outJ;
      const T* Y = HAS_Y ? YB + (int64_t)line * g.yLine + (int64_t)j * g.yJ : nullptr;
#pragma unroll
      for (int ibl = 0; ibl < NBT; ibl++) {
        Acc acc = (Acc){0, 0, 0, 0};
#pragma unroll
        for (int c0 = 0; c0 < PCMAX; c0 += 4) {
          if (c0 < (int)g.pcPad) {
            T f[4];
#pragma unroll
            for (int c = 0; c < 4; c++) f[c] = fa[(c0 + c) * Qp + 16 * ibl];
#pragma unroll
            for (int c = 0; c < 4; c++) acc = MF::mma(f[c], x[c0 + c], acc);
          }
        }
        T yv[4];
        if (HAS_Y) {
#pragma unroll
          for (int r = 0; r < 4; r++) yv[r] = Y[(int64_t)(16 * (ib0 + ibl) + MF::row(r, hi)) * g.yQ];
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {
          T v = acc[r] * alpha;
          if (HAS_Y) v += beta * yv[r];
          out[(int64_t)(16 * (ib0 + ibl) + MF::row(r, hi)) * g.outQ] = v;
        }
      }
    };
    if (wave >= g.totalTiles) return;
    loadTile(wave, xn);
    computeTile(wave);
    for (uint32_t t = wave + nWaves; t < g.totalTiles; t += nWaves) computeTile(t);
    return;
  }

  T xn[PREFETCH ? PCMAX : 1];
  if (PREFETCH && wave < g.totalTiles) loadTile(wave, (T(&)[PCMAX])xn);
  for (uint32_t t = wave; t < g.totalTiles; t += nWaves) {
    T x[PCMAX];
    if (PREFETCH) {
#pragma unroll
      for (int c = 0; c < PCMAX; c++) x[c] = xn[PREFETCH ? c : 0];
      if (t + nWaves < g.totalTiles) loadTile(t + nWaves, (T(&)[PCMAX])xn);   // the next tile streams in under the products
    } else {
      loadTile(t, x);
    }

    const uint32_t line = t / g.jBlocks, j = (t - line * g.jBlocks) * 16 + lo;
    const bool jOk = j < g.nJ;
    T* out = outB + (int64_t)line * g.outLine + (int64_t)j * g.outJ;
    const T* Y = HAS_Y ? YB + (int64_t)line * g.yLine + (int64_t)j * g.yJ : nullptr;
    for (uint32_t ibl = 0; ibl < nb; ibl++) {
      const uint32_t ib = ib0 + ibl;
      Acc acc = (Acc){0, 0, 0, 0};
      // four products per wave-uniform guard: straight-line groups let the operand reads run ahead of the products
#pragma unroll
      for (int c0 = 0; c0 < PCMAX; c0 += 4) {
        if (c0 < (int)g.pcPad) {
          T f[4];
#pragma unroll
          for (int c = 0; c < 4; c++) f[c] = fa[(c0 + c) * Qp + 16 * ibl];
#pragma unroll
          for (int c = 0; c < 4; c++) acc = MF::mma(f[c], x[c0 + c], acc);
        }
      }
      T yv[4];
      if (HAS_Y) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const uint32_t q = 16 * ib + MF::row(r, hi);
          yv[r] = (jOk && q < g.Q) ? Y[(int64_t)q * g.yQ] : (T)0;
        }
      }
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const uint32_t q = 16 * ib + MF::row(r, hi);
        if (!(jOk && q < g.Q)) continue;
        T v = acc[r] * alpha;
        if (HAS_Y) v += beta * yv[r];
        out[(int64_t)q * g.outQ] = v;
      }
    }
  }
}

static bool saOutRowsContiguous(const StepArgs& a) { return a.out_ldm == 1 && a.out_ldc != 1; }

static bool stepAnyGeometry(const StepArgs& a, DType dt, StepAnyGeom* g) {
  if (a.nf != 1 || a.M == 0) return false;
  const uint32_t P = a.p[0], Q = a.q[0];
  if (P == 0 || Q == 0 || P > kSaMaxP || Q > kSaMaxQ || a.Kin % P) return false;
  const uint64_t S = a.Kin / P;
  if (S >= (1ull << 31)) return false;
  g->P = P; g->Q = Q; g->pc = (P + 3) / 4; g->qb = (Q + 15) / 16;
  // slabs of output columns so that the padded copy of a slab fits the LDS target
  g->pcPad = (g->pc + 3) / 4 * 4;
  uint32_t slab = (uint32_t)(kSaLdsTarget / (4 * (size_t)g->pcPad * 16 * dtypeSize(dt)));
  if (slab < 1) slab = 1;
  if (slab > g->qb) slab = g->qb;
  g->qbSlab = slab; g->nSlabs = (g->qb + slab - 1) / slab;
  g->kStride = g->pcPad * slab * 16 + 16;
  uint64_t nLines;
  if (saOutRowsContiguous(a)) {        // KMM: lanes along the rows of one slice
    nLines = S; g->nJ = a.M;
    g->inLine = (int64_t)P * a.in_ldc;  g->inJ = a.in_ldm;  g->inP = a.in_ldc;
    g->outLine = a.out_ldc;             g->outJ = a.out_ldm; g->outQ = (int64_t)S * a.out_ldc;
    g->yLine = a.y_ldc;                 g->yJ = a.y_ldm;     g->yQ = (int64_t)S * a.y_ldc;
  } else {                             // MKM: lanes along the slices of one row
    nLines = a.M; g->nJ = (uint32_t)S;
    g->inLine = a.in_ldm;   g->inJ = (int64_t)P * a.in_ldc; g->inP = a.in_ldc;
    g->outLine = a.out_ldm; g->outJ = a.out_ldc;            g->outQ = (int64_t)S * a.out_ldc;
    g->yLine = a.y_ldm;     g->yJ = a.y_ldc;                g->yQ = (int64_t)S * a.y_ldc;
  }
  // vector loads: contiguous input, no ragged lane group, every lane's run aligned to the vector
  g->vecLoad = 0;
  if (g->inP == 1 && P % 4 == 0) {
    const uint32_t es = (uint32_t)dtypeSize(dt);
    for (uint32_t ve = 16 / es; ve >= 2; ve /= 2) {
      const bool ok = g->pc % ve == 0 && g->inLine % ve == 0 && g->inJ % ve == 0 && (a.in_batch % ve) == 0 &&
                      ((uintptr_t)a.in % (ve * es)) == 0;
      if (ok) { g->vecLoad = ve; break; }
    }
  }
  g->jBlocks = (g->nJ + 15) / 16;
  const uint64_t tiles = nLines * g->jBlocks;
  if (tiles >= (1ull << 31)) return false;
  g->totalTiles = (uint32_t)tiles;
  return a.batch <= 65535 && g->nSlabs <= 65535;
}

bool stepAnyMfmaSupported(const StepArgs& a, DType dt) {
  StepAnyGeom g;
  return stepAnyGeometry(a, dt, &g);
}

template <typename T, int PCMAX, int NBT = 0>
static hipError_t launchStepAnyT(const StepArgs& a, const StepAnyGeom& g, hipStream_t stream) {
  // the tile of the next iteration is held in registers too unless the two copies would not fit (fp64, P > 128)
  constexpr bool PF = PCMAX * sizeof(T) <= 256;
  static_assert(NBT == 0 || PF, "fixed block counts come with the prefetching loop");
  const size_t ldsBytes = (size_t)4 * g.kStride * sizeof(T);
  static PerDeviceOnce attrOnce;
  const int devIdx = launchDeviceIndex();
  if (!attrOnce.done(devIdx)) {
    hipError_t e = hipFuncSetAttribute((const void*)kron_step_any_kernel<T, PCMAX, true, PF, NBT>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute((const void*)kron_step_any_kernel<T, PCMAX, false, PF, NBT>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, 140 * 1024);
    if (e != hipSuccess) return e;
    attrOnce.mark(devIdx);
  }
  const int cus = deviceCUs();
  // persistent workgroups, as many per CU as registers and the factor's LDS copy allow: a wave has one tile in
  // flight, so the bytes in flight per CU (what hides the HBM latency) grow with the number of resident waves
  // (the last answer is kept per device, the LDS size and the count packed into one word)
  static std::atomic<uint64_t> occCache[kMaxDevices];
  const uint64_t cached = occCache[devIdx].load(std::memory_order_relaxed);
  int occ = (int)(cached & 15);
  if (occ == 0 || (cached >> 4) != ldsBytes) {
    int n = 0;
    const void* fn = (a.y && a.epilogue) ? (const void*)kron_step_any_kernel<T, PCMAX, true, PF, NBT>
                                         : (const void*)kron_step_any_kernel<T, PCMAX, false, PF, NBT>;
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&n, fn, kSaThreads, ldsBytes) != hipSuccess || n < 1) n = 1;
    occ = n > 8 ? 8 : n;
    occCache[devIdx].store(((uint64_t)ldsBytes << 4) | (uint64_t)occ, std::memory_order_relaxed);
  }
  uint32_t wgs = (uint32_t)cus * (uint32_t)occ;
  const uint32_t share = a.batch * g.nSlabs;                  // the other two grid dimensions
  if (share > 1) wgs = (wgs + share - 1) / share;
  const uint32_t need = (g.totalTiles + kSaWaves - 1) / kSaWaves;
  if (wgs > need) wgs = need;
  if (wgs == 0) wgs = 1;
  dim3 grid(wgs, a.batch, g.nSlabs), block(kSaThreads);
  if (a.y && a.epilogue)
    hipLaunchKernelGGL((kron_step_any_kernel<T, PCMAX, true, PF, NBT>), grid, block, ldsBytes, stream, a, g);
  else
    hipLaunchKernelGGL((kron_step_any_kernel<T, PCMAX, false, PF, NBT>), grid, block, ldsBytes, stream, a, g);
  return hipGetLastError();
}

template <typename T>
static hipError_t launchStepAnyD(const StepArgs& a, const StepAnyGeom& g, hipStream_t stream) {
  // 128-row factors in full blocks (128x128: one slab of eight blocks in fp32, two of four in fp64): the loop
  // without conditional memory operations
  // (fp32 in the KMM layout, 32 four-byte loads per tile, is 6 % faster on the guarded loop)
  const bool fullBlocks = g.P % 4 == 0 && g.Q % 16 == 0 && g.pc == g.pcPad && g.qb % g.qbSlab == 0 &&
                          (sizeof(T) == 8 || g.vecLoad != 0);
  if (g.pcPad == 32 && fullBlocks && g.qbSlab == 8) return launchStepAnyT<T, 32, 8>(a, g, stream);
  if (g.pcPad == 32 && fullBlocks && g.qbSlab == 4) return launchStepAnyT<T, 32, 4>(a, g, stream);
  if (g.pcPad <= 4)  return launchStepAnyT<T, 4>(a, g, stream);
  if (g.pcPad <= 8)  return launchStepAnyT<T, 8>(a, g, stream);
  if (g.pcPad <= 16) return launchStepAnyT<T, 16>(a, g, stream);
  if (g.pcPad <= 32) return launchStepAnyT<T, 32>(a, g, stream);
  return launchStepAnyT<T, 64>(a, g, stream);
}

hipError_t launchStepAnyMfma(const StepArgs& a, DType dt, hipStream_t stream) {
  StepAnyGeom g;
  if (!stepAnyGeometry(a, dt, &g)) return hipErrorInvalidValue;
  return dt == DType::F32 ? launchStepAnyD<float>(a, g, stream) : launchStepAnyD<double>(a, g, stream);
}

}  // namespace fk
