// Three fused 16x16 factors on contiguous blocks of 16^3 = 4096 elements (dgemkm with 16x16^3, or the three
// trailing factors of a longer chain applied block by block; fp32 where the 16x16^4 workgroup kernel does not
// apply): one wave owns a block, keeps it in registers and needs neither an LDS exchange nor a barrier.
//
//   Z[q1,q2,q3] = alpha * sum_{k1,k2,k3} X[k1,k2,k3] F1[k1,q1] F2[k2,q2] F3[k3,q3]  (+ beta*Y)
//
//   k3, k2   for every k1: V_MFMA_F64_16X16X4_F64 twice, chained in registers.  The first product contracts k3 with
//            the 256 values X[k1,:,:] as A operand (lane = (k2, 4 consecutive k3): two 16-byte loads, 2 KB contiguous
//            per wave) and leaves D[k2][q3] in register k2/4 of lane 16*(k2%4) + q3, which is the B-operand layout
//            of a product that contracts k2; its A operand is F2 with the rows permuted to match (4r + lane/16).
//   k1       the 16 results of a lane for its (q2, q3) sit in 16 x 4 registers: the last contraction runs over the
//            register index on the vector ALU (fp64 FMA runs at the matrix rate on this chip), F1 read from LDS as
//            broadcast 16-byte pairs.
//   store    per q1 a lane holds four doubles, rows q2 = 4r + lane/16: every quarter wave writes a 128-byte line.
// With two factors the leading digit is a row index (16 consecutive rows form a block) and F1 is the identity.
//
// The reference has no fp64 kernel that fuses this shape in one launch: its tile must fit 48 KB of shared memory
// (reference src/gen_tuner_kernels.py:10,366) and it runs one or two factors per launch.
// Algorithmic traffic: 8*4096 bytes read + 8*4096 bytes written per block (+ Y when beta != 0).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef double r3d4 __attribute__((ext_vector_type(4)));
typedef float r3f4 __attribute__((ext_vector_type(4)));

// accumulator layouts of the two 16x16x4 instructions: row(r, hi) = output row held by register r in the lane
// group hi = lane / 16
template <typename T> struct R3Mfma;
template <> struct R3Mfma<double> {
  using Acc = r3d4;
  static __device__ __forceinline__ Acc mma(double a, double b, Acc c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int row(int r, int hi) { return 4 * r + hi; }
};
template <> struct R3Mfma<float> {
  using Acc = r3f4;
  static __device__ __forceinline__ Acc mma(float a, float b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int row(int r, int hi) { return 4 * hi + r; }
};

constexpr int kR3Waves = 4;
// k1 slices of the next block requested before the last contraction / further slices in flight while a block is
// contracted: as many as the registers allow at two waves per SIMD
template <typename T> struct R3Depth { static constexpr int ahead = sizeof(T) == 4 ? 4 : 2, win = sizeof(T) == 4 ? 4 : 2; };

// EXACT: 16x16 factors (vector loads, no masks).  Otherwise PxP factors with 9 <= P <= 15 on blocks of P^3
// elements: the matrix-core operands are zero-padded to 16 and the lanes / registers beyond P are masked.
// WIDE (fp32, 16x16 factors, blocks of Z and Y on 16-byte boundaries): the second product with its operands exchanged,
// e[q3][q2] instead of e[q2][q3], leaves four consecutive q3 in a lane, and the results leave 16 bytes per lane, a
// wave instruction writing 1 KB in one piece (instead of 64-byte pieces 4 bytes per lane); results that nothing reads
// back soon go out at system scope (sgemkm 4096 x 16^3: 33.9 -> 24.6 us, 16384 x 16^3: 107.5 -> 104.6 us).
template <typename T, bool HAS_Y, bool EXACT, bool WIDE>
__global__ __launch_bounds__(256, 2) void kron_row16x3_kernel(const StepArgs a, const uint32_t blocksPerBatch,
                                                              const uint32_t totalBlocks) {
  using MF = R3Mfma<T>;
  using Acc = typename MF::Acc;
  typedef T V2 __attribute__((ext_vector_type(2)));
  constexpr int kR3Ahead = R3Depth<T>::ahead, kR3Win = R3Depth<T>::win;
  __shared__ __align__(16) T f1s[256];               // F1 transposed: f1s[q1*16 + k1]
  const int tid = threadIdx.x;
  const int l0 = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lo = l0 & 15, hi = l0 >> 4;
  const int P = EXACT ? 16 : (int)a.p[0];            // factor size; P2, P3: strides of k2 / k1 and the block length
  const int P2 = P * P, P3 = P2 * P;

  // a.f[0] is the last factor F3, a.f[1] = F2, a.f[2] = F1 (identity when only two factors are fused).
  // Factors shared by the whole launch only: per-batch factors are left to other kernels.
  {
    const int q1 = tid >> 4, k1 = tid & 15;
    const bool in = EXACT || (q1 < P && k1 < P);
    T v = (in && q1 == k1) ? (T)1 : (T)0;
    if (a.nf == 3 && in) v = ((const T*)a.f[2])[(int64_t)k1 * a.f_sp[2] + (int64_t)q1 * a.f_sq[2]];
    f1s[tid] = v;
  }
  // operands of the two products: F3[4*hi + c][lo] and F2[row(r, hi)][lo] (the rows the first product leaves
  // in register r of this lane group)
  T f3[4], f2[4];
  {
    const T* F3 = (const T*)a.f[0];
    const T* F2 = (const T*)a.f[1];
#pragma unroll
    for (int c = 0; c < 4; c++) {
      f3[c] = f2[c] = (T)0;
      if (EXACT || (4 * hi + c < P && lo < P)) f3[c] = F3[(int64_t)(4 * hi + c) * a.f_sp[0] + (int64_t)lo * a.f_sq[0]];
      if (EXACT || (MF::row(c, hi) < P && lo < P)) f2[c] = F2[(int64_t)MF::row(c, hi) * a.f_sp[1] + (int64_t)lo * a.f_sq[1]];
    }
  }
  __syncthreads();

  const uint32_t nWaves = gridDim.x * kR3Waves;
  uint32_t blk = blockIdx.x * kR3Waves + w;
  if (blk >= totalBlocks) return;

  auto blockPtr = [&](uint32_t b) {
    return (const T*)a.in + (size_t)(b / blocksPerBatch) * a.in_batch + (size_t)(b % blocksPerBatch) * P3;
  };
  // x[c] = X[k1][k2 = lo][k3 = 4*hi + c]: 16-byte loads (element by element, masked, for P < 16)
  auto loadSlice = [&](const T* X, int k1, T (&x)[4]) {
    const T* xp = X + k1 * P2 + lo * P + hi * 4;
    if (!EXACT) {
#pragma unroll
      for (int c = 0; c < 4; c++) {
        x[c] = (T)0;
        if (k1 < P && lo < P && 4 * hi + c < P) x[c] = xp[c];
      }
    } else if (sizeof(T) == 8) {
      const V2 v0 = *(const V2*)xp, v1 = *(const V2*)(xp + 2);
      x[0] = v0[0]; x[1] = v0[1]; x[2] = v1[0]; x[3] = v1[1];
    } else {
      const Acc v = *(const Acc*)xp;
      x[0] = v[0]; x[1] = v[1]; x[2] = v[2]; x[3] = v[3];
    }
  };

  T xa[kR3Ahead][4];                                 // the first slices of the block about to be processed
  {
    const T* X = blockPtr(blk);
#pragma unroll
    for (int k = 0; k < kR3Ahead; k++) loadSlice(X, k, xa[k]);
  }

  auto processBlock = [&](const uint32_t blk) {
    const T* X = blockPtr(blk);
    const size_t bt = blk / blocksPerBatch, m = blk % blocksPerBatch;
    T* Z = (T*)a.out + bt * a.out_batch + m * P3;
    const T* Y = HAS_Y ? (const T*)a.y + bt * a.y_batch + m * P3 : nullptr;

    // ---- k3 and k2, slice by slice; z[k1][r] = T[k1][q2 = row(r, hi)][q3 = lo] ----
    T z[16][4];
    T xb[kR3Win][4];                                 // rolling window of slices in flight
#pragma unroll
    for (int k = 0; k < kR3Win; k++) loadSlice(X, kR3Ahead + k, xb[k]);
#pragma unroll
    for (int k1 = 0; k1 < 16; k1++) {
      T x[4];
#pragma unroll
      for (int c = 0; c < 4; c++)
        x[c] = (k1 < kR3Ahead) ? xa[k1 < kR3Ahead ? k1 : 0][c] : xb[(k1 - kR3Ahead) % kR3Win][c];
      if (k1 >= kR3Ahead && k1 + kR3Win < 16) loadSlice(X, k1 + kR3Win, xb[(k1 - kR3Ahead) % kR3Win]);
      Acc e = (Acc){0, 0, 0, 0};
      if (EXACT || k1 < P) {
        Acc d = (Acc){0, 0, 0, 0};
#pragma unroll
        for (int c = 0; c < 4; c++) d = MF::mma(x[c], f3[c], d);       // d[k2][q3]
#pragma unroll
        for (int r = 0; r < 4; r++) e = WIDE ? MF::mma(d[r], f2[r], e) : MF::mma(f2[r], d[r], e);       // e[q2][q3] (WIDE: e[q3][q2])
      }
#pragma unroll
      for (int r = 0; r < 4; r++) z[k1][r] = e[r];
      __builtin_amdgcn_sched_barrier(0);             // keeps the loads of later slices from being hoisted up here
    }

    // ---- the first slices of the wave's next block stream in under the last contraction ----
    {
      const uint32_t nx = blk + nWaves;
      const T* Xn = blockPtr(nx < totalBlocks ? nx : blk);
#pragma unroll
      for (int k = 0; k < kR3Ahead; k++) loadSlice(Xn, k, xa[k]);
    }

    // ---- k1 on the vector ALU, one q1 at a time, and the stores ----
    const T alpha = a.epilogue ? (T)a.alpha : (T)1, beta = (T)a.beta;
    T* zp = Z + lo;
    const T* yp = HAS_Y ? Y + lo : nullptr;
    // (for P < 16: slices k1 >= P were not loaded, their z are exact zeros; rows and columns >= P are not stored)
    if constexpr (WIDE) {
      typedef T V4 __attribute__((ext_vector_type(4)));
      // z[k1][r] = T[k1][q2 = lo][q3 = 4*hi + r]
      T* zw = Z + lo * 16 + 4 * hi;
      const __amdgpu_buffer_rsrc_t zTarget = streamTarget((void*)Z, 4096 * 4u);
      const T* yw = HAS_Y ? Y + lo * 16 + 4 * hi : nullptr;
#pragma unroll 1
      for (int q1 = 0; q1 < 16; q1++) {
        V4 yv = {0, 0, 0, 0};
        if (HAS_Y) yv = *(const V4*)(yw + q1 * 256);
        T acc[4] = {0, 0, 0, 0};
#pragma unroll
        for (int k = 0; k < 16; k += 2) {
          const V2 f = *(const V2*)&f1s[q1 * 16 + k];
#pragma unroll
          for (int r = 0; r < 4; r++) acc[r] += f[0] * z[k][r];
#pragma unroll
          for (int r = 0; r < 4; r++) acc[r] += f[1] * z[k + 1][r];
        }
        V4 v = {acc[0] * alpha, acc[1] * alpha, acc[2] * alpha, acc[3] * alpha};
        if (HAS_Y) v += beta * yv;
        if (a.stream_out) streamStore16(v, zTarget, (uint32_t)(q1 * 256 + lo * 16 + 4 * hi) * 4u);
        else *(V4*)(zw + q1 * 256) = v;
      }
      return;
    }
#pragma unroll 1
    for (int q1 = 0; q1 < P; q1++) {
      T yv[4];
      if (HAS_Y) {
#pragma unroll
        for (int r = 0; r < 4; r++)
          yv[r] = (EXACT || (MF::row(r, hi) < P && lo < P)) ? yp[q1 * P2 + MF::row(r, hi) * P] : (T)0;
      }
      T acc[4] = {0, 0, 0, 0};
#pragma unroll
      for (int k = 0; k < 16; k += 2) {
        const V2 f = *(const V2*)&f1s[q1 * 16 + k];
#pragma unroll
        for (int r = 0; r < 4; r++) acc[r] += f[0] * z[k][r];
#pragma unroll
        for (int r = 0; r < 4; r++) acc[r] += f[1] * z[k + 1][r];
      }
#pragma unroll
      for (int r = 0; r < 4; r++) {
        T v = acc[r] * alpha;
        if (HAS_Y) v += beta * yv[r];
        if (EXACT || (MF::row(r, hi) < P && lo < P))
          zp[q1 * P2 + MF::row(r, hi) * P] = v;      // Z[q1][q2 = row(r, hi)][q3 = lo]
      }
    }
  };

  // The first block is peeled off the loop: the wait for the slices requested ahead is counted in younger memory
  // operations, and entering the loop only from a complete block lets that count include the block's stores.
  processBlock(blk);
  for (blk += nWaves; blk < totalBlocks; blk += nWaves) processBlock(blk);
}

bool row16x3Supported(const StepArgs& a, DType dt) {
  if (a.nf != 2 && a.nf != 3) return false;
  const uint32_t P = a.p[0];
  if (P < 9 || P > 16) return false;
  uint64_t k = 1;
  for (uint32_t j = 0; j < a.nf; j++) {
    if (a.p[j] != P || a.q[j] != P || (a.batch > 1 && a.f_batch[j] != 0)) return false;
    k *= P;
  }
  if (a.Kin != k || a.Kout != k) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  // the rows of a block must be contiguous, and M must be a whole number of blocks
  if ((uint64_t)a.in_ldm != k || (uint64_t)a.out_ldm != k || (a.y && (uint64_t)a.y_ldm != k)) return false;
  if (a.nf == 2 && a.M % P) return false;
  // 16-byte loads of the 16x16 form
  if (P == 16 && (((uintptr_t)a.in & 15) || (a.in_batch * dtypeSize(dt)) % 16)) return false;
  const uint64_t blocks = (uint64_t)(a.nf == 2 ? a.M / P : a.M) * a.batch;
  return blocks < (1ull << 32);
}

template <typename T, bool EXACT, bool WIDE>
static void launchRow16x3T(const StepArgs& a, dim3 grid, uint32_t blocksPerBatch, uint32_t total, hipStream_t stream) {
  dim3 block(256);
  if (a.y && a.epilogue)
    hipLaunchKernelGGL((kron_row16x3_kernel<T, true, EXACT, WIDE>), grid, block, 0, stream, a, blocksPerBatch, total);
  else
    hipLaunchKernelGGL((kron_row16x3_kernel<T, false, EXACT, WIDE>), grid, block, 0, stream, a, blocksPerBatch, total);
}

hipError_t launchRow16x3(const StepArgs& a, DType dt, hipStream_t stream) {
  if (!row16x3Supported(a, dt)) return hipErrorInvalidValue;
  const int cus = deviceCUs();
  const uint32_t P = a.p[0];
  const uint32_t blocksPerBatch = a.nf == 2 ? a.M / P : a.M;
  const uint64_t total = (uint64_t)blocksPerBatch * a.batch;
  // persistent waves: two workgroups of four waves per CU (more resident waves measured slightly slower)
  uint32_t wgs = (uint32_t)cus * 2;
  const uint64_t need = (total + kR3Waves - 1) / kR3Waves;
  if (wgs > need) wgs = (uint32_t)need;
  dim3 grid(wgs);
  const uint32_t tb = (uint32_t)total;
  if (dt == DType::F64) {
    if (P == 16) launchRow16x3T<double, true, false>(a, grid, blocksPerBatch, tb, stream);
    else         launchRow16x3T<double, false, false>(a, grid, blocksPerBatch, tb, stream);
  } else {
    // blocks of Z (and Y) on 16-byte boundaries: results 16 bytes per lane
    const bool wide = !(((uintptr_t)a.out & 15) || (a.out_batch & 3)) &&
                      !(a.y && a.epilogue && (((uintptr_t)a.y & 15) || (a.y_batch & 3)));
    if (P == 16 && wide) launchRow16x3T<float, true, true>(a, grid, blocksPerBatch, tb, stream);
    else if (P == 16)    launchRow16x3T<float, true, false>(a, grid, blocksPerBatch, tb, stream);
    else                 launchRow16x3T<float, false, false>(a, grid, blocksPerBatch, tb, stream);
  }
  return hipGetLastError();
}

}  // namespace fk
