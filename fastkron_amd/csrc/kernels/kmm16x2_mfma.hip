// Two fused 16x16 factors in the KMM layout (element (m, col) at m + col*M, the M index contiguous), fp32 or fp64:
// half the launches and half the HBM passes of sgekmm / dgekmm chains of 16x16 factors, and of the leading
// factors of long GeMKM chains (which run as KMM problems over contiguous blocks).
//
//   out[(q0, q1, s), m] = sum_{k0,k1} in[(s, k0, k1), m] * F0[k0,q0] * F1[k1,q1]      (s: slice, S = Kin / 256)
//
// A wave owns a tile of one slice and 16 consecutive m (fp32 with M a multiple of 32: 32 consecutive m, two per
// lane): 256 x 16 (32) elements, kept in registers; no LDS exchange, no barrier.
//   k1   for each k0 one V_MFMA_*_16X16X4 group, computed transposed: D[q1][m] = sum_k1 F1^T[q1][k1] X[k1][m].
//        B operand lane = 16*k + m reads rows k1 = 4*c + k (16 consecutive m per quarter wave and product), the A
//        operand is F1 in registers.  The results z[k0][r] = T[k0][q1 = row(r, lane/16)][m = lane%16] stay in
//        16 x 4 registers.
//   k0   contracted over the register index on the vector ALU, F0 read from LDS as broadcast pairs.
//   store  per q0 a lane holds four values, rows q1 = row(r, lane/16): every quarter wave writes 16 consecutive m.
//
// The reference's GPU kernels fuse factors through shared memory on CUDA cores (reference
// src/kernels/cuda/kernel.cuh:165-219); its x86 KMM kernels vectorise along M as this one does (reference
// src/kernels/cpu/kernel.h:124-126).
// Algorithmic traffic per launch: read M*Kin, write M*Kin elements (+ M*Kin for Y on the launch that writes Z).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef double k2d4 __attribute__((ext_vector_type(4)));
typedef float k2f4 __attribute__((ext_vector_type(4)));

template <typename T> struct K2Mfma;
template <> struct K2Mfma<double> {
  using Acc = k2d4;
  static __device__ __forceinline__ Acc mma(double a, double b, Acc c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int row(int r, int hi) { return 4 * r + hi; }
};
template <> struct K2Mfma<float> {
  using Acc = k2f4;
  static __device__ __forceinline__ Acc mma(float a, float b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int row(int r, int hi) { return 4 * hi + r; }
};

constexpr int kK2Waves = 4;
constexpr int kK2Win = 3;              // k0 slices of a tile in flight

// EXACT: 16x16 factors.  Otherwise PxP factors with 9 <= P <= 15: matrix-core operands zero-padded to 16, rows and
// registers beyond P masked.
// JW: columns m per lane.  With 2 (fp32, M a multiple of 32) a lane owns two neighbouring columns, reads and writes
// them as one 8-byte element, and a quarter wave covers a whole 128-byte line per row where JW = 1 covers half of
// one; the two columns go through the matrix cores as two column blocks.
template <typename T, bool HAS_Y, bool EXACT, int JW>
__global__ __launch_bounds__(256, 2) void kron_kmm16x2_kernel(const StepArgs a, const uint32_t mTiles,
                                                              const uint32_t totalTiles) {
  using MF = K2Mfma<T>;
  using Acc = typename MF::Acc;
  typedef T V2 __attribute__((ext_vector_type(2)));
  static_assert(JW == 1 || JW == 2, "one or two columns per lane");
  __shared__ __align__(16) T f0s[256];              // F0 transposed: f0s[q0*16 + k0]
  const int tid = threadIdx.x;
  const int l0 = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lo = l0 & 15, hi = l0 >> 4;
  const uint32_t bt = blockIdx.y;
  const int P = EXACT ? 16 : (int)a.p[0];
  const uint64_t S = a.Kin / (uint64_t)(P * P);
  const uint64_t M = a.M;

  // a.f[0] is the later factor F1 (contracts the fast digit k1), a.f[1] = F0
  {
    const T* F0 = (const T*)a.f[1] + (size_t)bt * a.f_batch[1];
    const int q0 = tid >> 4, k0 = tid & 15;
    T v = (T)0;
    if (EXACT || (q0 < P && k0 < P)) v = F0[(int64_t)k0 * a.f_sp[1] + (int64_t)q0 * a.f_sq[1]];
    f0s[tid] = v;
  }
  T f1[4];                                          // A operand: F1[k1 = 4*c + hi][q1 = lo]
  {
    const T* F1 = (const T*)a.f[0] + (size_t)bt * a.f_batch[0];
#pragma unroll
    for (int c = 0; c < 4; c++) {
      f1[c] = (T)0;
      if (EXACT || (4 * c + hi < P && lo < P)) f1[c] = F1[(int64_t)(4 * c + hi) * a.f_sp[0] + (int64_t)lo * a.f_sq[0]];
    }
  }
  __syncthreads();

  const T* inB = (const T*)a.in + (size_t)bt * a.in_batch;
  T* outB = (T*)a.out + (size_t)bt * a.out_batch;
  const T* YB = HAS_Y ? (const T*)a.y + (size_t)bt * a.y_batch : nullptr;
  const T alpha = a.epilogue ? (T)a.alpha : (T)1, beta = (T)a.beta;

  const uint32_t nWaves = gridDim.x * kK2Waves;
  // x[c] = X[(s, k0, k1 = 4*c + hi), m]; columns beyond M are clamped to the tile's first one (computed, not stored)
  // The rows are read in the order (k0, c): row k0*P + 4*c + hi, four rows further with every load and P - 16
  // back at the end of a slice, so one running pointer serves the whole tile.  Rows 4*c + hi >= P are not read.
  const int64_t rowStep = 4 * (int64_t)a.in_ldc, sliceFix = (int64_t)(P - 16) * (int64_t)a.in_ldc;
  auto loadSlice = [&](const T*& xp, T (&x)[JW][4]) {
#pragma unroll
    for (int c = 0; c < 4; c++) {
#pragma unroll
      for (int e = 0; e < JW; e++) x[e][c] = (T)0;
      if (EXACT || 4 * c + hi < P) {
        if (JW == 2) { const V2 v = *(const V2*)xp; x[0][c] = v[0]; x[JW - 1][c] = v[1]; }
        else x[0][c] = *xp;
      }
      xp += rowStep;
    }
    if (!EXACT) xp += sliceFix;
  };

  // first row of tile t that this lane reads
  auto tileRows = [&](uint32_t t) {
    const uint64_t s = t / mTiles;
    const uint32_t m0 = (uint32_t)(t - s * mTiles) * (16 * JW);
    const uint32_t m = (JW == 2 || m0 + lo < M) ? m0 + JW * lo : m0;
    return inB + m + (s * (uint64_t)(P * P) + hi) * (uint64_t)a.in_ldc;
  };
  // The first slices of a tile are requested while the tile before it is still in its vector-ALU and store phase
  // (the window's registers are free from the last matrix product on): a tile that requested them at its own start
  // sat out a memory round trip, behind the stores of the tile before, with nothing else in flight.
  T xw[kK2Win][JW][4];
  uint32_t t = blockIdx.x * kK2Waves + w;
  if (t >= totalTiles) return;
  const T* xp = tileRows(t);
#pragma unroll
  for (int k = 0; k < kK2Win; k++) loadSlice(xp, xw[k]);
  for (; t < totalTiles; t += nWaves) {
    const uint64_t s = t / mTiles;
    const uint32_t m0 = (uint32_t)(t - s * mTiles) * (16 * JW);
    const bool mOk = JW == 2 || m0 + lo < M;                      // two columns per lane: whole tiles only
    const uint32_t m = mOk ? m0 + JW * lo : m0;

    T z[JW][16][4];
#pragma unroll
    for (int k0 = 0; k0 < 16; k0++) {
      T x[JW][4];
#pragma unroll
      for (int e = 0; e < JW; e++)
#pragma unroll
        for (int c = 0; c < 4; c++) x[e][c] = xw[k0 % kK2Win][e][c];
      if (k0 + kK2Win < (EXACT ? 16 : P)) loadSlice(xp, xw[k0 % kK2Win]);
#pragma unroll
      for (int e = 0; e < JW; e++) {
        Acc d = (Acc){0, 0, 0, 0};
        if (EXACT || k0 < P) {
#pragma unroll
          for (int c = 0; c < 4; c++) d = MF::mma(f1[c], x[e][c], d);     // d[q1][m]
        }
#pragma unroll
        for (int r = 0; r < 4; r++) z[e][k0][r] = d[r];
      }
      __builtin_amdgcn_sched_barrier(0);             // keeps the loads of later slices from being hoisted up here
    }
    // (behind the last tile of a wave the requests go to that tile's own rows again and are dropped)
    xp = tileRows(t + nWaves < totalTiles ? t + nWaves : t);
#pragma unroll
    for (int k = 0; k < kK2Win; k++) loadSlice(xp, xw[k]);

    // ---- k0 on the vector ALU, one q0 at a time, and the stores ----
    // output row (q0, q1 = row(r, hi)): a running pointer per lane, 16 rows further with every q0
    const uint64_t oq = S * (uint64_t)a.out_ldc, yq = HAS_Y ? S * (uint64_t)a.y_ldc : 0;   // stride of one output row q
    const uint64_t rs = (uint64_t)(MF::row(1, 0) - MF::row(0, 0));                        // rows between two registers
    T* op = outB + m + s * (uint64_t)a.out_ldc + (uint64_t)MF::row(0, hi) * oq;
    const T* yp = HAS_Y ? YB + m + s * (uint64_t)a.y_ldc + (uint64_t)MF::row(0, hi) * yq : nullptr;
#pragma unroll 1
    for (int q0 = 0; q0 < P; q0++) {
      T yv[JW][4];
      if (HAS_Y) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const bool ok = mOk && (EXACT || MF::row(r, hi) < P);
          if (JW == 2) {
            const V2 v = ok ? *(const V2*)&yp[r * rs * yq] : (V2){0, 0};
            yv[0][r] = v[0]; yv[JW - 1][r] = v[1];
          } else {
            yv[0][r] = ok ? yp[r * rs * yq] : (T)0;
          }
        }
        yp += (uint64_t)P * yq;
      }
      T acc[JW][4];
#pragma unroll
      for (int e = 0; e < JW; e++)
#pragma unroll
        for (int r = 0; r < 4; r++) acc[e][r] = (T)0;
#pragma unroll
      for (int k = 0; k < 16; k += 2) {
        const V2 f = *(const V2*)&f0s[q0 * 16 + k];
#pragma unroll
        for (int e = 0; e < JW; e++) {
#pragma unroll
          for (int r = 0; r < 4; r++) acc[e][r] += f[0] * z[e][k][r];
#pragma unroll
          for (int r = 0; r < 4; r++) acc[e][r] += f[1] * z[e][k + 1][r];
        }
      }
      if (mOk) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
          T v[JW];
#pragma unroll
          for (int e = 0; e < JW; e++) {
            v[e] = acc[e][r] * alpha;
            if (HAS_Y) v[e] += beta * yv[e][r];
          }
          if (EXACT || MF::row(r, hi) < P) {
            if (JW == 2) *(V2*)&op[r * rs * oq] = (V2){v[0], v[JW - 1]};
            else op[r * rs * oq] = v[0];
          }
        }
      }
      op += (uint64_t)P * oq;
    }
  }
}

bool kmm16x2Supported(const StepArgs& a, DType dt) {
  if (a.nf != 2) return false;
  const uint32_t P = a.p[0];
  if (P < 9 || P > 16) return false;
  for (uint32_t j = 0; j < 2; j++) if (a.p[j] != P || a.q[j] != P) return false;
  if (a.Kin % (P * P) || a.Kout != a.Kin) return false;
  // the M index contiguous in the input, the output and Y
  if (a.in_ldm != 1 || a.out_ldm != 1 || (a.y && a.y_ldm != 1)) return false;
  const uint64_t tiles = (a.Kin / (P * P)) * ((a.M + 15) / 16);
  (void)dt;
  return tiles < (1ull << 31) && a.batch <= 65535;
}

// two columns per lane: fp32, whole tiles of 32 columns, every row and batch entry on an 8-byte boundary
static bool kmm16x2TwoColumns(const StepArgs& a, DType dt) {
  if (dt != DType::F32 || a.M % 32) return false;
  if (((uintptr_t)a.in & 7) || (a.in_ldc & 1) || (a.in_batch & 1)) return false;
  if (((uintptr_t)a.out & 7) || (a.out_ldc & 1) || (a.out_batch & 1)) return false;
  if (a.y && (((uintptr_t)a.y & 7) || (a.y_ldc & 1) || (a.y_batch & 1))) return false;
  return true;
}

template <typename T, bool EXACT, int JW>
static hipError_t launchKmm16x2T(const StepArgs& a, hipStream_t stream) {
  const int cus = deviceCUs();
  const uint32_t P = a.p[0];
  const uint32_t mTiles = (a.M + 16 * JW - 1) / (16 * JW);
  const uint32_t totalTiles = (uint32_t)((a.Kin / (P * P)) * mTiles);
  // persistent waves: two workgroups of four waves per CU (two waves per SIMD)
  uint32_t wgs = (uint32_t)cus * 2;
  if (a.batch > 1) wgs = (wgs + a.batch - 1) / a.batch;
  const uint32_t need = (totalTiles + kK2Waves - 1) / kK2Waves;
  if (wgs > need) wgs = need;
  if (wgs == 0) wgs = 1;
  dim3 grid(wgs, a.batch), block(256);
  if (a.y && a.epilogue)
    hipLaunchKernelGGL((kron_kmm16x2_kernel<T, true, EXACT, JW>), grid, block, 0, stream, a, mTiles, totalTiles);
  else
    hipLaunchKernelGGL((kron_kmm16x2_kernel<T, false, EXACT, JW>), grid, block, 0, stream, a, mTiles, totalTiles);
  return hipGetLastError();
}

hipError_t launchKmm16x2(const StepArgs& a, DType dt, hipStream_t stream) {
  if (!kmm16x2Supported(a, dt)) return hipErrorInvalidValue;
  const bool exact = a.p[0] == 16;
  if (dt == DType::F32) {
    if (kmm16x2TwoColumns(a, dt))
      return exact ? launchKmm16x2T<float, true, 2>(a, stream) : launchKmm16x2T<float, false, 2>(a, stream);
    return exact ? launchKmm16x2T<float, true, 1>(a, stream) : launchKmm16x2T<float, false, 1>(a, stream);
  }
  return exact ? launchKmm16x2T<double, true, 1>(a, stream) : launchKmm16x2T<double, false, 1>(a, stream);
}

}  // namespace fk
