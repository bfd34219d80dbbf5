// One sliced-multiply step with a square factor (P = Q in {16, 32, 64, 128}), MKM layout, fp64 or fp32, on the
// matrix cores (V_MFMA_F64_16X16X4_F64 / V_MFMA_F32_16X16X4_F32).  Used per factor for shapes like dgemkm 256 x 262144
// with 64x64^3, where every step is a real (M*Kin/P) x P x Q contraction.
//
//   out[m, q*S + s] = sum_p in[m, s*P + p] * F[p, q],   S = Kin / P
//
// Streaming design: a wave owns 16 consecutive slices of one row at a time and needs no LDS and no
// barrier.  The product is computed transposed, D[q][slice] = sum_p F^T[q][p] X^T[p][slice]:
//   * B operand (lane = 16*k + slice): the contraction index of product c is taken as
//     p = (P/4)*k + c, so a lane reads P/4 *consecutive* doubles of its slice (a full 128-byte line for
//     P = 64) with 128-bit loads, and the 4 lanes of a slice cover the slice exactly once;
//   * A operand (lane = 16*k + q): F[(P/4)*k + c][16*ib + q]; the whole factor sits in registers
//     (128 VGPRs for 64x64) for the life of the persistent wave, so the loop reads nothing but X;
//   * the next tile's loads are issued before the current tile's products (register double buffer);
//   * accumulator layout (fp64: register q/4, lane 16*(q%4) + slice; fp32: register q%4, lane
//     16*(q/4) + slice): each quarter wave stores 16 consecutive elements (a 128-byte line in fp64)
//     straight into the shuffled layout out[q*S + s].
// alpha / beta*Y are applied in the same store when this is the launch that writes Z.
//
// Role of the reference's CUDA kernel for large factors (reference src/kernels/cuda/kernel.cuh:53-224,
// which uses CUDA cores only, reference README.md:44-48); tiling, MFMA use, the permuted contraction
// index and the transposed accumulation are specific to this kernel.
// Algorithmic traffic per launch: read M*Kin, write M*Kout elements (+ M*Kout for Y on the last step).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef double d4 __attribute__((ext_vector_type(4)));
typedef float f4 __attribute__((ext_vector_type(4)));

template <typename T> struct Mfma16;
template <> struct Mfma16<double> {
  using Acc = d4;
  static __device__ __forceinline__ Acc mma(double a, double b, Acc c) {
    return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0);
  }
  // row index (0..15) of accumulator register r in the lane group hi = lane >> 4
  static __device__ __forceinline__ int row(int r, int hi) { return 4 * r + hi; }
};
template <> struct Mfma16<float> {
  using Acc = f4;
  static __device__ __forceinline__ Acc mma(float a, float b, Acc c) {
    return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0);
  }
  static __device__ __forceinline__ int row(int r, int hi) { return 4 * hi + r; }
};

constexpr int kStepWaves = 4;            // waves per workgroup

// QS > 1 splits the Q output columns of a tile over QS wave tasks (each keeps only its Q/QS columns of
// the factor in registers); used for 128x128, whose factor does not fit the register file of one wave.
//
// KMM = true is the same step on the KMM layout (element (m, col) at m + col*M, the M index contiguous): a
// tile is then 16 consecutive m of one slice, the B operand lane 16*k + m reads in[(s*P + p)*M + m] (16
// consecutive elements per quarter wave and product), and the stores are the same 16-element runs.
template <typename T, int P, int Q, int QS, bool HAS_Y, bool KMM>
__global__ __launch_bounds__(256, 2) void kron_step_mfma_kernel(const StepArgs a, const uint32_t tilesPerRow,
                                                                const uint32_t totalTiles) {
  using M16 = Mfma16<T>;
  using Acc = typename M16::Acc;
  constexpr int PC = P / 4;              // products per tile and elements per lane
  constexpr int NB = Q / 16 / QS;        // 16-column blocks per wave task
  constexpr int VE = 16 / sizeof(T);     // elements per 128-bit load
  typedef T VT __attribute__((ext_vector_type(VE)));
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);      // wave-uniform: keeps row addresses in SGPRs
  const int lo = l & 15, hi = l >> 4;
  const uint32_t bt = blockIdx.y;
  const uint64_t S = a.Kin / P;

  const T* inB = (const T*)a.in + (size_t)bt * a.in_batch;
  T* outB = (T*)a.out + (size_t)bt * a.out_batch;
  const T* F = (const T*)a.f[0] + (size_t)bt * a.f_batch[0];
  const T* YB = HAS_Y ? (const T*)a.y + (size_t)bt * a.y_batch : nullptr;

  const T alpha = (T)a.alpha, beta = (T)a.beta;
  // wave tasks: the QS column parts of a tile go to QS different waves, a wave keeps its part for life
  // Workgroups are dispatched round-robin over the 8 XCDs (each with its own L2): renumber them so that
  // consecutive ids, which share tiles when QS > kStepWaves and walk neighbouring tiles otherwise, sit on
  // one XCD.
  const uint32_t wg = (gridDim.x % 8 == 0) ? (blockIdx.x % 8) * (gridDim.x / 8) + blockIdx.x / 8 : blockIdx.x;
  const uint32_t gw = wg * kStepWaves + w;
  const uint32_t qpart = gw % QS, q0 = qpart * (Q / QS);
  const uint32_t waveId = gw / QS, nWaves = (gridDim.x * kStepWaves) / QS;

  // the factor columns of this wave as A operands, resident in registers:
  // fa[c][ib] = F[PC*hi + c][q0 + 16*ib + lo]
  T fa[PC][NB];
#pragma unroll
  for (int c = 0; c < PC; c++)
#pragma unroll
    for (int ib = 0; ib < NB; ib++)
      fa[c][ib] = F[(int64_t)(PC * hi + c) * a.f_sp[0] + (int64_t)(q0 + 16 * ib + lo) * a.f_sq[0]];

  auto loadTile = [&](uint32_t t, T (&x)[PC]) {
    if (KMM) {
      const uint64_t s = t / tilesPerRow;
      const uint32_t m0 = (t % tilesPerRow) * 16;
      const uint32_t m = (m0 + lo < a.M) ? m0 + lo : m0;
      const T* xp = inB + m + (s * P + PC * hi) * (uint64_t)a.in_ldc;
#pragma unroll
      for (int c = 0; c < PC; c++) x[c] = xp[(uint64_t)c * a.in_ldc];
      return;
    }
    const uint32_t m = t / tilesPerRow;
    const uint64_t s0 = (uint64_t)(t % tilesPerRow) * 16;
    const uint64_t s = (s0 + lo < S) ? s0 + lo : s0;
    const T* xp = inB + (size_t)m * a.in_ldm + s * P + PC * hi;
#pragma unroll
    for (int c = 0; c < PC; c += VE) {
      const VT v = *(const VT*)(xp + c);
#pragma unroll
      for (int e = 0; e < VE; e++) x[c + e] = v[e];
    }
  };

  // Loads and stores retire through one in-order counter, and the wait for the prefetched tile is counted in younger
  // operations: the number of stores behind the prefetch must be the same on every path into that wait, or the
  // compiler has to drain them all, which leaves a tile's stores uncovered by the next tile's products.  For 128x128
  // factors (64 to 128 products per tile) nothing is conditional therefore: lanes beyond the end of a ragged tile
  // work on a copy of the tile's first slice (column) and store the same values to the same places as its first
  // lane, the last tile of a wave prefetches itself again, and the first tile is peeled off the loop (sgemkm
  // 1024 x 128^2: 136.9 -> 119.7 us).  The smaller factors lose with stores kept in flight (32x32: 7 to 11 %) and
  // keep the guarded loop below.
  T xn[PC];
  if constexpr (P >= 128) {
    auto nextOf = [&](uint32_t t) { return t + nWaves < totalTiles ? t + nWaves : t; };
    auto computeTile = [&](uint32_t t) {
      T x[PC];
#pragma unroll
      for (int c = 0; c < PC; c++) x[c] = xn[c];
      loadTile(nextOf(t), xn);                                     // next tile streams in under the products

      Acc acc[NB];
#pragma unroll
      for (int ib = 0; ib < NB; ib++) acc[ib] = (Acc){0, 0, 0, 0};
#pragma unroll
      for (int c = 0; c < PC; c++)
#pragma unroll
        for (int ib = 0; ib < NB; ib++) acc[ib] = M16::mma(fa[c][ib], x[c], acc[ib]);

      // element (q, tile lane) of the output lives at out + q*qStride (+ the lane's own offset, in `out`)
      T* out;
      const T* Y = nullptr;
      uint64_t qStride, yStride = 0;
      if (KMM) {
        const uint64_t s = t / tilesPerRow;
        const uint32_t m0 = (t % tilesPerRow) * 16;
        const uint32_t m = (m0 + lo < a.M) ? m0 + lo : m0;
        out = outB + m + s * (uint64_t)a.out_ldc;
        qStride = S * (uint64_t)a.out_ldc;
        if (HAS_Y) { Y = YB + m + s * (uint64_t)a.y_ldc; yStride = S * (uint64_t)a.y_ldc; }
      } else {
        const uint32_t m = t / tilesPerRow;
        const uint64_t s0 = (uint64_t)(t % tilesPerRow) * 16;
        const uint64_t s = (s0 + lo < S) ? s0 + lo : s0;
        out = outB + (size_t)m * a.out_ldm + s;
        qStride = S;
        if (HAS_Y) { Y = YB + (size_t)m * a.y_ldm + s; yStride = S; }
      }
      // all Y loads of the tile before its first store
      T yv[HAS_Y ? NB : 1][4];
      if (HAS_Y) {
#pragma unroll
        for (int ib = 0; ib < NB; ib++)
#pragma unroll
          for (int r = 0; r < 4; r++) yv[ib][r] = Y[(uint64_t)(q0 + 16 * ib + M16::row(r, hi)) * yStride];
      }
      const T scale = a.epilogue ? alpha : (T)1;                   // multiplying by 1 is exact
#pragma unroll
      for (int ib = 0; ib < NB; ib++)
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const uint64_t col = (uint64_t)(q0 + 16 * ib + M16::row(r, hi)) * qStride;
          T v = acc[ib][r] * scale;
          if (HAS_Y) v += beta * yv[ib][r];
          out[col] = v;
        }
    };
    if (waveId >= totalTiles) return;
    loadTile(waveId, xn);
    computeTile(waveId);
    for (uint32_t t = waveId + nWaves; t < totalTiles; t += nWaves) computeTile(t);
    return;
  }

  if (waveId < totalTiles) loadTile(waveId, xn);
  for (uint32_t t = waveId; t < totalTiles; t += nWaves) {
    T x[PC];
#pragma unroll
    for (int c = 0; c < PC; c++) x[c] = xn[c];
    if (t + nWaves < totalTiles) loadTile(t + nWaves, xn);       // next tile streams in under the products

    Acc acc[NB];
#pragma unroll
    for (int ib = 0; ib < NB; ib++) acc[ib] = (Acc){0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < PC; c++)
#pragma unroll
      for (int ib = 0; ib < NB; ib++) acc[ib] = M16::mma(fa[c][ib], x[c], acc[ib]);

    // element (q, tile lane) of the output lives at out + q*qStride (+ the lane's own offset, in `out`)
    T* out;
    const T* Y = nullptr;
    uint64_t qStride, yStride = 0;
    if (KMM) {
      const uint64_t s = t / tilesPerRow;
      const uint32_t m = (t % tilesPerRow) * 16 + lo;
      if (m >= a.M) continue;
      out = outB + m + s * (uint64_t)a.out_ldc;
      qStride = S * (uint64_t)a.out_ldc;
      if (HAS_Y) { Y = YB + m + s * (uint64_t)a.y_ldc; yStride = S * (uint64_t)a.y_ldc; }
    } else {
      const uint32_t m = t / tilesPerRow;
      const uint64_t s = (uint64_t)(t % tilesPerRow) * 16 + lo;
      if (s >= S) continue;
      out = outB + (size_t)m * a.out_ldm + s;
      qStride = S;
      if (HAS_Y) { Y = YB + (size_t)m * a.y_ldm + s; yStride = S; }
    }
    // all Y loads of the tile before its first store (loads and stores share one in-order counter)
    T yv[HAS_Y ? NB : 1][4];
    if (HAS_Y) {
#pragma unroll
      for (int ib = 0; ib < NB; ib++)
#pragma unroll
        for (int r = 0; r < 4; r++) yv[ib][r] = Y[(uint64_t)(q0 + 16 * ib + M16::row(r, hi)) * yStride];
    }
#pragma unroll
    for (int ib = 0; ib < NB; ib++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const uint64_t col = (uint64_t)(q0 + 16 * ib + M16::row(r, hi)) * qStride;
        T v = acc[ib][r];
        if (a.epilogue) {
          v *= alpha;
          if (HAS_Y) v += beta * yv[ib][r];
        }
        out[col] = v;
      }
  }
}

// KMM layout: the M index is the contiguous one (and there is more than one row)
static bool stepMfmaIsKmm(const StepArgs& a) { return a.in_ldm == 1 && a.in_ldc != 1; }

bool stepMfmaSupported(const StepArgs& a, DType dt) {
  if (a.nf != 1) return false;
  const uint32_t P = a.p[0], Q = a.q[0];
  if (!((P == 128 && Q == 128) || (P == 64 && Q == 64) || (P == 32 && Q == 32) || (P == 16 && Q == 16))) return false;
  if (a.Kin % P) return false;
  const uint64_t S = a.Kin / P;
  if (stepMfmaIsKmm(a)) {
    if (a.out_ldm != 1 || (a.y && a.y_ldm != 1)) return false;
    return S * ((a.M + 15) / 16) < (1ull << 31) && a.batch <= 65535;
  }
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  // 16-byte alignment of every slice for the 128-bit loads
  const uint64_t vmask = 16 / dtypeSize(dt) - 1;
  if (((uintptr_t)a.in & 15) || ((uint64_t)a.in_ldm & vmask) || (a.in_batch & vmask)) return false;
  const uint64_t tiles = (S + 15) / 16;
  return tiles * a.M < (1ull << 31) && a.batch <= 65535;
}

template <typename T, int P, int Q, int QS>
static hipError_t launchStepMfmaT(const StepArgs& a, hipStream_t stream) {
  const uint64_t S = a.Kin / P;
  const bool kmm = stepMfmaIsKmm(a);
  const uint32_t tilesPerRow = kmm ? (a.M + 15) / 16 : (uint32_t)((S + 15) / 16);
  const uint32_t totalTiles = kmm ? (uint32_t)(tilesPerRow * S) : tilesPerRow * a.M;
  const int cus = deviceCUs();
  // persistent workgroups: 2 per CU (8 waves, 2 per SIMD at up to 256 VGPRs), fewer when there is not enough work
  uint32_t wgs = (uint32_t)cus * 2;
  if (a.batch > 1) wgs = (wgs + a.batch - 1) / a.batch;         // the batch index is the second grid dimension
  if (wgs < (uint32_t)(QS + kStepWaves - 1) / kStepWaves) wgs = (QS + kStepWaves - 1) / kStepWaves;
  const uint32_t need = (totalTiles * QS + kStepWaves - 1) / kStepWaves;
  if (wgs > need) wgs = need;
  static_assert(kStepWaves % QS == 0 || QS % kStepWaves == 0, "wave tasks must tile the workgroups");
  if (QS > kStepWaves) wgs = (wgs + QS / kStepWaves - 1) / (QS / kStepWaves) * (QS / kStepWaves);
  if (wgs >= 64) wgs = wgs / 8 * 8;      // a multiple of the XCD count keeps the renumbering on
  dim3 grid(wgs, a.batch), block(256);
  const bool y = a.y && a.epilogue;
  if (kmm) {
    if (y) hipLaunchKernelGGL((kron_step_mfma_kernel<T, P, Q, QS, true, true>), grid, block, 0, stream, a, tilesPerRow, totalTiles);
    else   hipLaunchKernelGGL((kron_step_mfma_kernel<T, P, Q, QS, false, true>), grid, block, 0, stream, a, tilesPerRow, totalTiles);
  } else {
    if (y) hipLaunchKernelGGL((kron_step_mfma_kernel<T, P, Q, QS, true, false>), grid, block, 0, stream, a, tilesPerRow, totalTiles);
    else   hipLaunchKernelGGL((kron_step_mfma_kernel<T, P, Q, QS, false, false>), grid, block, 0, stream, a, tilesPerRow, totalTiles);
  }
  return hipGetLastError();
}

hipError_t launchStepMfma(const StepArgs& a, DType dt, hipStream_t stream) {
  if (!stepMfmaSupported(a, dt)) return hipErrorInvalidValue;
  if (dt == DType::F64) {
    switch (a.p[0]) {
      case 16:  return launchStepMfmaT<double, 16, 16, 1>(a, stream);
      case 32:  return launchStepMfmaT<double, 32, 32, 1>(a, stream);
      case 64:  return launchStepMfmaT<double, 64, 64, 1>(a, stream);
      case 128: return launchStepMfmaT<double, 128, 128, 8>(a, stream);
    }
  } else {
    switch (a.p[0]) {
      case 16:  return launchStepMfmaT<float, 16, 16, 1>(a, stream);
      case 32:  return launchStepMfmaT<float, 32, 32, 1>(a, stream);
      case 64:  return launchStepMfmaT<float, 64, 64, 1>(a, stream);
      case 128: return launchStepMfmaT<float, 128, 128, 2>(a, stream);
    }
  }
  return hipErrorInvalidValue;
}

}  // namespace fk
