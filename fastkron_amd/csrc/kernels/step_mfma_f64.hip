// One sliced-multiply step with a square fp64 factor (P = Q in {16, 32, 64}), MKM layout, on the
// fp64 matrix cores (V_MFMA_F64_16X16X4_F64).  Used per factor for shapes like dgemkm 256 x 262144
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
//   * accumulator layout (register q/4, lane 16*(q%4) + slice): each quarter wave stores 16
//     consecutive doubles (one 128-byte line) straight into the shuffled layout out[q*S + s].
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

#define MFMA16D(a, b, c) __builtin_amdgcn_mfma_f64_16x16x4f64((a), (b), (c), 0, 0, 0)

constexpr int kF64Waves = 4;             // waves per workgroup

template <int P, int Q, bool HAS_Y>
__global__ __launch_bounds__(256, 2) void kron_step_mfma_f64_kernel(const StepArgs a, const uint32_t tilesPerRow,
                                                                    const uint32_t totalTiles) {
  constexpr int PC = P / 4;              // products per tile and doubles per lane
  constexpr int NB = Q / 16;
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);      // wave-uniform: keeps row addresses in SGPRs
  const int lo = l & 15, hi = l >> 4;
  const uint32_t bt = blockIdx.y;
  const uint64_t S = a.Kin / P;

  const double* inB = (const double*)a.in + (size_t)bt * a.in_batch;
  double* outB = (double*)a.out + (size_t)bt * a.out_batch;
  const double* F = (const double*)a.f[0] + (size_t)bt * a.f_batch[0];
  const double* YB = HAS_Y ? (const double*)a.y + (size_t)bt * a.y_batch : nullptr;

  // the whole factor as A operands, resident in registers: fa[c][ib] = F[PC*hi + c][16*ib + lo]
  double fa[PC][NB];
#pragma unroll
  for (int c = 0; c < PC; c++)
#pragma unroll
    for (int ib = 0; ib < NB; ib++)
      fa[c][ib] = F[(int64_t)(PC * hi + c) * a.f_sp[0] + (int64_t)(16 * ib + lo) * a.f_sq[0]];

  const double alpha = a.alpha, beta = a.beta;
  const uint32_t waveId = blockIdx.x * kF64Waves + w, nWaves = gridDim.x * kF64Waves;

  auto loadTile = [&](uint32_t t, double (&x)[PC]) {
    const uint32_t m = t / tilesPerRow;
    const uint64_t s0 = (uint64_t)(t % tilesPerRow) * 16;
    const uint64_t s = (s0 + lo < S) ? s0 + lo : s0;
    const double* xp = inB + (size_t)m * a.in_ldm + s * P + PC * hi;
#pragma unroll
    for (int c = 0; c < PC; c += 2) {
      const double2 v = *(const double2*)(xp + c);
      x[c] = v.x; x[c + 1] = v.y;
    }
  };

  double xn[PC];
  if (waveId < totalTiles) loadTile(waveId, xn);
  for (uint32_t t = waveId; t < totalTiles; t += nWaves) {
    double x[PC];
#pragma unroll
    for (int c = 0; c < PC; c++) x[c] = xn[c];
    if (t + nWaves < totalTiles) loadTile(t + nWaves, xn);       // next tile streams in under the products

    d4 acc[NB];
#pragma unroll
    for (int ib = 0; ib < NB; ib++) acc[ib] = (d4){0.0, 0.0, 0.0, 0.0};
#pragma unroll
    for (int c = 0; c < PC; c++)
#pragma unroll
      for (int ib = 0; ib < NB; ib++) acc[ib] = MFMA16D(fa[c][ib], x[c], acc[ib]);

    const uint32_t m = t / tilesPerRow;
    const uint64_t s = (uint64_t)(t % tilesPerRow) * 16 + lo;
    if (s >= S) continue;
    double* out = outB + (size_t)m * a.out_ldm;
    const double* Y = HAS_Y ? YB + (size_t)m * a.y_ldm : nullptr;
    // all Y loads of the tile before its first store (loads and stores share one in-order counter)
    double yv[HAS_Y ? NB : 1][4];
    if (HAS_Y) {
#pragma unroll
      for (int ib = 0; ib < NB; ib++)
#pragma unroll
        for (int r = 0; r < 4; r++) yv[ib][r] = Y[(uint64_t)(16 * ib + 4 * r + hi) * S + s];
    }
#pragma unroll
    for (int ib = 0; ib < NB; ib++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        const uint64_t col = (uint64_t)(16 * ib + 4 * r + hi) * S + s;
        double v = acc[ib][r];
        if (a.epilogue) {
          v *= alpha;
          if (HAS_Y) v += beta * yv[ib][r];
        }
        out[col] = v;
      }
  }
}

bool stepMfmaF64Supported(const StepArgs& a) {
  if (a.nf != 1) return false;
  const uint32_t P = a.p[0], Q = a.q[0];
  if (!((P == 64 && Q == 64) || (P == 32 && Q == 32) || (P == 16 && Q == 16))) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  if (a.Kin % P) return false;
  // 16-byte alignment of every slice for the 128-bit loads
  if (((uintptr_t)a.in & 15) || (a.in_ldm & 1) || (a.in_batch & 1)) return false;
  const uint64_t S = a.Kin / P;
  const uint64_t tiles = (S + 15) / 16;
  return tiles * a.M < (1ull << 31) && a.batch <= 65535;
}

template <int P, int Q>
static hipError_t launchStepMfmaF64T(const StepArgs& a, hipStream_t stream) {
  const uint64_t S = a.Kin / P;
  const uint32_t tilesPerRow = (uint32_t)((S + 15) / 16);
  const uint32_t totalTiles = tilesPerRow * a.M;
  const size_t ldsBytes = 0;
  static int cus = 0;
  if (!cus) {
    int dev = 0;
    hipDeviceProp_t prop;
    cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
              ? prop.multiProcessorCount : 256;
  }
  // persistent workgroups: 2 per CU (8 waves, 2 per SIMD at up to 256 VGPRs), fewer when there is not enough work
  uint32_t wgs = (uint32_t)cus * 2;
  const uint32_t need = (totalTiles + kF64Waves - 1) / kF64Waves;
  if (wgs > need) wgs = need;
  dim3 grid(wgs, a.batch), block(256);
  if (a.y && a.epilogue)
    hipLaunchKernelGGL((kron_step_mfma_f64_kernel<P, Q, true>), grid, block, ldsBytes, stream, a, tilesPerRow, totalTiles);
  else
    hipLaunchKernelGGL((kron_step_mfma_f64_kernel<P, Q, false>), grid, block, ldsBytes, stream, a, tilesPerRow, totalTiles);
  return hipGetLastError();
}

hipError_t launchStepMfmaF64(const StepArgs& a, hipStream_t stream) {
  if (!stepMfmaF64Supported(a)) return hipErrorInvalidValue;
  switch (a.p[0]) {
    case 16:  return launchStepMfmaF64T<16, 16>(a, stream);
    case 32:  return launchStepMfmaF64T<32, 32>(a, stream);
    case 64:  return launchStepMfmaF64T<64, 64>(a, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace fk
