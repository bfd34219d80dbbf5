// One sliced-multiply step with a large square-ish fp64 factor (P = Q in {16, 32, 64}),
// MKM layout, on the fp64 matrix cores (V_MFMA_F64_16X16X4_F64).  Used per factor for shapes like
// dgemkm 256 x 262144 with 64x64^3, where every step is a real (M*Kin/P) x P x Q contraction.
//
//   out[m, q*S + s] = sum_p in[m, s*P + p] * F[p, q],   S = Kin / P
//
// A workgroup (4 wave64s) owns TS = 64 consecutive slices of one row: a contiguous TS*P block of the
// input.  The block and the factor are staged in LDS (row strides padded to an odd number of doubles,
// so the 16 lanes served per LDS cycle hit 16 distinct bank pairs).  The product is computed
// transposed, D[q][slice] = sum_p F^T[q][p] * X^T[p][slice], so that the accumulator layout
// (register q/4, lane 16*(q%4) + slice) stores 16 consecutive doubles (a full 128-byte line) per
// quarter wave straight into the shuffled output layout out[q*S + s]; no transpose pass exists.
// alpha / beta*Y are applied in the same store when this is the launch that writes Z.
//
// Role of the reference's CUDA kernel for large factors (reference src/kernels/cuda/kernel.cuh:53-224,
// which uses CUDA cores only, reference README.md:44-48); the tiling, the use of MFMA and the
// transposed accumulation are specific to this kernel.
// Algorithmic traffic per launch: read M*Kin, write M*Kout elements (+ M*Kout for Y on the last step).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef double d4 __attribute__((ext_vector_type(4)));

#define MFMA16D(a, b, c) __builtin_amdgcn_mfma_f64_16x16x4f64((a), (b), (c), 0, 0, 0)

constexpr int kTS = 64;                  // slices per workgroup

template <int P, int Q, bool HAS_Y>
__global__ __launch_bounds__(256, 2) void kron_step_mfma_f64_kernel(const StepArgs a, const uint32_t sTiles) {
  constexpr int RX = P + 1;              // padded row strides (doubles)
  constexpr int RF = Q + 1;
  extern __shared__ double ldsd[];
  double* xs = ldsd;                     // [kTS][RX]
  double* fs = ldsd + kTS * RX;          // [P][RF]
  const int tid = threadIdx.x;
  const int l = tid & 63, w = tid >> 6;
  const int lo = l & 15, hi = l >> 4;
  const uint32_t st = blockIdx.x % sTiles, m = blockIdx.x / sTiles, bt = blockIdx.y;
  const uint64_t S = a.Kin / P;
  const uint64_t s0 = (uint64_t)st * kTS;

  const double* in = (const double*)a.in + (size_t)bt * a.in_batch + (size_t)m * a.in_ldm + s0 * P;
  double* out = (double*)a.out + (size_t)bt * a.out_batch + (size_t)m * a.out_ldm;
  const double* F = (const double*)a.f[0] + (size_t)bt * a.f_batch[0];

  // ---- stage the input block (contiguous kTS*P doubles) and the factor ----
  const uint32_t nS = (S - s0 < (uint64_t)kTS) ? (uint32_t)(S - s0) : kTS;   // valid slices in this tile
  for (int e = tid * 2; e < kTS * P; e += 512) {
    const int j = e / P, p = e % P;
    double2 v = make_double2(0.0, 0.0);
    if ((uint32_t)j < nS) v = *(const double2*)(in + e);
    xs[j * RX + p] = v.x;
    xs[j * RX + p + 1] = v.y;
  }
  for (int e = tid; e < P * Q; e += 256) {
    const int p = e / Q, q = e % Q;
    fs[p * RF + q] = F[(int64_t)p * a.f_sp[0] + (int64_t)q * a.f_sq[0]];
  }
  __syncthreads();

  // ---- each wave: 16 slices x Q outputs ----
  constexpr int NB = Q / 16;
  d4 acc[NB];
#pragma unroll
  for (int ib = 0; ib < NB; ib++) acc[ib] = (d4){0.0, 0.0, 0.0, 0.0};
  const double* xw = xs + (16 * w + lo) * RX + hi;          // B[k][j]: slice 16w+j, p = 4c + k
  const double* fw = fs + hi * RF + lo;                     // A[i][k]: q = 16ib + i, p = 4c + k
#pragma unroll 4
  for (int c = 0; c < P / 4; c++) {
    const double b = xw[4 * c];
#pragma unroll
    for (int ib = 0; ib < NB; ib++) acc[ib] = MFMA16D(fw[(4 * c) * RF + 16 * ib], b, acc[ib]);
  }

  // ---- store: acc[ib][r] is q = 16ib + 4r + hi, slice = s0 + 16w + lo ----
  const uint64_t s = s0 + 16 * w + lo;
  if (s >= S) return;
  const double alpha = a.alpha, beta = a.beta;
  const double* Y = HAS_Y ? (const double*)a.y + (size_t)bt * a.y_batch + (size_t)m * a.y_ldm : nullptr;
#pragma unroll
  for (int ib = 0; ib < NB; ib++)
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const uint64_t col = (uint64_t)(16 * ib + 4 * r + hi) * S + s;
      double v = acc[ib][r];
      if (a.epilogue) {
        v *= alpha;
        if (HAS_Y) v += beta * Y[col];
      }
      out[col] = v;
    }
}

bool stepMfmaF64Supported(const StepArgs& a) {
  if (a.nf != 1) return false;
  const uint32_t P = a.p[0], Q = a.q[0];
  if (!((P == 64 && Q == 64) || (P == 32 && Q == 32) || (P == 16 && Q == 16))) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  if (a.Kin % P) return false;
  // 16-byte alignment of every input block for the double2 loads
  if (((uintptr_t)a.in & 15) || (a.in_ldm & 1) || (a.in_batch & 1)) return false;
  const uint64_t S = a.Kin / P;
  const uint64_t tiles = (S + kTS - 1) / kTS;
  return tiles * a.M < (1ull << 31) && a.batch <= 65535;
}

template <int P, int Q>
static hipError_t launchStepMfmaF64T(const StepArgs& a, hipStream_t stream) {
  const uint64_t S = a.Kin / P;
  const uint32_t sTiles = (uint32_t)((S + kTS - 1) / kTS);
  const size_t ldsBytes = (size_t)(kTS * (P + 1) + P * (Q + 1)) * sizeof(double);
  static bool attrSet = false;
  if (!attrSet && ldsBytes > 65536) {
    hipError_t e = hipFuncSetAttribute((const void*)kron_step_mfma_f64_kernel<P, Q, true>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute((const void*)kron_step_mfma_f64_kernel<P, Q, false>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
    if (e != hipSuccess) return e;
    attrSet = true;
  }
  dim3 grid(sTiles * a.M, a.batch), block(256);
  if (a.y && a.epilogue)
    hipLaunchKernelGGL((kron_step_mfma_f64_kernel<P, Q, true>), grid, block, ldsBytes, stream, a, sTiles);
  else
    hipLaunchKernelGGL((kron_step_mfma_f64_kernel<P, Q, false>), grid, block, ldsBytes, stream, a, sTiles);
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
