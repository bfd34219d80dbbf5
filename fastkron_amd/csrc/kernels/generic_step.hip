// Fallback kernel: one sliced-multiply step for any P, Q, strides and operand transposes.
//
//   out[m, q*S + s] = sum_p in[m, s*P + p] * F[p, q],   S = Kin / P
//
// (step semantics as in reference tests/testBase.h:256-283; it plays the role of the reference's
// low-optimisation-level kernels, src/kernels/kernel_opt.h:42-84.)  Every thread owns one (row, slice)
// pair and TQ output columns; the factor chunk is staged in LDS and read as a broadcast.  Lanes run
// along the rows when rows are the contiguous dimension of the input (KMM layout) and along slices
// otherwise, so that stores are coalesced in both layouts.
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

constexpr int kGenThreads = 256;
constexpr int kGenTP = 32;

template <typename T, int TQ, bool LANES_M>
__global__ __launch_bounds__(kGenThreads) void kron_step_generic(const StepArgs a, const uint32_t qTiles) {
  __shared__ T fs[kGenTP][TQ];
  const uint32_t P = a.p[0], Q = a.q[0];
  const uint64_t S = a.Kin / P;
  const uint64_t tile = blockIdx.x / qTiles;
  const uint32_t q0 = (blockIdx.x % qTiles) * TQ;
  const uint32_t b = blockIdx.z;
  const T* in = (const T*)a.in + (size_t)b * a.in_batch;
  T* out = (T*)a.out + (size_t)b * a.out_batch;
  const T* y = a.y ? (const T*)a.y + (size_t)b * a.y_batch : nullptr;
  const T* F = (const T*)a.f[0] + (size_t)b * a.f_batch[0];

  const uint64_t g = tile * kGenThreads + threadIdx.x;
  const bool active = g < (uint64_t)a.M * S;
  uint64_t m, s;
  if (LANES_M) { m = g % a.M; s = g / a.M; } else { s = g % S; m = g / S; }

  T acc[TQ];
#pragma unroll
  for (int i = 0; i < TQ; i++) acc[i] = T(0);

  const T* xrow = in + (int64_t)m * a.in_ldm + (int64_t)(s * P) * a.in_ldc;
  for (uint32_t p0 = 0; p0 < P; p0 += kGenTP) {
    __syncthreads();
    for (int idx = threadIdx.x; idx < kGenTP * TQ; idx += kGenThreads) {
      const uint32_t pp = p0 + idx / TQ, qq = q0 + idx % TQ;
      fs[idx / TQ][idx % TQ] = (pp < P && qq < Q) ? F[(int64_t)pp * a.f_sp[0] + (int64_t)qq * a.f_sq[0]] : T(0);
    }
    __syncthreads();
    if (active) {
      const uint32_t pn = (P - p0 < (uint32_t)kGenTP) ? P - p0 : kGenTP;
      for (uint32_t pp = 0; pp < pn; pp++) {
        const T x = xrow[(int64_t)(p0 + pp) * a.in_ldc];
#pragma unroll
        for (int i = 0; i < TQ; i++) acc[i] += x * fs[pp][i];
      }
    }
  }
  if (!active) return;
  const T alpha = (T)a.alpha, beta = (T)a.beta;
#pragma unroll
  for (int i = 0; i < TQ; i++) {
    const uint32_t q = q0 + i;
    if (q >= Q) break;
    const uint64_t col = (uint64_t)q * S + s;
    T v = acc[i];
    if (a.epilogue) {
      v = alpha * v;
      if (y) v += beta * y[(int64_t)m * a.y_ldm + (int64_t)col * a.y_ldc];
    }
    out[(int64_t)m * a.out_ldm + (int64_t)col * a.out_ldc] = v;
  }
}

template <typename T, bool LANES_M>
static hipError_t launchGenericT(const StepArgs& a, hipStream_t stream) {
  const uint32_t Q = a.q[0];
  const uint64_t S = a.Kin / a.p[0];
  const uint64_t tiles = ((uint64_t)a.M * S + kGenThreads - 1) / kGenThreads;
  int tq = 1;
  while (tq < 16 && (uint32_t)tq < Q) tq *= 2;
  const uint32_t qTiles = (Q + tq - 1) / tq;
  if (tiles * qTiles >= (1ull << 31) || a.batch > 65535) return hipErrorInvalidValue;
  dim3 grid((uint32_t)(tiles * qTiles), 1, a.batch), block(kGenThreads);
  switch (tq) {
    case 1:  hipLaunchKernelGGL((kron_step_generic<T, 1, LANES_M>),  grid, block, 0, stream, a, qTiles); break;
    case 2:  hipLaunchKernelGGL((kron_step_generic<T, 2, LANES_M>),  grid, block, 0, stream, a, qTiles); break;
    case 4:  hipLaunchKernelGGL((kron_step_generic<T, 4, LANES_M>),  grid, block, 0, stream, a, qTiles); break;
    case 8:  hipLaunchKernelGGL((kron_step_generic<T, 8, LANES_M>),  grid, block, 0, stream, a, qTiles); break;
    default: hipLaunchKernelGGL((kron_step_generic<T, 16, LANES_M>), grid, block, 0, stream, a, qTiles); break;
  }
  return hipGetLastError();
}

hipError_t launchGenericStep(const StepArgs& a, DType dt, hipStream_t stream) {
  if (a.nf != 1 || a.M == 0 || a.batch == 0 || a.Kin == 0) return hipErrorInvalidValue;
  const bool lanesM = (a.in_ldm == 1 && a.M > 1);
  if (dt == DType::F32)
    return lanesM ? launchGenericT<float, true>(a, stream) : launchGenericT<float, false>(a, stream);
  return lanesM ? launchGenericT<double, true>(a, stream) : launchGenericT<double, false>(a, stream);
}

}  // namespace fk
