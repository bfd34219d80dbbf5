// Kronecker products of adjacent small factors, computed on the device into the handle's workspace:
// (F_i x F_{i+1} x ...) replaces its sources in the chain, which is exact algebra (the Kronecker product is
// associative), so that chains of 2x2 / 4x4 (and, in fp64, 8x8) factors run on the kernels built for 16x16
// and 64x64 factors instead of one generic launch per factor.
//
//   M[(p_0..p_{c-1}), (q_0..q_{c-1})] = prod_j F_j[p_j, q_j]      (source 0 owns the slowest digit)
//
// One workgroup per merged factor; sources are read through their strides (which absorb MKM/KMM storage and
// opF), the result is written with the same storage convention, so the merged chain keeps the call's opF.
// The reference has no counterpart: it compiles kernels per factor shape instead (reference
// src/kernels/best-kernels/*).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

template <typename T>
__global__ __launch_bounds__(256) void kron_merge_kernel(const MergeArgs a) {
  const MergeGroup g = a.g[blockIdx.x];
  uint32_t P = 1, Q = 1;
  for (uint32_t j = 0; j < g.count; j++) { P *= g.p[j]; Q *= g.q[j]; }
  T* dst = (T*)g.dst;
  for (uint32_t e = threadIdx.x; e < P * Q; e += 256) {
    uint32_t p = e / Q, q = e % Q;
    const uint32_t p0 = p, q0 = q;
    T v = (T)1;
    for (int j = (int)g.count - 1; j >= 0; j--) {          // the last source owns the fastest digit
      const uint32_t pj = p % g.p[j], qj = q % g.q[j];
      p /= g.p[j]; q /= g.q[j];
      v *= ((const T*)g.src[j])[(int64_t)pj * g.sp[j] + (int64_t)qj * g.sq[j]];
    }
    dst[(int64_t)p0 * g.dsp + (int64_t)q0 * g.dsq] = v;
  }
}

// Fills a buffer with values spread over [-1, 1] (a hash of the index): what the tuner times kernels on.  Zeros or a
// constant would let the device clock higher than real data does.
template <typename T>
__global__ __launch_bounds__(256) void kron_fill_kernel(T* dst, size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) {
    uint32_t h = (uint32_t)i * 2654435761u + (uint32_t)(i >> 32) * 40503u;
    h ^= h >> 15; h *= 2246822519u; h ^= h >> 13;
    dst[i] = (T)((double)(h & 0xffffff) / 8388608.0 - 1.0);
  }
}

hipError_t launchFill(void* dst, size_t elems, DType dt, hipStream_t stream) {
  if (elems == 0) return hipSuccess;
  const size_t want = (elems + 255) / 256;
  const uint32_t grid = want < 4096 ? (uint32_t)want : 4096;
  if (dt == DType::F32) hipLaunchKernelGGL(kron_fill_kernel<float>, dim3(grid), dim3(256), 0, stream, (float*)dst, elems);
  else                  hipLaunchKernelGGL(kron_fill_kernel<double>, dim3(grid), dim3(256), 0, stream, (double*)dst, elems);
  return hipGetLastError();
}

hipError_t launchMergeFactors(const MergeArgs& a, DType dt, hipStream_t stream) {
  if (a.groups == 0 || a.groups > kMaxMergeGroups) return hipErrorInvalidValue;
  if (dt == DType::F32) hipLaunchKernelGGL(kron_merge_kernel<float>, dim3(a.groups), dim3(256), 0, stream, a);
  else                  hipLaunchKernelGGL(kron_merge_kernel<double>, dim3(a.groups), dim3(256), 0, stream, a);
  return hipGetLastError();
}

}  // namespace fk
