// Copy kernels with the access patterns of the 4x4^6 GeKMM kernels and none of their arithmetic: what the memory
// system gives each pattern is the ceiling of the kernel that has it.  Z = 1.5 X + 0.5 Y on a 4096 x M fp32 matrix
// (M a multiple of 2048), all three operands touched exactly once:
//   0  contiguous: 16 bytes per lane, consecutive lanes on consecutive addresses (what any layout-free kernel could do);
//   1  strips: a workgroup owns 8 columns and all 4096 rows of them, 32 bytes of each row, rows M*4 bytes apart
//      (kmm4x6_mfma.hip);
//   2  two phases: 128 rows x 256 columns per workgroup (256-byte pieces), an intermediate T written and read back
//      through the XCD's L2 between them, 32 workgroups per column block waiting for each other (kmm4x6_twophase.hip).
// Run by `python bench.py --pattern-ceilings`; not used by any gemkm / gekmm call.
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float pp4 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void kron_probe_contiguous_kernel(const float* __restrict__ X, const float* __restrict__ Y,
                                                                    float* __restrict__ Z, size_t n4) {
  for (size_t i = blockIdx.x * (size_t)blockDim.x + threadIdx.x; i < n4; i += (size_t)gridDim.x * blockDim.x) {
    const pp4 x = __builtin_nontemporal_load((const pp4*)X + i), y = __builtin_nontemporal_load((const pp4*)Y + i);
    __builtin_nontemporal_store(x * 1.5f + y * 0.5f, (pp4*)Z + i);
  }
}

__device__ __forceinline__ int ppSpread(int v) { return (v & 1) | ((v & 2) << 1) | ((v & 4) << 2); }

__global__ __launch_bounds__(512) void kron_probe_strips_kernel(const float* __restrict__ X, const float* __restrict__ Y,
                                                                float* __restrict__ Z, uint32_t M) {
  __shared__ float mix[512];
  const int tid = threadIdx.x, l = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t tiles = M / 8;
  const uint32_t tile = (blockIdx.x % 8) * (tiles / 8) + blockIdx.x / 8;      // neighbouring tiles on one XCD
  const uint32_t m = tile * 8 + (l & 7);
  const int coord = (ppSpread(l >> 3) << 1) | ppSpread(w);
  float x[64], y[64];
#pragma unroll
  for (int r = 0; r < 64; r++) {
    const int row = (coord << 6) + (((r & 3) << 4) | ((r >> 2) & 3) | (((r >> 4) & 3) << 2));
    x[r] = X[(size_t)row * M + m];
  }
#pragma unroll
  for (int r = 0; r < 64; r++) y[r] = Y[(size_t)((r << 6) + coord) * M + m];
  // (an exchange between the lanes stands where the kernel has its LDS pass: the stores depend on every load)
  float s = 0.f;
#pragma unroll
  for (int r = 0; r < 64; r++) s += x[r];
  mix[tid] = s;
  __syncthreads();
  const float t = mix[(tid * 7 + 1) & 511] * 1e-30f;
#pragma unroll
  for (int r = 0; r < 64; r++) Z[(size_t)((r << 6) + coord) * M + m] = 1.5f * x[r] + 0.5f * y[r] + t;
}

// at most `n` vector memory operations outstanding
#define PP_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

__global__ __launch_bounds__(256) void kron_probe_twophase_kernel(const float* __restrict__ X, const float* __restrict__ Y,
                                                                  float* __restrict__ Z, float* __restrict__ T,
                                                                  uint32_t* sync, uint32_t M, uint32_t zero) {
  const int tid = threadIdx.x, l = tid & 63, w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = w >> 1, h = w & 1;
  const uint32_t q = (blockIdx.x & 7) + 8 * (blockIdx.x >> 8);                 // column block, all of it on one XCD
  const int j = (blockIdx.x >> 3) & 31;
  uint32_t* const words = sync + 16 + 4 * q;
  const int s = 2 * j + g;
  float xa[64], xb[64], ya[64], yb[64];
  const size_t col = (size_t)q * 256 + h * 64 + l;
  float* const t = T + (size_t)q * (4096 * 256) + h * 64 + l;
#pragma unroll
  for (int r = 0; r < 64; r++) xa[r] = __builtin_nontemporal_load(X + (size_t)(128 * j + 64 * g + r) * M + col);
#pragma unroll
  for (int r = 0; r < 64; r++) xb[r] = __builtin_nontemporal_load(X + (size_t)(128 * j + 64 * g + r) * M + col + 128);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r = 0; r < 64; r++) t[(size_t)r * (64 * 128) + (2 * j + g) * 128] = xa[r];
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r = 0; r < 63; r++) ya[r] = __builtin_nontemporal_load(Y + (size_t)(s + 64 * r) * M + col);
  __builtin_amdgcn_sched_barrier(0);
  PP_WAIT_VM(63);
  __builtin_amdgcn_sched_barrier(0);
  ya[63] = __builtin_nontemporal_load(Y + (size_t)(s + 64 * 63) * M + col);
  __syncthreads();
  if (tid == 0) (void)__hip_atomic_fetch_or(words + 0, 1u << j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r = 0; r < 64; r++) t[(size_t)(64 * 64 * 128) + (size_t)r * (64 * 128) + (2 * j + g) * 128] = xb[r];
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r = 0; r < 63; r++) yb[r] = __builtin_nontemporal_load(Y + (size_t)(s + 64 * r) * M + col + 128);
  __builtin_amdgcn_sched_barrier(0);
  PP_WAIT_VM(63);
  __builtin_amdgcn_sched_barrier(0);
  yb[63] = __builtin_nontemporal_load(Y + (size_t)(s + 64 * 63) * M + col + 128);
  __syncthreads();
  if (tid == 0) (void)__hip_atomic_fetch_or(words + 1, 1u << j, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  auto waitFor = [&](int u) __attribute__((always_inline)) {
    if (tid == 0)
      for (uint32_t spins = 0; spins < (1u << 22) &&
           __hip_atomic_fetch_or(words + u, zero, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) != ~0u; spins++)
        __builtin_amdgcn_s_sleep(4);
    __syncthreads();
  };
  waitFor(0);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r = 0; r < 64; r++) xa[r] = t[(size_t)s * (64 * 128) + r * 128];
#pragma unroll
  for (int r = 0; r < 64; r++) __builtin_nontemporal_store(1.5f * xa[r] + 0.5f * ya[r], Z + (size_t)(s + 64 * r) * M + col);
  __builtin_amdgcn_sched_barrier(0);
  waitFor(1);
  uint32_t through = 0;
  if (tid == 0) through = __hip_atomic_fetch_add(words + 2, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int r = 0; r < 64; r++) xb[r] = t[(size_t)(64 * 64 * 128) + (size_t)s * (64 * 128) + r * 128];
#pragma unroll
  for (int r = 0; r < 64; r++) __builtin_nontemporal_store(1.5f * xb[r] + 0.5f * yb[r], Z + (size_t)(s + 64 * r) * M + col + 128);
  if (tid == 0 && through + 1 == 32u) {
    (void)__hip_atomic_exchange(words + 0, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    (void)__hip_atomic_exchange(words + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    (void)__hip_atomic_exchange(words + 2, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
}

hipError_t launchPatternProbe(int pattern, const float* X, const float* Y, float* Z, float* T, void* sync, uint32_t M,
                              hipStream_t stream) {
  if (M == 0 || M % 2048 || M > 16384 || !X || !Y || !Z) return hipErrorInvalidValue;
  if (pattern == 0) {
    hipLaunchKernelGGL(kron_probe_contiguous_kernel, dim3(8192), dim3(256), 0, stream, X, Y, Z, (size_t)4096 * M / 4);
  } else if (pattern == 1) {
    hipLaunchKernelGGL(kron_probe_strips_kernel, dim3(M / 8), dim3(512), 0, stream, X, Y, Z, M);
  } else if (pattern == 2) {
    if (!T || !sync) return hipErrorInvalidValue;
    hipLaunchKernelGGL(kron_probe_twophase_kernel, dim3(256 * (M / 2048)), dim3(256), 0, stream, X, Y, Z, T, (uint32_t*)sync, M, 0u);
  } else {
    return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace fk
