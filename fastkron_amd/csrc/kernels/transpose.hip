// Transposed copy of X, batched: in is R x C row-major (element (r, c) at r*C + c), out is C x R.  Used ahead of the
// first launch when op(X) = T and the plan for the untransposed problem is enough faster than the kernels that read
// a transposed X directly (the whole-row kernels need their rows contiguous); the reference transposes X inside the
// first launch of any kernel (reference src/kmm/kmmalgo.cpp:186-190, src/kernels/cuda/shared-loads.cuh:4-88).
//
// A workgroup moves a tile of TR x TC elements through LDS (TC = min(C, 64) rounded up to a power of two,
// TR * TC = 4096): lanes run along c when reading (contiguous, or the whole tile contiguous when C <= 64) and along
// r when writing (TR >= 64 contiguous elements); the LDS rows are padded by one element, so both sides are free of
// bank conflicts.  Algorithmic traffic: R*C elements read and written.
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

constexpr int kTrTile = 4096;

template <typename T>
__global__ __launch_bounds__(256) void kron_transpose_kernel(const T* __restrict__ in, T* __restrict__ out, uint32_t R,
                                                             uint32_t C, uint32_t tcLog, uint32_t tilesC,
                                                             uint64_t inBatch, uint64_t outBatch) {
  __shared__ T tile[kTrTile + kTrTile / 4];            // TR rows of TC + 1 elements, TC >= 4
  const uint32_t TC = 1u << tcLog, TR = kTrTile >> tcLog;
  const uint32_t tr = blockIdx.x / tilesC, tc = blockIdx.x % tilesC;
  const uint32_t r0 = tr * TR, c0 = tc * TC;
  const T* src = in + (size_t)blockIdx.y * inBatch;
  T* dst = out + (size_t)blockIdx.y * outBatch;
  for (uint32_t i = threadIdx.x; i < (uint32_t)kTrTile; i += 256) {
    const uint32_t r = i >> tcLog, c = i & (TC - 1);
    if (r0 + r < R && c0 + c < C) tile[r * (TC + 1) + c] = src[(size_t)(r0 + r) * C + c0 + c];
  }
  __syncthreads();
  const uint32_t trLog = 12 - tcLog;
  for (uint32_t i = threadIdx.x; i < (uint32_t)kTrTile; i += 256) {
    const uint32_t c = i >> trLog, r = i & (TR - 1);
    if (r0 + r < R && c0 + c < C) dst[(size_t)(c0 + c) * R + r0 + r] = tile[r * (TC + 1) + c];
  }
}

hipError_t launchTranspose(const void* in, void* out, uint32_t R, uint32_t C, uint32_t batch, uint64_t inBatch,
                           uint64_t outBatch, DType dt, hipStream_t stream) {
  if (R == 0 || C == 0 || batch == 0 || batch > 65535) return hipErrorInvalidValue;
  uint32_t tcLog = 2;
  while (tcLog < 6 && (1u << tcLog) < C) tcLog++;
  const uint32_t TC = 1u << tcLog, TR = kTrTile >> tcLog;
  const uint64_t tilesC = (C + TC - 1) / TC, tilesR = (R + TR - 1) / TR;
  if (tilesC * tilesR >= (1ull << 31)) return hipErrorInvalidValue;
  dim3 grid((uint32_t)(tilesC * tilesR), batch), block(256);
  if (dt == DType::F32)
    hipLaunchKernelGGL(kron_transpose_kernel<float>, grid, block, 0, stream, (const float*)in, (float*)out, R, C, tcLog,
                       (uint32_t)tilesC, inBatch, outBatch);
  else
    hipLaunchKernelGGL(kron_transpose_kernel<double>, grid, block, 0, stream, (const double*)in, (double*)out, R, C, tcLog,
                       (uint32_t)tilesC, inBatch, outBatch);
  return hipGetLastError();
}

}  // namespace fk
