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

// The same with 16-byte global accesses and square tiles of TD x TD elements (128 x 128 in fp32, 64 x 64 in fp64:
// 512-byte pieces on both sides), for R and C multiples of the vector length and 16-byte aligned buffers.  LDS rows
// are TD + 1 elements, written and read element by element: a wave's writes go to (row, 4*c4 + k) with 16 lanes
// along c4, its reads to (4*r4 + k, col) with 16 lanes along r4, both on 64 distinct banks.
template <typename T, int TD>
__global__ __launch_bounds__(TD == 128 ? 1024 : 256) void kron_transpose_vec_kernel(const T* __restrict__ in, T* __restrict__ out,
                                                                                   uint32_t R, uint32_t C, uint32_t tilesC,
                                                                                   uint64_t inBatch, uint64_t outBatch) {
  constexpr int VE = 16 / sizeof(T), NTH = TD == 128 ? 1024 : 256, VPR = TD / VE;      // vectors per tile row
  typedef T VT __attribute__((ext_vector_type(VE)));
  extern __shared__ __align__(16) unsigned char trLds[];
  T* tile = (T*)trLds;                                                   // TD rows of TD + 1 elements
  const uint32_t tr = blockIdx.x / tilesC, tc = blockIdx.x % tilesC;
  const uint32_t r0 = tr * TD, c0 = tc * TD;
  const T* src = in + (size_t)blockIdx.y * inBatch;
  T* dst = out + (size_t)blockIdx.y * outBatch;
  constexpr int PER = TD * VPR / NTH;
  VT v[PER];
#pragma unroll
  for (int i = 0; i < PER; i++) {
    const uint32_t idx = threadIdx.x + i * NTH, row = idx / VPR, c4 = idx % VPR;
    const bool ok = r0 + row < R && c0 + VE * c4 < C;
    if (ok) v[i] = *(const VT*)(src + (size_t)(r0 + row) * C + c0 + VE * c4);
    else for (int k = 0; k < VE; k++) v[i][k] = (T)0;
  }
#pragma unroll
  for (int i = 0; i < PER; i++) {
    const uint32_t idx = threadIdx.x + i * NTH, row = idx / VPR, c4 = idx % VPR;
#pragma unroll
    for (int k = 0; k < VE; k++) tile[row * (TD + 1) + VE * c4 + k] = v[i][k];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < PER; i++) {
    const uint32_t idx = threadIdx.x + i * NTH, col = idx / VPR, r4 = idx % VPR;
    VT o;
#pragma unroll
    for (int k = 0; k < VE; k++) o[k] = tile[(VE * r4 + k) * (TD + 1) + col];
    if (c0 + col < C && r0 + VE * r4 < R) *(VT*)(dst + (size_t)(c0 + col) * R + r0 + VE * r4) = o;
  }
}

template <typename T, int TD>
static hipError_t launchTransposeVec(const void* in, void* out, uint32_t R, uint32_t C, uint32_t batch, uint64_t inBatch,
                                     uint64_t outBatch, hipStream_t stream) {
  const uint64_t tilesC = (C + TD - 1) / TD, tilesR = (R + TD - 1) / TD;
  if (tilesC * tilesR >= (1ull << 31)) return hipErrorInvalidValue;
  const size_t lds = (size_t)TD * (TD + 1) * sizeof(T);
  static PerDeviceOnce attrOnce;
  const int devIdx = launchDeviceIndex();
  if (!attrOnce.done(devIdx)) {
    hipError_t e = hipFuncSetAttribute((const void*)kron_transpose_vec_kernel<T, TD>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attrOnce.mark(devIdx);
  }
  dim3 grid((uint32_t)(tilesC * tilesR), batch), block(TD == 128 ? 1024 : 256);
  hipLaunchKernelGGL((kron_transpose_vec_kernel<T, TD>), grid, block, lds, stream, (const T*)in, (T*)out, R, C, (uint32_t)tilesC,
                     inBatch, outBatch);
  return hipGetLastError();
}

hipError_t launchTranspose(const void* in, void* out, uint32_t R, uint32_t C, uint32_t batch, uint64_t inBatch,
                           uint64_t outBatch, DType dt, hipStream_t stream) {
  if (R == 0 || C == 0 || batch == 0 || batch > 65535) return hipErrorInvalidValue;
  {
    const uint32_t ve = dt == DType::F32 ? 4 : 2;
    const bool vec = R % ve == 0 && C % ve == 0 && R >= 64 && C >= 64 && (((uintptr_t)in | (uintptr_t)out) & 15) == 0 &&
                     inBatch % ve == 0 && outBatch % ve == 0;
    if (vec) return dt == DType::F32 ? launchTransposeVec<float, 128>(in, out, R, C, batch, inBatch, outBatch, stream)
                                     : launchTransposeVec<double, 64>(in, out, R, C, batch, inBatch, outBatch, stream);
  }
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
