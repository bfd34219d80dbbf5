// Transposed copy of X, batched: in is R x C row-major (element (r, c) at r*C + c), out is C x R.  Used ahead of the
// first launch when op(X) = T and the plan for the untransposed problem is enough faster than the kernels that read
// a transposed X directly (the whole-row kernels need their rows contiguous); the reference transposes X inside the
// first launch of any kernel (reference src/kmm/kmmalgo.cpp:186-190, src/kernels/cuda/shared-loads.cuh:4-88).
//
// A workgroup moves a tile of TR x TC elements through LDS (TC = min(C, 64) rounded up to a power of two,
// TR * TC = 4096): lanes run along c when reading (contiguous, or the whole tile contiguous when C <= 64) and along
// r when writing (TR >= 64 contiguous elements); the LDS rows are padded by one element, so both sides are free of
// bank conflicts.  Algorithmic traffic: R*C elements read and written.
//
// The same kernels finish a GeKMM that ran as the GeMKM of its transposed operands: out = transpose(in) + beta * Y,
// Y laid out like out (HAS_Y).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

constexpr int kTrTile = 4096;

template <typename T, bool HAS_Y>
__global__ __launch_bounds__(256) void kron_transpose_kernel(const T* __restrict__ in, T* out, uint32_t R,
                                                             uint32_t C, uint32_t tcLog, uint32_t tilesC,
                                                             uint64_t inBatch, uint64_t outBatch, const T* y, uint64_t yBatch,
                                                             T beta) {
  __shared__ T tile[kTrTile + kTrTile / 4];            // TR rows of TC + 1 elements, TC >= 4
  const uint32_t TC = 1u << tcLog, TR = kTrTile >> tcLog;
  const uint32_t tr = blockIdx.x / tilesC, tc = blockIdx.x % tilesC;
  const uint32_t r0 = tr * TR, c0 = tc * TC;
  const T* src = in + (size_t)blockIdx.y * inBatch;
  T* dst = out + (size_t)blockIdx.y * outBatch;
  const T* ysrc = HAS_Y ? y + (size_t)blockIdx.y * yBatch : nullptr;
  for (uint32_t i = threadIdx.x; i < (uint32_t)kTrTile; i += 256) {
    const uint32_t r = i >> tcLog, c = i & (TC - 1);
    if (r0 + r < R && c0 + c < C) tile[r * (TC + 1) + c] = src[(size_t)(r0 + r) * C + c0 + c];
  }
  __syncthreads();
  const uint32_t trLog = 12 - tcLog;
  for (uint32_t i = threadIdx.x; i < (uint32_t)kTrTile; i += 256) {
    const uint32_t c = i >> trLog, r = i & (TR - 1);
    if (r0 + r < R && c0 + c < C) {
      T v = tile[r * (TC + 1) + c];
      if (HAS_Y) v += beta * ysrc[(size_t)(c0 + c) * R + r0 + r];
      dst[(size_t)(c0 + c) * R + r0 + r] = v;
    }
  }
}

// The same with 16-byte global accesses on tiles of TDR x TDC elements through LDS, for R and C multiples of the vector
// length and 16-byte aligned buffers: 128 x 128 in fp32 and 64 x 64 in fp64 (512-byte pieces on both sides), and
// tall or wide tiles of 16 KB for matrices with fewer than 64 rows or columns (16 or 32 columns: a tile is one
// contiguous piece of the input and 16 or 32 contiguous pieces of the output; 16 or 32 rows: the reverse).  LDS rows
// are TDC + 1 elements, written and read element by element.
// STREAM: the result goes to the caller and nothing reads it back soon: stores at system scope (launch.h), through a
// descriptor of the tile's span of the output (the launcher checks that it stays below 2 GB).
template <typename T, int TDR, int TDC, bool HAS_Y, bool STREAM>
__global__ __launch_bounds__(TDR * TDC * sizeof(T) >= 65536 ? 1024 : 256) void kron_transpose_vec_kernel(
    const T* __restrict__ in, T* out, uint32_t R, uint32_t C, uint32_t tilesC, uint64_t inBatch, uint64_t outBatch, const T* y,
    uint64_t yBatch, T beta) {
  constexpr int VE = 16 / sizeof(T), NTH = TDR * TDC * sizeof(T) >= 65536 ? 1024 : 256;
  constexpr int VPR = TDC / VE, VPC = TDR / VE;            // vectors per tile row (input side) / per tile column (output side)
  typedef T VT __attribute__((ext_vector_type(VE)));
  extern __shared__ __align__(16) unsigned char trLds[];
  T* tile = (T*)trLds;                                                   // TDR rows of TDC + 1 elements
  const uint32_t tr = blockIdx.x / tilesC, tc = blockIdx.x % tilesC;
  const uint32_t r0 = tr * TDR, c0 = tc * TDC;
  const T* src = in + (size_t)blockIdx.y * inBatch;
  T* dst = out + (size_t)blockIdx.y * outBatch;
  const T* ysrc = HAS_Y ? y + (size_t)blockIdx.y * yBatch : nullptr;
  constexpr int PER = TDR * VPR / NTH;
  static_assert(TDR * VPR % NTH == 0 && PER >= 1, "whole vectors per thread");
  const __amdgpu_buffer_rsrc_t oTarget =
      streamTarget((void*)(dst + (size_t)c0 * R + r0), STREAM ? (uint32_t)(((size_t)(TDC - 1) * R + TDR) * sizeof(T)) : 0u);
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
    for (int k = 0; k < VE; k++) tile[row * (TDC + 1) + VE * c4 + k] = v[i][k];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < PER; i++) {
    const uint32_t idx = threadIdx.x + i * NTH, col = idx / VPC, r4 = idx % VPC;
    VT o;
#pragma unroll
    for (int k = 0; k < VE; k++) o[k] = tile[(VE * r4 + k) * (TDC + 1) + col];
    if (c0 + col < C && r0 + VE * r4 < R) {
      if (HAS_Y) o += beta * *(const VT*)(ysrc + (size_t)(c0 + col) * R + r0 + VE * r4);
      if constexpr (STREAM) streamStore16(o, oTarget, (uint32_t)(((size_t)col * R + VE * r4) * sizeof(T)));
      else *(VT*)(dst + (size_t)(c0 + col) * R + r0 + VE * r4) = o;
    }
  }
}

template <typename T, int TDR, int TDC, bool HAS_Y, bool STREAM>
static hipError_t launchTransposeVec(const void* in, void* out, uint32_t R, uint32_t C, uint32_t batch, uint64_t inBatch,
                                     uint64_t outBatch, const void* y, uint64_t yBatch, double beta, hipStream_t stream) {
  const uint64_t tilesC = (C + TDC - 1) / TDC, tilesR = (R + TDR - 1) / TDR;
  if (tilesC * tilesR >= (1ull << 31)) return hipErrorInvalidValue;
  const size_t lds = (size_t)TDR * (TDC + 1) * sizeof(T);
  static PerDeviceOnce attrOnce;
  const int devIdx = launchDeviceIndex();
  if (!attrOnce.done(devIdx)) {
    hipError_t e = hipFuncSetAttribute((const void*)kron_transpose_vec_kernel<T, TDR, TDC, HAS_Y, STREAM>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    attrOnce.mark(devIdx);
  }
  dim3 grid((uint32_t)(tilesC * tilesR), batch), block(TDR * TDC * sizeof(T) >= 65536 ? 1024 : 256);
  hipLaunchKernelGGL((kron_transpose_vec_kernel<T, TDR, TDC, HAS_Y, STREAM>), grid, block, lds, stream, (const T*)in, (T*)out, R, C,
                     (uint32_t)tilesC, inBatch, outBatch, (const T*)y, yBatch, (T)beta);
  return hipGetLastError();
}

template <typename T, bool HAS_Y, bool STREAM>
static hipError_t launchTransposeT(const void* in, void* out, uint32_t R, uint32_t C, uint32_t batch, uint64_t inBatch,
                                   uint64_t outBatch, const void* y, uint64_t yBatch, double beta, hipStream_t stream) {
  constexpr uint32_t ve = 16 / sizeof(T);
  const bool vec = R % ve == 0 && C % ve == 0 && (((uintptr_t)in | (uintptr_t)out) & 15) == 0 && inBatch % ve == 0 &&
                   outBatch % ve == 0 && (!HAS_Y || (((uintptr_t)y & 15) == 0 && yBatch % ve == 0));
  if (vec) {
    constexpr int SQ = sizeof(T) == 4 ? 128 : 64, E = 16384 / sizeof(T);      // square tile edge; elements of a 16 KB tile
#define FK_TR(TDR, TDC) launchTransposeVec<T, TDR, TDC, HAS_Y, STREAM>(in, out, R, C, batch, inBatch, outBatch, y, yBatch, beta, stream)
    if (R >= 64 && C >= 64) return FK_TR(SQ, SQ);
    if (C < 64 && C >= 8 && R >= 256) return C <= 16 ? FK_TR(E / 16, 16) : FK_TR(E / 32, 32);
    if (R < 64 && R >= 8 && C >= 256) return R <= 16 ? FK_TR(16, E / 16) : FK_TR(32, E / 32);
#undef FK_TR
  }
  uint32_t tcLog = 2;
  while (tcLog < 6 && (1u << tcLog) < C) tcLog++;
  const uint32_t TC = 1u << tcLog, TR = kTrTile >> tcLog;
  const uint64_t tilesC = (C + TC - 1) / TC, tilesR = (R + TR - 1) / TR;
  if (tilesC * tilesR >= (1ull << 31)) return hipErrorInvalidValue;
  dim3 grid((uint32_t)(tilesC * tilesR), batch), block(256);
  hipLaunchKernelGGL((kron_transpose_kernel<T, HAS_Y>), grid, block, 0, stream, (const T*)in, (T*)out, R, C, tcLog,
                     (uint32_t)tilesC, inBatch, outBatch, (const T*)y, yBatch, (T)beta);
  return hipGetLastError();
}

// out (C x R) = transpose(in (R x C)) + beta * y (y null: the plain transposed copy), per batch entry; streamOut: the
// result is not read back soon (stores at system scope where the kernel with 16-byte accesses applies)
hipError_t launchTransposeAdd(const void* in, void* out, uint32_t R, uint32_t C, uint32_t batch, uint64_t inBatch,
                              uint64_t outBatch, const void* y, uint64_t yBatch, double beta, DType dt, hipStream_t stream,
                              bool streamOut) {
  if (R == 0 || C == 0 || batch == 0 || batch > 65535) return hipErrorInvalidValue;
  const bool hasY = y != nullptr && beta != 0.0;
  // a tile's span of the output, (tile columns) x R elements, has to stay below 2 GB for the descriptor's offsets
  const bool so = streamOut && (uint64_t)1024 * R * dtypeSize(dt) < (1ull << 31);
#define FK_TRT(T) (hasY ? (so ? launchTransposeT<T, true, true>(in, out, R, C, batch, inBatch, outBatch, y, yBatch, beta, stream)      \
                              : launchTransposeT<T, true, false>(in, out, R, C, batch, inBatch, outBatch, y, yBatch, beta, stream))    \
                        : (so ? launchTransposeT<T, false, true>(in, out, R, C, batch, inBatch, outBatch, nullptr, 0, 0.0, stream)    \
                              : launchTransposeT<T, false, false>(in, out, R, C, batch, inBatch, outBatch, nullptr, 0, 0.0, stream)))
  return dt == DType::F32 ? FK_TRT(float) : FK_TRT(double);
#undef FK_TRT
}

hipError_t launchTranspose(const void* in, void* out, uint32_t R, uint32_t C, uint32_t batch, uint64_t inBatch,
                           uint64_t outBatch, DType dt, hipStream_t stream) {
  return launchTransposeAdd(in, out, R, C, batch, inBatch, outBatch, nullptr, 0, 0.0, dt, stream, false);
}

}  // namespace fk
