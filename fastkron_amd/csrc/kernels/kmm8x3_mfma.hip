// Three fused 8x8 fp32 factors in the KMM layout (operands are K x M row-major, the M columns contiguous): sgekmm
// chains of 8x8 factors take one launch per three factors instead of one per two, and so do the leading factors of
// long GeMKM chains of 8x8 factors (which run as KMM problems over contiguous blocks).
//
//   out[(q1,q2,q3)*SG + sg, m] = sum_{k1,k2,k3} F1[q1,k1] F2[q2,k2] F3[q3,k3] * in[sg*512 + (k1,k2,k3), m],  SG = Kin / 512
//
// A workgroup of 8 waves owns 512 rows of one row group sg by 64 consecutive columns m, 128 KB kept in registers (64
// values per lane); two workgroups share a CU.  Lanes run along m, so every global access of a wave is a contiguous
// 256-byte row segment.
//   stage A  wave = k1, registers = (k2, k3): both contracted in registers with V_MFMA_F32_4X4X1_16B_F32 (16
//            independent 4x4 outer products: D[i][lane] += F[p][4*qq + i] * x_lane[p], every lane gets its own outputs);
//   exchange through LDS in two halves of 64 KB (q3 < 4, then q3 >= 4): wave = q2, registers = (k1, q3).  A lane
//            exchanges with the same lane of the other waves only, so consecutive lanes touch consecutive words;
//   stage B  k1 contracted the same way;
//   store    alpha / beta*Y applied in the launch that writes Z.
//
// The reference's GPU kernels fuse factors through shared memory on CUDA cores (reference
// src/kernels/cuda/kernel.cuh:165-219); its x86 KMM kernels vectorise along M as this one does (reference
// src/kernels/cpu/kernel.h:124-126).
// Algorithmic traffic per launch: read M*Kin, write M*Kin elements (+ M*Kin for Y on the launch that writes Z).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float k83f4 __attribute__((ext_vector_type(4)));

#define K83_MFMA4(a, b, c) __builtin_amdgcn_mfma_f32_4x4x1f32((a), (b), (c), 0, 0, 0)

constexpr int kK83LdsWords = 8 * 32 * 64 + 3 * 64;      // one half of the tile + the three factors

// Factor operand of the 4x4x1 products for this lane: fa[p][qq] = F[p][4*qq + (lane & 3)].
__device__ __forceinline__ void k83LoadFactor(const float* fl, int lane, float (&fa)[8][2]) {
#pragma unroll
  for (int p = 0; p < 8; p++)
#pragma unroll
    for (int qq = 0; qq < 2; qq++) fa[p][qq] = fl[p * 8 + 4 * qq + (lane & 3)];
}

// x[a][b]: contract the first index with F (a <- q).
__device__ __forceinline__ void k83ContractFirst(float (&x)[8][8], const float (&fa)[8][2]) {
#pragma unroll
  for (int b = 0; b < 8; b++) {
    k83f4 d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < 8; p++) {
      d0 = K83_MFMA4(fa[p][0], x[p][b], d0);
      d1 = K83_MFMA4(fa[p][1], x[p][b], d1);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) { x[i][b] = d0[i]; x[4 + i][b] = d1[i]; }
  }
}

// x[a][b]: contract the second index with F (b <- q).
__device__ __forceinline__ void k83ContractSecond(float (&x)[8][8], const float (&fa)[8][2]) {
#pragma unroll
  for (int a = 0; a < 8; a++) {
    k83f4 d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < 8; p++) {
      d0 = K83_MFMA4(fa[p][0], x[a][p], d0);
      d1 = K83_MFMA4(fa[p][1], x[a][p], d1);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) { x[a][i] = d0[i]; x[a][4 + i] = d1[i]; }
  }
}

// NT: 0 = ordinary accesses, 2 = non-temporal loads of X and stores (sgekmm 1024 x 8^6: 873 -> 832 us; small problems lose)
template <bool HAS_Y, int NT>
__global__ __launch_bounds__(512, 4) void kron_kmm8x3_kernel(const StepArgs a, const uint32_t mTiles) {
  extern __shared__ __align__(16) float k83Lds[];
  float* fl = k83Lds + 8 * 32 * 64;              // factors: fl[f*64 + p*8 + q]; f = 0 is F1 (slowest digit)
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t bt = blockIdx.y;
  const uint64_t SG = a.Kin / 512;
  const uint64_t sg = blockIdx.x / mTiles;
  const uint32_t m = (blockIdx.x % mTiles) * 64 + l;           // M is a multiple of 64

  // factors to LDS, ahead of the row loads.  a.f[0] is the factor of the fastest digit (F3), a.f[2] is F1; element
  // (p, q) of a factor, p the contracted index, lives at p*f_sp + q*f_sq.
  if (tid < 192) {
    const int f = tid >> 6, e = tid & 63, p = e >> 3, q = e & 7;
    const int j = 2 - f;
    const float* fp = (const float*)a.f[j] + (size_t)bt * a.f_batch[j];
    fl[tid] = fp[(int64_t)p * a.f_sp[j] + (int64_t)q * a.f_sq[j]];
  }

  // ---- load: x[k2][k3] = in[sg*512 + w*64 + k2*8 + k3, m] ----
  const float* in = (const float*)a.in + (size_t)bt * a.in_batch + m;
  float x[8][8];
  __builtin_amdgcn_s_setprio(3);                 // (the other workgroup of the CU is in its arithmetic: 3 % on large problems)
  {
    const float* xp = in + (sg * 512 + (uint64_t)w * 64) * (uint64_t)a.in_ldc;
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int j = 0; j < 8; j++) x[i][j] = FK_LD(NT, &xp[(uint64_t)(i * 8 + j) * (uint64_t)a.in_ldc]);
  }
  __builtin_amdgcn_s_setprio(0);
  __syncthreads();

  float fa[8][2];
  // ---- stage A: contract k3 then k2 ----
  k83LoadFactor(fl + 2 * 64, l, fa);
  k83ContractSecond(x, fa);
  k83LoadFactor(fl + 1 * 64, l, fa);
  k83ContractFirst(x, fa);                       // x[q2][q3], wave = k1

  // ---- exchange: half h holds q3 in [4h, 4h+4); word ((k1*8 + q2)*4 + q3%4)*64 + lane.  Afterwards wave = q2 and
  //      y[k1][q3] ----
  float y[8][8];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    if (h) __syncthreads();
#pragma unroll
    for (int q2 = 0; q2 < 8; q2++)
#pragma unroll
      for (int i = 0; i < 4; i++) k83Lds[((w * 8 + q2) * 4 + i) * 64 + l] = x[q2][4 * h + i];
    __syncthreads();
#pragma unroll
    for (int k1 = 0; k1 < 8; k1++)
#pragma unroll
      for (int i = 0; i < 4; i++) y[k1][4 * h + i] = k83Lds[((k1 * 8 + w) * 4 + i) * 64 + l];
  }

  // ---- stage B: contract k1 ----
  k83LoadFactor(fl + 0 * 64, l, fa);
  k83ContractFirst(y, fa);                       // y[q1][q3], wave = q2

  // ---- epilogue and store: row (q1*64 + q2*8 + q3)*SG + sg ----
  const float alpha = (float)a.alpha, beta = (float)a.beta;
  float* out = (float*)a.out + (size_t)bt * a.out_batch + m + (((uint64_t)w * 8) * SG + sg) * (uint64_t)a.out_ldc;
  const uint64_t rowStep = SG * (uint64_t)a.out_ldc;           // one step in (q1, q2, q3) as a number
  if (HAS_Y) {
    const float* Y = (const float*)a.y + (size_t)bt * a.y_batch + m + (((uint64_t)w * 8) * SG + sg) * (uint64_t)a.y_ldc;
    const uint64_t yStep = SG * (uint64_t)a.y_ldc;
    // a rolling window of 16 registers keeps the Y loads in flight ahead of the stores (loads and stores retire
    // through one in-order counter: a load issued behind a store could only be waited for together with that store)
    constexpr int YW = 16;
    float yw[YW];
#pragma unroll
    for (int e = 0; e < YW; e++) yw[e] = Y[(uint64_t)((e >> 3) * 64 + (e & 7)) * yStep];
#pragma unroll
    for (int e = 0; e < 64; e++) {
      const float v = alpha * y[e >> 3][e & 7] + beta * yw[e % YW];
      if (e + YW < 64) yw[e % YW] = Y[(uint64_t)(((e + YW) >> 3) * 64 + ((e + YW) & 7)) * yStep];
      FK_ST(NT, v, &out[(uint64_t)((e >> 3) * 64 + (e & 7)) * rowStep]);
    }
    return;
  }
  if (a.epilogue) {
#pragma unroll
    for (int q1 = 0; q1 < 8; q1++)
#pragma unroll
      for (int q3 = 0; q3 < 8; q3++) y[q1][q3] *= alpha;
  }
#pragma unroll
  for (int q1 = 0; q1 < 8; q1++)
#pragma unroll
    for (int q3 = 0; q3 < 8; q3++) FK_ST(NT, y[q1][q3], &out[(uint64_t)(q1 * 64 + q3) * rowStep]);
}

bool kmm8x3Supported(const StepArgs& a) {
  if (a.nf != 3) return false;
  for (uint32_t j = 0; j < 3; j++) if (a.p[j] != 8 || a.q[j] != 8) return false;
  if (a.Kin % 512 || a.Kout != a.Kin) return false;
  // the M index contiguous in the input, the output and Y; whole tiles of 64 columns
  if (a.in_ldm != 1 || a.out_ldm != 1 || (a.y && a.y_ldm != 1)) return false;
  if (a.M % 64) return false;
  const uint64_t tiles = (a.Kin / 512) * (a.M / 64);
  return tiles < (1ull << 31) && a.batch <= 65535;
}

hipError_t launchKmm8x3(const StepArgs& a, hipStream_t stream) {
  if (!kmm8x3Supported(a)) return hipErrorInvalidValue;
  static PerDeviceOnce attrOnce;
  const int devIdx = launchDeviceIndex();
  const size_t ldsBytes = kK83LdsWords * sizeof(float);
  using Kernel = void (*)(const StepArgs, const uint32_t);
  static const Kernel kernels[2][2] = {{kron_kmm8x3_kernel<false, 0>, kron_kmm8x3_kernel<false, 2>},
                                       {kron_kmm8x3_kernel<true, 0>, kron_kmm8x3_kernel<true, 2>}};
  if (!attrOnce.done(devIdx)) {
    for (int y = 0; y < 2; y++)
      for (int nt = 0; nt < 2; nt++) {
        hipError_t e = hipFuncSetAttribute((const void*)kernels[y][nt], hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
        if (e != hipSuccess) return e;
      }
    attrOnce.mark(devIdx);
  }
  const uint32_t mTiles = a.M / 64;
  dim3 grid((uint32_t)((a.Kin / 512) * mTiles), a.batch), block(512);
  hipLaunchKernelGGL(kernels[(a.y && a.epilogue) ? 1 : 0][(a.stream_in && a.stream_out) ? 1 : 0], grid, block, ldsBytes, stream, a,
                     mTiles);
  return hipGetLastError();
}

}  // namespace fk
