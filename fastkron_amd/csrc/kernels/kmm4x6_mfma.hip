// Six fused 4x4 fp32 factors in the KMM layout (X is 4096 x M row-major, the M columns are contiguous), one
// launch: sgekmm with 4x4^6 reads X and Y once and writes Z once instead of going through an intermediate.
//
//   Z[(q1..q6), m] = alpha * sum_{k1..k6} F1[q1,k1] ... F6[q6,k6] * X[(k1..k6), m]  (+ beta * Y)
//
// A workgroup of 8 waves owns 8 consecutive columns m and all 4096 rows of them: 32768 values, 64 per lane.
// The row index is six base-4 digits; digit 0 (row bits 0-1) is k6, the fastest, digit 5 (bits 10-11) is k1.
//   phase A  registers = the three fast digits, lanes and waves = the three slow ones: contracted in registers with
//            V_MFMA_F32_4X4X1_16B_F32 (16 independent 4x4 outer products per instruction: every lane gets its own
//            outputs, D[i][lane] += F[i][p] * x_lane[p]);
//   exchange one pass through LDS, element (c, s) of column m at m*4160 + shift(m) + c*65 + s, c = row bits 6-11,
//            s = row bits 0-5: the lanes of a wave differ in bits 1, 3, 5 of c when writing and of s when reading,
//            shift(m) puts the three bits of m on bits 0, 2, 4, so that both sides cover all 64 banks;
//   phase B  registers = the three slow digits, contracted the same way; the digits end up in place, so the result
//            is in its final order;
//   store    alpha / beta*Y applied.
// A wave-level memory instruction touches 8 rows x 32 bytes (the rows of X are M*4 bytes apart); the four tiles
// that share 128-byte lines are numbered onto the same XCD, so that they meet in its L2.  All workgroups (one per
// CU) move through the same phases together, so loads and stores never overlap and each phase runs at what this
// access pattern gets from the memory system by itself.  Which rows an instruction, a wave and a moment in time
// touch was chosen by timing every assignment of row bits to registers, lane groups and waves on the load and the
// store side (2400 of them; with operands that no cache holds, reading the 32 MB of one operand this way takes
// 13.6 to 17.5 us and writing them 9.1 to 23 us, against 6.4 / 7.3 us for a contiguous sweep: every request of a
// workgroup lies in another 8 KB row of the matrix, and wider tiles, 64 or 128 bytes per row, are no faster).
//
// The reference fuses at most as many factors as fit its shared-memory tile and runs this shape in several
// launches (reference src/kernel_db/kernel_db.cpp:152-290); its x86 KMM kernels vectorise along M likewise
// (reference src/kernels/cpu/kernel.h:124-126).
// Algorithmic traffic per launch: read 4096*M, write 4096*M elements (+ 4096*M for Y).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float k6f4 __attribute__((ext_vector_type(4)));

#define K6MFMA(a, b, c) __builtin_amdgcn_mfma_f32_4x4x1f32((a), (b), (c), 0, 0, 0)

constexpr int kK6Rows = 4096;               // 4^6
constexpr int kK6MStride = 64 * 65;          // LDS words per column m (+ the column's bank shift, at most 21)
constexpr size_t kK6LdsBytes = (8 * kK6MStride + 32) * sizeof(float);

// Row bits 0-5 (digits 0, 1, 2) of register r in phase A: register bits 0-1 hold digit 2, bits 2-3 digit 0, bits 4-5
// digit 1 (the order in which the loads go out: rows 16 apart first).
__host__ __device__ constexpr int k6RegRowA(int r) { return ((r & 3) << 4) | ((r >> 2) & 3) | (((r >> 4) & 3) << 2); }
// bits 0, 1, 2 -> bits 0, 2, 4
__device__ __forceinline__ int k6Spread(int v) { return (v & 1) | ((v & 2) << 1) | ((v & 4) << 2); }

// Contract the three digits held in the registers of x (digit j has register stride 4^j) with the factors
// fs[0..2]; fa[j][p] = F_j[q = lane & 3][p] is the A operand of the outer products.
__device__ __forceinline__ void k6Contract3(float (&x)[64], const float (&fa)[3][4]) {
#pragma unroll
  for (int j = 0; j < 3; j++) {
    const int st = (j == 0) ? 1 : (j == 1) ? 4 : 16;
#pragma unroll
    for (int s = 0; s < 16; s++) {
      const int base = (s / st) * st * 4 + (s % st);
      k6f4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int p = 0; p < 4; p++) d = K6MFMA(fa[j][p], x[base + p * st], d);
#pragma unroll
      for (int i = 0; i < 4; i++) x[base + i * st] = d[i];
    }
  }
}

template <bool HAS_Y>
__global__ __launch_bounds__(512) void kron_kmm4x6_kernel(const StepArgs a, const uint32_t mTiles) {
  extern __shared__ __align__(16) float lds[];
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t bt = blockIdx.y;
  // workgroups go round-robin over the 8 XCDs: neighbouring tiles (which share cache lines) onto one XCD
  const uint32_t tile = (mTiles % 8 == 0) ? (blockIdx.x % 8) * (mTiles / 8) + blockIdx.x / 8 : blockIdx.x;
  const int m8 = l & 7;
  // the lane's six row bits: bits 6-11 (c) in phase A, bits 0-5 (s) in phase B; lane group -> bits 1, 3, 5, wave -> 0, 2, 4
  const int coord = (k6Spread(l >> 3) << 1) | k6Spread(w);
  const uint64_t ldi = (uint64_t)a.in_ldc, ldo = (uint64_t)a.out_ldc, ldy = (uint64_t)a.y_ldc;
  const uint32_t m = tile * 8 + m8;

  // factor operands: fa[j][p] = F_j[q = l & 3][p]; a.f[j] is the factor of digit j (a.f[0]: the fastest digit, k6).
  // Element (p, q) of a factor lives at p*f_sp + q*f_sq.  Requested ahead of the bulk loads.
  float fa[6][4];
#pragma unroll
  for (int j = 0; j < 6; j++) {
    const float* F = (const float*)a.f[j] + (size_t)bt * a.f_batch[j];
#pragma unroll
    for (int p = 0; p < 4; p++) fa[j][p] = F[(int64_t)p * a.f_sp[j] + (int64_t)(l & 3) * a.f_sq[j]];
  }

  // Y is requested right behind X.  Measured with operands from HBM (no cache holding them) against requesting it
  // behind the first contraction or behind the exchange barrier: 36.6 / 37.7 / 40.4 us.  Holding Y back lets X
  // arrive sooner, but the more requests are in flight the better this access pattern is served.
  float yv[HAS_Y ? 64 : 1];
  auto loadY = [&]() {
    if (HAS_Y) {
      const float* Y = (const float*)a.y + (size_t)bt * a.y_batch + m + (uint64_t)coord * ldy;
#pragma unroll
      for (int r = 0; r < 64; r++) yv[r] = Y[(uint64_t)(r << 6) * ldy];
    }
  };
  float x[64];
  {
    const float* in = (const float*)a.in + (size_t)bt * a.in_batch + m + (uint64_t)(coord << 6) * ldi;
#pragma unroll
    for (int r = 0; r < 64; r++) x[r] = in[(uint64_t)k6RegRowA(r) * ldi];
  }
  loadY();
  {
    // register stride 1 = digit 2, stride 4 = digit 0, stride 16 = digit 1
    const float fA[3][4] = {{fa[2][0], fa[2][1], fa[2][2], fa[2][3]}, {fa[0][0], fa[0][1], fa[0][2], fa[0][3]},
                            {fa[1][0], fa[1][1], fa[1][2], fa[1][3]}};
    k6Contract3(x, fA);                     // registers: (q4,q5,q6) in the same arrangement
  }
  __builtin_amdgcn_sched_barrier(0);
  float* col = lds + m8 * kK6MStride + k6Spread(m8);
#pragma unroll
  for (int r = 0; r < 64; r++) col[coord * 65 + k6RegRowA(r)] = x[r];
  __syncthreads();
#pragma unroll
  for (int r = 0; r < 64; r++) x[r] = col[r * 65 + coord];  // registers: row bits 6-11 = (k1,k2,k3), k3 fastest
  {
    const float fB[3][4] = {{fa[3][0], fa[3][1], fa[3][2], fa[3][3]}, {fa[4][0], fa[4][1], fa[4][2], fa[4][3]},
                            {fa[5][0], fa[5][1], fa[5][2], fa[5][3]}};
    k6Contract3(x, fB);                     // registers: (q1,q2,q3)
  }

  float* out = (float*)a.out + (size_t)bt * a.out_batch + m + (uint64_t)coord * ldo;
  const float alpha = a.epilogue ? (float)a.alpha : 1.f, beta = (float)a.beta;
#pragma unroll
  for (int r = 0; r < 64; r++) {
    float v = x[r] * alpha;
    if (HAS_Y) v += beta * yv[r];
    out[(uint64_t)(r << 6) * ldo] = v;
  }
}

bool kmm4x6Supported(const StepArgs& a) {
  if (a.nf != 6 || a.Kin != kK6Rows || a.Kout != kK6Rows) return false;
  for (uint32_t j = 0; j < 6; j++) if (a.p[j] != 4 || a.q[j] != 4) return false;
  if (a.in_ldm != 1 || a.out_ldm != 1 || (a.y && a.y_ldm != 1)) return false;
  return a.M % 8 == 0 && a.batch <= 65535;
}

hipError_t launchKmm4x6(const StepArgs& a, hipStream_t stream) {
  if (!kmm4x6Supported(a)) return hipErrorInvalidValue;
  static PerDeviceOnce attrOnce;
  const int devIdx = launchDeviceIndex();
  if (!attrOnce.done(devIdx)) {
    hipError_t e = hipFuncSetAttribute((const void*)kron_kmm4x6_kernel<true>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)kK6LdsBytes);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute((const void*)kron_kmm4x6_kernel<false>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kK6LdsBytes);
    if (e != hipSuccess) return e;
    attrOnce.mark(devIdx);
  }
  const uint32_t mTiles = a.M / 8;
  dim3 grid(mTiles, a.batch), block(512);
  if (a.y && a.epilogue) hipLaunchKernelGGL(kron_kmm4x6_kernel<true>, grid, block, kK6LdsBytes, stream, a, mTiles);
  else                   hipLaunchKernelGGL(kron_kmm4x6_kernel<false>, grid, block, kK6LdsBytes, stream, a, mTiles);
  return hipGetLastError();
}

}  // namespace fk
