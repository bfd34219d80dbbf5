// Whole-row kernel for five fused 8x8 fp32 factors (row length 8^5 = 32768, e.g. sgemkm
// 1024 x 32768 with 8x8^5).  One workgroup of 8 wave64s owns one row and keeps it in VGPRs (64 per
// lane); two workgroups share a CU, so one row's HBM traffic overlaps the other row's arithmetic.
//
//   Z[q1..q5] = alpha * sum_{k1..k5} X[k1..k5] * F1[k1,q1] * ... * F5[k5,q5]  (+ beta * Y)
//
// Every lane owns whole "slices": for the digit being contracted it holds all 8 inputs of a slice in
// registers and produces the 8 outputs of that slice in registers.  The contraction runs on the
// matrix cores with V_MFMA_F32_4X4X1_16B_F32: 16 independent 4x4 outer products per instruction, so
// D[i][lane] += F[p][4*qq+i] * x_lane[p] gives each lane its own outputs at the full fp32 MFMA rate.
//
//   load     lane = (k4,k5) (256 contiguous bytes per wave instruction), wave = k3, regs = (k1,k2)
//   stage A  contract k1, k2
//   exch. 1  through LDS (two 64 KB halves, XOR-swizzled 16-byte chunks): regs become (k4,k5)
//   stage B  contract k5, k4
//   exch. 2  through LDS: regs become (k3, 3 spectator bits), lanes (q4lo,q5) + 1 bit of q2
//   stage C  contract k3
//   store    every wave instruction writes two full 128-byte lines
//
// The reference fuses at most as many factors as fit its 48 KB shared-memory tile (three 8x8 factors
// of a 4096-column tile for this shape: reference kernel X86/CUDA "..._8x8_8x8_3_1x4096_..."), i.e. two
// launches and one HBM round trip for the intermediate; here the row never leaves the CU.
// Algorithmic traffic: 4*32768 bytes read + 4*32768 bytes written per row (+ Y when beta != 0).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float f4 __attribute__((ext_vector_type(4)));

#define MFMA4(a, b, c) __builtin_amdgcn_mfma_f32_4x4x1f32((a), (b), (c), 0, 0, 0)


constexpr int kRow8Len = 32768;
// The two workgroups of a CU would load, compute and store in lockstep; the later one starts 5 us behind (measured
// on 1024 x 8^5 with cold operands: 59.5 us without, 57.7 with 5 us, 57.9 with 6, 58.0 with 7, 63 with 12; 512 rows
// 31.1 -> 29.3 us, 768 rows 52.8 -> 47.8, 4096 rows 213.3 -> 211.7; one workgroup per CU is not delayed).
constexpr uint32_t kRow8SlotDelayTicks = 500;
constexpr int kRow8LdsWords = 16384 + 5 * 64;     // one half row + the five factors

// Factor operand of the 4x4x1 products for this lane: fa[p][qq] = F[p][4*qq + (lane & 3)].
__device__ __forceinline__ void loadFactor8(const float* fl, int lane, float (&fa)[8][2]) {
#pragma unroll
  for (int p = 0; p < 8; p++)
#pragma unroll
    for (int qq = 0; qq < 2; qq++) fa[p][qq] = fl[p * 8 + 4 * qq + (lane & 3)];
}

// x[a][b]: contract the first index with F (a <- q).
__device__ __forceinline__ void contractFirst(float (&x)[8][8], const float (&fa)[8][2]) {
#pragma unroll
  for (int b = 0; b < 8; b++) {
    f4 d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < 8; p++) {
      d0 = MFMA4(fa[p][0], x[p][b], d0);
      d1 = MFMA4(fa[p][1], x[p][b], d1);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) { x[i][b] = d0[i]; x[4 + i][b] = d1[i]; }
  }
}

// x[a][b]: contract the second index with F (b <- q).
__device__ __forceinline__ void contractSecond(float (&x)[8][8], const float (&fa)[8][2]) {
#pragma unroll
  for (int a = 0; a < 8; a++) {
    f4 d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int p = 0; p < 8; p++) {
      d0 = MFMA4(fa[p][0], x[a][p], d0);
      d1 = MFMA4(fa[p][1], x[a][p], d1);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) { x[a][i] = d0[i]; x[a][4 + i] = d1[i]; }
  }
}

template <bool HAS_Y, int NT>
__global__ __launch_bounds__(512, 4) void kron_row8x5_kernel(const StepArgs a, const uint32_t firstRound, const uint32_t delayTicks) {
  extern __shared__ __align__(16) float lds[];
  float* fl = lds + 16384;                       // factors: fl[f*64 + p*8 + q], f = 0 is F1
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);      // wave-uniform: keeps row addresses in SGPRs
  const uint32_t m = blockIdx.x, bt = blockIdx.y;

  // m counts blocks of 32768 contiguous elements: one row for five factors, 8^(5-nf) rows otherwise
  const float* X = (const float*)a.in + (size_t)bt * a.in_batch + (size_t)m * kRow8Len;
  float* Z = (float*)a.out + (size_t)bt * a.out_batch + (size_t)m * kRow8Len;

  // factors to LDS, ahead of the row loads (vector memory operations retire in order, so these small
  // loads must not queue behind 128 KB of row data).  a.f[0] is the last factor F5 ... a.f[nf-1] the first.  With fewer than five
  // factors the leading digits are row indices (8^(5-nf) consecutive rows form the same contiguous
  // 32768-element block) and their factor slots hold the identity.
  delayLaterWorkgroupOfCU(firstRound, delayTicks);
  if (tid < 320) {
    const int f = tid >> 6, e = tid & 63, p = e >> 3, q = e & 7;
    const int j = 4 - f;
    float v = (p == q) ? 1.f : 0.f;
    if (j < (int)a.nf) {
      const float* fp = (const float*)a.f[j] + (size_t)bt * a.f_batch[j];
      v = fp[(int64_t)p * a.f_sp[j] + (int64_t)q * a.f_sq[j]];
    }
    fl[tid] = v;
  }
  // ---- load: x[k1][k2] = X[k1][k2][k3 = w][(k4,k5) = l]; k2 outermost, so the slices of the first
  //      contraction (all k1 for one k2) complete in issue order ----
  float x[8][8];
  // (issued at raised priority: the other workgroup of the CU is in its arithmetic then, and its older waves would
  // otherwise win the instruction arbiter; 55.7 -> 53.2 us)
  __builtin_amdgcn_s_setprio(3);
  {
    const float* xp = X + w * 64 + l;
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
      for (int i = 0; i < 8; i++) x[i][j] = FK_LD(NT, &xp[i * 4096 + j * 512]);
  }
  __builtin_amdgcn_s_setprio(0);
  __syncthreads();

  float fa[8][2];
  // ---- stage A: contract k1 then k2 ----
  loadFactor8(fl + 0 * 64, l, fa);
  contractFirst(x, fa);
  loadFactor8(fl + 1 * 64, l, fa);
  contractSecond(x, fa);                         // x[q1][q2], wave = k3, lane = (k4,k5)

  // ---- exchange 1: half h holds q1 in [4h, 4h+4).  Group id = (q1 & 3, q2, k3) owns 64 floats
  //      (k4,k5) stored as 16 chunks of 4, chunk index XORed with the low 4 bits of the id.  Readers:
  //      thread tid' = (q1, q2, k3) reads its 64 floats as regs [k4][k5]; waves q1>>2 == h read. ----
  float y[8][8];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    if (h) __syncthreads();
    // id & 15 = (j & 1)*8 + w: two base addresses (even and odd j) plus constant offsets, so that the writes
    // pair up into two-address LDS instructions
    {
      float* const base0 = lds + w * 64 + ((((l >> 2) ^ w) << 2) | (l & 3));
      float* const base1 = lds + w * 64 + ((((l >> 2) ^ (w + 8)) << 2) | (l & 3));
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int jj = 0; jj < 8; jj++) {
          const int j = (jj < 4) ? 2 * jj : 2 * (jj - 4) + 1;          // even columns, then odd ones
          ((j & 1) ? base1 : base0)[(i * 64 + j * 8) * 64] = x[4 * h + i][j];
        }
    }
    __syncthreads();
    if ((w >> 2) == h) {
      const int id = (w & 3) * 64 + l;
#pragma unroll
      for (int c = 0; c < 16; c++) {
        const f4 v = *(const f4*)&lds[id * 64 + ((c ^ (id & 15)) << 2)];
#pragma unroll
        for (int e = 0; e < 4; e++) y[c >> 1][(c & 1) * 4 + e] = v[e];
      }
    }
  }
  // now thread = (q1 = w, q2 = l >> 3, k3 = l & 7), y[k4][k5]

  // ---- stage B: contract k5 then k4 ----
  loadFactor8(fl + 4 * 64, l, fa);
  contractSecond(y, fa);
  loadFactor8(fl + 3 * 64, l, fa);
  contractFirst(y, fa);                          // y[q4][q5]

  // ---- exchange 2: half h holds q4 in [4h, 4h+4).  Group = (q1, q2>>1, k3) owns 64 floats
  //      (q2&1, q4lo, q5) as 16 chunks, chunk index XORed with k3.  Readers: wave = q1,
  //      lane = (q2&1, q4lo, q5), regs z[k3][g], g = q4hi*4 + (q2>>1). ----
  float z[8][8];
  {
    const int q2 = l >> 3, k3 = l & 7;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      __syncthreads();
      const int grp = (w * 4 + (q2 >> 1)) * 8 + k3;
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int c2 = 0; c2 < 2; c2++) {
          f4 v;
#pragma unroll
          for (int e = 0; e < 4; e++) v[e] = y[4 * h + i][c2 * 4 + e];
          const int ch = ((q2 & 1) * 8 + i * 2 + c2) ^ k3;
          *(f4*)&lds[grp * 64 + (ch << 2)] = v;
        }
      __syncthreads();
#pragma unroll
      for (int d3 = 0; d3 < 8; d3++)
#pragma unroll
        for (int s = 0; s < 4; s++) {
          const int g2 = (w * 4 + s) * 8 + d3;
          z[d3][4 * h + s] = lds[g2 * 64 + ((((l >> 2) ^ d3) << 2) | (l & 3))];
        }
    }
  }
  // thread = (q1 = w, lane = (q2&1, q4lo, q5)), z[k3][g], g = q4hi*4 + (q2>>1)

  // ---- stage C: contract k3 ----
  loadFactor8(fl + 2 * 64, l, fa);
  contractFirst(z, fa);

  // ---- epilogue and store ----
  const float alpha = (float)a.alpha, beta = (float)a.beta;
  const float* Y = HAS_Y ? (const float*)a.y + (size_t)bt * a.y_batch + (size_t)m * kRow8Len : nullptr;
  const int lo = (l & 31), q2b = l >> 5;
#pragma unroll
  for (int q3 = 0; q3 < 8; q3++)
#pragma unroll
    for (int g = 0; g < 8; g++) {
      const int q2 = 2 * (g & 3) + q2b;
      const int col = w * 4096 + q2 * 512 + q3 * 64 + (g >> 2) * 32 + lo;
      float v = z[q3][g];
      if (a.epilogue) {
        v *= alpha;
        if (HAS_Y) v += beta * Y[col];
      }
      FK_ST(NT, v, &Z[col]);
    }
}

// Rows per workgroup: 8^(5-nf).
static uint32_t row8Rows(const StepArgs& a) { uint32_t r = 1; for (uint32_t j = a.nf; j < 5; j++) r *= 8; return r; }

bool row8x5Supported(const StepArgs& a) {
  if (a.nf < 2 || a.nf > 5) return false;
  uint64_t k = 1;
  for (uint32_t j = 0; j < a.nf; j++) { if (a.p[j] != 8 || a.q[j] != 8) return false; k *= 8; }
  if (a.Kin != k || a.Kout != k) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  // the rows of a block must be contiguous, and M must be a whole number of blocks
  if ((uint64_t)a.in_ldm != k || (uint64_t)a.out_ldm != k || (a.y && (uint64_t)a.y_ldm != k)) return false;
  if (a.M % row8Rows(a)) return false;
  return a.batch <= 65535;
}

// schedule: 0 = two workgroups per CU, the later one of a CU started kRow8SlotDelayTicks behind (the online choice);
// 1 = one workgroup per CU (the launch asks for more LDS than two workgroups can have); 2 = two per CU without the delay.
hipError_t launchRow8x5(const StepArgs& a, hipStream_t stream, int schedule) {
  if (!row8x5Supported(a)) return hipErrorInvalidValue;
  static PerDeviceOnce attrOnce;
  const int devIdx = launchDeviceIndex();
  const size_t ldsMax = 96 * 1024;
  const size_t ldsBytes = schedule == 1 ? ldsMax : kRow8LdsWords * sizeof(float);
  using Kernel = void (*)(const StepArgs, const uint32_t, const uint32_t);
  static const Kernel kernels[2][3] = {
      {kron_row8x5_kernel<false, 0>, kron_row8x5_kernel<false, 1>, kron_row8x5_kernel<false, 2>},
      {kron_row8x5_kernel<true, 0>, kron_row8x5_kernel<true, 1>, kron_row8x5_kernel<true, 2>}};
  if (!attrOnce.done(devIdx)) {
    for (int y = 0; y < 2; y++)
      for (int nt = 0; nt < 3; nt++) {
        hipError_t e = hipFuncSetAttribute((const void*)kernels[y][nt], hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsMax);
        if (e != hipSuccess) return e;
      }
    attrOnce.mark(devIdx);
  }
  dim3 grid(a.M / row8Rows(a), a.batch), block(512);
  const uint32_t firstRound = 2u * (uint32_t)deviceCUs();
  hipLaunchKernelGGL(kernels[(a.y && a.epilogue) ? 1 : 0][streamMode(a)], grid, block, ldsBytes, stream, a, firstRound,
                     schedule == 0 ? kRow8SlotDelayTicks : 0u);
  return hipGetLastError();
}

}  // namespace fk
