// Whole-row kernel for four fused 16x16 fp32 factors (row length 16^4 = 65536, e.g. sgemkm
// 1024 x 65536 with 16x16^4): one workgroup of 16 wave64s owns one row, keeps it in VGPRs
// (64 per lane) and touches HBM exactly once for the read and once for the write.
//
//   Z[q1,q2,q3,q4] = alpha * sum_{k1..k4} X[k1,k2,k3,k4] F1[k1,q1] F2[k2,q2] F3[k3,q3] F4[k4,q4] (+ beta*Y)
//
// The reference cannot fuse this shape in one launch (its tile must fit 48 KB of shared memory,
// reference src/gen_tuner_kernels.py:10,366; it runs 2 launches of 2 fused factors each).  Here the
// row (256 KB) does not fit the 160 KB LDS either, so the LDS is only the exchange buffer:
//
//   stage 1  contract k3 then k4 with V_MFMA_F32_16X16X4_F32, chained in registers: the first
//            product leaves D[i][j] in register i%4 of lane 16*(i/4)+j, which is exactly the A-operand
//            layout (lane 16*k+i) of a second product that contracts the *row* index i of the first;
//            the factor operand of the second product is loaded with its rows permuted (4*k + r)
//            to match.  No data movement between the two steps.
//   exch. 1  transpose (k1,k2) <-> (q3,q4) through LDS, in two halves of 128 KB, XOR-swizzled so that
//            both the ds_write_b32 and the ds_read_b32 side hit 64 distinct banks.
//   stage 2  contract k1 then k2 the same way.
//   exch. 2  bring the result to the store layout (lane = 4 consecutive columns, 1 KB per wave store),
//            again in two swizzled halves; ds_read_b128 on the way out.
//
// Algorithmic traffic: 4*65536 bytes read + 4*65536 bytes written per row (+ Y when beta != 0).
#include <hip/hip_runtime.h>
#include <cstdio>
#include <cstdlib>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float f4 __attribute__((ext_vector_type(4)));

#define MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x4f32((a), (b), (c), 0, 0, 0)

#ifdef FK_ROW_TIMING
// Experiment-only build: phase time stamps (s_memtime) of wave 0 of every workgroup.
__device__ unsigned long long g_rowTiming[1024 * 8];
#define FK_STAMP(k) do { if (tid == 0 && blockIdx.x < 1024) g_rowTiming[blockIdx.x * 8 + (k)] = __builtin_readcyclecounter(); } while (0)
extern "C" void fkDebugReadRowTiming(unsigned long long* out) {
  (void)hipMemcpyFromSymbol(out, HIP_SYMBOL(g_rowTiming), sizeof(unsigned long long) * 1024 * 8);
}
#else
#define FK_STAMP(k)
#endif

constexpr int kRowLen = 65536;
constexpr int kLdsWords = 32768;           // 128 KB: one half of a row

template <bool HAS_Y>
__global__ __launch_bounds__(1024, 1) void kron_row16x4_kernel(const StepArgs a, const uint32_t firstWave,
                                                               const uint32_t groups, const uint32_t delayCycles) {
  extern __shared__ float lds[];
  const int tid = threadIdx.x;
  // One workgroup fills a CU, so every CU alternates between an HBM phase (load, store) and an
  // on-chip phase (MFMA, LDS exchange).  Workgroups that start together stay in lockstep and leave
  // HBM idle during the on-chip phases; delaying a part of the first wave of workgroups by a fraction
  // of the row period interleaves the phases of different CUs.  Later workgroups inherit the offset.
  if (groups > 1) {
    const uint32_t wg = blockIdx.x + blockIdx.y * gridDim.x;
    const uint32_t g = (wg >> 3) % groups;   // workgroups go round-robin over the 8 XCDs: keep every group on every XCD
    if (wg < firstWave && g != 0) {
      // pure s_sleep (64 cycles per unit): polling a clock from thousands of waves would itself load the memory path
      const uint32_t n = (g * delayCycles) >> 12;                 // units of 64*64 cycles
      for (uint32_t k = 0; k < n; k++) __builtin_amdgcn_s_sleep(64);
    }
  }
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);      // wave-uniform: keeps row addresses in SGPRs
  const int i = l & 15, kb = l >> 4;
  const uint32_t m = blockIdx.x, b = blockIdx.y;
  FK_STAMP(0);
#ifdef FK_ROW_TIMING
  if (tid == 0 && blockIdx.x < 1024) g_rowTiming[blockIdx.x * 8 + 6] = wall_clock64();
#endif

  // m counts blocks of 65536 contiguous elements: one row for four factors, 16^(4-nf) rows otherwise
  const float* X = (const float*)a.in + (size_t)b * a.in_batch + (size_t)m * kRowLen;
  float* Z = (float*)a.out + (size_t)b * a.out_batch + (size_t)m * kRowLen;

  // Factor operands (B side of every product).  a.f[0] is the last factor (F4) ... a.f[3] the first (F1).
  // First product of a chain: B_c[k][j] = F[4c + k][j]; second product: B_r[k][j] = F[4k + r][j].
  // With fewer than four factors the leading digits are row indices (16^(4-nf) consecutive rows form the
  // same contiguous 65536-element block) and their factor slots hold the identity.
  float FA[4], FB[4], FC[4], FD[4];
  {
    auto fetch = [&](int j, int p, int q) -> float {
      if (j >= (int)a.nf) return (p == q) ? 1.f : 0.f;
      const float* f = (const float*)a.f[j] + (size_t)b * a.f_batch[j];
      return f[(int64_t)p * a.f_sp[j] + (int64_t)q * a.f_sq[j]];
    };
#pragma unroll
    for (int c = 0; c < 4; c++) {
      FA[c] = fetch(1, 4 * c + kb, i);      // F3: first product of stage 1
      FB[c] = fetch(0, 4 * kb + c, i);      // F4: second product of stage 1
      FC[c] = fetch(3, 4 * c + kb, i);      // F1: first product of stage 2
      FD[c] = fetch(2, 4 * kb + c, i);      // F2: second product of stage 2
    }
  }

  // ---- load: wave w reads the 16 KB of k1 = w; x[t][c] = X[k1=w][k2=t][k3=4c+kb][k4=i] ----
  float x[16][4];
  {
    const float* xp = X + w * 4096 + l;
#pragma unroll
    for (int t = 0; t < 16; t++)
#pragma unroll
      for (int c = 0; c < 4; c++) x[t][c] = xp[t * 256 + c * 64];
  }

  // ---- stage 1: contract k3 (first product) and k4 (second product) ----
#pragma unroll
  for (int t = 0; t < 16; t++) {
    f4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 4; c++) d = MFMA16(x[t][c], FA[c], d);
    f4 e = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 4; r++) e = MFMA16(d[r], FB[r], e);
#pragma unroll
    for (int r = 0; r < 4; r++) x[t][r] = e[r];       // = Y[k1=w][k2=t][q3=4kb+r][q4=i]
    // half 0 of exchange 1 goes out as soon as it exists, under the products of the next blocks
#pragma unroll
    for (int rr = 0; rr < 2; rr++)
      lds[((kb * 2 + rr) * 16 + i) * 256 + ((w * 16 + t) ^ l)] = e[rr];
  }

  FK_STAMP(1);
  // ---- exchange 1: rows (q3,q4), columns (k1,k2); half h holds the rows with bit 1 of q3 == h ----
  float z[16][4];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    if (h) {
      __syncthreads();
#pragma unroll
      for (int t = 0; t < 16; t++)
#pragma unroll
        for (int rr = 0; rr < 2; rr++) {
          const int row = (kb * 2 + rr) * 16 + i;
          lds[row * 256 + ((w * 16 + t) ^ l)] = x[t][2 + rr];
        }
    }
    __syncthreads();
#pragma unroll
    for (int u = 0; u < 16; u++) {
      if (((u >> 1) & 1) != h) continue;
      const int row = ((u >> 2) * 2 + (u & 1)) * 16 + w;
      const int swz = w + 16 * (u >> 2);
#pragma unroll
      for (int c = 0; c < 4; c++) z[u][c] = lds[row * 256 + ((c * 64 + l) ^ swz)];   // Y[k1=4c+kb][k2=i][q3=u][q4=w]
    }
  }
  __syncthreads();
  FK_STAMP(2);

  // ---- stage 2: contract k1 (first product) and k2 (second product) ----
#pragma unroll
  for (int u = 0; u < 16; u++) {
    f4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 4; c++) d = MFMA16(z[u][c], FC[c], d);
    f4 e = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 4; r++) e = MFMA16(d[r], FD[r], e);
#pragma unroll
    for (int r = 0; r < 4; r++) z[u][r] = e[r];       // = Z[q1=4kb+r][q2=i][q3=u][q4=w]
    // half 0 of exchange 2 (every wave passed the barrier after its last read of exchange 1)
#pragma unroll
    for (int rr = 0; rr < 2; rr++)
      lds[((kb * 2 + rr) * 16 + i) * 256 + ((u * 16 + w) ^ (i * 4) ^ kb)] = e[rr];
  }

  FK_STAMP(3);
  // ---- exchange 2: rows (q1,q2), columns (q3,q4); half h holds the rows with bit 1 of q1 == h.
  //      Reader: wave w owns q2 = w, lane owns columns 4l .. 4l+3, register index is q1. ----
  f4 o[16];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    if (h) {
      __syncthreads();
#pragma unroll
      for (int u = 0; u < 16; u++)
#pragma unroll
        for (int rr = 0; rr < 2; rr++) {
          const int row = (kb * 2 + rr) * 16 + i;
          lds[row * 256 + ((u * 16 + w) ^ (i * 4) ^ kb)] = z[u][2 + rr];
        }
    }
    __syncthreads();
#pragma unroll
    for (int q1hi = 0; q1hi < 4; q1hi++)
#pragma unroll
      for (int rr = 0; rr < 2; rr++) {
        const int row = (q1hi * 2 + rr) * 16 + w;
        const f4 v = *(const f4*)&lds[row * 256 + ((l * 4) ^ (w * 4))];
        f4 p;                                           // word e of v is column 4l + (e ^ q1hi)
        p[0] = v[0 ^ q1hi]; p[1] = v[1 ^ q1hi]; p[2] = v[2 ^ q1hi]; p[3] = v[3 ^ q1hi];
        o[4 * q1hi + 2 * h + rr] = p;
      }
  }

  FK_STAMP(4);
  // ---- epilogue and store: every wave-level store covers 1 KB of contiguous columns ----
  const float alpha = (float)a.alpha, beta = (float)a.beta;
  const float* Y = HAS_Y ? (const float*)a.y + (size_t)b * a.y_batch + (size_t)m * kRowLen : nullptr;
#pragma unroll
  for (int q1 = 0; q1 < 16; q1++) {
    const int col = q1 * 4096 + w * 256 + l * 4;
    f4 v = o[q1];
    if (a.epilogue) {
      v = v * alpha;
      if (HAS_Y) {
        const f4 yv = *(const f4*)(Y + col);
        v = v + yv * beta;
      }
    }
    *(f4*)(Z + col) = v;
  }
  FK_STAMP(5);
#ifdef FK_ROW_TIMING
  if (tid == 0 && blockIdx.x < 1024) g_rowTiming[blockIdx.x * 8 + 7] = wall_clock64();
#endif
}

// Rows per workgroup: 16^(4-nf).
static uint32_t row16Rows(const StepArgs& a) { uint32_t r = 1; for (uint32_t j = a.nf; j < 4; j++) r *= 16; return r; }

bool row16x4Supported(const StepArgs& a) {
  if (a.nf < 2 || a.nf > 4) return false;
  uint64_t k = 1;
  for (uint32_t j = 0; j < a.nf; j++) { if (a.p[j] != 16 || a.q[j] != 16) return false; k *= 16; }
  if (a.Kin != k || a.Kout != k) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  // the rows of a block must be contiguous, and M must be a whole number of blocks
  if ((uint64_t)a.in_ldm != k || (uint64_t)a.out_ldm != k || (a.y && (uint64_t)a.y_ldm != k)) return false;
  if (a.M % row16Rows(a)) return false;
  // 16-byte aligned blocks for the vector stores / Y loads
  if (((uintptr_t)a.out & 15) || (a.out_batch & 3)) return false;
  if (a.y && (((uintptr_t)a.y & 15) || (a.y_batch & 3))) return false;
  return a.batch <= 65535;
}

hipError_t launchRow16x4(const StepArgs& a, hipStream_t stream) {
  if (!row16x4Supported(a)) return hipErrorInvalidValue;
  static bool attrSet = false;
  const size_t ldsBytes = kLdsWords * sizeof(float);
  if (!attrSet) {
    hipError_t e = hipFuncSetAttribute((const void*)kron_row16x4_kernel<true>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute((const void*)kron_row16x4_kernel<false>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
    if (e != hipSuccess) return e;
    attrSet = true;
  }
  dim3 grid(a.M / row16Rows(a), a.batch), block(1024);
  static int cus = 0;
  static uint32_t groups = 3, delay = 20000;           // three start groups, 20000 cycles (about 9 us) apart
  if (!cus) {
    int dev = 0;
    hipDeviceProp_t prop;
    if (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess) cus = prop.multiProcessorCount;
    else cus = 256;
    if (const char* e = getenv("FASTKRON_ROW_STAGGER")) {   // "<groups>,<ticks>" for experiments
      unsigned g = 0, d = 0;
      if (sscanf(e, "%u,%u", &g, &d) == 2) { groups = g; delay = d; }
    }
  }
  const uint32_t firstWave = (uint32_t)cus;
  const uint32_t g = ((uint64_t)grid.x * a.batch > (uint64_t)cus) ? groups : 1;   // a single wave of rows gains nothing
  if (a.y && a.epilogue)
    hipLaunchKernelGGL(kron_row16x4_kernel<true>, grid, block, ldsBytes, stream, a, firstWave, g, delay);
  else
    hipLaunchKernelGGL(kron_row16x4_kernel<false>, grid, block, ldsBytes, stream, a, firstWave, g, delay);
  return hipGetLastError();
}

}  // namespace fk
