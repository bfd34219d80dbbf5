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
//   load     one 16-byte load per lane and 256-element block (k3 = lane%16, k4 = 4*(lane/16) + register)
//   stage 1  contract k4 then k3 with V_MFMA_F32_16X16X4_F32, chained in registers: the first
//            product leaves D[i][j] in register i%4 of lane 16*(i/4)+j, which is exactly the A-operand
//            layout (lane 16*k+i) of a second product that contracts the *row* index i of the first;
//            the factor operand of the second product is loaded with its rows permuted (4*k + r)
//            to match.  No data movement between the two steps.
//   exch. 1  transpose (k1,k2) <-> (q3,q4) through LDS, in two halves of 128 KB: 16-byte writes (four blocks
//            of a lane are four adjacent columns of its row), 4-byte reads, chunks XOR-swizzled so that both
//            sides are free of bank conflicts.
//   stage 2  contract k1 then k2 the same way.
//   exch. 2  bring the result to the store layout (lane = 4 consecutive columns, 1 KB per wave store),
//            again in two swizzled halves; 16-byte LDS writes and reads (the LDS pipeline is bound by its
//            instruction rate, about 3-4 cycles per wave instruction whatever the width).
//
// Algorithmic traffic: 4*65536 bytes read + 4*65536 bytes written per row (+ Y when beta != 0).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float f4 __attribute__((ext_vector_type(4)));

#define MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x4f32((a), (b), (c), 0, 0, 0)



constexpr int kRowLen = 65536;
constexpr int kLdsWords = 32768;           // 128 KB: one half of a row
#ifndef ROW16_KPF
#define ROW16_KPF 5
#endif
constexpr int kPF = ROW16_KPF;                     // blocks (of 16) of the next item loaded one item ahead

template <bool HAS_Y>
__global__ __launch_bounds__(1024, 1) void kron_row16x4_kernel(const StepArgs a, const uint32_t blocksPerBatch,
                                                               const uint32_t totalItems) {
  extern __shared__ __align__(16) float lds[];
  const int tid = threadIdx.x;
  const int l0 = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);      // wave-uniform: keeps row addresses in SGPRs

  uint32_t item = blockIdx.x;
  if (item >= totalItems) return;

  // Factors: a.f[0] is the last factor (F4) ... a.f[3] the first (F1); with fewer than four factors the
  // leading digits are row indices (16^(4-nf) consecutive rows form the same contiguous 65536-element
  // block) and their factor slots hold the identity.  The four 16x16 matrices are staged in LDS behind
  // the exchange buffer, fl[j*256 + p*16 + q], and the B operands of a stage are read from there right
  // before the stage: LDS reads do not queue behind the row loads the way small global loads would
  // (vector memory operations retire in order).
  float* fl = lds + kLdsWords;
  auto stageFactors = [&](uint32_t b) {
    const int j = tid >> 8, p = (tid >> 4) & 15, q = tid & 15;
    float v = (p == q) ? 1.f : 0.f;
    if (j < (int)a.nf) {
      const float* f = (const float*)a.f[j] + (size_t)b * a.f_batch[j];
      v = f[(int64_t)p * a.f_sp[j] + (int64_t)q * a.f_sq[j]];
    }
    fl[tid] = v;
  };
  bool perBatchFactors = false;
  for (uint32_t j = 0; j < a.nf; j++) perBatchFactors |= (a.f_batch[j] != 0);
  stageFactors(item / blocksPerBatch);
  __syncthreads();

  // An item is a block of 65536 contiguous elements: one row for four factors, 16^(4-nf) rows otherwise.
  // xa holds blocks t = 0..kPF-1 (k2) of the item about to be processed; it is loaded one item ahead, under the
  // second stage, the second exchange and the stores of the previous item.
  // One 16-byte load per lane and block: x[t][r] = X[k1=w][k2=t][k3=i][k4=4kb+r] (i = l%16, kb = l/16), 1 KB per
  // wave instruction; a quarter as many memory instructions as 4-byte loads would take.
  f4 xa[kPF];
  {
    const float* xp = (const float*)a.in + (size_t)(item / blocksPerBatch) * a.in_batch +
                      (size_t)(item % blocksPerBatch) * kRowLen + w * 4096 + (l0 & 15) * 16 + (l0 >> 4) * 4;
#pragma unroll
    for (int t = 0; t < kPF; t++) xa[t] = *(const f4*)(xp + t * 256);
  }

  auto processItem = [&](const uint32_t item) {
    // The lane id is laundered once per item: the hundreds of lane-dependent LDS offsets below are
    // loop invariant, and hoisting them out of the item loop would pin them all in registers.
    int l = l0;
    asm volatile("" : "+v"(l));
    const int i = l & 15, kb = l >> 4;
    const uint32_t m = item % blocksPerBatch, b = item / blocksPerBatch;
    const float* X = (const float*)a.in + (size_t)b * a.in_batch + (size_t)m * kRowLen;
    float* Z = (float*)a.out + (size_t)b * a.out_batch + (size_t)m * kRowLen;
    if (perBatchFactors && item != blockIdx.x && b != (item - gridDim.x) / blocksPerBatch) {   // a new batch: restage its factors
      stageFactors(b);                                               // (all waves are past the closing barrier of the previous item)
      __syncthreads();
    }

    // ---- the rest of the row: blocks t = kPF..15 ----
    f4 xb[16 - kPF];
    {
      const float* xp = X + w * 4096 + i * 16 + kb * 4 + kPF * 256;
#pragma unroll
      for (int t = 0; t < 16 - kPF; t++) xb[t] = *(const f4*)(xp + t * 256);
    }

    // LDS column of (k1 = w, k2 = t) is w*16 + t: the four blocks t = 4g .. 4g+3 of a lane are one 16-byte chunk
    // of its row.  The chunk index is XORed with q3 = i so that the 64 rows of a wave-level write spread over
    // the banks.
    auto writeGroup = [&](const int g, const int h) {
#pragma unroll
      for (int rr = 0; rr < 2; rr++) {
        f4 v;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          const int t = 4 * g + e;
          v[e] = (t < kPF) ? xa[t < kPF ? t : 0][2 * h + rr] : xb[t < kPF ? 0 : t - kPF][2 * h + rr];
        }
        *(f4*)&lds[((kb * 2 + rr) * 16 + i) * 256 + (((w * 4 + g) ^ i) << 2)] = v;
      }
    };

    // ---- stage 1: contract k3 (first product) and k4 (second product), block by block.  The half of
    //      the result with bit 1 of q3 clear goes to LDS at once, under the products of the next blocks. ----
    {
      // both products of this chain take the contraction index as 4*k + r (lane group k, instruction r): the
      // first contracts k4, which the 16-byte loads put in the registers of a lane, the second k3, which
      // the first leaves in the registers of its accumulator: B_r[k][j] = F[4k + r][j]
      float FA[4], FB[4];
#pragma unroll
      for (int c = 0; c < 4; c++) {
        FA[c] = fl[1 * 256 + (4 * kb + c) * 16 + i];      // F3
        FB[c] = fl[0 * 256 + (4 * kb + c) * 16 + i];      // F4
      }
      auto stage1 = [&](auto& x, const int nt, const int t0) {
#pragma unroll
        for (int t = 0; t < nt; t++) {
          f4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int r = 0; r < 4; r++) d = MFMA16(x[t][r], FB[r], d);     // d[k3][q4]
          f4 e = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int r = 0; r < 4; r++) e = MFMA16(d[r], FA[r], e);        // e[q4][q3]
          // e[r] = Y[k1=w][k2=t0+t][q4=4kb+r][q3=i]: from here to the second exchange q3 and q4 appear with their
          // roles swapped with respect to the comments below (the first exchange treats them alike)
          x[t] = e;
          if (((t0 + t) & 3) == 3) writeGroup((t0 + t) >> 2, 0);
        }
      };
      stage1(xa, kPF, 0);
      stage1(xb, 16 - kPF, kPF);
    }

    // ---- exchange 1: rows (q3,q4), columns (k1,k2); half h holds the rows with bit 1 of q3 == h.
    //      Reader layout: z[u][c] = Y[k1=4c+kb][k2=i][q3=u][q4=w]. ----
    float z[16][4];
#pragma unroll
    for (int h = 0; h < 2; h++) {
      if (h) {
        __syncthreads();
#pragma unroll
        for (int g = 0; g < 4; g++) writeGroup(g, 1);
      }
      __syncthreads();
#pragma unroll
      for (int u = 0; u < 16; u++) {
        if (((u >> 1) & 1) != h) continue;
        const int row = ((u >> 2) * 2 + (u & 1)) * 16 + w;
        // column (k1 = 4c + kb, k2 = i) = c*64 + l: chunk c*16 + l/4, XORed with the row's q3 = w as written
#pragma unroll
        for (int c = 0; c < 4; c++) z[u][c] = lds[row * 256 + ((((c * 16 + (l >> 2)) ^ w) << 2) | (l & 3))];
      }
    }
    __syncthreads();

    // ---- the first half of the next item streams in from here on ----
    {
      const uint32_t nx = item + gridDim.x;
      if (nx < totalItems) {
        const float* xp = (const float*)a.in + (size_t)(nx / blocksPerBatch) * a.in_batch +
                          (size_t)(nx % blocksPerBatch) * kRowLen + w * 4096 + i * 16 + kb * 4;
#pragma unroll
        for (int t = 0; t < kPF; t++) xa[t] = *(const f4*)(xp + t * 256);
      }
    }

    // ---- stage 2: contract k1 (first product) and k2 (second product); half 0 of exchange 2 goes out
    //      at once (rows (q1,q2), columns (q3,q4); half h holds the rows with bit 1 of q1 == h) ----
    {
      float FC[4], FD[4];
#pragma unroll
      for (int c = 0; c < 4; c++) {
        FC[c] = fl[3 * 256 + (4 * c + kb) * 16 + i];      // F1
        FD[c] = fl[2 * 256 + (4 * kb + c) * 16 + i];      // F2
      }
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
        // four consecutive columns (w*16 + u, u = 4g .. 4g+3) of a row go out as one 16-byte write; the chunk
        // index is XORed with q2 so that the lanes of a write (same chunk, 64 rows) spread over the banks
        if ((u & 3) == 3) {
          const int g = u >> 2;
#pragma unroll
          for (int rr = 0; rr < 2; rr++) {
            const f4 v = {z[4 * g][rr], z[4 * g + 1][rr], z[4 * g + 2][rr], z[4 * g + 3][rr]};
            *(f4*)&lds[((kb * 2 + rr) * 16 + i) * 256 + (((w * 4 + g) ^ i) << 2)] = v;
          }
        }
      }
    }

    // ---- exchange 2 and store, half by half.  Reader: wave w owns q2 = w, lane owns columns 4l..4l+3,
    //      register index is q1; every wave-level store covers 1 KB of contiguous columns. ----
    const float alpha = (float)a.alpha, beta = (float)a.beta;
    const float* Y = HAS_Y ? (const float*)a.y + (size_t)b * a.y_batch + (size_t)m * kRowLen : nullptr;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      if (h) {
        __syncthreads();
#pragma unroll
        for (int g = 0; g < 4; g++)
#pragma unroll
          for (int rr = 0; rr < 2; rr++) {
            const int row = (kb * 2 + rr) * 16 + i;
            const f4 v = {z[4 * g][2 + rr], z[4 * g + 1][2 + rr], z[4 * g + 2][2 + rr], z[4 * g + 3][2 + rr]};
            *(f4*)&lds[row * 256 + (((w * 4 + g) ^ i) << 2)] = v;
          }
      }
      __syncthreads();
      // four vectors at a time: their Y values are fetched before their first store (loads and stores
      // share one in-order counter)
#pragma unroll
      for (int g = 0; g < 2; g++) {
        f4 o[4], yv[HAS_Y ? 4 : 1];
#pragma unroll
        for (int k = 0; k < 4; k++) {
          const int q1hi = 2 * g + (k >> 1), rr = k & 1;
          const int row = (q1hi * 2 + rr) * 16 + w;
          o[k] = *(const f4*)&lds[row * 256 + ((l * 4) ^ (w * 4))];     // chunk l of the row of (q1, q2 = w)
          if (HAS_Y) yv[k] = *(const f4*)(Y + (4 * q1hi + 2 * h + rr) * 4096 + w * 256 + l * 4);
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
          const int q1hi = 2 * g + (k >> 1), rr = k & 1;
          const int col = (4 * q1hi + 2 * h + rr) * 4096 + w * 256 + l * 4;
          f4 v = o[k];
          if (a.epilogue) {
            v = v * alpha;
            if (HAS_Y) v = v + yv[k] * beta;
          }
          *(f4*)(Z + col) = v;
        }
      }
    }
    __syncthreads();      // every wave has read its last LDS word before the next item's stage 1 writes
  };

  // The first item is peeled off the loop.  Loads and stores retire through one in-order counter, and the
  // wait for the prefetched blocks is counted in younger operations: entering the loop only from a complete
  // item lets that count include the stores issued behind the prefetch, so that the wait at the top of an
  // item does not drain the previous item's stores.
  processItem(item);
  for (item += gridDim.x; item < totalItems; item += gridDim.x) processItem(item);
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
  const size_t ldsBytes = (kLdsWords + 4 * 256) * sizeof(float);
  if (!attrSet) {
    hipError_t e = hipFuncSetAttribute((const void*)kron_row16x4_kernel<true>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute((const void*)kron_row16x4_kernel<false>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
    if (e != hipSuccess) return e;
    attrSet = true;
  }
  static int cus = 0;
  if (!cus) {
    int dev = 0;
    hipDeviceProp_t prop;
    cus = (hipGetDevice(&dev) == hipSuccess && hipGetDeviceProperties(&prop, dev) == hipSuccess)
              ? prop.multiProcessorCount : 256;
  }
  const uint32_t blocksPerBatch = a.M / row16Rows(a);
  const uint64_t total = (uint64_t)blocksPerBatch * a.batch;
  if (total >= (1ull << 32)) return hipErrorInvalidValue;
  // persistent workgroups, one per CU.  (Delaying a part of the workgroups at start to interleave the HBM and
  // on-chip phases of different CUs was measured and gains nothing once the next item is prefetched.)
  const uint32_t wgs = total < (uint64_t)cus ? (uint32_t)total : (uint32_t)cus;
  dim3 grid(wgs), block(1024);
  if (a.y && a.epilogue)
    hipLaunchKernelGGL(kron_row16x4_kernel<true>, grid, block, ldsBytes, stream, a, blocksPerBatch, (uint32_t)total);
  else
    hipLaunchKernelGGL(kron_row16x4_kernel<false>, grid, block, ldsBytes, stream, a, blocksPerBatch, (uint32_t)total);
  return hipGetLastError();
}

}  // namespace fk
