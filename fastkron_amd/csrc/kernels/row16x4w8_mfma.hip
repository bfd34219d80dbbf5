// Whole-block kernel for up to four fused 16x16 fp32 factors on contiguous blocks of 16^4 = 65536 elements,
// eight-wave variant: the same two chained matrix-core stages and two LDS exchanges as row16x4_mfma.hip,
// but the block is held by 512 threads with 128 values each instead of 1024 threads with 64.
//
//   Z[q1,q2,q3,q4] = alpha * sum_{k1..k4} X[k1,k2,k3,k4] F1[k1,q1] F2[k2,q2] F3[k3,q3] F4[k4,q4] (+ beta*Y)
//
// Why fewer, fatter waves: a CU holds one block at a time, so its HBM phases (load, store) and on-chip
// phases (two MFMA stages, two exchanges) overlap only through what is prefetched for the next block.
// With two waves per SIMD a lane has 256 registers: the stage-1 operand registers x[2][16][4] are dead once
// the first exchange has read them out, and the stage-2 registers z[2][16][4] die block by block as their
// results go to LDS, so the *whole* next block is requested under stage 2, the second exchange and the
// stores of the current one - 64 registers' worth when stage 2 starts, 4 more after every second stage-2
// block - and no load is left for the top of the next item.
//
// Index map (wave w owns the two "virtual waves" vw = w and w + 8; lane l: i = l%16, kb = l/16):
//   stage 1   x[v][t][r] = X[k1=vw][k2=t][k3=i][k4=4kb+r]      -> Y[k1=vw][k2=t][q3=i][q4=4kb+r] in register r
//             (one 16-byte load per lane and block: fewer, wider memory instructions stall the waves less;
//             below, q3 and q4 appear with their roles swapped until the second exchange restores the order)
//   exch. 1   rows (q3,q4), columns (k1,k2), two halves by bit 1 of q3, XOR-swizzled by the writer's lane
//   stage 2   z[v][u][c] = Y[k1=4c+kb][k2=i][q3=u][q4=vw]      -> Z[q1=4kb+r][q2=i][q3=u][q4=vw] in register r
//   exch. 2   rows (q1,q2), columns (q3,q4), two halves by bit 1 of q1; reader: q2 = vw, lane = 4 columns
// The chained products, the swizzles and the factor slots (identity for fewer than four factors) are those
// of row16x4_mfma.hip.  Loads and stores retire through one in-order counter: the first item is peeled off
// the persistent loop so that the wait for prefetched registers is counted in younger operations (the
// stores issued behind the prefetch) and does not drain them.
//
// Measured on sgemkm 1024 x 16^4 this build and the 16-wave build run within 1 % of each other (the on-chip
// phases, about 24 us per block, are the critical path of both), so it is registered as an alternative that
// the tuner may pick; the online selection prefers the 16-wave build.
//
// Algorithmic traffic: 4*65536 bytes read + 4*65536 bytes written per block (+ Y when beta != 0).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float w8f4 __attribute__((ext_vector_type(4)));

#define W8MFMA(a, b, c) __builtin_amdgcn_mfma_f32_16x16x4f32((a), (b), (c), 0, 0, 0)

constexpr int kW8RowLen = 65536;
constexpr int kW8LdsWords = 32768;          // 128 KB: one half of a block
constexpr int kW8Early = 16;                // (v,t) register blocks of the next item requested when stage 2 starts

template <bool HAS_Y>
__global__ __launch_bounds__(512, 2) void kron_row16x4w8_kernel(const StepArgs a, const uint32_t blocksPerBatch,
                                                                const uint32_t totalItems) {
  extern __shared__ __align__(16) float lds[];
  const int tid = threadIdx.x;
  const int l0 = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);      // wave-uniform: keeps row addresses in SGPRs

  uint32_t item = blockIdx.x;
  if (item >= totalItems) return;

  // Factors: a.f[0] is the last factor (F4) ... a.f[3] the first (F1); missing leading factors are identity
  // slots (their digits are row indices).  Staged in LDS behind the exchange buffer, fl[j*256 + p*16 + q].
  float* fl = lds + kW8LdsWords;
  auto stageFactors = [&](uint32_t b) {
#pragma unroll
    for (int h = 0; h < 2; h++) {
      const int e = tid + 512 * h;
      const int j = e >> 8, p = (e >> 4) & 15, q = e & 15;
      float v = (p == q) ? 1.f : 0.f;
      if (j < (int)a.nf) {
        const float* f = (const float*)a.f[j] + (size_t)b * a.f_batch[j];
        v = f[(int64_t)p * a.f_sp[j] + (int64_t)q * a.f_sq[j]];
      }
      fl[e] = v;
    }
  };
  bool perBatchFactors = false;
  for (uint32_t j = 0; j < a.nf; j++) perBatchFactors |= (a.f_batch[j] != 0);
  stageFactors(item / blocksPerBatch);
  __syncthreads();

  // x[v*16 + t][c]: registers of stage 1; block (v,t) of an item is one 1 KB row segment per c
  w8f4 x[32];
  auto itemBase = [&](uint32_t it) {
    return (const float*)a.in + (size_t)(it / blocksPerBatch) * a.in_batch + (size_t)(it % blocksPerBatch) * kW8RowLen;
  };
  // one 16-byte load per lane and block: x[vt][r] = X[k1=vw][k2=t][k3=i][k4=4kb+r] (a wave reads 1 KB per instruction)
  const int ldOfs = (l0 & 15) * 16 + (l0 >> 4) * 4;
  auto loadBlock = [&](const float* X, int vt) {
    x[vt] = *(const w8f4*)(X + ((vt >> 4) * 8 + w) * 4096 + (vt & 15) * 256 + ldOfs);
  };
  // The last item of a workgroup has nothing to prefetch.  Its registers are then *overwritten* rather than
  // left alone: a register that keeps its old value on one path stays live from stage 1 to this point on
  // every path, and 128 such registers on top of the stage-2 operands do not fit.
  auto prefetchBlock = [&](bool hasNext, const float* X, int vt) {
    if (hasNext) {
      loadBlock(X, vt);
    } else {
      x[vt] = (w8f4){0.f, 0.f, 0.f, 0.f};
    }
  };
  {
    const float* X = itemBase(item);
#pragma unroll
    for (int vt = 0; vt < 32; vt++) loadBlock(X, vt);
  }

  auto processItem = [&](const uint32_t item) {
    // The lane id is laundered once per item: the hundreds of lane-dependent LDS offsets below are
    // loop invariant, and hoisting them out of the item loop would pin them all in registers.
    int l = l0;
    asm volatile("" : "+v"(l));
    const int i = l & 15, kb = l >> 4;
    const uint32_t m = item % blocksPerBatch, b = item / blocksPerBatch;
    float* Z = (float*)a.out + (size_t)b * a.out_batch + (size_t)m * kW8RowLen;
    if (perBatchFactors && item != blockIdx.x && b != (item - gridDim.x) / blocksPerBatch) {   // a new batch: restage its factors
      stageFactors(b);                                               // (all waves are past the closing barrier of the previous item)
      __syncthreads();
    }
    // the next item of this workgroup (uniform: the prefetch below is skipped as a whole for the last one)
    const bool hasNext = item + gridDim.x < totalItems;
    const float* XN = itemBase(hasNext ? item + gridDim.x : item);

    float xk[32][2], zk[32][2];                           // the halves of the stage results that wait for exchange half 1
    // ---- stage 1: contract k3 (first product) and k4 (second product), block by block.  The half of
    //      the result with bit 1 of q3 clear goes to LDS at once, under the products of the next blocks. ----
    {
      // both products of this chain take the contraction index as 4*k + r (lane group k, instruction r):
      // the first contracts k4, which the 16-byte loads put in the registers of a lane, the second k3,
      // which the first leaves in the registers of its accumulator: B_r[k][j] = F[4k + r][j]
      float FA[4], FB[4];
#pragma unroll
      for (int c = 0; c < 4; c++) {
        FA[c] = fl[1 * 256 + (4 * kb + c) * 16 + i];      // F3
        FB[c] = fl[0 * 256 + (4 * kb + c) * 16 + i];      // F4
      }
#pragma unroll
      for (int vt = 0; vt < 32; vt++) {
        const int vw = (vt >> 4) * 8 + w, t = vt & 15;
        w8f4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < 4; r++) d = W8MFMA(x[vt][r], FB[r], d);      // d[k3][q4]
        w8f4 e = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < 4; r++) e = W8MFMA(d[r], FA[r], e);          // e[q4][q3]
        // e[r] = Y[k1=vw][k2=t][q4=4kb+r][q3=i]: from here to the second exchange the roles of q3 and q4 are
        // swapped with respect to the index map in the header (the exchange treats them alike).  Elements 0, 1 go to LDS at once; 2, 3 are *moved* out of the
        // accumulator tuple (an opaque move the compiler cannot fold): a tuple with two live elements would pin
        // four aligned registers, and 32 such tuples leave no room for the 32 of the next phase.
#pragma unroll
        for (int rr = 0; rr < 2; rr++)
          lds[((kb * 2 + rr) * 16 + i) * 256 + ((vw * 16 + t) ^ l)] = e[rr];
#pragma unroll
        for (int rr = 0; rr < 2; rr++) asm volatile("v_mov_b32 %0, %1" : "=v"(xk[vt][rr]) : "v"(e[2 + rr]));
        __builtin_amdgcn_sched_barrier(0);                // keep the blocks in program order: the scheduler otherwise
      }                                                   // runs ahead with loads and offsets and overflows the registers
    }

    // ---- exchange 1: rows (q3,q4), columns (k1,k2); half h holds the rows with bit 1 of q3 == h.
    //      Reader layout: z[v*16 + u][c] = Y[k1=4c+kb][k2=i][q3=u][q4=vw]. ----
    float z[32][4];
#pragma unroll
    for (int h = 0; h < 2; h++) {
      if (h) {
        __syncthreads();
        // a fresh opaque lane id per phase: otherwise the 64 offsets of the stage-1 writes above are kept
        // in registers for these writes, which use the same ones
        int lw = l0;
        asm volatile("" : "+v"(lw));
        const int iw = lw & 15, kbw = lw >> 4;
#pragma unroll
        for (int vt = 0; vt < 32; vt++)
#pragma unroll
          for (int rr = 0; rr < 2; rr++) {
            const int vw = (vt >> 4) * 8 + w, t = vt & 15;
            lds[((kbw * 2 + rr) * 16 + iw) * 256 + ((vw * 16 + t) ^ lw)] = xk[vt][rr];
          }
      }
      __syncthreads();
#pragma unroll
      for (int vu = 0; vu < 32; vu++) {
        const int vw = (vu >> 4) * 8 + w, u = vu & 15;
        if (((u >> 1) & 1) != h) continue;
        const int row = ((u >> 2) * 2 + (u & 1)) * 16 + vw;
        const int swz = vw + 16 * (u >> 2);
#pragma unroll
        for (int c = 0; c < 4; c++) z[vu][c] = lds[row * 256 + ((c * 64 + l) ^ swz)];
        if ((vu & 3) == 3) __builtin_amdgcn_sched_barrier(0);
      }
    }
    __syncthreads();

    // ---- the next item streams in from here on: kW8Early register blocks now, the rest as stage 2 frees
    //      registers (two per finished block) ----
#pragma unroll
    for (int vt = 0; vt < kW8Early; vt++) prefetchBlock(hasNext, XN, vt);

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
      for (int vu = 0; vu < 32; vu++) {
        const int vw = (vu >> 4) * 8 + w, u = vu & 15;
        w8f4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int c = 0; c < 4; c++) d = W8MFMA(z[vu][c], FC[c], d);
        w8f4 e = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < 4; r++) e = W8MFMA(d[r], FD[r], e);
        // e[r] = Z[q1=4kb+r][q2=i][q4=u][q3=vw]: column q3*16 + q4 = vw*16 + u
#pragma unroll
        for (int rr = 0; rr < 2; rr++)
          lds[((kb * 2 + rr) * 16 + i) * 256 + ((vw * 16 + u) ^ (i * 4) ^ kb)] = e[rr];
#pragma unroll
        for (int rr = 0; rr < 2; rr++) asm volatile("v_mov_b32 %0, %1" : "=v"(zk[vu][rr]) : "v"(e[2 + rr]));
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // the rest of the next item: the stage-2 operands are dead now (loads issued between the products of stage 2
    // stall the wave, and with it the matrix pipe, whenever the memory path is backed up)
#pragma unroll
    for (int vt = kW8Early; vt < 32; vt++) prefetchBlock(hasNext, XN, vt);

    // ---- exchange 2 and store, half by half.  Reader: q2 = vw, lane owns columns 4l..4l+3, register
    //      index is q1; every wave-level store covers 1 KB of contiguous columns. ----
    const float alpha = (float)a.alpha, beta = (float)a.beta;
    const float* Y = HAS_Y ? (const float*)a.y + (size_t)b * a.y_batch + (size_t)m * kW8RowLen : nullptr;
#pragma unroll
    for (int h = 0; h < 2; h++) {
      if (h) {
        __syncthreads();
        int lw = l0;
        asm volatile("" : "+v"(lw));
        const int iw = lw & 15, kbw = lw >> 4;
#pragma unroll
        for (int vu = 0; vu < 32; vu++)
#pragma unroll
          for (int rr = 0; rr < 2; rr++) {
            const int vw = (vu >> 4) * 8 + w, u = vu & 15;
            lds[((kbw * 2 + rr) * 16 + iw) * 256 + ((vw * 16 + u) ^ (iw * 4) ^ kbw)] = zk[vu][rr];
          }
      }
      __syncthreads();
      // four vectors at a time: their Y values are fetched before their first store (loads and stores
      // share one in-order counter)
#pragma unroll
      for (int vg = 0; vg < 4; vg++) {
        const int vw = (vg >> 1) * 8 + w, g = vg & 1;
        w8f4 o[4], yv[HAS_Y ? 4 : 1];
#pragma unroll
        for (int k = 0; k < 4; k++) {
          const int q1hi = 2 * g + (k >> 1), rr = k & 1;
          const int row = (q1hi * 2 + rr) * 16 + vw;
          const w8f4 v = *(const w8f4*)&lds[row * 256 + ((l * 4) ^ (vw * 4))];
          w8f4 p;                                         // word e of v is column 4l + (e ^ q1hi)
          p[0] = v[0 ^ q1hi]; p[1] = v[1 ^ q1hi]; p[2] = v[2 ^ q1hi]; p[3] = v[3 ^ q1hi];
          o[k] = p;
          if (HAS_Y) yv[k] = *(const w8f4*)(Y + (4 * q1hi + 2 * h + rr) * 4096 + vw * 256 + l * 4);
        }
#pragma unroll
        for (int k = 0; k < 4; k++) {
          const int q1hi = 2 * g + (k >> 1), rr = k & 1;
          const int col = (4 * q1hi + 2 * h + rr) * 4096 + vw * 256 + l * 4;
          w8f4 v = o[k];
          if (a.epilogue) {
            v = v * alpha;
            if (HAS_Y) v = v + yv[k] * beta;
          }
          *(w8f4*)(Z + col) = v;
        }
      }
    }
    __syncthreads();      // every wave has read its last LDS word before the next item's stage 1 writes
  };

  processItem(item);
  for (item += gridDim.x; item < totalItems; item += gridDim.x) processItem(item);
}

// Rows per workgroup: 16^(4-nf).
static uint32_t w8Rows(const StepArgs& a) { uint32_t r = 1; for (uint32_t j = a.nf; j < 4; j++) r *= 16; return r; }

bool row16x4W8Supported(const StepArgs& a) {
  if (a.nf < 2 || a.nf > 4) return false;
  uint64_t k = 1;
  for (uint32_t j = 0; j < a.nf; j++) { if (a.p[j] != 16 || a.q[j] != 16) return false; k *= 16; }
  if (a.Kin != k || a.Kout != k) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  // the rows of a block must be contiguous, and M must be a whole number of blocks
  if ((uint64_t)a.in_ldm != k || (uint64_t)a.out_ldm != k || (a.y && (uint64_t)a.y_ldm != k)) return false;
  if (a.M % w8Rows(a)) return false;
  // 16-byte aligned blocks for the vector loads, stores and Y loads
  if (((uintptr_t)a.in & 15) || (a.in_batch & 3)) return false;
  if (((uintptr_t)a.out & 15) || (a.out_batch & 3)) return false;
  if (a.y && (((uintptr_t)a.y & 15) || (a.y_batch & 3))) return false;
  return a.batch <= 65535;
}

hipError_t launchRow16x4W8(const StepArgs& a, hipStream_t stream) {
  if (!row16x4W8Supported(a)) return hipErrorInvalidValue;
  static PerDeviceOnce attrOnce;
  const int devIdx = launchDeviceIndex();
  const size_t ldsBytes = (kW8LdsWords + 4 * 256) * sizeof(float);
  if (!attrOnce.done(devIdx)) {
    hipError_t e = hipFuncSetAttribute((const void*)kron_row16x4w8_kernel<true>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute((const void*)kron_row16x4w8_kernel<false>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
    if (e != hipSuccess) return e;
    attrOnce.mark(devIdx);
  }
  const int cus = deviceCUs();
  const uint32_t blocksPerBatch = a.M / w8Rows(a);
  const uint64_t total = (uint64_t)blocksPerBatch * a.batch;
  if (total >= (1ull << 32)) return hipErrorInvalidValue;
  const uint32_t wgs = total < (uint64_t)cus ? (uint32_t)total : (uint32_t)cus;     // persistent, one per CU
  dim3 grid(wgs), block(512);
  if (a.y && a.epilogue)
    hipLaunchKernelGGL(kron_row16x4w8_kernel<true>, grid, block, ldsBytes, stream, a, blocksPerBatch, (uint32_t)total);
  else
    hipLaunchKernelGGL(kron_row16x4w8_kernel<false>, grid, block, ldsBytes, stream, a, blocksPerBatch, (uint32_t)total);
  return hipGetLastError();
}

}  // namespace fk
