// Whole-row kernel for four fused 16x16 fp32 factors (row length 16^4 = 65536, e.g. sgemkm
// 1024 x 65536 with 16x16^4): one persistent workgroup of 16 wave64s per CU owns one row at a time, keeps it in
// VGPRs and touches HBM exactly once for the read and once for the write.
//
//   Z[q1,q2,q3,q4] = alpha * sum_{k1..k4} X[k1,k2,k3,k4] F1[k1,q1] F2[k2,q2] F3[k3,q3] F4[k4,q4] (+ beta*Y)
//
// The reference cannot fuse this shape in one launch (its tile must fit 48 KB of shared memory,
// reference src/gen_tuner_kernels.py:10,366; it runs 2 launches of 2 fused factors each).  Here the
// row (256 KB) does not fit the 160 KB LDS either, so the LDS is only an exchange buffer, crossed once:
//
//   load     wave w owns the block k1 = w (4096 contiguous elements): one 16-byte load per lane and
//            256-element slice (k3 = lane%16, k4 = 4*(lane/16) + register), a window of kWin slices in flight
//            (kCarry of them, the first of the next row, across the exchange)
//   k4, k3   per slice, V_MFMA_F32_16X16X4_F32 chained in registers: the first product leaves D[i][j] in
//            register i%4 of lane 16*(i/4)+j, which is exactly the A-operand layout (lane 16*k+i) of a
//            second product that contracts the *row* index i of the first; the factor operand of the
//            second product is loaded with its rows permuted (4*k + r) to match.  No data movement.
//   k2       the slice index: V_MFMA_F32_4X4X1_16B_F32 (16 independent 4x4 outer products per instruction)
//            adds every slice's share to the lane's 16 x 4 accumulators, acc[q2][r] += F2[k2][q2] * T[k2][r].
//            Up to here a wave works on its own: no barrier, no LDS traffic but operands, and every slice
//            worked on frees the registers for the request of the slice kWin later, so the loads of a row
//            are spread over this phase (and run on into the first kCarry slices of the next row).
//   k1       the one digit that couples the waves: quarter by quarter (q2 = 4*qq .. 4*qq+3, 64 KB) through
//            a double-buffered LDS exchange, 16-byte writes and reads; the quarter qq+1 is written between
//            the same two barriers in which the quarter qq is consumed: one 16x16x4 product per 16 columns,
//            D[q1][col] = sum_k1 F1[k1][q1] T2[k1][col], stored straight from the accumulators (a lane holds
//            four consecutive columns of four rows q1; 256 contiguous bytes per quarter wave).  The stores
//            of a row are spread over this phase.  Four barriers per row.
//
// Vector memory instructions of a CU pass through one in-order pipeline: stores issued behind a burst of loads
// wait for it, and so do the waves that issue them.  Hence the spreading above (a burst of 16 loads per lane
// behind the last quarter, with the stores of two quarters behind it, costs 14 us per row), and the register
// budget (64 accumulators + the window out of 128) is what limits the window: one window slot that the compiler
// has to spill right after its load makes the wave wait for that load, and costs 8 % of the launch.
// The CUs start in lockstep and would alternate between a phase in which all of them wait for HBM and a phase in
// which none uses it; the workgroups start in kStaggerGroups groups, kStaggerTicks apart (when a workgroup has more
// than one row to work on), which interleaves the phases of neighbouring CUs.
//
// Algorithmic traffic: 4*65536 bytes read + 4*65536 bytes written per row (+ Y when beta != 0).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float f4 __attribute__((ext_vector_type(4)));

#define MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x4f32((a), (b), (c), 0, 0, 0)
#define MFMA4(a, b, c) __builtin_amdgcn_mfma_f32_4x4x1f32((a), (b), (c), 0, 0, 0)

constexpr int kRowLen = 65536;
constexpr int kWin = 6;            // slices in flight per wave while it works on slices (registers: 64 accumulators + 4*kWin + operands)
constexpr int kCarry = 2;        // slices of the next row in flight during the exchange (<= kWin)
constexpr uint32_t kStaggerGroups = 5;     // measured: 5 groups 2.5 us apart or 3 groups 4 us apart; 2 or 4 groups lose to no stagger
constexpr uint32_t kStaggerTicks = 250;    // of the 100 MHz wall clock
constexpr int kQuarterWords = 16384;       // 64 KB: 16 rows k1 of 1024 columns (four values of q2)
constexpr int kFacWords = 320;            // a staged factor: element (p, q) at 16*(p + p/4) + q (rows padded so that lanes
                                          // reading rows 4k + c, k = lane/16, cover all 64 banks)
constexpr int kLdsWords = 2 * kQuarterWords + 4 * kFacWords + 256;   // two quarters + the four factors + F2 transposed

// NT: 0 = ordinary accesses, 1 = streaming stores, 2 = non-temporal loads of X as well.  The streaming stores are
// 16-byte stores at system scope through a buffer descriptor of the row (sgemkm 1024 x 16^4: 103.7 us with
// non-temporal stores, 99.1 us with these).
template <bool HAS_Y, int NT>
__global__ __launch_bounds__(1024, 1) void kron_row16x4_kernel(const StepArgs a, const uint32_t blocksPerBatch,
                                                               const uint32_t totalItems, const uint32_t staggerTicks) {
  extern __shared__ __align__(16) float lds[];
  const int tid = threadIdx.x;
  const int l0 = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);      // wave-uniform: keeps row addresses in SGPRs

  uint32_t item = blockIdx.x;
  if (item >= totalItems) return;

  // Factors: a.f[0] is the last factor (F4) ... a.f[3] the first (F1); with fewer than four factors the
  // leading digits are row indices (16^(4-nf) consecutive rows form the same contiguous 65536-element
  // block) and their factor slots hold the identity.  The four 16x16 matrices are staged in LDS behind
  // the exchange buffers, fl[j*320 + 16*(p + p/4) + q], F2 a second time as f2t[k2*16 + (q2%4)*4 + q2/4] (the 4x4x1 operand of a lane, the four
  // values F2[k2][4*qq + lane%4], is one 16-byte read), and operands
  // are read from there right before use: LDS reads do not queue behind the row loads the way small global
  // loads would (vector memory operations retire in order).
  float* fl = lds + 2 * kQuarterWords;
  float* f2t = fl + 4 * kFacWords;
  auto stageFactors = [&](uint32_t b) {
    const int j = tid >> 8, p = (tid >> 4) & 15, q = tid & 15;
    float v = (p == q) ? 1.f : 0.f;
    if (j < (int)a.nf) {
      const float* f = (const float*)a.f[j] + (size_t)b * a.f_batch[j];
      v = f[(int64_t)p * a.f_sp[j] + (int64_t)q * a.f_sq[j]];
    }
    fl[j * kFacWords + 16 * (p + (p >> 2)) + q] = v;
    if (j == 2) f2t[p * 16 + (q & 3) * 4 + (q >> 2)] = v;      // [k2][q2 % 4][q2 / 4]
  };
  bool perBatchFactors = false;
  for (uint32_t j = 0; j < a.nf; j++) perBatchFactors |= (a.f_batch[j] != 0);
  stageFactors(item / blocksPerBatch);

  // An item is a block of 65536 contiguous elements: one row for four factors, 16^(4-nf) rows otherwise.
  // x[t][r] = X[k1=w][k2=t][k3=i][k4=4kb+r] (i = l%16, kb = l/16): 1 KB per wave instruction.
  // kWin slices are in flight: slice t + kWin is requested when slice t has been read, and the first kCarry slices
  // of the next item behind the last ones of this item; the other kWin - kCarry follow at the start of that item.
  f4 xw[kWin];
  // uniform part of a slice address (scalar registers) and the lane's part (one 32-bit register)
  auto slicePtr = [&](const uint32_t it) {
    return (const float*)a.in + (size_t)(it / blocksPerBatch) * a.in_batch + (size_t)(it % blocksPerBatch) * kRowLen +
           w * 4096;
  };
  const uint32_t laneOff = (l0 & 15) * 16 + (l0 >> 4) * 4;
  if (staggerTicks) {
    const uint32_t grp = (blockIdx.x >> 3) % kStaggerGroups;      // blockIdx % 8 is the XCD
    if (grp) {
      const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
      while (__builtin_amdgcn_s_memrealtime() - t0 < (unsigned long long)grp * staggerTicks) __builtin_amdgcn_s_sleep(16);
    }
  }
  {
    const float* xp = slicePtr(item);
#pragma unroll
    for (int t = 0; t < kCarry; t++) xw[t] = FK_LD(NT, (const f4*)(xp + (laneOff + t * 256)));
  }
  __syncthreads();

  const float alpha = a.epilogue ? (float)a.alpha : 1.f, beta = (float)a.beta;    // HAS_Y implies a.epilogue
  uint32_t batchOfFactors = item / blocksPerBatch;

  for (;;) {
    // The lane id is laundered once per item: the lane-dependent LDS offsets below are loop invariant, and
    // hoisting them out of the item loop would pin them in registers.
    int l = l0;
    asm volatile("" : "+v"(l));
    const int i = l & 15, kb = l >> 4;
    const uint32_t m = item % blocksPerBatch, b = item / blocksPerBatch;
    // row bases pinned to scalar registers: the stores then take one 32-bit lane offset each instead of an address pair
    typedef __attribute__((address_space(1))) float GlobalFloat;
    typedef __attribute__((address_space(1))) f4 GlobalF4;
    auto uniformPtr = [](const void* p) {
      const uintptr_t v = (uintptr_t)p;
      const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)v), hi = __builtin_amdgcn_readfirstlane((uint32_t)(v >> 32));
      return (GlobalFloat*)(((uintptr_t)hi << 32) | lo);
    };
    GlobalFloat* const Z = uniformPtr((float*)a.out + (size_t)b * a.out_batch + (size_t)m * kRowLen);
    const __amdgpu_buffer_rsrc_t zTarget = streamTarget((void*)(float*)Z, kRowLen * 4u);
    const GlobalFloat* const Y = HAS_Y ? uniformPtr((const float*)a.y + (size_t)b * a.y_batch + (size_t)m * kRowLen) : nullptr;
    if (perBatchFactors && b != batchOfFactors) {      // a new batch: restage its factors
      __syncthreads();                                 // every wave has read its last operand of the previous item
      stageFactors(b);
      __syncthreads();
      batchOfFactors = b;
    }
    const uint32_t nx = item + gridDim.x;

    // ---- k4 and k3 slice by slice, then the slice's share of k2: acc[qq][r][j] += F2[k2=t][4qq+j] * T[k2=t][q3=i][q4=4kb+r] ----
    f4 acc[4][4];
#pragma unroll
    for (int qq = 0; qq < 4; qq++)
#pragma unroll
      for (int r = 0; r < 4; r++) acc[qq][r] = (f4){0.f, 0.f, 0.f, 0.f};
    {
      // both products of the chain take the contraction index as 4*k + r (lane group k, instruction r): the
      // first contracts k4, which the 16-byte loads put in the registers of a lane, the second k3, which
      // the first leaves in the registers of its accumulator: B_r[k][j] = F[4k + r][j]
      float FA[4], FB[4];
#pragma unroll
      for (int c = 0; c < 4; c++) {
        FA[c] = fl[1 * kFacWords + (5 * kb + c) * 16 + i];      // F3
        FB[c] = fl[0 * kFacWords + (5 * kb + c) * 16 + i];      // F4
      }
      const float* const xcur = slicePtr(item);
#pragma unroll
      for (int t = kCarry; t < kWin; t++) xw[t] = FK_LD(NT, (const f4*)(xcur + (laneOff + t * 256)));
      // behind the last item the requests go to one cached kilobyte of the current row instead, and are dropped
      const float* const xnext = slicePtr(nx < totalItems ? nx : item);
      const int nextStride = nx < totalItems ? 256 : 0;
#pragma unroll
      for (int t = 0; t < 16; t++) {
        const f4 fa = *(const f4*)&f2t[t * 16 + (l & 3) * 4];          // fa[qq] = F2[k2 = t][q2 = 4qq + l%4]
        f4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < 4; r++) d = MFMA16(xw[t % kWin][r], FB[r], d);     // d[k3][q4]
        // the slot is free: request the slice that comes kWin later
        if (t + kWin < 16) xw[t % kWin] = FK_LD(NT, (const f4*)(xcur + (laneOff + (t + kWin) * 256)));
        else if (t + kWin - 16 < kCarry) xw[t % kWin] = FK_LD(NT, (const f4*)(xnext + (laneOff + (t + kWin - 16) * nextStride)));
        f4 e = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < 4; r++) e = MFMA16(d[r], FA[r], e);        // e[q4][q3]: e[r] = T[k2=t][q3=i][q4=4kb+r]
#pragma unroll
        for (int qq = 0; qq < 4; qq++)
#pragma unroll
          for (int r = 0; r < 4; r++) acc[qq][r] = MFMA4(fa[qq], e[r], acc[qq][r]);
        __builtin_amdgcn_sched_barrier(0);
      }
      // slice j of the next item sits in the slot that fell free for it, (16 - kWin + j) % kWin: to slot j
      if (16 % kWin) {
        f4 nxt[kCarry];
#pragma unroll
        for (int j = 0; j < kCarry; j++) nxt[j] = xw[(16 - kWin + j) % kWin];
#pragma unroll
        for (int j = 0; j < kCarry; j++) xw[j] = nxt[j];
      }
    }

    // Exchange geometry.  A quarter buffer holds T2[k1][q2l][piece][4]: row k1 (1024 words), q2l = q2 % 4, and the
    // 256 columns (q3,q4) of one q2 as 64 pieces of four.  Column piece o = 4*q3 + q4/4 sits at position
    // (o & 48) | (swap(o & 15) ^ 4*((o >> 4) & 1)), swap exchanging the two bit pairs of its argument.  The LDS takes a
    // 16-byte write eight consecutive lanes at a time and a 16-byte read sixteen at a time (measured: patterns that
    // repeat a bank within such a group count as conflicts, others do not): the eight writers (one kb, i = 8h .. 8h+7:
    // pieces 4 apart) land on positions that differ modulo 8, the sixteen readers (consecutive pieces) on positions
    // that differ modulo 16.
    const int wo = i * 4 + kb;
    float* const wbase = lds + w * 1024 + (((wo & 48) | ((((wo & 15) >> 2) | ((wo & 3) << 2)) ^ (((wo >> 4) & 1) << 2))) << 2);
    // reader: wave w takes q2l = w/4 and the 64 columns g = w%4 of it; lane (kb, i) reads row k1 = 4c + kb,
    // piece 16*g + i, and ends up with Z[q1 = 4kb + r][q2][64*g + 4*i + e] in register r of accumulator e
    const int g = w & 3, q2l = w >> 2;
    const float* const rbase = lds + kb * 1024 + q2l * 256 + g * 64 + ((((i >> 2) | ((i & 3) << 2)) ^ ((g & 1) << 2)) << 2);
    float f1[4];
#pragma unroll
    for (int c = 0; c < 4; c++) f1[c] = fl[3 * kFacWords + (5 * c + kb) * 16 + i];      // A operand: F1[k1 = 4c+kb][q1 = i]

    // quarter qq of the k2 result, written to buffer qq % 2
    auto produce = [&](const int qq) {
      float* const wb = wbase + (qq & 1) * kQuarterWords;
#pragma unroll
      for (int j = 0; j < 4; j++) *(f4*)(wb + j * 256) = (f4){acc[qq][0][j], acc[qq][1][j], acc[qq][2][j], acc[qq][3][j]};
    };
    // quarter qq of the k1 contraction, read from buffer qq % 2, and its stores
    auto consume = [&](const int qq) {
      const float* const rb = rbase + (qq & 1) * kQuarterWords;
      const uint32_t col = kb * 4 * 4096 + (4 * qq + q2l) * 256 + g * 64 + 4 * i;   // unsigned: uniform base + 32-bit lane offset
      f4 yv[HAS_Y ? 4 : 1];
      if (HAS_Y) {
#pragma unroll
        for (int r = 0; r < 4; r++) yv[r] = *(const GlobalF4*)(Y + (col + r * 4096));
      }
      f4 D[4];
#pragma unroll
      for (int e = 0; e < 4; e++) D[e] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < 4; c++) {
        const f4 v = *(const f4*)(rb + c * 4096);
#pragma unroll
        for (int e = 0; e < 4; e++) D[e] = MFMA16(f1[c], v[e], D[e]);
      }
#pragma unroll
      for (int r = 0; r < 4; r++) {
        f4 o = (f4){D[0][r], D[1][r], D[2][r], D[3][r]} * alpha;
        if (HAS_Y) o = o + yv[r] * beta;
        if (NT) streamStore16(o, zTarget, (col + r * 4096) * 4u);
        else *(GlobalF4*)(Z + (col + r * 4096)) = o;
      }
    };

    produce(0);
    __syncthreads();
    produce(1);
    consume(0);
    __syncthreads();
    produce(2);
    consume(1);
    __syncthreads();
    produce(3);
    consume(2);
    __syncthreads();
    consume(3);
    // no barrier here: the next item's first quarter goes to buffer 0, last read before the barrier above, and its
    // second quarter to buffer 1 only behind the next barrier, which every wave reaches after consume(3)

    item = nx;
    if (item >= totalItems) break;
  }
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
  // 16-byte aligned blocks for the vector loads, stores and Y loads
  if (((uintptr_t)a.in & 15) || (a.in_batch & 3)) return false;
  if (((uintptr_t)a.out & 15) || (a.out_batch & 3)) return false;
  if (a.y && (((uintptr_t)a.y & 15) || (a.y_batch & 3))) return false;
  return a.batch <= 65535;
}

// stagger: start the workgroups in groups some microseconds apart (the online choice) or all at once (a tuner candidate)
hipError_t launchRow16x4(const StepArgs& a, hipStream_t stream, bool staggered) {
  if (!row16x4Supported(a)) return hipErrorInvalidValue;
  static PerDeviceOnce attrOnce;
  const int devIdx = launchDeviceIndex();
  const size_t ldsBytes = kLdsWords * sizeof(float);
  using Kernel = void (*)(const StepArgs, const uint32_t, const uint32_t, const uint32_t);
  static const Kernel kernels[2][3] = {
      {kron_row16x4_kernel<false, 0>, kron_row16x4_kernel<false, 1>, kron_row16x4_kernel<false, 2>},
      {kron_row16x4_kernel<true, 0>, kron_row16x4_kernel<true, 1>, kron_row16x4_kernel<true, 2>}};
  if (!attrOnce.done(devIdx)) {
    for (int y = 0; y < 2; y++)
      for (int nt = 0; nt < 3; nt++) {
        hipError_t e = hipFuncSetAttribute((const void*)kernels[y][nt], hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
        if (e != hipSuccess) return e;
      }
    attrOnce.mark(devIdx);
  }
  const int cus = deviceCUs();
  const uint32_t blocksPerBatch = a.M / row16Rows(a);
  const uint64_t total = (uint64_t)blocksPerBatch * a.batch;
  if (total >= (1ull << 32) - 65536) return hipErrorInvalidValue;      // item + gridDim.x stays a 32-bit number
  // persistent workgroups, one per CU
  const uint32_t wgs = total < (uint64_t)cus ? (uint32_t)total : (uint32_t)cus;
  const uint32_t stagger = (staggered && total >= 2ull * wgs) ? kStaggerTicks : 0;
  dim3 grid(wgs), block(1024);
  hipLaunchKernelGGL(kernels[(a.y && a.epilogue) ? 1 : 0][streamMode(a)], grid, block, ldsBytes, stream, a, blocksPerBatch,
                     (uint32_t)total, stagger);
  return hipGetLastError();
}

}  // namespace fk
