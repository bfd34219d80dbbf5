// Whole-row kernel for three fused 32x32 fp32 factors (row length 32^3 = 32768), persistent form: one workgroup of 16
// wave64s per CU goes from row to row and keeps the loads of the next row in flight while it works on this one.
//
//   Z[q1,q2,q3] = alpha * sum_{k1,k2,k3} X[k1,k2,k3] F1[k1,q1] F2[k2,q2] F3[k3,q3] (+ beta * Y)
//
// The kernel with two independent workgroups of 8 waves per CU (row32x3_mfma.hip) spends half of a launch without
// memory traffic: a workgroup requests its whole row at once, the second workgroup of a CU receives its row behind
// the first one's, and neither has registers for the row after.  Here:
//
//   load     wave w owns the blocks k1 = 2w, 2w+1 (1024 contiguous elements each): four 16-byte loads per lane and
//            block, lane = (k2 % 16, (k3 % 16) / 4), register = k3 % 4.  Three block slots per lane: the block worked
//            on and the two after it, which may belong to the next row; a slot is requested again as soon as its
//            block has been multiplied, so the loads of a row are spread over the whole time of the row before.
//   k3, k2   per block, V_MFMA_F32_16X16X4_F32 in 2 x 2 blocks of 16 x 16, chained in registers: the first product
//            leaves D[i][j] (i = k2 % 16, j = q3 % 16) in register i%4 of lane 16*(i/4)+j, which is the A-operand
//            layout of a second product that contracts i; the rows of F2 are taken in the order 4*k + r to match.
//            The block ends up as T[k1][q2 = 16*jq + lane%16][q3 = 16*jh + 4*(lane/16) + r] and goes straight to LDS.
//   k1       the digit that couples the waves: the four quarters (jq, jh) of 256 columns each have an LDS buffer of
//            their own (4 x 32 KB, 16-byte writes and reads, XOR-swizzled pieces), written by every wave between two
//            barriers; behind the second barrier wave (t, jq1, g) takes the two quarters jq = t, 64 columns g of
//            each and the rows q1 = 16*jq1 .. +15, D[q1][col] = sum_k1 F1[k1][q1] T[k1][col], and stores straight
//            from the accumulators (a lane holds four consecutive columns q3 of four rows q1; both quarters are
//            multiplied first, so that the two halves of a 128-byte line are stored one behind the other).  Two
//            barriers per row.
//
// Vector memory instructions of a CU retire in order, so the requests for later blocks sit between the stores of
// this row; they are few (four per lane and block) and were issued a row earlier, which is what keeps the stores
// from waiting for them.
// Measured against the kernel with two workgroups per CU (operands from HBM): 768 rows 57.8 against 59.6 us, 1024 rows
// 70.6 against 74.9, 2048 rows 129 against 146, 32768 rows 1.89 against 2.04 ms; with 512 rows or fewer (two rows per CU
// at most) it loses, 44.0 against 39.2 us.  Builds with parts removed, per row of a long launch: 16.4 us as it is, 13.0 us
// without the matrix products, 12.8 us without global memory accesses (the products alone would take 10.2 us), 3.9 us with
// neither (exchange, barriers, operand reads); starting the workgroups in groups some microseconds apart gains nothing.
// Algorithmic traffic: 4*32768 bytes read + 4*32768 bytes written per row (+ Y when beta != 0).
#include <hip/hip_runtime.h>
#include <type_traits>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float p3f4 __attribute__((ext_vector_type(4)));

#define P3MFMA(a, b, c) __builtin_amdgcn_mfma_f32_16x16x4f32((a), (b), (c), 0, 0, 0)

constexpr int kP3Len = 32768;
constexpr int kP3QuarterWords = 32 * 256;                          // 32 rows k1 of 256 columns
constexpr int kP3LdsWords = 4 * kP3QuarterWords + 3 * 1024;        // the four quarters + the three factors: 143 360 bytes

// NT: 0 = ordinary stores, 1 = streaming stores (16 bytes at system scope through a descriptor of the row)
template <bool HAS_Y, int NT>
__global__ __launch_bounds__(1024, 1) void kron_row32x3p_kernel(const StepArgs a, const uint32_t totalItems) {
  extern __shared__ __align__(16) float p3lds[];
  float* const fl = p3lds + 4 * kP3QuarterWords;                   // fl[j*1024 + p*32 + q]; j = 0: F3, 1: F2, 2: F1
  const int tid = threadIdx.x;
  const int l0 = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);          // wave-uniform: keeps row addresses in SGPRs

  uint32_t item = blockIdx.x;                                      // an item is a row: items = M * batch
  if (item >= totalItems) return;

  // factors to LDS; a.f[0] is the factor of the fastest digit (F3), element (p, q) at p*f_sp + q*f_sq
  auto stageFactors = [&](uint32_t b) {
    float v[3];
#pragma unroll
    for (int j = 0; j < 3; j++) {
      const int p = tid >> 5, q = tid & 31;
      const float* F = (const float*)a.f[j] + (size_t)b * a.f_batch[j];
      v[j] = F[(int64_t)p * a.f_sp[j] + (int64_t)q * a.f_sq[j]];
    }
#pragma unroll
    for (int j = 0; j < 3; j++) fl[j * 1024 + tid] = v[j];
  };
  bool perBatchFactors = false;
  for (uint32_t j = 0; j < 3; j++) perBatchFactors |= (a.f_batch[j] != 0);
  uint32_t batchOfFactors = item / a.M;
  stageFactors(batchOfFactors);

  // block b of an item: the 1024 elements k1 = 2w + b; a lane's part of it is four 16-byte pieces
  const uint32_t laneOff = (l0 & 15) * 32 + (l0 >> 4) * 4;
  auto blockPtr = [&](uint32_t it, int b) {
    // behind the last item the requests go to the workgroup's last row again (cached, and never used)
    const uint32_t i2 = it < totalItems ? it : (totalItems - 1 - (totalItems - 1 - blockIdx.x) % gridDim.x);
    return (const float*)a.in + (size_t)(i2 / a.M) * a.in_batch + (size_t)(i2 % a.M) * (size_t)a.in_ldm + (2 * w + b) * 1024 + laneOff;
  };
  p3f4 xw[3][4];                                                   // slot, piece (h, c): X[k2 = 16h + lo][k3 = 16c + 4hi + r]
  auto request = [&](p3f4 (&x)[4], const float* p) __attribute__((always_inline)) {
#pragma unroll
    for (int h = 0; h < 2; h++)
#pragma unroll
      for (int c = 0; c < 2; c++) x[h * 2 + c] = *(const p3f4*)(p + h * 512 + c * 16);
  };
  request(xw[0], blockPtr(item, 0));
  request(xw[1], blockPtr(item, 1));
  request(xw[2], blockPtr(item + gridDim.x, 0));
  __syncthreads();

  const float alpha = a.epilogue ? (float)a.alpha : 1.f, beta = (float)a.beta;

  // One item: its blocks sit in the slots SA and SB; the slot SA is refilled with block 1 of the next item, the slot
  // SB with block 0 of the item after that.  Returns false behind the workgroup's last item.
  auto processItem = [&](auto SA, auto SB) __attribute__((always_inline)) -> bool {
    constexpr int sa = decltype(SA)::value, sb = decltype(SB)::value;
    // The lane id is laundered once per item: the lane-dependent LDS offsets and factor operands below are loop
    // invariant, and hoisting them out of the item loop would pin them in registers.
    int l = l0;
    asm volatile("" : "+v"(l));
    const int lo = l & 15, hi = l >> 4;
    const uint32_t m = item % a.M, b = item / a.M;
    const uint32_t nx = item + gridDim.x;
    if (perBatchFactors && b != batchOfFactors) {      // a new batch: restage its factors
      __syncthreads();                                 // every wave has read its last operand of the previous item
      stageFactors(b);
      __syncthreads();
      batchOfFactors = b;
    }
    float* const Z = (float*)a.out + (size_t)b * a.out_batch + (size_t)m * (size_t)a.out_ldm;
    const float* const Y = HAS_Y ? (const float*)a.y + (size_t)b * a.y_batch + (size_t)m * (size_t)a.y_ldm : nullptr;
    const __amdgpu_buffer_rsrc_t zTarget = streamTarget((void*)Z, kP3Len * 4u);

    // factor operands of the two chained products: both take the contraction index as 16*c + 4*hi + r
    float f3[2][4][2], f2[2][4][2];
#pragma unroll
    for (int c = 0; c < 2; c++)
#pragma unroll
      for (int r = 0; r < 4; r++)
#pragma unroll
        for (int j = 0; j < 2; j++) {
          f3[c][r][j] = fl[0 * 1024 + (16 * c + 4 * hi + r) * 32 + 16 * j + lo];      // B: F3[k3 = 16c + 4hi + r][q3 = 16j + lo]
          f2[c][r][j] = fl[1 * 1024 + (16 * c + 4 * hi + r) * 32 + 16 * j + lo];      // B: F2[k2 = 16h + 4hi + r][q2 = 16j + lo]
        }
    // x[h*2 + c][r] = X[k2 = 16h + lo][k3 = 16c + 4hi + r] becomes t[jh][jq][r] = T[q2 = 16jq + lo][q3 = 16jh + 4hi + r]
    auto multiply = [&](const p3f4 (&x)[4], p3f4 (&t)[2][2]) __attribute__((always_inline)) {
#pragma unroll
      for (int jh = 0; jh < 2; jh++) {
        p3f4 d1[2];                                   // d1[h][r] = D1[k2 = 16h + 4hi + r][q3 = 16jh + lo]
#pragma unroll
        for (int h = 0; h < 2; h++) {
          d1[h] = (p3f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int c = 0; c < 2; c++)
#pragma unroll
            for (int r = 0; r < 4; r++) d1[h] = P3MFMA(x[h * 2 + c][r], f3[c][r][jh], d1[h]);
        }
#pragma unroll
        for (int jq = 0; jq < 2; jq++) {
          t[jh][jq] = (p3f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int h = 0; h < 2; h++)
#pragma unroll
            for (int r = 0; r < 4; r++) t[jh][jq] = P3MFMA(d1[h][r], f2[h][r][jq], t[jh][jq]);
        }
      }
    };
    // Exchange geometry.  The buffer of quarter (jq, jh) holds T[k1][piece][4]: row k1 (256 words), and the 256
    // columns of the quarter, numbered (q2 % 16)*16 + q3 % 16, as 64 pieces of four.  Piece o sits at position
    // (o & 48) | ((o & 15) ^ (o >> 4)): the writers of a quarter wave (one hi, 16 values of lo: pieces 4 apart) and
    // the readers of a quarter wave (16 consecutive pieces) both cover all 64 banks.
    const int wo = lo * 4 + hi;
    float* const wbase = p3lds + (2 * w) * 256 + (((wo & 48) | ((wo & 15) ^ (wo >> 4))) << 2);
    auto produce = [&](const p3f4 (&t)[2][2], int blk) __attribute__((always_inline)) {
#pragma unroll
      for (int jq = 0; jq < 2; jq++)
#pragma unroll
        for (int jh = 0; jh < 2; jh++) *(p3f4*)(wbase + (2 * jq + jh) * kP3QuarterWords + blk * 256) = t[jh][jq];
    };

    p3f4 t[2][2];
    multiply(xw[sa], t);
    __builtin_amdgcn_sched_barrier(0);
    request(xw[sa], blockPtr(nx, 1));                  // the slot is free: block 1 of the next item
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();                                   // every wave has read the last quarter of the item before
    produce(t, 0);
    multiply(xw[sb], t);
    __builtin_amdgcn_sched_barrier(0);
    request(xw[sb], blockPtr(nx + gridDim.x, 0));      // block 0 of the item after the next
    __builtin_amdgcn_sched_barrier(0);
    produce(t, 1);
    __syncthreads();

    // reader: wave (t, jq1, g) takes the quarters jq = t (jh = 0, 1), the 64 columns g of each and the rows
    // q1 = 16*jq1 .. +15; lane (hi, lo) reads row k1 = 4c + hi, piece 16*g + lo, and ends up with
    // Z[q1 = 16*jq1 + 4hi + r][column 64g + 4lo + e] in register r of accumulator e
    const int g = w & 3, jq1 = (w >> 2) & 1, jq = w >> 3;
    float f1[8];
#pragma unroll
    for (int c = 0; c < 8; c++) f1[c] = fl[2 * 1024 + (4 * c + hi) * 32 + 16 * jq1 + lo];     // A: F1[k1 = 4c + hi][q1 = 16jq1 + lo]
    // both halves jh of the lines first, then the stores of a line's two halves one behind the other (the halves
    // stored a quarter's products apart: 32768 rows 1.89 -> 1.82 ms)
    // column 64g + 4lo + e of quarter (jq, jh) is q2 = 16jq + 4g + lo/4, q3 = 16jh + 4*(lo%4) + e
    const uint32_t col = (16 * jq1 + 4 * hi) * 1024 + (16 * jq + 4 * g + (lo >> 2)) * 32 + 4 * (lo & 3);
    p3f4 D[2][4];
#pragma unroll
    for (int jh = 0; jh < 2; jh++) {
      const float* const rb = p3lds + (2 * jq + jh) * kP3QuarterWords + hi * 256 + g * 64 + ((lo ^ g) << 2);
#pragma unroll
      for (int e = 0; e < 4; e++) D[jh][e] = (p3f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < 8; c++) {
        const p3f4 v = *(const p3f4*)(rb + c * 1024);
#pragma unroll
        for (int e = 0; e < 4; e++) D[jh][e] = P3MFMA(f1[c], v[e], D[jh][e]);
      }
    }
#pragma unroll
    for (int r = 0; r < 4; r++) {
      p3f4 yv[HAS_Y ? 2 : 1];
      if (HAS_Y) {
#pragma unroll
        for (int jh = 0; jh < 2; jh++) yv[jh] = *(const p3f4*)(Y + (col + 16 * jh + r * 1024));
      }
#pragma unroll
      for (int jh = 0; jh < 2; jh++) {
        p3f4 o = (p3f4){D[jh][0][r], D[jh][1][r], D[jh][2][r], D[jh][3][r]} * alpha;
        if (HAS_Y) o = o + yv[jh] * beta;
        if (NT) streamStore16(o, zTarget, (col + 16 * jh + r * 1024) * 4u);
        else *(p3f4*)(Z + (col + 16 * jh + r * 1024)) = o;
      }
    }
    item = nx;
    return item < totalItems;
  };

  using I0 = std::integral_constant<int, 0>;
  using I1 = std::integral_constant<int, 1>;
  using I2 = std::integral_constant<int, 2>;
  // the slots of an item's two blocks rotate with a period of three items
  for (;;) {
    if (!processItem(I0{}, I1{})) break;
    if (!processItem(I2{}, I0{})) break;
    if (!processItem(I1{}, I2{})) break;
  }
}

bool row32x3pSupported(const StepArgs& a) {
  if (a.nf != 3 || a.Kin != (uint64_t)kP3Len || a.Kout != (uint64_t)kP3Len) return false;
  for (uint32_t j = 0; j < 3; j++) if (a.p[j] != 32 || a.q[j] != 32) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  // 16-byte vector accesses
  if (((uintptr_t)a.in & 15) || (a.in_ldm & 3) || (a.in_batch & 3)) return false;
  if (((uintptr_t)a.out & 15) || (a.out_ldm & 3) || (a.out_batch & 3)) return false;
  if (a.y && (((uintptr_t)a.y & 15) || (a.y_ldm & 3) || (a.y_batch & 3))) return false;
  return (uint64_t)a.M * a.batch < (1ull << 32) - 65536;           // item + 2 * gridDim.x stays a 32-bit number
}

hipError_t launchRow32x3p(const StepArgs& a, hipStream_t stream) {
  if (!row32x3pSupported(a)) return hipErrorInvalidValue;
  static PerDeviceOnce attrOnce;
  const int devIdx = launchDeviceIndex();
  const size_t ldsBytes = kP3LdsWords * sizeof(float);
  using Kernel = void (*)(const StepArgs, const uint32_t);
  static const Kernel kernels[2][2] = {{kron_row32x3p_kernel<false, 0>, kron_row32x3p_kernel<false, 1>},
                                       {kron_row32x3p_kernel<true, 0>, kron_row32x3p_kernel<true, 1>}};
  if (!attrOnce.done(devIdx)) {
    for (int y = 0; y < 2; y++)
      for (int nt = 0; nt < 2; nt++) {
        hipError_t e = hipFuncSetAttribute((const void*)kernels[y][nt], hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
        if (e != hipSuccess) return e;
      }
    attrOnce.mark(devIdx);
  }
  const uint64_t total = (uint64_t)a.M * a.batch;
  const uint32_t cus = (uint32_t)deviceCUs();
  dim3 grid(total < cus ? (uint32_t)total : cus), block(1024);
  hipLaunchKernelGGL(kernels[(a.y && a.epilogue) ? 1 : 0][a.stream_out ? 1 : 0], grid, block, ldsBytes, stream, a, (uint32_t)total);
  return hipGetLastError();
}

}  // namespace fk
