// Whole-row kernel for three fused 32x32 fp32 factors (row length 32^3 = 32768, e.g. sgemkm 1024 x 32768 with
// 32x32^3, or the three trailing factors of a longer chain of 32x32 factors on its contiguous blocks of 32768
// columns).  One workgroup of 8 wave64s owns one row and keeps it in VGPRs (64 per lane); two workgroups share a
// CU.  The reference fuses at most as many factors as fit its shared-memory tile (two 32x32 factors of a
// 1024-column tile, reference src/gen_tuner_kernels.py:10,366) and runs this shape in two or three launches; here
// the row is read once and written once.
//
//   Z[q1,q2,q3] = alpha * sum_{k1,k2,k3} X[k1,k2,k3] F1[k1,q1] F2[k2,q2] F3[k3,q3] (+ beta * Y)
//
//   load     wave w owns the four slices k1 = 4w .. 4w+3 (1024 contiguous elements each): 16-byte loads, lane =
//            (k2 % 16, (k3 % 16) / 4), register = k3 % 4, one instruction per half of k2 and of k3
//   k3, k2   per slice, V_MFMA_F32_16X16X4_F32 in 2 x 2 blocks of 16 x 16, chained in registers: the first product
//            leaves D[i][j] (i = k2 % 16, j = q3 % 16) in register i%4 of lane 16*(i/4)+j, which is the A-operand
//            layout of a second product that contracts i; the rows of F2 are taken in the order 4*k + r to match.
//            The slice ends up as T[k1][q2 = 16*jq + lane%16][q3 = 16*jh + 4*(lane/16) + r], in place.
//   k1       the digit that couples the waves: four quarters (jq, jh) of 256 columns each go through a
//            double-buffered LDS exchange (32 KB per quarter, 16-byte writes and reads, XOR-swizzled pieces); the
//            quarter n+1 is written between the same two barriers in which the quarter n is consumed by
//            D[q1][col] = sum_k1 F1[k1][q1] T[k1][col] and stored straight from the accumulators (a lane holds four
//            consecutive columns q3 of four rows q1).  Four barriers per row.
//
// Algorithmic traffic: 4*32768 bytes read + 4*32768 bytes written per row (+ Y when beta != 0).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float r3f4 __attribute__((ext_vector_type(4)));

#define R32MFMA(a, b, c) __builtin_amdgcn_mfma_f32_16x16x4f32((a), (b), (c), 0, 0, 0)

constexpr int kR32Len = 32768;
constexpr int kR32QuarterWords = 32 * 256;                         // 32 rows k1 of 256 columns
constexpr int kR32LdsWords = 2 * kR32QuarterWords + 3 * 1024;      // two quarters + the three factors

// NT: 0 = ordinary stores, 1 = streaming stores (1024 x 32^3: 85.0 -> 78.0 us with non-temporal stores, non-temporal loads
// of X as well: 81.6; at system scope through a descriptor of the row: 4096 rows 286 -> 279 us)
template <bool HAS_Y, int NT>
__global__ __launch_bounds__(512, 4) void kron_row32x3_kernel(const StepArgs a) {
  extern __shared__ __align__(16) float r32lds[];
  float* const fl = r32lds + 2 * kR32QuarterWords;                 // fl[j*1024 + p*32 + q]; j = 0: F3, 1: F2, 2: F1
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);          // wave-uniform: keeps row addresses in SGPRs
  const int lo = l & 15, hi = l >> 4;
  const uint32_t m = blockIdx.x, bt = blockIdx.y;

  const float* X = (const float*)a.in + (size_t)bt * a.in_batch + (size_t)m * a.in_ldm;
  float* Z = (float*)a.out + (size_t)bt * a.out_batch + (size_t)m * a.out_ldm;
  const float* Y = HAS_Y ? (const float*)a.y + (size_t)bt * a.y_batch + (size_t)m * a.y_ldm : nullptr;
  const __amdgpu_buffer_rsrc_t zTarget = streamTarget((void*)Z, 32768 * 4u);

  // factors to LDS ahead of the row loads (vector memory operations retire in order); a.f[0] is the factor of the
  // fastest digit (F3), element (p, q) at p*f_sp + q*f_sq
  // (all six loads of a thread go out before the first LDS write waits for one: a loop of load, wait, write would
  // put six memory round trips in front of the first barrier)
  {
    float v[6];
#pragma unroll
    for (int k = 0; k < 6; k++) {
      const int j = k >> 1, e = tid + 512 * (k & 1), p = e >> 5, q = e & 31;
      const float* F = (const float*)a.f[j] + (size_t)bt * a.f_batch[j];
      v[k] = F[(int64_t)p * a.f_sp[j] + (int64_t)q * a.f_sq[j]];
    }
#pragma unroll
    for (int k = 0; k < 6; k++) fl[tid + 512 * k] = v[k];
  }

  // x[s][h][c][r] = X[k1 = 4w+s][k2 = 16h + lo][k3 = 16c + 4hi + r]
  r3f4 x[4][2][2];
  {
    const float* xp = X + w * 4096 + lo * 32 + hi * 4;
#pragma unroll
    for (int s = 0; s < 4; s++)
#pragma unroll
      for (int h = 0; h < 2; h++)
#pragma unroll
        for (int c = 0; c < 2; c++) x[s][h][c] = *(const r3f4*)(xp + s * 1024 + h * 512 + c * 16);
  }
  __syncthreads();

  // ---- k3 and k2, slice by slice, in place: x[s][jh][jq][r] becomes T[k1 = 4w+s][q2 = 16jq + lo][q3 = 16jh + 4hi + r] ----
  {
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
#pragma unroll
    for (int s = 0; s < 4; s++) {
      r3f4 d2[2][2];
#pragma unroll
      for (int jh = 0; jh < 2; jh++) {
        r3f4 d1[2];                                   // d1[h][r] = D1[k2 = 16h + 4hi + r][q3 = 16jh + lo]
#pragma unroll
        for (int h = 0; h < 2; h++) {
          d1[h] = (r3f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int c = 0; c < 2; c++)
#pragma unroll
            for (int r = 0; r < 4; r++) d1[h] = R32MFMA(x[s][h][c][r], f3[c][r][jh], d1[h]);
        }
#pragma unroll
        for (int jq = 0; jq < 2; jq++) {
          d2[jh][jq] = (r3f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int h = 0; h < 2; h++)
#pragma unroll
            for (int r = 0; r < 4; r++) d2[jh][jq] = R32MFMA(d1[h][r], f2[h][r][jq], d2[jh][jq]);
        }
      }
#pragma unroll
      for (int jh = 0; jh < 2; jh++)
#pragma unroll
        for (int jq = 0; jq < 2; jq++) x[s][jh][jq] = d2[jh][jq];
    }
  }

  // Exchange geometry.  A quarter buffer holds T[k1][piece][4]: row k1 (256 words), and the 256 columns of the
  // quarter (jq, jh), numbered (q2 % 16)*16 + q3 % 16, as 64 pieces of four.  Piece o sits at position
  // (o & 48) | ((o & 15) ^ (o >> 4)): the writers of a quarter wave (one hi, 16 values of lo: pieces 4 apart) and
  // the readers of a quarter wave (16 consecutive pieces) both cover all 64 banks.
  const int wo = lo * 4 + hi;
  float* const wbase = r32lds + (4 * w) * 256 + (((wo & 48) | ((wo & 15) ^ (wo >> 4))) << 2);
  // reader: wave w takes the 64 columns g = w%4 of the quarter and the rows q1 = 16*(w/4) .. +15; lane (hi, lo)
  // reads row k1 = 4c + hi, piece 16*g + lo, and ends up with Z[q1 = 16*(w/4) + 4hi + r][column 64g + 4lo + e]
  // in register r of accumulator e
  const int g = w & 3, jq1 = w >> 2;
  const float* const rbase = r32lds + hi * 256 + g * 64 + ((lo ^ g) << 2);
  float f1[8];
#pragma unroll
  for (int c = 0; c < 8; c++) f1[c] = fl[2 * 1024 + (4 * c + hi) * 32 + 16 * jq1 + lo];     // A: F1[k1 = 4c + hi][q1 = 16jq1 + lo]
  const float alpha = a.epilogue ? (float)a.alpha : 1.f, beta = (float)a.beta;

  // quarter n = 2*jq + jh (the two halves of a 128-byte line in consecutive quarters), buffer n % 2
  auto produce = [&](const int n) {
    const int jq = n >> 1, jh = n & 1;
    float* const wb = wbase + (n & 1) * kR32QuarterWords;
#pragma unroll
    for (int s = 0; s < 4; s++) *(r3f4*)(wb + s * 256) = x[s][jh][jq];
  };
  auto consume = [&](const int n) {
    const int jq = n >> 1, jh = n & 1;
    const float* const rb = rbase + (n & 1) * kR32QuarterWords;
    // column 64g + 4lo + e of the quarter is q2 = 16jq + 4g + lo/4, q3 = 16jh + 4*(lo%4) + e
    const uint32_t col = (16 * jq1 + 4 * hi) * 1024 + (16 * jq + 4 * g + (lo >> 2)) * 32 + 16 * jh + 4 * (lo & 3);
    r3f4 yv[HAS_Y ? 4 : 1];
    if (HAS_Y) {
#pragma unroll
      for (int r = 0; r < 4; r++) yv[r] = *(const r3f4*)(Y + (col + r * 1024));
    }
    r3f4 D[4];
#pragma unroll
    for (int e = 0; e < 4; e++) D[e] = (r3f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 8; c++) {
      const r3f4 v = *(const r3f4*)(rb + c * 1024);
#pragma unroll
      for (int e = 0; e < 4; e++) D[e] = R32MFMA(f1[c], v[e], D[e]);
    }
#pragma unroll
    for (int r = 0; r < 4; r++) {
      r3f4 o = (r3f4){D[0][r], D[1][r], D[2][r], D[3][r]} * alpha;
      if (HAS_Y) o = o + yv[r] * beta;
      if (NT) streamStore16(o, zTarget, (col + r * 1024) * 4u);
      else *(r3f4*)(Z + (col + r * 1024)) = o;
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
}

bool row32x3Supported(const StepArgs& a) {
  if (a.nf != 3 || a.Kin != (uint64_t)kR32Len || a.Kout != (uint64_t)kR32Len) return false;
  for (uint32_t j = 0; j < 3; j++) if (a.p[j] != 32 || a.q[j] != 32) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  // 16-byte vector accesses
  if (((uintptr_t)a.in & 15) || (a.in_ldm & 3) || (a.in_batch & 3)) return false;
  if (((uintptr_t)a.out & 15) || (a.out_ldm & 3) || (a.out_batch & 3)) return false;
  if (a.y && (((uintptr_t)a.y & 15) || (a.y_ldm & 3) || (a.y_batch & 3))) return false;
  return a.batch <= 65535;
}

hipError_t launchRow32x3(const StepArgs& a, hipStream_t stream) {
  if (!row32x3Supported(a)) return hipErrorInvalidValue;
  static PerDeviceOnce attrOnce;
  const int devIdx = launchDeviceIndex();
  const size_t ldsBytes = kR32LdsWords * sizeof(float);
  using Kernel = void (*)(const StepArgs);
  static const Kernel kernels[2][2] = {{kron_row32x3_kernel<false, 0>, kron_row32x3_kernel<false, 1>},
                                       {kron_row32x3_kernel<true, 0>, kron_row32x3_kernel<true, 1>}};
  if (!attrOnce.done(devIdx)) {
    for (int y = 0; y < 2; y++)
      for (int nt = 0; nt < 2; nt++) {
        hipError_t e = hipFuncSetAttribute((const void*)kernels[y][nt], hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
        if (e != hipSuccess) return e;
      }
    attrOnce.mark(devIdx);
  }
  dim3 grid(a.M, a.batch), block(512);
  hipLaunchKernelGGL(kernels[(a.y && a.epilogue) ? 1 : 0][a.stream_out ? 1 : 0], grid, block, ldsBytes, stream, a);
  return hipGetLastError();
}

}  // namespace fk
