// Whole-row kernel for three fused 32x16 fp32 factors (row length 32^3 = 32768 -> 16^3 = 4096, e.g.
// sgemkmStridedBatched with 32x16^3).  One workgroup of 8 wave64s owns one (batch, row) pair, two
// workgroups share a CU.  The reference never fuses non-square factors (reference
// src/kernel_db/kernel_db.cpp:164-181) and runs three launches with two HBM round trips; here the
// row is read once (128 KB), Y once and Z written once (16 KB each).
//
//   Z[q1,q2,q3] = alpha * sum_{k1,k2,k3} X[k1,k2,k3] F1[k1,q1] F2[k2,q2] F3[k3,q3] + beta * Y[q1,q2,q3]
//
//   load     lane = (k3 & 15, k2 & 3): 64-byte runs, both halves of a line by consecutive instructions
//   stage 1  V_MFMA_F32_16X16X4_F32 chain in registers: contract k2 with the 16 values k3 & 15 as the
//            row index (8 products per k3 half), then contract k3 by feeding the two results straight
//            back as A operands (their register/lane layout is the A layout of a product over the row
//            index) with the rows of F3 permuted to match.  64 registers shrink to 16.
//   exch.    32 KB through LDS (XOR-swizzled, conflict-free both ways): lanes become (q3, k1 & 3)
//   stage 2  contract k1 with the data on the B side, so that q3 stays in the lanes
//   store    64-byte runs, both halves of a line by consecutive instructions of one wave
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float f4 __attribute__((ext_vector_type(4)));

#define MFMA16(a, b, c) __builtin_amdgcn_mfma_f32_16x16x4f32((a), (b), (c), 0, 0, 0)

constexpr int kRow32In = 32768, kRow32Out = 4096;
constexpr int kRow32LdsWords = 8192;

// NT: 0 = ordinary stores, 1 = non-temporal stores (non-temporal loads of X lose here: 127.7 against 126.2 us)
// WIDE: the last product with its operands exchanged, D[q3][q1] instead of D[q1][q3], leaves four consecutive q3 in a
// lane: Z is written and Y read 16 bytes per lane (rows of Z and Y 16-byte aligned), streamed results at system
// scope (8 x 512 x (32x16)^3 with beta = 1: 120.9 -> 117.9 us)
template <bool HAS_Y, int NT, bool WIDE>
__global__ __launch_bounds__(512, 4) void kron_row32x16x3_kernel(const StepArgs a) {
  extern __shared__ __align__(16) float lds[];
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);      // wave-uniform: keeps row addresses in SGPRs
  const int lo = l & 15, hi = l >> 4;
  const uint32_t m = blockIdx.x, bt = blockIdx.y;

  const float* X = (const float*)a.in + (size_t)bt * a.in_batch + (size_t)m * a.in_ldm;
  float* Z = (float*)a.out + (size_t)bt * a.out_batch + (size_t)m * a.out_ldm;
  const __amdgpu_buffer_rsrc_t zTarget = streamTarget((void*)Z, kRow32Out * 4u);

  // a.f[0] = F3 (applied to the fastest digit), a.f[1] = F2, a.f[2] = F1; element (p,q) at p*sp + q*sq.
  const float* F3p = (const float*)a.f[0] + (size_t)bt * a.f_batch[0];
  const float* F2p = (const float*)a.f[1] + (size_t)bt * a.f_batch[1];
  const float* F1p = (const float*)a.f[2] + (size_t)bt * a.f_batch[2];

  // factor operands: first product B_c[k][j] = F2[4c+k][j]; second product B_{h,r}[k][j] = F3[16h+4k+r][j]
  float FA[8], FB[2][4];
#pragma unroll
  for (int c = 0; c < 8; c++) FA[c] = F2p[(int64_t)(4 * c + hi) * a.f_sp[1] + (int64_t)lo * a.f_sq[1]];
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int r = 0; r < 4; r++)
      FB[h][r] = F3p[(int64_t)(16 * h + 4 * hi + r) * a.f_sp[0] + (int64_t)lo * a.f_sq[0]];
  // (the small factor loads go out before the row data: vector memory operations retire in order)

  float FC[8];
#pragma unroll
  for (int c = 0; c < 8; c++) FC[c] = F1p[(int64_t)(4 * c + hi) * a.f_sp[2] + (int64_t)lo * a.f_sq[2]];

  // Y next (8 values per lane, in the store layout): on gfx9 loads and stores share one in-order
  // counter, so a load issued after a store could only be waited for together with that store.
  const float* Y = HAS_Y ? (const float*)a.y + (size_t)bt * a.y_batch + (size_t)m * a.y_ldm : nullptr;
  float yv[2][4];
  if (HAS_Y) {
#pragma unroll
    for (int bq = 0; bq < 2; bq++) {
      if (WIDE) {
        const f4 v = *(const f4*)&Y[lo * 256 + (2 * w + bq) * 16 + 4 * hi];
#pragma unroll
        for (int r = 0; r < 4; r++) yv[bq][r] = v[r];
      } else {
#pragma unroll
        for (int r = 0; r < 4; r++) yv[bq][r] = Y[(4 * hi + r) * 256 + (2 * w + bq) * 16 + lo];
      }
    }
  }

  // ---- load: x[g][h][c] = X[k1 = 4w+g][k2 = 4c+hi][k3 = 16h+lo] ----
  float x[4][2][8];
  {
    const float* xp = X + (size_t)(4 * w) * 1024 + hi * 32 + lo;
#pragma unroll
    for (int g = 0; g < 4; g++)
#pragma unroll
      for (int c = 0; c < 8; c++)
#pragma unroll
        for (int h = 0; h < 2; h++) x[g][h][c] = xp[g * 1024 + c * 128 + h * 16];
  }

  // ---- stage 1 ----
  float y[4][4];
#pragma unroll
  for (int g = 0; g < 4; g++) {
    f4 d0 = {0.f, 0.f, 0.f, 0.f}, d1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 8; c++) {
      d0 = MFMA16(x[g][0][c], FA[c], d0);     // d_h[r] @ lane(lo = q2, hi): k3 = 16h + 4*hi + r
      d1 = MFMA16(x[g][1][c], FA[c], d1);
    }
    f4 e = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int r = 0; r < 4; r++) {
      e = MFMA16(d0[r], FB[0][r], e);
      e = MFMA16(d1[r], FB[1][r], e);
    }
#pragma unroll
    for (int r = 0; r < 4; r++) y[g][r] = e[r];   // lane (lo = q3, hi): q2 = 4*hi + r, k1 = 4w + g
  }

  // ---- exchange: lds[q2*512 + ((k1*16 + q3) ^ (16 * (q2 >> 2)))] ----
#pragma unroll
  for (int g = 0; g < 4; g++)
#pragma unroll
    for (int r = 0; r < 4; r++)
      lds[(4 * hi + r) * 512 + ((((4 * w + g) << 4) | lo) ^ (hi << 4))] = y[g][r];
  __syncthreads();

  // reader: block bq -> q2 = 2w + bq; lane (lo = q3, hi = k1 & 3); z[bq][c]: k1 = 4c + hi
  float z[2][8];
#pragma unroll
  for (int bq = 0; bq < 2; bq++) {
    const int q2 = 2 * w + bq;
#pragma unroll
    for (int c = 0; c < 8; c++) z[bq][c] = lds[q2 * 512 + ((((4 * c + hi) << 4) | lo) ^ ((q2 >> 2) << 4))];
  }

  // ---- stage 2: D[i = q1][j = q3] = sum_k1 F1[k1][q1] * z[k1][q3]; A_c[i][k] = F1[4c+k][i] (FC, loaded up front) ----
  const float alpha = (float)a.alpha, beta = (float)a.beta;
#pragma unroll
  for (int bq = 0; bq < 2; bq++) {
    f4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < 8; c++) d = WIDE ? MFMA16(z[bq][c], FC[c], d) : MFMA16(FC[c], z[bq][c], d);
    // d[r] @ lane (lo = q3, hi): q1 = 4*hi + r; WIDE: lane (lo = q1, hi): q3 = 4*hi + r
    const int q2 = 2 * w + bq;
    if (WIDE) {
      if (a.epilogue) {
        d *= alpha;
        if (HAS_Y) d += beta * (f4){yv[bq][0], yv[bq][1], yv[bq][2], yv[bq][3]};
      }
      const int col = lo * 256 + q2 * 16 + 4 * hi;
      if (NT) streamStore16(d, zTarget, (uint32_t)col * 4u);
      else *(f4*)&Z[col] = d;
      continue;
    }
#pragma unroll
    for (int r = 0; r < 4; r++) {
      const int col = (4 * hi + r) * 256 + q2 * 16 + lo;
      float v = d[r];
      if (a.epilogue) {
        v *= alpha;
        if (HAS_Y) v += beta * yv[bq][r];
      }
      FK_ST(NT, v, &Z[col]);
    }
  }
}

bool row32x16x3Supported(const StepArgs& a) {
  if (a.nf != 3 || a.Kin != (uint64_t)kRow32In || a.Kout != (uint64_t)kRow32Out) return false;
  for (int j = 0; j < 3; j++) if (a.p[j] != 32 || a.q[j] != 16) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1) return false;
  if (a.y && a.y_ldc != 1) return false;
  return a.batch <= 65535;
}

hipError_t launchRow32x16x3(const StepArgs& a, hipStream_t stream) {
  if (!row32x16x3Supported(a)) return hipErrorInvalidValue;
  const size_t ldsBytes = kRow32LdsWords * sizeof(float);
  dim3 grid(a.M, a.batch), block(512);
  const bool y = a.y && a.epilogue, nt = a.stream_out != 0;
  // rows of Z (and Y) on 16-byte boundaries: results 16 bytes per lane
  const bool wide = !(((uintptr_t)a.out & 15) || (a.out_ldm & 3) || (a.out_batch & 3)) &&
                    !(y && (((uintptr_t)a.y & 15) || (a.y_ldm & 3) || (a.y_batch & 3)));
  using Kernel = void (*)(const StepArgs);
  static const Kernel kernels[2][2][2] = {
      {{kron_row32x16x3_kernel<false, 0, false>, kron_row32x16x3_kernel<false, 0, true>},
       {kron_row32x16x3_kernel<false, 1, false>, kron_row32x16x3_kernel<false, 1, true>}},
      {{kron_row32x16x3_kernel<true, 0, false>, kron_row32x16x3_kernel<true, 0, true>},
       {kron_row32x16x3_kernel<true, 1, false>, kron_row32x16x3_kernel<true, 1, true>}}};
  hipLaunchKernelGGL(kernels[y][nt][wide], grid, block, ldsBytes, stream, a);
  return hipGetLastError();
}

}  // namespace fk
