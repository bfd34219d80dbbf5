// Fused steps for small square fp32 factors in the KMM layout (operands are K x M row-major, the M
// columns are the contiguous dimension): NF factors of P x P with G = P^NF <= 64 values per lane, e.g.
// three 4x4 or two 8x8 factors per launch (sgekmm with 4x4^6 runs as two launches of three factors),
// or a single 8x8 / 16x16 factor.
//
//   out[(q_1..q_NF)*SG + sg, m] = sum_{k_1..k_NF} F_1[q_1,k_1] ... F_NF[q_NF,k_NF] * in[sg*64 + (k_1..k_NF), m]
//
// Lanes run along m, so every global access of a wave is a contiguous 256-byte row segment, and a
// lane holds the 64 values (k_1..k_NF) of its column in registers: all NF contractions happen in
// registers with no LDS and no barrier.  The arithmetic uses V_MFMA_F32_4X4X1_16B_F32 (16 independent
// 4x4 outer products): D[i][lane] += F[q = 4*qq + i][p] * x_lane[p], i.e. every lane gets its own
// outputs at the full fp32 MFMA rate; the factor values sit in P*P/4 registers per factor.
// alpha / beta*Y are applied in the store of the launch that writes Z.
//
// The reference's x86 KMM kernels vectorise along M in the same spirit (reference
// src/kernels/cpu/kernel.h:124-126, vector-types.h); its CUDA KMM kernels tile through shared memory.
// Algorithmic traffic per launch: read K*M, write K*M elements (+ K*M for Y on the last launch).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float f4 __attribute__((ext_vector_type(4)));

#define MFMA4(a, b, c) __builtin_amdgcn_mfma_f32_4x4x1f32((a), (b), (c), 0, 0, 0)

template <int P, int NF> struct KmmRegCfg {
  static constexpr int G = (NF == 1) ? P : (NF == 2) ? P * P : P * P * P;
  static_assert(G <= 64 && P % 4 == 0 && NF >= 1 && NF <= 3, "unsupported KMM register tile");
};

constexpr int kKmmWaves = 4;

// NT: 0 = ordinary, 2 = non-temporal loads of X and stores (sgekmm 1024 x 8^6: 1175 -> 1127 us)
template <int P, int NF, bool HAS_Y, int NT>
__global__ __launch_bounds__(256, HAS_Y ? 3 : 4) void kron_kmm_reg_kernel(const StepArgs a, const uint32_t mTiles,
                                                              const uint32_t totalTiles) {
  constexpr int G = KmmRegCfg<P, NF>::G;
  constexpr int QQ = P / 4;
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);      // wave-uniform: keeps row addresses in SGPRs
  const uint32_t bt = blockIdx.y;
  const uint64_t SG = a.Kin / G;
  const uint32_t t = blockIdx.x * kKmmWaves + w;
  if (t >= totalTiles) return;
  const uint64_t sg = t / mTiles;
  const uint32_t m0 = (t % mTiles) * 64;
  const bool valid = m0 + l < a.M;
  const uint32_t m = valid ? m0 + l : m0;

  // factor operands: fa[f][p][qq] = F_f[q = 4*qq + (l & 3)][p]; a.f[0] is the factor of the fastest
  // digit.  Element (p, q) of a factor lives at p*f_sp + q*f_sq.
  float fa[NF][P][QQ];
#pragma unroll
  for (int f = 0; f < NF; f++) {
    const float* F = (const float*)a.f[f] + (size_t)bt * a.f_batch[f];
#pragma unroll
    for (int p = 0; p < P; p++)
#pragma unroll
      for (int qq = 0; qq < QQ; qq++)
        fa[f][p][qq] = F[(int64_t)p * a.f_sp[f] + (int64_t)(4 * qq + (l & 3)) * a.f_sq[f]];
  }

  const float* in = (const float*)a.in + (size_t)bt * a.in_batch + (size_t)m * a.in_ldm;
  float x[G];
#pragma unroll
  for (int e = 0; e < G; e++) x[e] = FK_LD(NT, &in[(int64_t)(sg * G + e) * a.in_ldc]);

  // contract digit f (f = 0 is the fastest digit, register stride 1; digit f has stride P^f)
#pragma unroll
  for (int f = 0; f < NF; f++) {
    int st = 1;
#pragma unroll
    for (int i = 0; i < f; i++) st *= P;
#pragma unroll
    for (int s = 0; s < G / P; s++) {
      const int base = (s / st) * st * P + (s % st);
      f4 d[QQ];
#pragma unroll
      for (int qq = 0; qq < QQ; qq++) d[qq] = (f4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int p = 0; p < P; p++)
#pragma unroll
        for (int qq = 0; qq < QQ; qq++) d[qq] = MFMA4(fa[f][p][qq], x[base + p * st], d[qq]);
#pragma unroll
      for (int qq = 0; qq < QQ; qq++)
#pragma unroll
        for (int i = 0; i < 4; i++) x[base + (4 * qq + i) * st] = d[qq][i];
    }
  }

  if (!valid) return;
  float* out = (float*)a.out + (size_t)bt * a.out_batch + (size_t)m * a.out_ldm;
  const float alpha = (float)a.alpha, beta = (float)a.beta;
  if (a.epilogue) {
    if (HAS_Y) {
      // Every Y load is issued before the first store (on gfx9 loads and stores share one in-order
      // counter, so a load behind a store could only be waited for together with that store); a
      // rolling window of 16 registers keeps the loads in flight.
      const float* Y = (const float*)a.y + (size_t)bt * a.y_batch + (size_t)m * a.y_ldm;
      constexpr int YW = (G < 16) ? G : 16;
      float yw[YW];
#pragma unroll
      for (int e = 0; e < YW; e++) yw[e] = Y[(int64_t)((uint64_t)e * SG + sg) * a.y_ldc];
#pragma unroll
      for (int e = 0; e < G; e++) {
        x[e] = alpha * x[e] + beta * yw[e % YW];
        if (e + YW < G) yw[e % YW] = Y[(int64_t)((uint64_t)(e + YW) * SG + sg) * a.y_ldc];
      }
    } else {
#pragma unroll
      for (int e = 0; e < G; e++) x[e] *= alpha;
    }
  }
#pragma unroll
  for (int e = 0; e < G; e++) FK_ST(NT, x[e], &out[(int64_t)((uint64_t)e * SG + sg) * a.out_ldc]);
}

// Tile width (values per lane) for a supported (P, nf) pair, 0 otherwise.
static uint32_t kmmRegTile(uint32_t P, uint32_t nf) {
  if (P == 4 && nf >= 1 && nf <= 3) return nf == 1 ? 4 : nf == 2 ? 16 : 64;
  if (P == 8 && nf >= 1 && nf <= 2) return nf == 1 ? 8 : 64;
  if (P == 16 && nf == 1) return 16;
  return 0;
}

bool kmmRegSupported(const StepArgs& a) {
  const uint32_t G = kmmRegTile(a.p[0], a.nf);
  if (!G) return false;
  for (uint32_t j = 0; j < a.nf; j++) if (a.p[j] != a.p[0] || a.q[j] != a.p[0]) return false;
  if (a.in_ldm != 1 || a.out_ldm != 1 || (a.y && a.y_ldm != 1)) return false;
  if (a.Kin % G) return false;
  const uint64_t tiles = (a.Kin / G) * ((a.M + 63) / 64);
  return tiles < (1ull << 31) && a.batch <= 65535;
}

template <int P, int NF>
static hipError_t launchKmmRegT(const StepArgs& a, hipStream_t stream) {
  constexpr int G = KmmRegCfg<P, NF>::G;
  const uint32_t mTiles = (a.M + 63) / 64;
  const uint32_t totalTiles = (uint32_t)((a.Kin / G) * mTiles);
  dim3 grid((totalTiles + kKmmWaves - 1) / kKmmWaves, a.batch), block(256);
  const bool y = a.y && a.epilogue, nt = a.stream_in && a.stream_out;
  if (y && nt)  hipLaunchKernelGGL((kron_kmm_reg_kernel<P, NF, true, 2>), grid, block, 0, stream, a, mTiles, totalTiles);
  else if (y)   hipLaunchKernelGGL((kron_kmm_reg_kernel<P, NF, true, 0>), grid, block, 0, stream, a, mTiles, totalTiles);
  else if (nt)  hipLaunchKernelGGL((kron_kmm_reg_kernel<P, NF, false, 2>), grid, block, 0, stream, a, mTiles, totalTiles);
  else          hipLaunchKernelGGL((kron_kmm_reg_kernel<P, NF, false, 0>), grid, block, 0, stream, a, mTiles, totalTiles);
  return hipGetLastError();
}

hipError_t launchKmmReg(const StepArgs& a, hipStream_t stream) {
  if (!kmmRegSupported(a)) return hipErrorInvalidValue;
  switch (a.p[0] * 10 + a.nf) {
    case 41:  return launchKmmRegT<4, 1>(a, stream);
    case 42:  return launchKmmRegT<4, 2>(a, stream);
    case 43:  return launchKmmRegT<4, 3>(a, stream);
    case 81:  return launchKmmRegT<8, 1>(a, stream);
    case 82:  return launchKmmRegT<8, 2>(a, stream);
    case 161: return launchKmmRegT<16, 1>(a, stream);
  }
  return hipErrorInvalidValue;
}

}  // namespace fk
