// One sliced-multiply step with a 64x64 fp64 factor on the KMM layout (element (m, col) at m + col*M, the M
// index contiguous), on the matrix cores with V_MFMA_F64_4X4X4_4B_F64, which sustains about 1.5 times the
// rate of the 16x16x4 instruction on this device.  Serves dgekmm with 64x64 factors and the leading factors
// of long dgemkm chains, which the planner runs as a KMM over the row blocks.
//
//   out[(q*S + s)*M + m] = sum_p F[p, q] * in[(s*64 + p)*M + m],   S = Kin / 64
//
// A wave owns a tile of one slice s and 64 consecutive m:
//   * B operand = the data as loaded: lane 16*k + n of the register for (t, g) holds in[(s*64 + 4t + k)*M + m]
//     with m = m0 + 32*(g/2) + 2*n + g%2, so a lane loads 16 bytes and a quarter wave 256 contiguous bytes
//     per contraction row;
//   * A operand = F[4t + k][4u + i], the same for the four 4x4 blocks of an instruction: read from LDS with
//     four lanes per address; the factor is staged there once per workgroup, XOR-swizzled so that the 16
//     addresses of one read fall into 16 different bank pairs.  Every read feeds four products;
//   * the result for (u, g) sits at lane 16*(q%4) + n: 16-byte stores, 256 contiguous bytes per quarter wave.
// One wave per SIMD: its 512 registers hold the tile (128), which is refilled row by row for the wave's next
// tile as soon as a row has been consumed, and the 64 accumulators of the tile's whole 64 x 64 result (128).
// No barrier after the factor is staged.  alpha / beta*Y are applied in the store when this launch writes Z.
//
// Role of the reference's CUDA kernel for large factors on the KMM layout (reference
// src/kernels/cuda/kernel.cuh:53-224 with OpX/KMM template arguments; CUDA cores only).
// Algorithmic traffic per launch: read M*Kin, write M*Kout elements (+ M*Kout for Y).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef double kd2 __attribute__((ext_vector_type(2)));

constexpr int kKmm64Waves = 4;

// NT: 0 = ordinary, 2 = non-temporal loads of X and stores (dgekmm 1024 x 64^3: 2684 -> 2566 us)
// FLAT: the batch entries share one factor and the workgroups of the launch walk the tiles of all entries as one
// sequence (entry after entry), so that at any moment the launch reads and writes a few entries completely instead of
// a 2 KB wide strip of every entry (the leading 64x64 factor of dgemkm 256 x 64^3, 256 entries of 64 x 4096: 225 ->
// 208 us; memory accesses alone take 176 us in this order and 208 us entry by entry, the products alone 127 us)
template <bool HAS_Y, int NT, bool FLAT>
__global__ __launch_bounds__(256, 1) void kron_kmm64_f64_kernel(const StepArgs a, const uint32_t mBlocks,
                                                                const uint32_t tilesPerEntry, const uint32_t totalTiles) {
  constexpr int P = 64;
  __shared__ double fB[P * P];                       // F[p][q] at p*64 + (q ^ 4*(p%4))
  const int tid = threadIdx.x;
  const int l0 = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t bt = FLAT ? 0 : blockIdx.y;
  const uint64_t S = a.Kin / P;
  const uint64_t ldi = (uint64_t)a.in_ldc, ldo = (uint64_t)a.out_ldc, ldy = (uint64_t)a.y_ldc;

  const double* inB = (const double*)a.in + (size_t)bt * a.in_batch;
  double* outB = (double*)a.out + (size_t)bt * a.out_batch;
  const double* YB = HAS_Y ? (const double*)a.y + (size_t)bt * a.y_batch : nullptr;
  // multiplying by 1.0 is exact: launches that do not write Z need no branch around the scaling
  const double alpha = a.epilogue ? a.alpha : 1.0, beta = a.beta;

  {
    const double* F = (const double*)a.f[0] + (size_t)bt * a.f_batch[0];
    // all loads of a thread go out before the first LDS write waits for one (a loop of load, wait, write puts one
    // memory round trip per iteration in front of the first product)
    double v[P * P / 256];
#pragma unroll
    for (int k = 0; k < P * P / 256; k++) {
      const int i = tid + 256 * k, p = i / P, q = i % P;
      v[k] = F[(int64_t)p * a.f_sp[0] + (int64_t)q * a.f_sq[0]];
    }
#pragma unroll
    for (int k = 0; k < P * P / 256; k++) {
      const int i = tid + 256 * k, p = i / P, q = i % P;
      fB[p * P + (q ^ (4 * (p & 3)))] = v[k];
    }
  }
  __syncthreads();

  const uint32_t stride = gridDim.x * kKmm64Waves;
  const int n2 = 2 * (l0 & 15), k4l = l0 >> 4;

  // d[t][h] = the two consecutive m (m0 + 32h + n2, +1) of contraction row 4t + k.  One register buffer:
  // the rows of step t are loaded for the wave's next tile as soon as step t of the current tile has issued
  // its products, so every load has a whole tile of products to arrive under.  (M is a multiple of 64 and
  // the last tile of a wave prefetches itself again: no predicates, no branches around memory operations.)
  kd2 d[16][2];
  auto loadStep = [&](uint32_t tile, int t) {
    const uint32_t e = FLAT ? tile / tilesPerEntry : 0;
    if (FLAT) tile -= e * tilesPerEntry;
    const uint64_t s = tile / mBlocks;
    const uint32_t m0 = (tile % mBlocks) * 64;
    const double* xp = inB + (size_t)e * a.in_batch + (s * P + 4 * t + k4l) * ldi + m0 + n2;
#pragma unroll
    for (int h = 0; h < 2; h++) d[t][h] = FK_LD(NT, (const kd2*)(xp + 32 * h));
  };

  auto computeTile = [&](uint32_t tile, uint32_t next) {
    // the lane id is made opaque once per tile: the LDS reads of the factor are the same for every tile and
    // must not be hoisted out of the loop into registers
    int l = l0;
    asm volatile("" : "+v"(l));
    const int i4 = l & 3, k4 = l >> 4;               // operand lane = i + 4*blk + 16*k
    const uint32_t e = FLAT ? tile / tilesPerEntry : 0;
    if (FLAT) tile -= e * tilesPerEntry;
    const uint64_t s = tile / mBlocks;
    const uint32_t m0 = (tile % mBlocks) * 64;
    const int orow = l >> 4;                         // result lane = 16*(q%4) + n
    double* out = outB + (size_t)e * a.out_batch + s * ldo + m0 + n2;
    const double* Y = HAS_Y ? YB + (size_t)e * a.y_batch + s * ldy + m0 + n2 : nullptr;

    // F[4t + k][16ub + 4uu + i] at (4t + k)*64 + 16ub + 4*(uu ^ k) + i
    int fo[4];
#pragma unroll
    for (int uu = 0; uu < 4; uu++) {
      fo[uu] = k4 * 64 + 4 * (uu ^ k4) + i4;
      asm volatile("" : "+v"(fo[uu]));
    }
    double acc[16][4];
#pragma unroll
    for (int u = 0; u < 16; u++)
#pragma unroll
      for (int g = 0; g < 4; g++) acc[u][g] = 0.0;
    // the factor operands of step (t, ub) + 1 are read before the products of step (t, ub) are issued:
    // with one wave per SIMD nothing else hides the LDS latency
    double fn[4];
#pragma unroll
    for (int uu = 0; uu < 4; uu++) fn[uu] = fB[fo[uu]];
#pragma unroll
    for (int t = 0; t < 16; t++) {
#pragma unroll
      for (int ub = 0; ub < 4; ub++) {
        double fc[4];
#pragma unroll
        for (int uu = 0; uu < 4; uu++) fc[uu] = fn[uu];
        const int nx = 4 * t + ub + 1;               // next step: t' = nx / 4, ub' = nx % 4
        if (nx < 64) {
#pragma unroll
          for (int uu = 0; uu < 4; uu++) fn[uu] = fB[fo[uu] + 4 * (nx / 4) * 64 + 16 * (nx % 4)];
        }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int uu = 0; uu < 4; uu++)
#pragma unroll
          for (int g = 0; g < 4; g++)
            acc[4 * ub + uu][g] =
                __builtin_amdgcn_mfma_f64_4x4x4f64(fc[uu], d[t][g >> 1][g & 1], acc[4 * ub + uu][g], 0, 0, 0);
      }
      loadStep(next, t);
    }
    // q = 4u + orow; the 16-byte element pair (g = 2h, 2h+1) at m0 + 32h + n2.  Y is read in four parts,
    // each before the stores of its part.
#pragma unroll
    for (int ub = 0; ub < 4; ub++) {
      kd2 yv[4][2];
      if (HAS_Y) {
#pragma unroll
        for (int uu = 0; uu < 4; uu++)
#pragma unroll
          for (int h = 0; h < 2; h++)
            yv[uu][h] = *(const kd2*)(Y + (uint64_t)(16 * ub + 4 * uu + orow) * S * ldy + 32 * h);
      }
#pragma unroll
      for (int uu = 0; uu < 4; uu++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
          kd2 v = {acc[4 * ub + uu][2 * h] * alpha, acc[4 * ub + uu][2 * h + 1] * alpha};
          if (HAS_Y) v += beta * yv[uu][h];
          FK_ST(NT, v, (kd2*)(out + (uint64_t)(16 * ub + 4 * uu + orow) * S * ldo + 32 * h));
        }
    }
  };

  uint32_t tile = blockIdx.x * kKmm64Waves + w;
  if (tile >= totalTiles) return;
#pragma unroll
  for (int t = 0; t < 16; t++) loadStep(tile, t);
  // The first tile is peeled off the loop.  Loads and stores retire through one in-order counter and the
  // wait for prefetched rows is counted in younger operations; entering the loop only from a complete tile
  // lets that count include the stores issued behind the prefetch, so that the wait at the top of a tile
  // does not drain the previous tile's stores.
  auto nextOf = [&](uint32_t t) { return t + stride < totalTiles ? t + stride : t; };
  computeTile(tile, nextOf(tile));
  for (tile += stride; tile < totalTiles; tile += stride) computeTile(tile, nextOf(tile));
}

bool kmm64F64Supported(const StepArgs& a) {
  if (a.nf != 1 || a.p[0] != 64 || a.q[0] != 64 || a.Kin % 64) return false;
  if (a.in_ldm != 1 || a.out_ldm != 1 || (a.y && a.y_ldm != 1)) return false;
  // whole 64-column tiles of 16-byte element pairs: even strides, 16-byte aligned bases
  if ((a.M % 64) || (a.in_ldc & 1) || (a.out_ldc & 1) || (a.in_batch & 1) || (a.out_batch & 1)) return false;
  if (((uintptr_t)a.in & 15) || ((uintptr_t)a.out & 15)) return false;
  if (a.y && (((uintptr_t)a.y & 15) || (a.y_ldc & 1) || (a.y_batch & 1))) return false;
  const uint64_t S = a.Kin / 64;
  return S * ((a.M + 63) / 64) < (1ull << 31) && a.batch <= 65535;
}

hipError_t launchKmm64F64(const StepArgs& a, hipStream_t stream) {
  if (!kmm64F64Supported(a)) return hipErrorInvalidValue;
  const int cus = deviceCUs();
  const uint64_t S = a.Kin / 64;
  const uint32_t mBlocks = (a.M + 63) / 64;
  const uint32_t tilesPerEntry = (uint32_t)(S * mBlocks);
  // one factor for every batch entry: the entries' tiles as one sequence
  const bool flat = a.batch > 1 && a.f_batch[0] == 0 && (uint64_t)tilesPerEntry * a.batch < (1ull << 31);
  const uint32_t totalTiles = flat ? tilesPerEntry * a.batch : tilesPerEntry;
  uint32_t wgs = (uint32_t)cus;                      // persistent, one workgroup per CU, one wave per SIMD
  if (!flat && a.batch > 1) wgs = (wgs + a.batch - 1) / a.batch;
  const uint32_t need = (totalTiles + kKmm64Waves - 1) / kKmm64Waves;
  if (wgs > need) wgs = need;
  if (wgs == 0) wgs = 1;
  dim3 grid(wgs, flat ? 1 : a.batch), block(256);
  const bool y = a.y && a.epilogue, nt = a.stream_in && a.stream_out;
  using Kernel = void (*)(const StepArgs, const uint32_t, const uint32_t, const uint32_t);
  static const Kernel kernels[2][2][2] = {
      {{kron_kmm64_f64_kernel<false, 0, false>, kron_kmm64_f64_kernel<false, 0, true>},
       {kron_kmm64_f64_kernel<false, 2, false>, kron_kmm64_f64_kernel<false, 2, true>}},
      {{kron_kmm64_f64_kernel<true, 0, false>, kron_kmm64_f64_kernel<true, 0, true>},
       {kron_kmm64_f64_kernel<true, 2, false>, kron_kmm64_f64_kernel<true, 2, true>}}};
  hipLaunchKernelGGL(kernels[y][nt][flat], grid, block, 0, stream, a, mBlocks, tilesPerEntry, totalTiles);
  return hipGetLastError();
}

}  // namespace fk
