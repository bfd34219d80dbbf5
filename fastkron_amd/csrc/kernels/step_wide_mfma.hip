// One sliced-multiply step with a square fp32 factor of 64x64 or 128x128, MKM or KMM layout, every global access a
// whole 128-byte line or more.
//
//   MKM  out[m, q*S + s] = sum_p in[m, s*P + p] * F[p, q]          S = Kin / P
//   KMM  out[(q*S + s), m] = sum_p in[(s*P + p), m] * F[p, q]      (the M index contiguous)
//
// The streaming step kernel (step_mfma.hip) gives a wave 16 slices and lets every lane read its own 16-byte pieces
// and write 4-byte elements: its load instructions touch 64 lines each and its stores write 64-byte halves of lines,
// which costs a third of the time once the operands are far larger than the caches (sgemkm 320 x 128^3: 6.3 ms
// against 4.4 ms here; 1024 x 128^2: 120 against 85 us).  Here a workgroup of four waves owns a tile of 4096 input
// elements: in the MKM layout TS = 4096/P consecutive slices of a row (contiguous), in the KMM layout the P rows
// of a slice by TS consecutive columns m.
//   * The tile is read with 16-byte accesses, consecutive lanes on consecutive addresses, one tile ahead into
//     registers, and passed on through LDS (two buffers, one barrier per tile).
//   * Wave w owns the output columns q in [w*P/4, (w+1)*P/4): its part of the factor stays in registers as the A
//     operands of V_MFMA_F32_16X16X4_F32, D[q][j] += F^T[q][p] * X^T[p][j].  The 16 columns j of product e are the
//     slices (MKM) or columns m (KMM) JH*lane + e, JH = TS/16: a lane's results for one q are then JH consecutive
//     output elements, and 16 lanes store 128 (128x128) or 256 (64x64) contiguous bytes.
//   * MKM: the contraction index of product c in lane group k is p = (P/4)*k + c, so a lane's B operands are P/4
//     consecutive elements of its slice, read from LDS 16 bytes at a time; 16-byte chunk `ch` of slice `s` sits at
//     chunk s*(P/4) + (ch ^ ((s / JH) % 16)), which keeps the writers, eight lanes with consecutive chunks, and the
//     readers, sixteen lanes with the same chunk of slices JH apart, on distinct banks.
//     KMM: p = 4*c + k, a lane reads its JH consecutive columns of row p; rows are TS elements apart, which puts
//     the lane groups of one read on distinct banks without padding.
// alpha / beta*Y are applied in the store of the launch that writes Z.  Loads and stores retire through one in-order
// counter and the wait for the tile read ahead is counted in younger operations, so nothing in the loop is
// conditional: the last tile of a workgroup requests itself again and the first one is peeled off the loop.
//
// Role of the reference's CUDA kernel for large factors (reference src/kernels/cuda/kernel.cuh:53-224: shared-memory
// tiles of X and F, CUDA cores; reference src/kernels/cuda/shared-loads.cuh:4-88 for its staging of X).
// Algorithmic traffic per launch: read M*Kin, write M*Kout elements (+ M*Kout for Y on the launch that writes Z).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float swf4 __attribute__((ext_vector_type(4)));
typedef float swf2 __attribute__((ext_vector_type(2)));

constexpr int kSwTile = 4096;                 // input elements per tile
constexpr int kSwWaves = 4;
constexpr size_t kSwLdsBytes = 2 * kSwTile * sizeof(float);

template <int JH> struct SwVec;
template <> struct SwVec<4> { using type = swf4; };
template <> struct SwVec<2> { using type = swf2; };

template <int P, bool KMM, bool HAS_Y>
__global__ __launch_bounds__(256, 2) void kron_step_wide_kernel(const StepArgs a, const uint32_t tilesPerLine,
                                                                const uint32_t totalTiles) {
  constexpr int PC = P / 4;                   // products per column block; 16-byte chunks per slice (MKM)
  constexpr int TS = kSwTile / P;             // slices (MKM) or columns m (KMM) per tile
  constexpr int JH = TS / 16;                 // column blocks per tile = consecutive output elements per lane and q
  constexpr int NBW = P / 64;                 // 16-column blocks of the factor per wave
  constexpr int RW = 16 * NBW;                // output columns q per wave
  using Vec = typename SwVec<JH>::type;
  extern __shared__ __align__(16) float swLds[];
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lo = l & 15, hi = l >> 4;
  const uint32_t bt = blockIdx.y;
  const uint64_t S = a.Kin / P;

  const float* inB = (const float*)a.in + (size_t)bt * a.in_batch;
  float* outB = (float*)a.out + (size_t)bt * a.out_batch;
  const float* YB = HAS_Y ? (const float*)a.y + (size_t)bt * a.y_batch : nullptr;
  const float alpha = a.epilogue ? (float)a.alpha : 1.f, beta = (float)a.beta;   // multiplying by 1 is exact

  // this wave's columns of the factor as A operands: fa[c][ib] = F[p(c, hi)][RW*w + 16*ib + lo]
  float fa[PC][NBW];
  {
    const float* F = (const float*)a.f[0] + (size_t)bt * a.f_batch[0];
#pragma unroll
    for (int c = 0; c < PC; c++)
#pragma unroll
      for (int ib = 0; ib < NBW; ib++) {
        const int p = KMM ? 4 * c + hi : PC * hi + c;
        fa[c][ib] = F[(int64_t)p * a.f_sp[0] + (int64_t)(RW * w + 16 * ib + lo) * a.f_sq[0]];
      }
  }

  // tile t: MKM row t / tilesPerLine, slices TS*(t % tilesPerLine) ...; KMM slice t / tilesPerLine, columns likewise
  swf4 pre[4];
  auto request = [&](uint32_t t) {
    const size_t line = t / tilesPerLine, part = t % tilesPerLine;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int g = 256 * i + tid;                             // 16-byte chunk of the tile
      if (KMM) {
        const int p = g / (TS / 4), ch = g % (TS / 4);
        pre[i] = *(const swf4*)(inB + (line * P + p) * (size_t)a.in_ldc + part * TS + 4 * ch);
      } else {
        pre[i] = *(const swf4*)(inB + line * (size_t)a.in_ldm + part * kSwTile + 4 * g);
      }
    }
  };
  auto nextOf = [&](uint32_t t) { return t + gridDim.x < totalTiles ? t + gridDim.x : t; };

  auto computeTile = [&](uint32_t t, int buf) {
    float* xs = swLds + buf * kSwTile;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int g = 256 * i + tid;
      if (KMM) {
        *(swf4*)&xs[4 * g] = pre[i];                           // row p = g / (TS/4), TS elements per row
      } else {
        const int s = g / PC, ch = g % PC;
        *(swf4*)&xs[4 * (s * PC + (ch ^ ((s / JH) & 15)))] = pre[i];
      }
    }
    request(nextOf(t));                                        // the next tile streams in under the products
    __syncthreads();
    // B operands: x[e][c] = X[p(c, hi)][column JH*lo + e]
    float x[JH][PC];
    if (KMM) {
#pragma unroll
      for (int c = 0; c < PC; c++) {
        const Vec v = *(const Vec*)&xs[(4 * c + hi) * TS + JH * lo];
#pragma unroll
        for (int e = 0; e < JH; e++) x[e][c] = v[e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < JH; e++)
#pragma unroll
        for (int c4 = 0; c4 < PC / 4; c4++) {
          const int ch = (PC / 4) * hi + c4;
          const swf4 v = *(const swf4*)&xs[4 * ((JH * lo + e) * PC + (ch ^ lo))];
#pragma unroll
          for (int k = 0; k < 4; k++) x[e][4 * c4 + k] = v[k];
        }
    }

    swf4 acc[NBW][JH];
#pragma unroll
    for (int ib = 0; ib < NBW; ib++)
#pragma unroll
      for (int e = 0; e < JH; e++) acc[ib][e] = (swf4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < PC; c++)
#pragma unroll
      for (int ib = 0; ib < NBW; ib++)
#pragma unroll
        for (int e = 0; e < JH; e++)
          acc[ib][e] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[c][ib], x[e][c], acc[ib][e], 0, 0, 0);

    // accumulator register r of lane (hi, lo) and product e: output column q = RW*w + 16*ib + 4*hi + r, element
    // JH*lo + e of the tile's TS
    const size_t line = t / tilesPerLine, part = t % tilesPerLine;
    const size_t qStride = KMM ? S * (size_t)a.out_ldc : S, yStride = KMM ? S * (size_t)a.y_ldc : S;
    float* out = KMM ? outB + line * (size_t)a.out_ldc + part * TS + JH * lo
                     : outB + line * (size_t)a.out_ldm + part * TS + JH * lo;
    const float* Y = nullptr;
    if (HAS_Y) Y = KMM ? YB + line * (size_t)a.y_ldc + part * TS + JH * lo : YB + line * (size_t)a.y_ldm + part * TS + JH * lo;
    Vec yv[NBW][4];
    if (HAS_Y) {
#pragma unroll
      for (int ib = 0; ib < NBW; ib++)
#pragma unroll
        for (int r = 0; r < 4; r++) yv[ib][r] = *(const Vec*)(Y + (size_t)(RW * w + 16 * ib + 4 * hi + r) * yStride);
    }
#pragma unroll
    for (int ib = 0; ib < NBW; ib++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        Vec v;
#pragma unroll
        for (int e = 0; e < JH; e++) v[e] = acc[ib][e][r] * alpha;
        if (HAS_Y) v += yv[ib][r] * beta;
        *(Vec*)(out + (size_t)(RW * w + 16 * ib + 4 * hi + r) * qStride) = v;
      }
  };

  uint32_t t = blockIdx.x;
  if (t >= totalTiles) return;
  request(t);
  computeTile(t, 0);
  int buf = 1;
  for (t += gridDim.x; t < totalTiles; t += gridDim.x, buf ^= 1) computeTile(t, buf);
}

static bool stepWideIsKmm(const StepArgs& a) { return a.in_ldm == 1 && a.in_ldc != 1; }

bool stepWideSupported(const StepArgs& a) {
  if (a.nf != 1) return false;
  const uint32_t P = a.p[0];
  if ((P != 64 && P != 128) || a.q[0] != P) return false;
  if (a.Kin % P || a.Kout != a.Kin) return false;
  const uint64_t S = a.Kin / P, TS = kSwTile / P;
  if (stepWideIsKmm(a)) {
    if (a.out_ldm != 1 || (a.y && a.y_ldm != 1)) return false;
    if (a.M % TS) return false;                               // whole tiles
    if (((uintptr_t)a.in & 15) || (a.in_ldc & 3) || (a.in_batch & 3)) return false;
    if (((uintptr_t)a.out & 15) || (a.out_ldc & 3) || (a.out_batch & 3)) return false;
    if (a.y && (((uintptr_t)a.y & 15) || (a.y_ldc & 3) || (a.y_batch & 3))) return false;
    return S * (a.M / TS) < (1ull << 31) && a.batch <= 65535;
  }
  if (S % TS) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  // 16-byte accesses: rows and batch entries start on 16-byte boundaries
  if (((uintptr_t)a.in & 15) || (a.in_ldm & 3) || (a.in_batch & 3)) return false;
  if (((uintptr_t)a.out & 15) || (a.out_ldm & 3) || (a.out_batch & 3)) return false;
  if (a.y && (((uintptr_t)a.y & 15) || (a.y_ldm & 3) || (a.y_batch & 3))) return false;
  return (a.Kin / kSwTile) * a.M < (1ull << 31) && a.batch <= 65535;
}

template <int P, bool KMM>
static hipError_t launchStepWideT(const StepArgs& a, hipStream_t stream) {
  const uint32_t TS = kSwTile / P;
  const uint32_t tilesPerLine = KMM ? a.M / TS : (uint32_t)(a.Kin / kSwTile);
  const uint32_t totalTiles = KMM ? (uint32_t)(a.Kin / P) * tilesPerLine : tilesPerLine * a.M;
  uint32_t wgs = 2u * (uint32_t)deviceCUs();                   // persistent, two workgroups per CU
  if (a.batch > 1) wgs = (wgs + a.batch - 1) / a.batch;
  if (wgs > totalTiles) wgs = totalTiles;
  if (wgs == 0) wgs = 1;
  dim3 grid(wgs, a.batch), block(64 * kSwWaves);
  if (a.y && a.epilogue)
    hipLaunchKernelGGL((kron_step_wide_kernel<P, KMM, true>), grid, block, kSwLdsBytes, stream, a, tilesPerLine, totalTiles);
  else
    hipLaunchKernelGGL((kron_step_wide_kernel<P, KMM, false>), grid, block, kSwLdsBytes, stream, a, tilesPerLine, totalTiles);
  return hipGetLastError();
}

hipError_t launchStepWide(const StepArgs& a, hipStream_t stream) {
  if (!stepWideSupported(a)) return hipErrorInvalidValue;
  if (stepWideIsKmm(a)) return a.p[0] == 128 ? launchStepWideT<128, true>(a, stream) : launchStepWideT<64, true>(a, stream);
  return a.p[0] == 128 ? launchStepWideT<128, false>(a, stream) : launchStepWideT<64, false>(a, stream);
}

}  // namespace fk
