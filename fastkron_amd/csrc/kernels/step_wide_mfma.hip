// One sliced-multiply step with a square factor of 64x64 or 128x128, fp32 or fp64, MKM or KMM layout, every global
// access a whole 128-byte line or more.
//
//   MKM  out[m, q*S + s] = sum_p in[m, s*P + p] * F[p, q]          S = Kin / P
//   KMM  out[(q*S + s), m] = sum_p in[(s*P + p), m] * F[p, q]      (the M index contiguous)
//
// The streaming step kernel (step_mfma.hip) gives a wave 16 slices and lets every lane read its own 16-byte pieces
// and write 4-byte elements: its load instructions touch 64 lines each and its stores write 64-byte halves of lines,
// which costs a third of the time once the operands are far larger than the caches (sgemkm 320 x 128^3: 6.3 ms
// against 4.4 ms here; 1024 x 128^2: 120 against 85 us).  Here a workgroup of four waves owns a tile of 16 KB of input
// (E = 4096 fp32 or 2048 fp64 elements): in the MKM layout TS = E/P consecutive slices of a row (contiguous), in the
// KMM layout the P rows of a slice by TS consecutive columns m.
//   * The tile is read with 16-byte accesses, consecutive lanes on consecutive addresses, one tile ahead into
//     registers, and passed on through LDS (two buffers, one barrier per tile).
//   * Wave w owns the output columns q in [w*P/4, (w+1)*P/4): its part of the factor stays in registers as the A
//     operands of V_MFMA_F32_16X16X4_F32 / V_MFMA_F64_16X16X4_F64, D[q][j] += F^T[q][p] * X^T[p][j].  The 16 columns j of product e are the
//     slices (MKM) or columns m (KMM) JH*lane + e, JH = TS/16: a lane's results for one q are then JH consecutive
//     output elements, and 16 lanes store 128 (128x128) or 256 (64x64) contiguous bytes in either type.
//   * MKM: the contraction index of product c in lane group k is p = (P/4)*k + c, so a lane's B operands are P/4
//     consecutive elements of its slice, read from LDS 16 bytes at a time; 16-byte chunk `ch` of slice `s` (of CPS
//     chunks) sits at chunk s*CPS + (ch ^ ((s / JH) % min(CPS, 16))), which keeps the writers, eight lanes with consecutive chunks, and the
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
typedef double swd2 __attribute__((ext_vector_type(2)));
typedef double swd4 __attribute__((ext_vector_type(4)));

constexpr int kSwTileBytes = 16384;           // input bytes per tile
constexpr int kSwWaves = 4;
constexpr size_t kSwLdsBytes = 2 * kSwTileBytes;

template <typename T> struct SwType;
template <> struct SwType<float> {
  using Acc = swf4;
  using Chunk = swf4;                          // 16 bytes
  static __device__ __forceinline__ Acc mma(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ int row(int r, int hi) { return 4 * hi + r; }   // row of accumulator register r
};
template <> struct SwType<double> {
  using Acc = swd4;
  using Chunk = swd2;
  static __device__ __forceinline__ Acc mma(double a, double b, Acc c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ int row(int r, int hi) { return 4 * r + hi; }
};
// JH consecutive output elements of a lane
template <typename T, int JH> struct SwVec { typedef T type __attribute__((ext_vector_type(JH))); };
template <typename T> struct SwVec<T, 1> { using type = T; };
template <typename V, int JH> struct SwLane {
  template <typename T> static __device__ __forceinline__ T get(const V& v, int e) { return v[e]; }
  template <typename T> static __device__ __forceinline__ void set(V& v, int e, T x) { v[e] = x; }
};
template <typename V> struct SwLane<V, 1> {
  template <typename T> static __device__ __forceinline__ T get(const V& v, int) { return v; }
  template <typename T> static __device__ __forceinline__ void set(V& v, int, T x) { v = x; }
};

// MKM tiles in LDS: slice s of CPS 16-byte chunks.  With 8 chunks per slice the sixteen lanes of a read (slices 4
// apart) would meet on two bank groups of eight: slices 32 apart swap places with their neighbours, which moves the
// upper eight lanes to the other group.
template <int CPS> __device__ __forceinline__ int swSlot(int s) { return CPS < 16 ? s ^ ((s >> 5) & 1) : s; }

template <typename T, int P, bool KMM, bool HAS_Y, bool STREAM>
__global__ __launch_bounds__(256, 2) void kron_step_wide_kernel(const StepArgs a, const uint32_t tilesPerLine,
                                                                const uint32_t totalTiles) {
  using ST = SwType<T>;
  using Acc = typename ST::Acc;
  using Chunk = typename ST::Chunk;
  constexpr int EPC = 16 / sizeof(T);         // elements per 16-byte chunk
  constexpr int E = kSwTileBytes / sizeof(T); // elements per tile
  constexpr int PC = P / 4;                   // products per column block, elements per lane and slice
  constexpr int CPS = P / EPC;                // 16-byte chunks per slice (MKM)
  constexpr int TS = E / P;                   // slices (MKM) or columns m (KMM) per tile
  // the four waves split the factor's columns q into QG groups and the tile's TS slices / columns into JG parts
  constexpr int QG = P >= 64 ? 4 : P / 16, JG = 4 / QG;
  constexpr int JH = TS / 16 / JG;            // column blocks per wave = consecutive output elements per lane and q
  constexpr int NBW = P / 16 / QG;            // 16-column blocks of the factor per wave
  constexpr int RW = 16 * NBW;                // output columns q per wave
  constexpr int KEY = (CPS < 16 ? CPS : 16) - 1;
  using Vec = typename SwVec<T, JH>::type;
  using VL = SwLane<Vec, JH>;
  extern __shared__ __align__(16) unsigned char swLdsRaw[];
  T* swLds = (T*)swLdsRaw;
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lo = l & 15, hi = l >> 4;
  const int qg = w % QG, j0 = (w / QG) * (TS / JG);            // this wave's column group and first slice / column
  const uint32_t bt = blockIdx.y;
  const uint64_t S = a.Kin / P;

  const T* inB = (const T*)a.in + (size_t)bt * a.in_batch;
  T* outB = (T*)a.out + (size_t)bt * a.out_batch;
  const T* YB = HAS_Y ? (const T*)a.y + (size_t)bt * a.y_batch : nullptr;
  const T alpha = a.epilogue ? (T)a.alpha : (T)1, beta = (T)a.beta;   // multiplying by 1 is exact

  // this wave's columns of the factor as A operands: fa[c][ib] = F[p(c, hi)][RW*qg + 16*ib + lo]
  T fa[PC][NBW];
  {
    const T* F = (const T*)a.f[0] + (size_t)bt * a.f_batch[0];
#pragma unroll
    for (int c = 0; c < PC; c++)
#pragma unroll
      for (int ib = 0; ib < NBW; ib++) {
        const int p = KMM ? 4 * c + hi : PC * hi + c;
        fa[c][ib] = F[(int64_t)p * a.f_sp[0] + (int64_t)(RW * qg + 16 * ib + lo) * a.f_sq[0]];
      }
  }

  // tile t: MKM row t / tilesPerLine, slices TS*(t % tilesPerLine) ...; KMM slice t / tilesPerLine, columns likewise
  Chunk pre[4];
  auto request = [&](uint32_t t) {
    const size_t line = t / tilesPerLine, part = t % tilesPerLine;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int g = 256 * i + tid;                             // 16-byte chunk of the tile
      if (KMM) {
        const int p = g / (TS / EPC), ch = g % (TS / EPC);
        pre[i] = *(const Chunk*)(inB + (line * P + p) * (size_t)a.in_ldc + part * TS + EPC * ch);
      } else {
        pre[i] = *(const Chunk*)(inB + line * (size_t)a.in_ldm + part * E + EPC * g);
      }
    }
  };
  auto nextOf = [&](uint32_t t) { return t + gridDim.x < totalTiles ? t + gridDim.x : t; };

  auto computeTile = [&](uint32_t t, int buf) {
    T* xs = swLds + buf * E;
#pragma unroll
    for (int i = 0; i < 4; i++) {
      const int g = 256 * i + tid;
      if (KMM) {
        *(Chunk*)&xs[EPC * g] = pre[i];                        // row p = g / (TS/EPC), TS elements per row
      } else {
        const int s = g / CPS, ch = g % CPS;
        *(Chunk*)&xs[EPC * (swSlot<CPS>(s) * CPS + (ch ^ ((s / JH) & KEY)))] = pre[i];
      }
    }
    request(nextOf(t));                                        // the next tile streams in under the products
    __syncthreads();
    // B operands: x[e][c] = X[p(c, hi)][column j0 + JH*lo + e]
    T x[JH][PC];
    if (KMM) {
#pragma unroll
      for (int c = 0; c < PC; c++) {
        const Vec v = *(const Vec*)&xs[(4 * c + hi) * TS + j0 + JH * lo];
#pragma unroll
        for (int e = 0; e < JH; e++) x[e][c] = VL::template get<T>(v, e);
      }
    } else {
#pragma unroll
      for (int e = 0; e < JH; e++)
#pragma unroll
        for (int c4 = 0; c4 < PC / EPC; c4++) {
          const int ch = (PC / EPC) * hi + c4;
          const Chunk v = *(const Chunk*)&xs[EPC * (swSlot<CPS>(j0 + JH * lo + e) * CPS + (ch ^ (lo & KEY)))];
#pragma unroll
          for (int k = 0; k < EPC; k++) x[e][EPC * c4 + k] = v[k];
        }
    }

    Acc acc[NBW][JH];
#pragma unroll
    for (int ib = 0; ib < NBW; ib++)
#pragma unroll
      for (int e = 0; e < JH; e++) acc[ib][e] = (Acc){0, 0, 0, 0};
#pragma unroll
    for (int c = 0; c < PC; c++)
#pragma unroll
      for (int ib = 0; ib < NBW; ib++)
#pragma unroll
        for (int e = 0; e < JH; e++) acc[ib][e] = ST::mma(fa[c][ib], x[e][c], acc[ib][e]);

    // accumulator register r of lane (hi, lo) and product e: output column q = RW*qg + 16*ib + row(r, hi), element
    // j0 + JH*lo + e of the tile's TS
    const size_t line = t / tilesPerLine, part = t % tilesPerLine;
    const size_t qStride = KMM ? S * (size_t)a.out_ldc : S, yStride = KMM ? S * (size_t)a.y_ldc : S;
    T* const outTile = KMM ? outB + line * (size_t)a.out_ldc + part * TS : outB + line * (size_t)a.out_ldm + part * TS;
    T* out = outTile + j0 + JH * lo;
    // results that nothing reads back soon: 16-byte stores at system scope through a descriptor of the tile's span
    // (sgekmm 1024 x 32^3: 156.5 -> 139.8 us, 1024 x 64^3: 1.31 -> 1.26 ms; as the leading step of a GeMKM, one batch
    // entry per row, the same stores lose 2 to 3 %: sgemkm 1024 x 32^4 and 1024 x 64^3, which keep ordinary ones)
    // (STREAM: chosen by the launcher for single-entry launches with stream_out whose tiles span less than 2 GB)
    const __amdgpu_buffer_rsrc_t oTarget = streamTarget((void*)outTile, STREAM ? (uint32_t)(P * qStride * sizeof(T)) : 0u);
    const T* Y = nullptr;
    if (HAS_Y) Y = KMM ? YB + line * (size_t)a.y_ldc + part * TS + j0 + JH * lo : YB + line * (size_t)a.y_ldm + part * TS + j0 + JH * lo;
    Vec yv[NBW][4];
    if (HAS_Y) {
#pragma unroll
      for (int ib = 0; ib < NBW; ib++)
#pragma unroll
        for (int r = 0; r < 4; r++) yv[ib][r] = *(const Vec*)(Y + (size_t)(RW * qg + 16 * ib + ST::row(r, hi)) * yStride);
    }
#pragma unroll
    for (int ib = 0; ib < NBW; ib++)
#pragma unroll
      for (int r = 0; r < 4; r++) {
        Vec v;
#pragma unroll
        for (int e = 0; e < JH; e++) VL::template set<T>(v, e, acc[ib][e][r] * alpha);
        if (HAS_Y) v += yv[ib][r] * beta;
        const size_t at = (size_t)(RW * qg + 16 * ib + ST::row(r, hi)) * qStride;
        if constexpr (STREAM && sizeof(Vec) == 16) streamStore16(v, oTarget, (uint32_t)((at + j0 + JH * lo) * sizeof(T)));
        else *(Vec*)(out + at) = v;
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

bool stepWideSupported(const StepArgs& a, DType dt) {
  if (a.nf != 1) return false;
  const uint32_t P = a.p[0];
  if ((P != 32 && P != 64 && P != 128) || a.q[0] != P) return false;
  if (a.Kin % P || a.Kout != a.Kin) return false;
  const uint64_t es = dtypeSize(dt), E = kSwTileBytes / es, S = a.Kin / P, TS = E / P, vm = 16 / es - 1;
  if (stepWideIsKmm(a)) {
    if (a.out_ldm != 1 || (a.y && a.y_ldm != 1)) return false;
    if (a.M % TS) return false;                               // whole tiles
    if (((uintptr_t)a.in & 15) || ((uint64_t)a.in_ldc & vm) || (a.in_batch & vm)) return false;
    if (((uintptr_t)a.out & 15) || ((uint64_t)a.out_ldc & vm) || (a.out_batch & vm)) return false;
    if (a.y && (((uintptr_t)a.y & 15) || ((uint64_t)a.y_ldc & vm) || (a.y_batch & vm))) return false;
    return S * (a.M / TS) < (1ull << 31) && a.batch <= 65535;
  }
  if (S % TS) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  // 16-byte accesses: rows and batch entries start on 16-byte boundaries
  if (((uintptr_t)a.in & 15) || ((uint64_t)a.in_ldm & vm) || (a.in_batch & vm)) return false;
  if (((uintptr_t)a.out & 15) || ((uint64_t)a.out_ldm & vm) || (a.out_batch & vm)) return false;
  if (a.y && (((uintptr_t)a.y & 15) || ((uint64_t)a.y_ldm & vm) || (a.y_batch & vm))) return false;
  return (a.Kin / E) * a.M < (1ull << 31) && a.batch <= 65535;
}

template <typename T, int P, bool KMM>
static hipError_t launchStepWideT(const StepArgs& a, hipStream_t stream, int maxPerCU) {
  const uint32_t E = kSwTileBytes / sizeof(T), TS = E / P;
  const uint32_t tilesPerLine = KMM ? a.M / TS : (uint32_t)(a.Kin / E);
  const uint32_t totalTiles = KMM ? (uint32_t)(a.Kin / P) * tilesPerLine : tilesPerLine * a.M;
  // persistent workgroups, as many per CU as registers and LDS allow (two for 128x128, more for the smaller factors)
  static std::atomic<int> occCache[kMaxDevices];
  const int devIdx = launchDeviceIndex();
  int occ = occCache[devIdx].load(std::memory_order_relaxed);
  if (occ == 0) {
    if (hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, (const void*)kron_step_wide_kernel<T, P, KMM, false, false>, 64 * kSwWaves,
                                                     kSwLdsBytes) != hipSuccess || occ < 1) occ = 2;
    if (occ > 4) occ = 4;
    occCache[devIdx].store(occ, std::memory_order_relaxed);
  }
  if (maxPerCU > 0 && occ > maxPerCU) occ = maxPerCU;          // (a tuner candidate: fewer, longer-running workgroups)
  uint32_t wgs = (uint32_t)occ * (uint32_t)deviceCUs();
  if (a.batch > 1) wgs = (wgs + a.batch - 1) / a.batch;
  if (wgs > totalTiles) wgs = totalTiles;
  if (wgs == 0) wgs = 1;
  dim3 grid(wgs, a.batch), block(64 * kSwWaves);
  // streamed results at system scope: 16 bytes per lane (not the 128x128 form), one batch entry, tiles spanning < 2 GB
  const uint64_t qStride = KMM ? (a.Kin / P) * (uint64_t)a.out_ldc : a.Kin / P;
  const bool streamOut = P != 128 && a.stream_out && a.batch == 1 && (uint64_t)P * qStride * sizeof(T) < (1ull << 31);
  using Kernel = void (*)(const StepArgs, const uint32_t, const uint32_t);
  static const Kernel kernels[2][2] = {
      {kron_step_wide_kernel<T, P, KMM, false, false>, kron_step_wide_kernel<T, P, KMM, false, P != 128>},
      {kron_step_wide_kernel<T, P, KMM, true, false>, kron_step_wide_kernel<T, P, KMM, true, P != 128>}};
  hipLaunchKernelGGL(kernels[(a.y && a.epilogue) ? 1 : 0][streamOut ? 1 : 0], grid, block, kSwLdsBytes, stream, a, tilesPerLine,
                     totalTiles);
  return hipGetLastError();
}

template <typename T>
static hipError_t launchStepWideD(const StepArgs& a, hipStream_t stream, int maxPerCU) {
  const uint32_t P = a.p[0];
  if (stepWideIsKmm(a))
    return P == 128 ? launchStepWideT<T, 128, true>(a, stream, maxPerCU) : P == 64 ? launchStepWideT<T, 64, true>(a, stream, maxPerCU)
                                                                         : launchStepWideT<T, 32, true>(a, stream, maxPerCU);
  return P == 128 ? launchStepWideT<T, 128, false>(a, stream, maxPerCU) : P == 64 ? launchStepWideT<T, 64, false>(a, stream, maxPerCU)
                                                                        : launchStepWideT<T, 32, false>(a, stream, maxPerCU);
}

hipError_t launchStepWide(const StepArgs& a, DType dt, hipStream_t stream, int maxWorkgroupsPerCU) {
  if (!stepWideSupported(a, dt)) return hipErrorInvalidValue;
  return dt == DType::F32 ? launchStepWideD<float>(a, stream, maxWorkgroupsPerCU) : launchStepWideD<double>(a, stream, maxWorkgroupsPerCU);
}

}  // namespace fk
