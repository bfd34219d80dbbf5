// Whole-row kernel for five fused 8x8 fp64 factors (row length 8^5 = 32768 doubles = 256 KB, e.g. dgemkm
// 1024 x 32768 with 8x8^5).  One workgroup of 8 wave64s owns one row and keeps it in VGPRs (64 doubles = 128
// registers per lane); the row is half of a CU's register file, so one workgroup runs per CU.
//
//   Z[q1..q5] = alpha * sum_{k1..k5} X[k1..k5] * F1[k1,q1] * ... * F5[k5,q5]  (+ beta * Y)
//
// Every lane owns whole slices: for the digit being contracted it holds the 8 inputs of a slice in registers and
// produces the 8 outputs in registers.  The contractions run on the vector ALU: on this chip its fp64 FMA rate equals
// the matrix cores' (128 flop per clock and CU either way), a lane's FMA needs no particular operand layout, and the
// factor element of an FMA is the same for all lanes, so it comes from a scalar register (the factors are read with
// scalar loads, half a factor = 64 scalar registers at a time).  The fp64 matrix instruction (4x4x4) contracts an
// index that lies in lane bits 4-5: it could contract the digits where the loads put them, in the lanes, and spare the
// in-wave exchange below, which costs 1 us of a row's 28 (measured with the exchange removed).
//
//   load     lane = (k4,k5) (512 contiguous bytes per wave instruction), wave = k3, regs = (k1,k2)
//   stage A  contract k1, k2
//   exch. 1  across the waves through LDS (two 128 KB halves, XOR-swizzled 16-byte chunks): wave = q1,
//            lane = (q2,k3), regs = (k4,k5)
//   stage B  contract k5, k4
//   exch. 2  inside each wave (a 64 x 64 transposition through the wave's own LDS region, two halves, rows padded to
//            65 doubles): lane = (q4,q5), regs = (k3,q2); no workgroup barrier
//   stage C  contract k3
//   store    512 contiguous bytes per wave instruction
// The workgroups that start together (one per CU) begin in three groups a few microseconds apart, so that not every
// CU waits for HBM at the same moment.
//
// The reference fuses at most as many factors as fit its shared-memory tile (two launches and one HBM round trip of
// the intermediate for this shape, kernel "..._8x8_8x8_3_1x4096_..."); here the row never leaves the CU.
// Algorithmic traffic: 8*32768 bytes read + 8*32768 bytes written per row (+ Y when beta != 0); arithmetic:
// 5 * 32768 * 8 FMAs per row = 8.5 us of one CU's vector ALUs.
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef double d2 __attribute__((ext_vector_type(2)));
// Factor elements are read through the constant address space: the address is wave-uniform and nothing in the launch
// writes the factors, so the loads are scalar loads whatever else the kernel has stored by then.
typedef const double __attribute__((address_space(4))) * FactorPtr;

constexpr int kRow8dLen = 32768;
// Start groups of the first round of workgroups (measured on dgemkm 1024 / 2048 x 8^5: no stagger 125 / 242 us; three
// groups 6 us apart 121 / 228, 7 us apart 119 / 232, 8 to 10 us apart 131-135 / 247; two, four, five, six or eight
// groups at spacings from 2 to 14 us 124-137 / 237-252).
constexpr uint32_t kRow8dStaggerGroups = 3;
constexpr uint32_t kRow8dStaggerTicks = 650;      // of the 100 MHz wall clock
constexpr int kRow8dWaveRegion = 32 * 65;                       // doubles per wave in exchange 2
constexpr int kRow8dLdsDoubles = 8 * kRow8dWaveRegion;          // 133 120 bytes; exchange 1 needs 131 072

struct Factor8 {
  FactorPtr f;
};

// Half a factor, the columns q0 .. q0+3, in 64 scalar registers: element (p, i) is F(p, q0 + i).  Stored with q
// fastest these are eight pieces of four doubles, stored with p fastest four pieces of eight.  The loads are written
// out because the compiler merges the two halves of a factor into one fetch and then spills scalar registers by
// the hundred.  `fetch` waits for its loads before it returns: the compiler does not know of a load inside an asm
// statement, so a value must not be in flight anywhere it might copy the register (the factors are 2.5 KB that
// every wave of the launch reads, a scalar-cache hit each time).  One asm statement holds the loads of a half and
// their wait, with early-clobber results, so nothing can come between them.
typedef double d4s __attribute__((ext_vector_type(4)));
typedef double d8s __attribute__((ext_vector_type(8)));
template <bool PMAJOR> struct HalfFactor;
template <> struct HalfFactor<true> {
  d4s v[8];                                     // v[p][i]
  __device__ __forceinline__ void fetch(FactorPtr f, int q0) {
    // (q0 is 0 or 4: the offsets are immediates)
#define ROW8D_FETCH(o)                                                                                        \
    asm volatile("s_load_dwordx8 %0, %8, " #o "+0\n\ts_load_dwordx8 %1, %8, " #o "+64\n\t"                     \
                 "s_load_dwordx8 %2, %8, " #o "+128\n\ts_load_dwordx8 %3, %8, " #o "+192\n\t"                  \
                 "s_load_dwordx8 %4, %8, " #o "+256\n\ts_load_dwordx8 %5, %8, " #o "+320\n\t"                  \
                 "s_load_dwordx8 %6, %8, " #o "+384\n\ts_load_dwordx8 %7, %8, " #o "+448\n\t"                  \
                 "s_waitcnt lgkmcnt(0)"                                                                       \
                 : "=&s"(v[0]), "=&s"(v[1]), "=&s"(v[2]), "=&s"(v[3]), "=&s"(v[4]), "=&s"(v[5]), "=&s"(v[6]), \
                   "=&s"(v[7])                                                                                \
                 : "s"(f))
    if (q0 == 0) ROW8D_FETCH(0); else ROW8D_FETCH(32);
#undef ROW8D_FETCH
  }
  __device__ __forceinline__ double at(int p, int i) const { return v[p][i]; }
};
template <> struct HalfFactor<false> {
  d8s v[4];                                     // v[i][p]
  __device__ __forceinline__ void fetch(FactorPtr f, int q0) {
#define ROW8D_FETCH(o)                                                                                        \
    asm volatile("s_load_dwordx16 %0, %4, " #o "+0\n\ts_load_dwordx16 %1, %4, " #o "+64\n\t"                   \
                 "s_load_dwordx16 %2, %4, " #o "+128\n\ts_load_dwordx16 %3, %4, " #o "+192\n\t"                \
                 "s_waitcnt lgkmcnt(0)"                                                                       \
                 : "=&s"(v[0]), "=&s"(v[1]), "=&s"(v[2]), "=&s"(v[3])                                         \
                 : "s"(f))
    if (q0 == 0) ROW8D_FETCH(0); else ROW8D_FETCH(256);
#undef ROW8D_FETCH
  }
  __device__ __forceinline__ double at(int p, int i) const { return v[i][p]; }
};

// One 8-point contraction per slice s: v(s, p) names the register of input / output p of slice s.  The outputs 0..3
// of all eight slices are kept aside while the outputs 4..7 are formed, so that one half of the factor is in scalar
// registers at a time and a lane holds at most 96 doubles.
#define ROW8D_CONTRACT(v)                                                                                   \
  {                                                                                                         \
    double keep[8][4];                                                                                      \
    HalfFactor<PMAJOR> f;                                                                                   \
    f.fetch(F.f, 0);                                                                                        \
    _Pragma("unroll") for (int s = 0; s < 8; s++)                                                           \
      _Pragma("unroll") for (int i = 0; i < 4; i++) {                                                       \
        double t = f.at(0, i) * v(s, 0);                                                                    \
        _Pragma("unroll") for (int p = 1; p < 8; p++) t = __builtin_fma(f.at(p, i), v(s, p), t);            \
        keep[s][i] = t;                                                                                     \
      }                                                                                                     \
    f.fetch(F.f, 4);                                                                                        \
    _Pragma("unroll") for (int s = 0; s < 8; s++) {                                                         \
      double o[4];                                                                                          \
      _Pragma("unroll") for (int i = 0; i < 4; i++) {                                                       \
        double t = f.at(0, i) * v(s, 0);                                                                    \
        _Pragma("unroll") for (int p = 1; p < 8; p++) t = __builtin_fma(f.at(p, i), v(s, p), t);            \
        o[i] = t;                                                                                           \
      }                                                                                                     \
      _Pragma("unroll") for (int i = 0; i < 4; i++) { v(s, i) = keep[s][i]; v(s, 4 + i) = o[i]; }           \
    }                                                                                                       \
  }

// x[a][b] <- sum_p F[p][a] x[p][b]
template <bool PMAJOR>
__device__ __forceinline__ void contractFirst(double (&x)[8][8], const Factor8& F) {
#define ROW8D_V(s, p) x[p][s]
  ROW8D_CONTRACT(ROW8D_V)
#undef ROW8D_V
}

// x[a][b] <- sum_p F[p][b] x[a][p]
template <bool PMAJOR>
__device__ __forceinline__ void contractSecond(double (&x)[8][8], const Factor8& F) {
#define ROW8D_V(s, p) x[s][p]
  ROW8D_CONTRACT(ROW8D_V)
#undef ROW8D_V
}

// PMAJOR: the factors are stored with q fastest (element (p,q) at 8p + q), otherwise with p fastest (the other op)
template <bool HAS_Y, int NT, bool PMAJOR>
__global__ __launch_bounds__(512) void kron_row8x5_f64_kernel(const StepArgs a, const uint32_t firstRound,
                                                              const uint32_t staggerGroups, const uint32_t staggerTicks) {
  extern __shared__ __align__(16) double ldsd[];
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t m = blockIdx.x, bt = blockIdx.y;
  // The workgroups that the device starts together (one per CU) would load, compute and store in lockstep, all of
  // them waiting for HBM in one phase and none using it in the next: they start in groups, staggerTicks of the 100 MHz
  // clock apart; later workgroups start whenever a predecessor ends and keep that spread.
  if (staggerTicks) {
    const uint32_t idx = blockIdx.x + gridDim.x * blockIdx.y;
    const uint32_t grp = (idx >> 3) % staggerGroups;              // idx % 8 is the XCD
    if (idx < firstRound && grp) {
      const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
      while (__builtin_amdgcn_s_memrealtime() - t0 < (unsigned long long)grp * staggerTicks) __builtin_amdgcn_s_sleep(16);
    }
  }

  const double* X = (const double*)a.in + (size_t)bt * a.in_batch + (size_t)m * kRow8dLen;
  double* Z = (double*)a.out + (size_t)bt * a.out_batch + (size_t)m * kRow8dLen;

  // a.f[0] is the last factor F5 ... a.f[nf-1] the first; F[d] below is the factor of digit d+1
  Factor8 F[5];
#pragma unroll
  for (int d = 0; d < 5; d++) {
    const int j = 4 - d;
    F[d].f = (FactorPtr)((const double*)a.f[j] + (size_t)bt * a.f_batch[j]);
  }

  // ---- load: x[k1][k2] = X[k1][k2][k3 = w][(k4,k5) = l]; k2 outermost, so the slices of the first contraction (all
  //      k1 for one k2) complete in issue order ----
  double x[8][8];
  {
    const double* xp = X + w * 64 + l;
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
      for (int i = 0; i < 8; i++) x[i][j] = FK_LD(NT, &xp[i * 4096 + j * 512]);
  }

  // ---- stage A ----
  contractFirst<PMAJOR>(x, F[0]);
  contractSecond<PMAJOR>(x, F[1]);                       // x[q1][q2], wave = k3, lane = (k4,k5)

  // ---- exchange 1: half h holds q1 in [4h, 4h+4).  Group g = (q1 & 3, q2, k3) owns 64 doubles (k4,k5) stored as 32
  //      chunks of 2, chunk index XORed with the low 5 bits of g.  Reader: thread (q1, q2, k3) reads its group as regs
  //      [k4][k5]; the waves with q1 >> 2 == h read. ----
  double y[8][8];
#pragma unroll
  for (int h = 0; h < 2; h++) {
    if (h) __syncthreads();
    {
      // g & 31 = (q2 & 3) * 8 + w: four base addresses, the rest are constant offsets
      double* base[4];
#pragma unroll
      for (int s = 0; s < 4; s++) base[s] = ldsd + w * 64 + ((((l >> 1) ^ (s * 8 + w)) << 1) | (l & 1));
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) base[j & 3][(i * 8 + j) * 512] = x[4 * h + i][j];
    }
    __syncthreads();
    if ((w >> 2) == h) {
      const int g = (w & 3) * 64 + l;
#pragma unroll
      for (int c = 0; c < 32; c++) {
        const d2 v = *(const d2*)&ldsd[g * 64 + ((c ^ (g & 31)) << 1)];
        y[c >> 2][(c & 3) * 2] = v[0];
        y[c >> 2][(c & 3) * 2 + 1] = v[1];
      }
    }
  }
  // thread = (q1 = w, q2 = l >> 3, k3 = l & 7), y[k4][k5]

  // ---- stage B ----
  contractSecond<PMAJOR>(y, F[4]);
  contractFirst<PMAJOR>(y, F[3]);                        // y[q4][q5]

  // ---- exchange 2, inside the wave: writer lane (q2,k3) holds y[q4][q5], reader lane (q4,q5) wants z[k3][q2].
  //      Half h: the reader lanes with q4 >> 2 == h.  T[reader lane & 31][writer lane], rows of 65 doubles.  The
  //      wave's region is part of what other waves read in exchange 1, hence one workgroup barrier ahead of the
  //      first write. ----
  double z[8][8];
  __syncthreads();
  {
    double* const T = ldsd + w * kRow8dWaveRegion;
#pragma unroll
    for (int h = 0; h < 2; h++) {
#pragma unroll
      for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 8; j++) T[(i * 8 + j) * 65 + l] = y[4 * h + i][j];
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      if ((l >> 5) == h) {
#pragma unroll
        for (int q2 = 0; q2 < 8; q2++)
#pragma unroll
          for (int k3 = 0; k3 < 8; k3++) z[k3][q2] = T[(l & 31) * 65 + q2 * 8 + k3];
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    }
  }
  // thread = (q1 = w, lane = (q4,q5)), z[k3][q2]

  // ---- stage C ----
  contractFirst<PMAJOR>(z, F[2]);

  // ---- epilogue and store ----
  const double alpha = a.alpha, beta = a.beta;
  const double* Y = HAS_Y ? (const double*)a.y + (size_t)bt * a.y_batch + (size_t)m * kRow8dLen : nullptr;
#pragma unroll
  for (int q2 = 0; q2 < 8; q2++)
#pragma unroll
    for (int q3 = 0; q3 < 8; q3++) {
      const int col = w * 4096 + q2 * 512 + q3 * 64 + l;
      double v = z[q3][q2];
      if (a.epilogue) {
        v *= alpha;
        if (HAS_Y) v += beta * Y[col];
      }
      FK_ST(NT, v, &Z[col]);
    }
}

static bool row8dPMajor(const StepArgs& a) { return a.f_sq[0] == 1; }

bool row8x5F64Supported(const StepArgs& a) {
  if (a.nf != 5) return false;
  for (uint32_t j = 0; j < 5; j++) {
    if (a.p[j] != 8 || a.q[j] != 8) return false;
    // dense 8x8 factors, all stored the same way round
    if (!((a.f_sp[j] == 8 && a.f_sq[j] == 1) || (a.f_sp[j] == 1 && a.f_sq[j] == 8))) return false;
    if (a.f_sq[j] != a.f_sq[0]) return false;
  }
  const uint64_t k = kRow8dLen;
  if (a.Kin != k || a.Kout != k) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  if ((uint64_t)a.in_ldm != k || (uint64_t)a.out_ldm != k || (a.y && (uint64_t)a.y_ldm != k)) return false;
  return a.batch <= 65535;
}

hipError_t launchRow8x5F64(const StepArgs& a, hipStream_t stream) {
  if (!row8x5F64Supported(a)) return hipErrorInvalidValue;
  static PerDeviceOnce attrOnce;
  const int devIdx = launchDeviceIndex();
  const size_t ldsBytes = kRow8dLdsDoubles * sizeof(double);
  using Kernel = void (*)(const StepArgs, const uint32_t, const uint32_t, const uint32_t);
  static const Kernel kernels[2][2][3] = {
      {{kron_row8x5_f64_kernel<false, 0, false>, kron_row8x5_f64_kernel<false, 1, false>, kron_row8x5_f64_kernel<false, 2, false>},
       {kron_row8x5_f64_kernel<true, 0, false>, kron_row8x5_f64_kernel<true, 1, false>, kron_row8x5_f64_kernel<true, 2, false>}},
      {{kron_row8x5_f64_kernel<false, 0, true>, kron_row8x5_f64_kernel<false, 1, true>, kron_row8x5_f64_kernel<false, 2, true>},
       {kron_row8x5_f64_kernel<true, 0, true>, kron_row8x5_f64_kernel<true, 1, true>, kron_row8x5_f64_kernel<true, 2, true>}}};
  if (!attrOnce.done(devIdx)) {
    for (int f = 0; f < 2; f++)
      for (int y = 0; y < 2; y++)
        for (int nt = 0; nt < 3; nt++) {
          hipError_t e = hipFuncSetAttribute((const void*)kernels[f][y][nt], hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
          if (e != hipSuccess) return e;
        }
    attrOnce.mark(devIdx);
  }
  dim3 grid(a.M, a.batch), block(512);
  const uint32_t cus = (uint32_t)deviceCUs();
  const bool stagger = (uint64_t)a.M * a.batch >= 2ull * cus;     // with one row per CU there is nothing to interleave
  hipLaunchKernelGGL(kernels[row8dPMajor(a) ? 1 : 0][(a.y && a.epilogue) ? 1 : 0][streamMode(a)], grid, block, ldsBytes, stream, a,
                     cus, kRow8dStaggerGroups, stagger ? kRow8dStaggerTicks : 0u);
  return hipGetLastError();
}

}  // namespace fk
