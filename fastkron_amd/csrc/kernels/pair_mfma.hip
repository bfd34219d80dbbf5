// Two fused square factors (P = Q in {32, 64}, fp64 or fp32) on rows of exactly P*P columns, MKM layout, on the
// matrix cores (V_MFMA_F64_16X16X4_F64 / V_MFMA_F32_16X16X4_F32): Z = X (F_b x F_a) with one read of X and one
// write of Z.  Serves gemkm with two such factors directly and, on "virtual rows" (every contiguous block of P*P columns of a
// longer row), the trailing two factors of longer chains; the leading factors are then applied across the
// blocks by the KMM-layout step kernel.
//
//   out[q_b*P + q_a] = sum_{k_b, k_a} in[k_b*P + k_a] * F_a[k_a, q_a] * F_b[k_b, q_b]
//
// A wave owns one row (a P x P tile, 32 KB for P = 64) at a time; no exchange through LDS is needed
// because the accumulator layout of the first product is an operand layout of the second:
//   * product 1, D1[k_b][q_a] = sum_{k_a} X[k_b][k_a] F_a[k_a][q_a]: X is the A operand (lane = 16*k + k_b,
//     contraction index k_a = (P/4)*k + c, so a lane reads P/4 consecutive doubles of its row), F_a the B
//     operand from LDS.  D1 sits at register k_b/4, lane 16*(k_b%4) + q_a;
//   * product 2, D2[q_b][q_a] = sum_{k_b} F_b^T[q_b][k_b] D1[k_b][q_a]: register r of D1 *is* a B operand
//     (lane = 16*k' + q_a) for the contraction indices k_b = 16*g + 4*r + k'; F_b^T comes from LDS as the
//     A operand.  D2 sits at register q_b/4, lane 16*(q_b%4) + q_a: a quarter wave stores 16 consecutive
//     doubles (one 128-byte line).
// Both factors are staged in LDS once per workgroup.  Workgroups are persistent, one per CU with one wave
// per SIMD: that leaves a wave 512 registers, enough to hold the next row (128 registers for P = 64) while
// the current one is multiplied, so memory and matrix pipe overlap inside every wave.
// alpha / beta*Y are applied in the store when this launch writes Z.
//
//
// The 64x64 case is bound by the matrix pipe, and V_MFMA_F64_4X4X4_4B_F64 sustains about 1.5 times the rate
// of the 16x16x4 instruction on this device, so 64x64 has its own kernel built on it (kron_pair64_f64_kernel;
// the chained-product kernel above serves 32x32, which is bound by memory).  One instruction multiplies four
// independent 4x4x4 blocks; the blocks are four neighbouring groups of four output columns q_a, so the
// factor operand is used as stored and the other operand is the same for the four blocks:
//   * product 1: A = X[k_b = 4t+i][k_a = 16k+c], the same for every block: read from LDS (the wave stages 16
//     rows of its tile at a time there) with four lanes per address; B = F_a[16k+c][16g+4blk+j], also from
//     LDS.  The 16 columns of product g are q_a = 32*(g/2) + 2n + g%2 (n = lane%16), so that a lane ends up with
//     pairs of neighbouring columns; D1[t][g] sits at lane 16*(k_b%4) + n;
//   * product 2: that register is the B operand for the contraction indices k_b = 4t+k; A = F_b[4t+k][4u+i]
//     comes from LDS, again one address per four lanes.  D2 sits at lane 16*(q_b%4) + n: 16-byte stores, a
//     quarter wave writes 32 consecutive doubles with two of them.
// Every LDS read feeds four products (two reads per four products in product 1).  Waves work independently
// (no barrier after the factors are staged), two per SIMD - the instruction only reaches its rate with two
// waves issuing - which leaves a wave 256 registers: 128 for D1, 32 for the quarter tile in flight.
//
// Role of the reference's fused shared-memory kernel (reference src/kernels/cuda/kernel.cuh:53-224 with
// FusedFacs = 2, CUDA cores only); the chained matrix-core products are specific to this kernel.
// Algorithmic traffic per launch: read M*P*P, write M*P*P elements (+ M*P*P for Y).
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef double pd4 __attribute__((ext_vector_type(4)));
typedef double pd2 __attribute__((ext_vector_type(2)));
typedef float pf4 __attribute__((ext_vector_type(4)));

constexpr int kPairWaves = 4;

// The 16x16x4 instruction per element type; row(r, hi) = row index, within a 16x16 accumulator, of register r
// in the lane group hi = lane / 16 (fp64: register i/4, lane group i%4; fp32: register i%4, lane group i/4).
template <typename T> struct PairMfma;
template <> struct PairMfma<double> {
  using Acc = pd4;
  static __device__ __forceinline__ Acc mma(double a, double b, Acc c) { return __builtin_amdgcn_mfma_f64_16x16x4f64(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ int row(int r, int hi) { return 4 * r + hi; }
};
template <> struct PairMfma<float> {
  using Acc = pf4;
  static __device__ __forceinline__ Acc mma(float a, float b, Acc c) { return __builtin_amdgcn_mfma_f32_16x16x4f32(a, b, c, 0, 0, 0); }
  static __device__ __forceinline__ int row(int r, int hi) { return 4 * hi + r; }
};

// EXACT = false: factors of R x R with 16 < R < P, operands zero-padded to the P x P tile: a row is R*R contiguous
// elements, loaded and stored element by element with indices >= R masked (what the padded lanes and registers
// compute is exact zeros and is never stored).
// Q != P: two factors of P x Q each (32 x 64, 64 x 32): the row is a P x P tile, the first product leaves P x Q, the
// result is a Q x Q tile; exact sizes only.
// SPLIT: a row is shared by 2^splitArg waves, each of which loads the whole row and produces Q / 16 / 2^splitArg of
// the 16-wide blocks of output columns q_a (few rows: more waves than rows, and the products of a block are one
// dependent chain).
template <typename T, int P, bool HAS_Y, bool EXACT = true, int Q = P, bool SPLIT = false>
__global__ __launch_bounds__(256, 2) void kron_pair_kernel(const StepArgs a, const uint32_t splitArg) {
  const uint32_t splitShift = SPLIT ? splitArg : 0;   // a constant in the kernels of whole rows
  static_assert(EXACT || P == Q, "the zero-padded form is square");
  using MF = PairMfma<T>;
  using Acc = typename MF::Acc;
  constexpr int PB = P / 16;             // 16-wide blocks of an input digit
  constexpr int QB = Q / 16;             // 16-wide blocks of an output digit
  constexpr int PC = P / 4;              // products per block of product 1, elements per lane and row
  constexpr int VE = 16 / sizeof(T);     // elements per 128-bit load
  typedef T VT __attribute__((ext_vector_type(VE)));
  extern __shared__ double pairLdsRaw[];
  T* fA = (T*)pairLdsRaw;                // F_a[k_a][q_a], row-major P x Q
  T* fB = fA + P * Q;                    // F_b[k_b][q_b]
  const int tid = threadIdx.x;
  const int l0 = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t bt = blockIdx.y;
  // exact tiles: a wave's own stage for 16 rows of its tile, 16 bytes of padding per row
  constexpr int kPitch = P + VE;
  T* stage = fB + P * Q + w * (16 * kPitch);

  const T* inB = (const T*)a.in + (size_t)bt * a.in_batch;
  T* outB = (T*)a.out + (size_t)bt * a.out_batch;
  const T* YB = HAS_Y ? (const T*)a.y + (size_t)bt * a.y_batch : nullptr;
  // multiplying by 1 is exact: launches that do not write Z need no branch around the scaling
  const T alpha = a.epilogue ? (T)a.alpha : (T)1, beta = (T)a.beta;
  const int R = EXACT ? P : (int)a.p[0];            // the factors' real size; the row is R * R elements
  const int RO = EXACT ? Q : R;                     // pitch of the result tile

  {
    const T* Fa = (const T*)a.f[0] + (size_t)bt * a.f_batch[0];
    const T* Fb = (const T*)a.f[1] + (size_t)bt * a.f_batch[1];
    // all loads of a thread go out before the first LDS write waits for one (a loop of load, wait, write puts one
    // memory round trip per iteration in front of the first product)
    T va[P * Q / 256], vb[P * Q / 256];
#pragma unroll
    for (int k = 0; k < P * Q / 256; k++) {
      const int i = tid + 256 * k, p = i / Q, q = i % Q;
      const bool in = EXACT || (p < R && q < R);
      va[k] = in ? Fa[(int64_t)p * a.f_sp[0] + (int64_t)q * a.f_sq[0]] : (T)0;
      vb[k] = in ? Fb[(int64_t)p * a.f_sp[1] + (int64_t)q * a.f_sq[1]] : (T)0;
    }
#pragma unroll
    for (int k = 0; k < P * Q / 256; k++) { fA[tid + 256 * k] = va[k]; fB[tid + 256 * k] = vb[k]; }
  }
  __syncthreads();

  const uint32_t stride = gridDim.x * kPairWaves;
  const uint32_t items = a.M << splitShift;         // an item: one row, one share of its q_a blocks
  const int jbPer = QB >> splitShift;
  // A row arrives in whole 1 KB pieces, lane l the 16 bytes l of a piece (an instruction that gave each lane 16 bytes
  // of its own tile row, 16 rows to a wave, kept the address path of the CU busy for 40 % of the kernel's time), and is
  // turned into operands through the stage, 16 tile rows at a time: lane (lo, hi) holds the columns PC*hi .. PC*hi+PC-1
  // of the rows 16g + lo.  The padded form loads its operands element by element.
  auto loadRow = [&](uint32_t item, T (&x)[PB][PC]) {
    const uint32_t row = item >> splitShift;
    if (!EXACT) {
      const int lo = l0 & 15, hi = l0 >> 4;
      const T* xp = inB + (size_t)row * a.in_ldm + lo * R + PC * hi;
#pragma unroll
      for (int g = 0; g < PB; g++)
#pragma unroll
        for (int c = 0; c < PC; c++)
          x[g][c] = (16 * g + lo < R && PC * hi + c < R) ? xp[g * 16 * R + c] : (T)0;
      return;
    }
    const VT* src = (const VT*)(inB + (size_t)row * a.in_ldm) + l0;
#pragma unroll
    for (int g = 0; g < PB; g++)
#pragma unroll
      for (int c = 0; c < PC; c += VE) {
        const VT v = src[64 * (g * (PC / VE) + c / VE)];
#pragma unroll
        for (int e = 0; e < VE; e++) x[g][c + e] = v[e];
      }
  };
  auto toOperands = [&](const T (&raw)[PB][PC], T (&x)[PB][PC]) {
    if (!EXACT) {
#pragma unroll
      for (int g = 0; g < PB; g++)
#pragma unroll
        for (int c = 0; c < PC; c++) x[g][c] = raw[g][c];
      return;
    }
    constexpr int CPR = P / VE;                     // 16-byte pieces of a tile row
    const int lo = l0 & 15, hi = l0 >> 4;
    T* wr = stage + (l0 / CPR) * kPitch + (l0 % CPR) * VE;
    const T* rd = stage + lo * kPitch + PC * hi;
#pragma unroll
    for (int g = 0; g < PB; g++) {
#pragma unroll
      for (int c = 0; c < PC; c += VE) {
        VT v;
#pragma unroll
        for (int e = 0; e < VE; e++) v[e] = raw[g][c + e];
        *(VT*)(wr + (c / VE) * (64 / CPR) * kPitch) = v;
      }
#pragma unroll
      for (int c = 0; c < PC; c += VE) {
        const VT v = *(const VT*)(rd + c);
#pragma unroll
        for (int e = 0; e < VE; e++) x[g][c + e] = v[e];
      }
    }
  };

  auto computeRow = [&](uint32_t item, const T (&x)[PB][PC]) {
    // the lane id is made opaque once per row so that the LDS reads below (the same for every row) are
    // not hoisted out of the loop into registers
    int l = l0;
    asm volatile("" : "+v"(l));
    const int lo = l & 15, hi = l >> 4;
    const uint32_t row = item >> splitShift;
    const int jb0 = SPLIT ? (int)(item & ((1u << splitShift) - 1)) * jbPer : 0;
    T* out = outB + (size_t)row * a.out_ldm;
    const T* Y = HAS_Y ? YB + (size_t)row * a.y_ldm : nullptr;

    // Factor operands come from LDS one group of products ahead: those of group n+1 are requested before the
    // products of group n are issued (left to itself the compiler requests an operand right in front of the two
    // products that take it, and the wave sits out an LDS round trip per 64 cycles of matrix work).
    auto readA = [&](int jb, int cg, T (&b)[4]) {        // product 1: F_a rows PC*hi + 4cg .. +3, column 16jb + lo
#pragma unroll
      for (int cc = 0; cc < 4; cc++) b[cc] = fA[(PC * hi + 4 * cg + cc) * Q + 16 * jb + lo];
    };
    auto readB = [&](int step, T (&f)[4][2]) {           // product 2: step = (pair of column blocks, row block g)
      const int jb2 = 2 * (step / PB), g = step % PB;
#pragma unroll
      for (int r = 0; r < 4; r++)
#pragma unroll
        for (int u = 0; u < 2; u++) f[r][u] = fB[(16 * g + MF::row(r, hi)) * Q + 16 * (jb2 + u) + lo];
    };
    constexpr int CG = PC / 4, STEPS = (QB / 2) * PB;
    // fp32: the operands of product 2 change places, which leaves the result transposed in the accumulators, a lane's
    // four registers four neighbouring columns q_a: 16-byte stores, a quarter of the store instructions (the fp64
    // instruction spreads a lane's registers over rows 4 apart either way)
    constexpr bool kTransposed = sizeof(T) == 4 && EXACT;
    T bn[4], fn[4][2];
    readA(jb0, 0, bn);
    // whole rows: unrolled, so that the stores of a row are counted and the wait for the next row's loads, which are
    // older, does not drain them (loads and stores share one in-order counter; behind a loop the wait is for all)
#pragma unroll
    for (int jb = jb0; jb < jb0 + jbPer; jb++) {
      const int ofs = 16 * jb + lo;
      Acc d1[PB];
#pragma unroll
      for (int g = 0; g < PB; g++) d1[g] = (Acc){0, 0, 0, 0};
#pragma unroll
      for (int cg = 0; cg < CG; cg++) {
        T bc[4];
#pragma unroll
        for (int cc = 0; cc < 4; cc++) bc[cc] = bn[cc];
        if (cg + 1 < CG) readA(jb, cg + 1, bn); else readB(0, fn);
        asm volatile("" ::: "memory");
#pragma unroll
        for (int cc = 0; cc < 4; cc++)
#pragma unroll
          for (int g = 0; g < PB; g++) d1[g] = MF::mma(x[g][4 * cg + cc], bc[cc], d1[g]);
      }
      // register r of d1[g] holds the rows k_b = 16g + row(r, hi): the B operand of product 2 for them;
      // two independent accumulator chains at a time
      Acc acc[2];
#pragma unroll
      for (int step = 0; step < STEPS; step++) {
        const int jb2 = 2 * (step / PB), g = step % PB;
        if (g == 0) { acc[0] = (Acc){0, 0, 0, 0}; acc[1] = (Acc){0, 0, 0, 0}; }
        T fc[4][2];
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
          for (int u = 0; u < 2; u++) fc[r][u] = fn[r][u];
        // (behind the last block of columns the request runs into the rows of F_b: inside LDS, never used)
        if (step + 1 < STEPS) readB(step + 1, fn); else readA(jb + 1, 0, bn);
        asm volatile("" ::: "memory");
#pragma unroll
        for (int r = 0; r < 4; r++)
#pragma unroll
          for (int u = 0; u < 2; u++)
            acc[u] = kTransposed ? MF::mma(d1[g][r], fc[r][u], acc[u]) : MF::mma(fc[r][u], d1[g][r], acc[u]);
        if (g != PB - 1) continue;
        if constexpr (kTransposed) {
          // lane (lo, hi), register e: Z[q_b = 16*(jb2+u) + lo][q_a = 16*jb + 4*hi + e], four neighbours per lane
#pragma unroll
          for (int u = 0; u < 2; u++) {
            const int qb = 16 * (jb2 + u) + lo, qa = 16 * jb + 4 * hi;
            if (EXACT) {
              Acc v = acc[u] * alpha;
              if (HAS_Y) v += beta * *(const Acc*)(Y + qb * RO + qa);
              // non-temporal: 4 to 7 % on the forms with a 64-wide factor, also where the next launch reads the
              // result (64x64^3: 1083 -> 1058 us); the same stores at system scope gain on 64x64, lose on 32x64
              __builtin_nontemporal_store(v, (Acc*)(out + qb * RO + qa));
            } else {
#pragma unroll
              for (int e = 0; e < 4; e++)
                if (qb < R && qa + e < R) {
                  T v = acc[u][e] * alpha;
                  if (HAS_Y) v += beta * Y[qb * RO + qa + e];
                  out[qb * RO + qa + e] = v;
                }
            }
          }
          continue;
        }
        T yv[2][4];
        if (HAS_Y) {
#pragma unroll
          for (int u = 0; u < 2; u++)
#pragma unroll
            for (int r = 0; r < 4; r++)
              yv[u][r] = (EXACT || (16 * (jb2 + u) + MF::row(r, hi) < R && ofs < R))
                             ? Y[(16 * (jb2 + u) + MF::row(r, hi)) * RO + ofs] : (T)0;
        }
#pragma unroll
        for (int u = 0; u < 2; u++)
#pragma unroll
          for (int r = 0; r < 4; r++) {               // q_b = 16*(jb2+u) + row(r, hi), q_a = 16*jb + lo
            T v = acc[u][r] * alpha;
            if (HAS_Y) v += beta * yv[u][r];
            if (EXACT || (16 * (jb2 + u) + MF::row(r, hi) < R && ofs < R))
              out[(16 * (jb2 + u) + MF::row(r, hi)) * RO + ofs] = v;
          }
      }
    }
  };

  // the next row streams into registers under the products of the current one (the last row of a wave requests
  // itself again rather than branching around the loads)
  uint32_t row = blockIdx.x * kPairWaves + w;
  if (row >= items) return;
  auto nextOf = [&](uint32_t r) { return r + stride < items ? r + stride : r; };
  T raw[PB][PC];
  loadRow(row, raw);
  auto oneRow = [&](uint32_t r) {
    T x[PB][PC];
    toOperands(raw, x);
    loadRow(nextOf(r), raw);
    computeRow(r, x);
  };
  // The first row is peeled off the loop.  Loads and stores retire through one in-order counter and the wait for the
  // prefetched row is counted in younger operations: entering the loop only behind a complete row lets that count
  // include the row's stores (otherwise the loop's wait is the first row's, which drains every store).
  oneRow(row);
  for (row += stride; row < items; row += stride) oneRow(row);
}


constexpr int kP64 = 64;
constexpr int kPair64Waves = 8;                     // one workgroup of 8 waves per CU, two waves per SIMD
constexpr int kPair64XWords = 16 * 64;              // doubles of X staging per wave: 16 rows of the tile
constexpr size_t kPair64LdsBytes = (2 * kP64 * kP64 + kPair64Waves * kPair64XWords) * sizeof(double);

// GN: 16-wide groups of output columns q_a a wave produces.  4: whole rows.  2 / 1: a row is shared by 2 / 4 waves, each
// of which loads it whole and works on its own columns (for row counts that leave waves without a row: the products
// of a row in one wave are latency bound, about 35 us whatever else runs).  Columns of group g and lane n: with
// GN >= 2 the pairs 32*(g/2) + 2n + g%2 (128-bit accesses), with GN = 1 the 16 neighbours 16*g + n.
template <bool HAS_Y, int NT, int GN = 4>
__global__ __launch_bounds__(512, 2) void kron_pair64_f64_kernel(const StepArgs a) {
  constexpr int P = kP64;
  constexpr int HN = GN >= 2 ? GN / 2 : 1;          // 128-bit column pairs (GN = 1: the one column) per lane
  constexpr uint32_t SHARE = 4 / GN;                // waves per row
  extern __shared__ double pairLds[];
  double* fA = pairLds;                              // F_a[k_a][q_a], row-major
  double* fB = pairLds + P * P;                      // F_b[k_b][q_b] at k_b*64 + (q_b ^ 4*(k_b%4))
  const int tid = threadIdx.x;
  const int l0 = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  double* xs = pairLds + 2 * P * P + w * kPair64XWords;   // this wave's X staging
  const uint32_t bt = blockIdx.y;

  const double* inB = (const double*)a.in + (size_t)bt * a.in_batch;
  double* outB = (double*)a.out + (size_t)bt * a.out_batch;
  const double* YB = HAS_Y ? (const double*)a.y + (size_t)bt * a.y_batch : nullptr;
  // multiplying by 1.0 is exact: launches that do not write Z need no branch around the scaling
  const double alpha = a.epilogue ? a.alpha : 1.0, beta = a.beta;

  {
    const double* Fa = (const double*)a.f[0] + (size_t)bt * a.f_batch[0];
    const double* Fb = (const double*)a.f[1] + (size_t)bt * a.f_batch[1];
    // (loads first, then the LDS writes: one memory round trip in front of the first product, not eight)
    double va[P * P / 512], vb[P * P / 512];
#pragma unroll
    for (int k = 0; k < P * P / 512; k++) {
      const int i = tid + 512 * k, p = i / P, q = i % P;
      va[k] = Fa[(int64_t)p * a.f_sp[0] + (int64_t)q * a.f_sq[0]];
      vb[k] = Fb[(int64_t)p * a.f_sp[1] + (int64_t)q * a.f_sq[1]];
    }
#pragma unroll
    for (int k = 0; k < P * P / 512; k++) {
      const int i = tid + 512 * k, p = i / P, q = i % P;
      fA[i] = va[k];
      fB[p * P + (q ^ (4 * (p & 3)))] = vb[k];
    }
  }
  __syncthreads();

  const uint32_t stride = gridDim.x * kPair64Waves;
  // lane l holds, of the 16 rows of a part, the doubles (j*64 + l)*2 + {0, 1}, j = 0..7.  One part (a
  // quarter of the tile) is in flight at a time: it is requested when the part before it has been written
  // to LDS, and arrives under that part's products (part 0 of the next tile under all of product 2).
  pd2 x[8];
  auto loadPart = [&](uint32_t row, int tb) {
    const double* xp = inB + (size_t)row * a.in_ldm + 2 * l0 + tb * 1024;
#pragma unroll
    for (int j = 0; j < 8; j++) x[j] = FK_LD(NT, (const pd2*)(xp + j * 128));
  };

  auto computeRow = [&](uint32_t item, uint32_t next) {
    // the lane id is made opaque once per row: the LDS reads of the factors are the same for every row and
    // must not be hoisted out of the loop into registers
    int l = l0;
    asm volatile("" : "+v"(l));
    const int i4 = l & 3, k4 = l >> 4, n16 = l & 15;  // operand lane = i + 4*blk + 16*k = n + 16*k
    const uint32_t row = item / SHARE;
    // first column of this wave's share, and the lane's place in a group
    const int colB = (int)(item % SHARE) * (GN == 1 ? 16 : 32), colL = GN == 1 ? n16 : 2 * n16;
    double* out = outB + (size_t)row * a.out_ldm;
    const double* Y = HAS_Y ? YB + (size_t)row * a.y_ldm : nullptr;

    // staging position of element (r, col) of a 16-row part: r*64 + 16*k + ((c + 4*(r%4) + k) % 16),
    // col = 16*k + c: the 16 addresses (i, k) of one operand read fall into 16 different bank pairs
    const int wr = l >> 5, wk = (l & 31) >> 3, wc = 2 * (l & 7);
    double d1[16][GN];
    auto loadB = [&](int c, double (&b)[GN]) {
      if (GN == 1) {
        b[0] = fA[(16 * k4 + c) * 64 + colB + colL];
      } else {
#pragma unroll
        for (int h = 0; h < HN; h++) {
          const pd2 v = *(const pd2*)&fA[(16 * k4 + c) * 64 + colB + 32 * h + colL];
          b[2 * h] = v[0]; b[(2 * h + 1) % GN] = v[1];
        }
      }
    };
#pragma unroll
    for (int tb = 0; tb < 4; tb++) {
#pragma unroll
      for (int j = 0; j < 8; j++) {
        const int r = 2 * j + wr;
#pragma unroll
        for (int e = 0; e < 2; e++) xs[r * 64 + 16 * wk + ((wc + e + 4 * (r & 3) + wk) & 15)] = x[j][e];
      }
      if (tb < 3) loadPart(row, tb + 1); else loadPart(next / SHARE, 0);
#pragma unroll
      for (int tt = 0; tt < 4; tt++)
#pragma unroll
        for (int g = 0; g < GN; g++) d1[4 * tb + tt][g] = 0.0;
      // operands of step c+1 are read before the products of step c are issued
      double an[4], bn[GN];
#pragma unroll
      for (int tt = 0; tt < 4; tt++) an[tt] = xs[(4 * tt + i4) * 64 + 16 * k4 + ((4 * i4 + k4) & 15)];
      loadB(0, bn);
#pragma unroll
      for (int c = 0; c < 16; c++) {
        double ac[4], bc[GN];
#pragma unroll
        for (int tt = 0; tt < 4; tt++) ac[tt] = an[tt];
#pragma unroll
        for (int g = 0; g < GN; g++) bc[g] = bn[g];
        if (c + 1 < 16) {
#pragma unroll
          for (int tt = 0; tt < 4; tt++) an[tt] = xs[(4 * tt + i4) * 64 + 16 * k4 + ((c + 1 + 4 * i4 + k4) & 15)];
          loadB(c + 1, bn);
        }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int tt = 0; tt < 4; tt++)
#pragma unroll
          for (int g = 0; g < GN; g++)
            d1[4 * tb + tt][g] = __builtin_amdgcn_mfma_f64_4x4x4f64(ac[tt], bc[g], d1[4 * tb + tt][g], 0, 0, 0);
      }
    }

    const int orow = l >> 4, ocol = l & 15;         // result lane = 16*(q_b%4) + q_a%16
    // fully unrolled, so that the 64 stores of a row are counted when the next row waits for its
    // prefetched part (see the note on the peeled first row)
#pragma unroll
    for (int ub = 0; ub < 4; ub++) {
      // F_b[4t + k][16ub + 4uu + i] at (4t + k)*64 + 16ub + 4*(uu ^ k) + i
      int fo[4];
#pragma unroll
      for (int uu = 0; uu < 4; uu++) {
        fo[uu] = k4 * 64 + 16 * ub + 4 * (uu ^ k4) + i4;
        asm volatile("" : "+v"(fo[uu]));
      }
      double acc[4][GN];
#pragma unroll
      for (int uu = 0; uu < 4; uu++)
#pragma unroll
        for (int g = 0; g < GN; g++) acc[uu][g] = 0.0;
      double fn[4];
#pragma unroll
      for (int uu = 0; uu < 4; uu++) fn[uu] = fB[fo[uu]];
#pragma unroll
      for (int t = 0; t < 16; t++) {
        double fc[4];
#pragma unroll
        for (int uu = 0; uu < 4; uu++) fc[uu] = fn[uu];
        if (t + 1 < 16) {
#pragma unroll
          for (int uu = 0; uu < 4; uu++) fn[uu] = fB[fo[uu] + 4 * (t + 1) * 64];
        }
        asm volatile("" ::: "memory");
#pragma unroll
        for (int uu = 0; uu < 4; uu++)
#pragma unroll
          for (int g = 0; g < GN; g++)
            acc[uu][g] = __builtin_amdgcn_mfma_f64_4x4x4f64(fc[uu], d1[t][g], acc[uu][g], 0, 0, 0);
      }
      // q_b = 16ub + 4uu + orow; the products g = 2h, 2h+1 hold the neighbouring columns q_a = 32h + 2*ocol, +1
      // (one group: the column 16*share + ocol)
      const int o0 = (16 * ub + orow) * 64 + colB + (GN == 1 ? ocol : 2 * ocol);
      // Y in two halves, each read before the stores of its half (registers are short with Y)
#pragma unroll
      for (int uh = 0; uh < 4; uh += 2) {
        if (GN == 1) {
          double yv[2];
          if (HAS_Y) {
#pragma unroll
            for (int uu = 0; uu < 2; uu++) yv[uu] = Y[o0 + 4 * (uh + uu) * 64];
          }
#pragma unroll
          for (int uu = 0; uu < 2; uu++) {
            double v = acc[uh + uu][0] * alpha;
            if (HAS_Y) v += beta * yv[uu];
            out[o0 + 4 * (uh + uu) * 64] = v;
          }
        } else {
          pd2 yv[2][HN];
          if (HAS_Y) {
#pragma unroll
            for (int uu = 0; uu < 2; uu++)
#pragma unroll
              for (int h = 0; h < HN; h++) yv[uu][h] = *(const pd2*)(Y + o0 + 4 * (uh + uu) * 64 + 32 * h);
          }
#pragma unroll
          for (int uu = 0; uu < 2; uu++)
#pragma unroll
            for (int h = 0; h < HN; h++) {
              pd2 v = {acc[uh + uu][2 * h] * alpha, acc[uh + uu][(2 * h + 1) % GN] * alpha};
              if (HAS_Y) v += beta * yv[uu][h];
              FK_ST(NT, v, (pd2*)(out + o0 + 4 * (uh + uu) * 64 + 32 * h));
            }
        }
      }
    }
  };

  const uint32_t items = a.M * SHARE;               // an item: one row, one share of its columns
  uint32_t row = blockIdx.x * kPair64Waves + w;
  if (row >= items) return;
  // the last row of a wave prefetches its own first part again: no branch around memory operations
  auto nextOf = [&](uint32_t r) { return r + stride < items ? r + stride : r; };
  loadPart(row / SHARE, 0);
  // The first row is peeled off the loop.  Loads and stores retire through one in-order counter and
  // the wait for a prefetched part is counted in younger operations; entering the loop only from a
  // complete row lets that count include the 64 stores issued behind the prefetch, so that the wait
  // at the top of a row does not drain the previous row's stores.
  computeRow(row, nextOf(row));
  for (row += stride; row < items; row += stride) computeRow(row, nextOf(row));
}

// Rectangular pairs with exact tiles: 32x64 and 64x32 in fp32, 32x64 in fp64 (a 64 x 64 tile of doubles, twice over
// for the row in flight, would not leave this kernel's waves enough registers).
static bool pairRectShape(uint32_t P, uint32_t Q, DType dt) {
  return (P == 32 && Q == 64) || (P == 64 && Q == 32 && dt == DType::F32);
}

bool pairMfmaSupported(const StepArgs& a, DType dt) {
  if (a.nf != 2) return false;
  const uint32_t P = a.p[0], Q = a.q[0];
  if (a.p[1] != P || a.q[1] != Q) return false;
  if (P != Q) {
    if (!pairRectShape(P, Q, dt)) return false;
  } else if (P != 64 && (P < 17 || P > 32)) return false;
  if (a.Kin != (uint64_t)P * P || a.Kout != (uint64_t)Q * Q) return false;
  if (a.in_ldc != 1 || a.out_ldc != 1 || (a.y && a.y_ldc != 1)) return false;
  if (P < 32) return a.batch <= 65535;                                                // padded form: element-wise accesses
  const uint64_t vmask = 16 / dtypeSize(dt) - 1;                                      // 128-bit loads
  if (((uintptr_t)a.in & 15) || ((uint64_t)a.in_ldm & vmask) || (a.in_batch & vmask)) return false;
  if (dt == DType::F32 || (P == 64 && Q == 64)) {                                     // and 128-bit stores / Y loads
    if (((uintptr_t)a.out & 15) || ((uint64_t)a.out_ldm & vmask) || (a.out_batch & vmask)) return false;
    if (a.y && (((uintptr_t)a.y & 15) || ((uint64_t)a.y_ldm & vmask) || (a.y_batch & vmask))) return false;
  }
  return a.batch <= 65535;
}

template <typename T, int P, bool EXACT = true, int Q = P>
static hipError_t launchPairT(const StepArgs& a, hipStream_t stream) {
  const int cus = deviceCUs();
  const size_t ldsBytes = (2 * P * Q + (EXACT ? kPairWaves * 16 * (P + 16 / sizeof(T)) : 0)) * sizeof(T);
  uint32_t wgs = (uint32_t)cus * (P == 32 && Q == 32 ? 4 : 2);   // persistent; the 32x32 kernels need few registers
  if (a.batch > 1) wgs = (wgs + a.batch - 1) / a.batch;
  // fewer rows than the waves of one workgroup per CU: the rows are shared out by blocks of output columns (a second
  // workgroup of a CU starts microseconds behind the first, which costs more than the shorter chains gain)
  uint32_t splitShift = 0;
  while ((Q / 16) >> (splitShift + 1) >= 1 &&
         ((uint64_t)a.M << (splitShift + 1)) * a.batch <= (uint64_t)cus * kPairWaves)
    splitShift++;
  const uint32_t need = ((a.M << splitShift) + kPairWaves - 1) / kPairWaves;
  if (wgs > need) wgs = need;
  if (wgs == 0) wgs = 1;
  dim3 grid(wgs, a.batch), block(256);
  static PerDeviceOnce attrOnce[2];
  const int devIdx = launchDeviceIndex();
  const bool y = a.y && a.epilogue;
  if (!attrOnce[y].done(devIdx)) {
    using Kernel = void (*)(const StepArgs, const uint32_t);
    const Kernel all[4] = {kron_pair_kernel<T, P, false, EXACT, Q, false>, kron_pair_kernel<T, P, false, EXACT, Q, true>,
                           kron_pair_kernel<T, P, true, EXACT, Q, false>, kron_pair_kernel<T, P, true, EXACT, Q, true>};
    for (int k = 2 * y; k < 2 * y + 2; k++) {
      hipError_t e = hipFuncSetAttribute((const void*)all[k], hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
      if (e != hipSuccess) return e;
    }
    attrOnce[y].mark(devIdx);
  }
  if (y) {
    if (splitShift) hipLaunchKernelGGL((kron_pair_kernel<T, P, true, EXACT, Q, true>), grid, block, ldsBytes, stream, a, splitShift);
    else hipLaunchKernelGGL((kron_pair_kernel<T, P, true, EXACT, Q, false>), grid, block, ldsBytes, stream, a, 0u);
  } else {
    if (splitShift) hipLaunchKernelGGL((kron_pair_kernel<T, P, false, EXACT, Q, true>), grid, block, ldsBytes, stream, a, splitShift);
    else hipLaunchKernelGGL((kron_pair_kernel<T, P, false, EXACT, Q, false>), grid, block, ldsBytes, stream, a, 0u);
  }
  return hipGetLastError();
}

static hipError_t launchPair64(const StepArgs& a, hipStream_t stream) {
  const int cus = deviceCUs();
  uint32_t wgs = (uint32_t)cus;                     // persistent, one workgroup per CU
  if (a.batch > 1) wgs = (wgs + a.batch - 1) / a.batch;
  // rows for at most half (a quarter) of the waves: two (four) waves per row
  const uint64_t waves = (uint64_t)wgs * kPair64Waves;
  const uint32_t share = 4ull * a.M <= waves ? 4 : 2ull * a.M <= waves ? 2 : 1;
  const uint32_t need = (a.M * share + kPair64Waves - 1) / kPair64Waves;
  if (wgs > need) wgs = need;
  if (wgs == 0) wgs = 1;
  dim3 grid(wgs, a.batch), block(64 * kPair64Waves);
  static PerDeviceOnce attrOnce;
  const int devIdx = launchDeviceIndex();
  using Kernel = void (*)(const StepArgs);
  // (the shared forms run on rows that stay in the caches: ordinary loads and stores)
  static const Kernel kernels[2][5] = {
      {kron_pair64_f64_kernel<false, 0>, kron_pair64_f64_kernel<false, 1>, kron_pair64_f64_kernel<false, 2>,
       kron_pair64_f64_kernel<false, 0, 2>, kron_pair64_f64_kernel<false, 0, 1>},
      {kron_pair64_f64_kernel<true, 0>, kron_pair64_f64_kernel<true, 1>, kron_pair64_f64_kernel<true, 2>,
       kron_pair64_f64_kernel<true, 0, 2>, kron_pair64_f64_kernel<true, 0, 1>}};
  if (!attrOnce.done(devIdx)) {
    for (int y = 0; y < 2; y++)
      for (int k = 0; k < 5; k++) {
        hipError_t e = hipFuncSetAttribute((const void*)kernels[y][k], hipFuncAttributeMaxDynamicSharedMemorySize,
                                           (int)kPair64LdsBytes);
        if (e != hipSuccess) return e;
      }
    attrOnce.mark(devIdx);
  }
  const int which = share == 4 ? 4 : share == 2 ? 3 : streamMode(a);
  hipLaunchKernelGGL(kernels[(a.y && a.epilogue) ? 1 : 0][which], grid, block, kPair64LdsBytes, stream, a);
  return hipGetLastError();
}

hipError_t launchPairMfma(const StepArgs& a, DType dt, hipStream_t stream) {
  if (!pairMfmaSupported(a, dt)) return hipErrorInvalidValue;
  if (a.p[0] != a.q[0]) {
    if (dt == DType::F64) return launchPairT<double, 32, true, 64>(a, stream);
    return a.p[0] == 32 ? launchPairT<float, 32, true, 64>(a, stream) : launchPairT<float, 64, true, 32>(a, stream);
  }
  if (a.p[0] < 32) return dt == DType::F64 ? launchPairT<double, 32, false>(a, stream) : launchPairT<float, 32, false>(a, stream);
  if (dt == DType::F64) return a.p[0] == 64 ? launchPair64(a, stream) : launchPairT<double, 32>(a, stream);
  return a.p[0] == 64 ? launchPairT<float, 64>(a, stream) : launchPairT<float, 32>(a, stream);
}

}  // namespace fk
