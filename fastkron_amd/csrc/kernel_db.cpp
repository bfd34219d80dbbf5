#include "kernel_db.h"

#include <dlfcn.h>

#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <sstream>

#include "kernels/launch.h"

namespace fk {

std::string KronProblem::str() const {
  std::ostringstream o;
  auto facs = [&]() {
    if (sameShapes(0, N - 1)) o << P[0] << "x" << Q[0] << "^" << N;
    else for (uint32_t i = 0; i < N; i++) { o << P[i] << "x" << Q[i]; if (i + 1 < N) o << "(x)"; }
  };
  if (mm == MMType::MKM) { o << M << "x" << K() << "*("; facs(); o << ")"; }
  else                   { o << "("; facs(); o << ")*" << K() << "x" << M; }
  o << "_" << (opX == 2 ? "T" : "N") << (opF == 2 ? "T" : "N") << "_" << (dt == DType::F32 ? "f" : "d");
  if (strided) {
    o << "_stridedBatched_" << batch;
    // the stride class: a shared X and shared factors change which kernels and rewritings apply (merging, the
    // two-part plan), so plans of one class are not looked up for another.  Per-batch operands carry no suffix.
    if (batch > 1) {
      if (strideX == 0) o << "_Xs";
      uint64_t shared = 0;
      for (uint32_t i = 0; i < N; i++) if (strideF[i] == 0) shared |= 1ull << i;
      if (shared) o << "_Fs" << std::hex << shared << std::dec;
    }
  }
  return o.str();
}

static bool genericCanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool, bool,
                          const DeviceInfo&) {
  return lo == hi && k.dt == p.dt;
}
static hipError_t genericLaunch(const KernelInfo& k, const StepArgs& a, hipStream_t s) {
  return launchGenericStep(a, k.dt, s);
}

// ---- several small factors of any shape fused through LDS ----
static bool fusedSmallCanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                             const DeviceInfo& dev) {
  const uint32_t nf = hi - lo + 1;
  if (k.dt != p.dt || nf < 2 || nf > kMaxFused || p.forward) return false;
  if (first && p.opX == 2) return false;                   // input and output in the same layout only
  // groups made of sizes that have matrix-core kernels are left to those
  bool dedicated = true;
  for (uint32_t i = lo; i <= hi; i++) {
    const bool sq = p.P[i] == p.Q[i];
    const bool mfma = sq && (p.P[i] == 16 || (p.dt == DType::F32 && p.mm == MMType::KMM && (p.P[i] == 4 || p.P[i] == 8)));
    if (!mfma) dedicated = false;
  }
  if (dedicated && dev.rulesOfThumb) return false;
  uint32_t ps[kMaxFused], qs[kMaxFused];
  for (uint32_t j = 0; j < nf; j++) { ps[j] = p.P[hi - j]; qs[j] = p.Q[hi - j]; }
  const bool kmm = p.mm == MMType::KMM && p.M > 1;
  // In the KMM layout the plain kernel already runs every factor at about 5 TB/s: fusing pays off only for
  // groups of three or more factors of at most 6 rows (measured against tuned plans).
  if (kmm && dev.rulesOfThumb) {
    if (nf < 3) return false;
    for (uint32_t j = 0; j < nf; j++) if (ps[j] > 6) return false;
  }
  return fusedSmallFits(nf, ps, qs, p.colsBefore(hi), p.M, kmm, p.dt);
}
static hipError_t fusedSmallLaunch(const KernelInfo& k, const StepArgs& a, hipStream_t s) {
  return launchFusedSmall(a, k.dt, s);
}
static bool fusedSmallCheck(const KernelInfo& k, const StepArgs& a) { return fusedSmallSupported(a, k.dt); }

// ---- one factor of any shape up to 256x512 on the matrix cores (zero padded) ----
static bool stepAnyCanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                          const DeviceInfo& dev) {
  if (k.dt != p.dt || lo != hi) return false;
  const uint32_t P = p.P[lo], Q = p.Q[lo];
  if (P > 256 || Q > 512) return false;
  // Small factors are bound by memory on the plain kernel already; the padded tiles pay off from these sizes on
  // (measured per layout and type: e.g. fp32 MKM 18x18, fp64 MKM 12x12, fp32 KMM 31x31, fp64 KMM 20x20).
  const bool kmm = p.mm == MMType::KMM && p.M > 1;
  uint64_t minPQ = kmm ? (p.dt == DType::F32 ? 900 : 400) : (p.dt == DType::F32 ? 256 : 144);
  // a first launch that reads a transposed X: the plain kernel's lanes then run across the strided dimension, and the
  // padded tiles win from 8x8 on (tuned plans: 16x16 chains with op(X) = T 2.6 times faster)
  if (first && p.opX == 2) minPQ = 64;
  // fp64 in the KMM layout with more than 128 rows that do not fill the padded groups of four: the plain kernel is
  // 1.8 times faster (dgekmm 1024 x 129^2 and 200^2; 160^2 the same, 255^2 slower)
  if (dev.rulesOfThumb && kmm && p.dt == DType::F64 && P > 128 && ((P + 3) / 4) % 4 != 0) return false;
  // shrinking factors with 16 rows or more (tuned plans: gemkm 1024 x (16x8)^5 1.4 times faster in both types)
  if (!kmm && P >= 16 && Q < P && minPQ > 128) minPQ = 128;
  return ((uint64_t)P * Q >= minPQ || !dev.rulesOfThumb) && P >= 4;
}
static hipError_t stepAnyLaunch(const KernelInfo& k, const StepArgs& a, hipStream_t s) {
  return launchStepAnyMfma(a, k.dt, s);
}
static bool stepAnyCheck(const KernelInfo& k, const StepArgs& a) { return stepAnyMfmaSupported(a, k.dt); }

void registerGenericKernels(std::vector<KernelInfo>& out) {
  for (DType dt : {DType::F32, DType::F64}) {
    KernelInfo k{};
    k.name = std::string("gekmm_hip_gfx950_512_") + (dt == DType::F32 ? "f" : "d") + "_anyxany_256x512_1_16xany_mfma16x16x4";
    k.dt = dt; k.P = 1; k.Q = 1; k.fused = 1; k.tileM = 0; k.tileK = 0; k.threads = 256; k.variant = 0;
    k.canRun = stepAnyCanRun; k.launch = stepAnyLaunch; k.check = stepAnyCheck;
    out.push_back(k);
  }
  for (DType dt : {DType::F32, DType::F64}) {
    KernelInfo k{};
    k.name = std::string("gekmm_hip_gfx950_512_") + (dt == DType::F32 ? "f" : "d") + "_small_fused_lds_8";
    k.dt = dt; k.P = 1; k.Q = 1; k.fused = kMaxFused; k.tileM = 0; k.tileK = 0; k.threads = 512; k.variant = 0;
    k.canRun = fusedSmallCanRun; k.launch = fusedSmallLaunch; k.check = fusedSmallCheck;
    out.push_back(k);
  }
  for (DType dt : {DType::F32, DType::F64}) {
    KernelInfo k{};
    k.name = std::string("gekmm_hip_gfx950_256_") + (dt == DType::F32 ? "f" : "d") + "_generic_1";
    k.dt = dt; k.P = 0; k.Q = 0; k.fused = 1; k.tileM = 0; k.tileK = 0; k.threads = 256; k.variant = 0;
    k.canRun = genericCanRun; k.launch = genericLaunch; k.check = nullptr;
    out.push_back(k);
  }
}

// ---- whole-row kernel for four fused 16x16 fp32 factors ----
constexpr uint64_t kRow16MinBlocks = 96;
static bool row16CanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                        const DeviceInfo& dev) {
  const uint32_t nf = hi - lo + 1;
  if (p.dt != DType::F32 || p.mm != MMType::MKM || nf < 2 || nf > 4 || p.forward) return false;
  uint64_t kk = 1, rows = 1;
  for (uint32_t i = lo; i <= hi; i++) { if (p.P[i] != 16 || p.Q[i] != 16) return false; kk *= 16; }
  for (uint32_t i = nf; i < 4; i++) rows *= 16;
  if (p.colsBefore(hi) != kk || p.M % rows) return false;   // the group covers whole rows, M a whole number of blocks
  if (first && p.opX == 2) return false;
  // A block is one workgroup's work for about 20 us (256 KB through one CU, 14 us of its matrix pipes): with few
  // blocks the kernels that spread a block over many CUs finish sooner (measured crossover between 64 and 128 blocks).
  // (Shorter chains have no such alternative when their factors differ per batch entry, and go to the wave-per-block
  // kernel anyway when they do not.)
  if (dev.rulesOfThumb && nf == 4 && (uint64_t)p.M * p.batch < kRow16MinBlocks) return false;
  return dev.ldsPerBlock >= 131072 && k.dt == p.dt;
}
static hipError_t row16Launch(const KernelInfo& k, const StepArgs& a, hipStream_t s) {
  return k.threads == 512 ? launchRow16x4W8(a, s) : launchRow16x4(a, s, k.variant == 0);
}
static bool row16Check(const KernelInfo& k, const StepArgs& a) {
  return k.threads == 512 ? row16x4W8Supported(a) : row16x4Supported(a);
}

// ---- whole-row kernel for five fused 8x8 fp32 factors ----
static bool row8CanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                       const DeviceInfo& dev) {
  const uint32_t nf = hi - lo + 1;
  if (p.dt != DType::F32 || p.mm != MMType::MKM || nf < 2 || nf > 5 || p.forward) return false;
  uint64_t kk = 1, rows = 1;
  for (uint32_t i = lo; i <= hi; i++) { if (p.P[i] != 8 || p.Q[i] != 8) return false; kk *= 8; }
  for (uint32_t i = nf; i < 5; i++) rows *= 8;
  if (p.colsBefore(hi) != kk || p.M % rows) return false;
  if (first && p.opX == 2) return false;
  return dev.ldsPerBlock >= 67000 && k.dt == p.dt;
}
static hipError_t row8Launch(const KernelInfo& k, const StepArgs& a, hipStream_t s) { return launchRow8x5(a, s, (int)k.variant); }
static bool row8Check(const KernelInfo&, const StepArgs& a) { return row8x5Supported(a); }

// ---- whole-row kernel for five fused 8x8 fp64 factors ----
// A row is one workgroup's work for about 25 us whatever the number of rows (one workgroup fills a CU); tuned against
// the merged 64x64 products on kernels that spread a row over many CUs it still wins at 32 rows (26.7 us), the
// smallest count measured.
constexpr uint64_t kRow8dMinRows = 32;
static bool row8dCanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                        const DeviceInfo& dev) {
  if (p.dt != DType::F64 || p.mm != MMType::MKM || hi - lo + 1 != 5 || p.forward) return false;
  for (uint32_t i = lo; i <= hi; i++) if (p.P[i] != 8 || p.Q[i] != 8) return false;
  if (p.colsBefore(hi) != 32768) return false;
  if (first && p.opX == 2) return false;
  if (dev.rulesOfThumb && (uint64_t)p.M * p.batch < kRow8dMinRows) return false;
  return dev.ldsPerBlock >= 133120 && k.dt == p.dt;
}
static hipError_t row8dLaunch(const KernelInfo&, const StepArgs& a, hipStream_t s) { return launchRow8x5F64(a, s); }
static bool row8dCheck(const KernelInfo&, const StepArgs& a) { return row8x5F64Supported(a); }

// ---- wave-per-block kernel for two or three fused PxP factors, 9 <= P <= 16 ----
static bool row16x3CanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                          const DeviceInfo&) {
  const uint32_t nf = hi - lo + 1;
  if (p.dt != k.dt || p.mm != MMType::MKM || nf < 2 || nf > 3 || p.forward) return false;
  const uint32_t P = p.P[hi];
  if (P < 9 || P > 16) return false;
  uint64_t kk = 1;
  for (uint32_t i = lo; i <= hi; i++) {
    if (p.P[i] != P || p.Q[i] != P) return false;
    if (p.batch > 1 && p.strideF[i] != 0) return false;     // the factors are staged once per workgroup
    kk *= P;
  }
  if (p.colsBefore(hi) != kk || (nf == 2 && p.M % P)) return false;
  return !(first && p.opX == 2);
}
static hipError_t row16x3Launch(const KernelInfo& k, const StepArgs& a, hipStream_t s) { return launchRow16x3(a, k.dt, s); }
static bool row16x3Check(const KernelInfo& k, const StepArgs& a) { return row16x3Supported(a, k.dt); }

// ---- whole-row kernel for three fused 32x16 fp32 factors ----
static bool row32CanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                        const DeviceInfo&) {
  if (p.dt != DType::F32 || p.mm != MMType::MKM || hi - lo + 1 != 3 || p.forward) return false;
  for (uint32_t i = lo; i <= hi; i++) if (p.P[i] != 32 || p.Q[i] != 16) return false;
  if (p.colsBefore(hi) != 32768) return false;
  if (first && p.opX == 2) return false;
  return k.dt == p.dt;
}
static hipError_t row32Launch(const KernelInfo&, const StepArgs& a, hipStream_t s) { return launchRow32x16x3(a, s); }
static bool row32Check(const KernelInfo&, const StepArgs& a) { return row32x16x3Supported(a); }

// ---- whole-row kernel for three fused 32x32 fp32 factors ----
constexpr uint64_t kRow32MinRows = 96;
static bool row32x3CanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                          const DeviceInfo& dev) {
  if (p.dt != DType::F32 || p.mm != MMType::MKM || hi - lo + 1 != 3 || p.forward) return false;
  for (uint32_t i = lo; i <= hi; i++) if (p.P[i] != 32 || p.Q[i] != 32) return false;
  if (p.colsBefore(hi) != 32768) return false;
  if (first && p.opX == 2) return false;
  // a row is one workgroup's work for about 17 us: with few rows the pair kernel (a wave per 1024-column block) plus
  // one step across the blocks finishes sooner (measured crossover between 64 and 128 rows)
  if (dev.rulesOfThumb && (uint64_t)p.M * p.batch < kRow32MinRows) return false;
  // the persistent form (four quarter buffers in LDS) from three rows per CU on; with fewer the two workgroups of a CU
  // that start together are faster (768 rows 57.8 against 59.6 us, 512 rows 44.0 against 39.2)
  if (k.threads == 1024 && (dev.ldsPerBlock < 143360 || (dev.rulesOfThumb && (uint64_t)p.M * p.batch < 3ull * dev.cus))) return false;
  return k.dt == p.dt;
}
static hipError_t row32x3Launch(const KernelInfo& k, const StepArgs& a, hipStream_t s) {
  return k.threads == 1024 ? launchRow32x3p(a, s) : launchRow32x3(a, s);
}
static bool row32x3Check(const KernelInfo& k, const StepArgs& a) { return k.threads == 1024 ? row32x3pSupported(a) : row32x3Supported(a); }

// ---- single-factor fp32 step for 64x64 and 128x128, whole-line accesses through LDS (variant 3: MKM, 4: KMM) ----
static bool stepWideCanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                           const DeviceInfo&) {
  const MMType mm = ((k.variant & 255) == 4) ? MMType::KMM : MMType::MKM;
  if (p.dt != k.dt || p.mm != mm || lo != hi) return false;
  if (p.P[lo] != k.P || p.Q[lo] != k.Q) return false;
  if (first && p.opX == 2) return false;
  // whole tiles of 16 KB of input: slices of a row (MKM), columns of a slice (KMM)
  const uint64_t TS = 16384 / dtypeSize(k.dt) / k.P;
  return mm == MMType::KMM ? p.M % TS == 0 : (p.colsBefore(hi) / k.P) % TS == 0;
}
static hipError_t stepWideLaunch(const KernelInfo& k, const StepArgs& a, hipStream_t s) { return launchStepWide(a, k.dt, s, (int)(k.variant >> 8)); }
static bool stepWideCheck(const KernelInfo& k, const StepArgs& a) { return stepWideSupported(a, k.dt); }

// ---- single-factor MFMA step (fp64 and fp32) ----
static bool stepF64CanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                          const DeviceInfo& dev) {
  const MMType mm = (k.variant == 1) ? MMType::KMM : MMType::MKM;
  if (p.dt != k.dt || p.mm != mm || lo != hi) return false;
  if (p.P[lo] != k.P || p.Q[lo] != k.Q) return false;
  if (first && p.opX == 2) return false;

  (void)dev;
  return true;
}
static hipError_t stepF64Launch(const KernelInfo& k, const StepArgs& a, hipStream_t s) { return launchStepMfma(a, k.dt, s); }
static bool stepF64Check(const KernelInfo& k, const StepArgs& a) { return stepMfmaSupported(a, k.dt); }

// ---- two fused square factors covering whole rows ----
static bool pairCanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                       const DeviceInfo& dev) {
  if (p.dt != k.dt || p.mm != MMType::MKM || hi - lo + 1 != 2 || p.forward) return false;
  if (k.P != k.Q) {
    // two rectangular factors of exactly the kernel's shape (32x64, 64x32): rows of P*P elements become Q*Q
    for (uint32_t i = lo; i <= hi; i++) if (p.P[i] != k.P || p.Q[i] != k.Q) return false;
    if (p.colsBefore(hi) != (uint64_t)k.P * k.P) return false;
    return !(first && p.opX == 2) && dev.ldsPerBlock >= (int)(2 * k.P * k.Q * 8 + 4 * 16 * (k.P + 4) * 8);   // factors and the waves' stages
  }
  // the 32x32 kernel also takes factors of 17x17 ... 31x31, zero-padded to its tile
  const uint32_t P = p.P[hi];
  if (!(P == k.P || (k.P == 32 && P >= 17 && P < 32))) return false;
  for (uint32_t i = lo; i <= hi; i++) if (p.P[i] != P || p.Q[i] != P) return false;
  if (p.colsBefore(hi) != (uint64_t)P * P) return false;
  if (first && p.opX == 2) return false;
  // one wave per 64x64 block: with few blocks two single-factor launches, whose tiles are 16 times smaller, fill the
  // device better (tuned plans at 256 blocks: 1.4 times faster in fp32, 1.9 times in fp64; at 1024 blocks the pair wins)
  // fp64, a block per wave and two waves per SIMD: from 8 blocks per CU on; with up to 4 per CU two or four waves share a
  // block and the pair wins again (1024 blocks: 25.8 against 31 us, 512: 17.3 against 22.4, 320: 16.2 against 18.1; at
  // 256 blocks two single steps on tiles passed through LDS take 14.9 us and the pair does not beat them; between 4 and
  // 8 blocks per CU a wave's chain of one whole block, 35 us, loses to them too)
  if (dev.rulesOfThumb && P == 64) {
    const uint64_t blocks = (uint64_t)p.M * p.batch, cus = (uint64_t)dev.cus;
    if (p.dt == DType::F64 ? (4 * blocks < 5 * cus || (blocks > 4 * cus && blocks < 8 * cus)) : blocks < 2 * cus) return false;
  }
  return dev.ldsPerBlock >= (int)(2 * k.P * k.P * 8 + 8 * 8192);
}
static hipError_t pairLaunch(const KernelInfo& k, const StepArgs& a, hipStream_t s) { return launchPairMfma(a, k.dt, s); }
static bool pairCheck(const KernelInfo& k, const StepArgs& a) { return pairMfmaSupported(a, k.dt); }

// ---- KMM-layout step with a 64x64 fp64 factor ----
static bool kmm64CanRun(const KernelInfo&, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                        const DeviceInfo& dev) {
  if (p.dt != DType::F64 || p.mm != MMType::KMM || lo != hi || p.P[lo] != 64 || p.Q[lo] != 64) return false;
  if (first && p.opX == 2) return false;
  // made for the leading factors of long MKM chains (many batch entries of 4096 contiguous columns); a KMM problem
  // proper, one entry of a few hundred columns, runs 1.1 to 1.8 times faster on the tiles passed through LDS
  // (up to 1 GB of X; at 2 GB this kernel is 4 % ahead again)
  if (dev.rulesOfThumb && p.batch < 8 && (uint64_t)p.M * p.K() < (1ull << 27)) return false;
  return p.M % 64 == 0;
}
static hipError_t kmm64Launch(const KernelInfo&, const StepArgs& a, hipStream_t s) { return launchKmm64F64(a, s); }
static bool kmm64Check(const KernelInfo&, const StepArgs& a) { return kmm64F64Supported(a); }

// ---- KMM layout: two fused 16x16 factors ----
static bool kmm16x2CanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                          const DeviceInfo&) {
  if (p.dt != k.dt || p.mm != MMType::KMM || p.M < 2 || hi - lo + 1 != 2 || p.forward) return false;
  const uint32_t P = p.P[hi];
  if (P < 9 || P > 16) return false;                       // 9 ... 15: zero-padded to the 16x16 tile
  for (uint32_t i = lo; i <= hi; i++) if (p.P[i] != P || p.Q[i] != P) return false;
  return !(first && p.opX == 2);
}
static hipError_t kmm16x2Launch(const KernelInfo& k, const StepArgs& a, hipStream_t s) { return launchKmm16x2(a, k.dt, s); }
static bool kmm16x2Check(const KernelInfo& k, const StepArgs& a) { return kmm16x2Supported(a, k.dt); }

// ---- KMM layout: six fused 4x4 fp32 factors covering all 4096 rows ----
static bool kmm4x6CanRun(const KernelInfo&, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                         const DeviceInfo& dev) {
  if (p.dt != DType::F32 || p.mm != MMType::KMM || hi - lo + 1 != 6 || p.forward) return false;
  for (uint32_t i = lo; i <= hi; i++) if (p.P[i] != 4 || p.Q[i] != 4) return false;
  if (p.colsBefore(hi) != 4096 || p.M % 8) return false;
  if (first && p.opX == 2) return false;
  // Only while all column tiles are resident at once (one per CU): the tiles of an XCD then walk the rows of X
  // together and their 32-byte pieces meet in its L2.  With more tiles than CUs that order is lost and the
  // two-launch plan, which reads 256 bytes per row and wave, is faster (measured from M = 4096 on).
  if (dev.rulesOfThumb && (uint64_t)(p.M / 8) * p.batch > (uint64_t)dev.cus) return false;
  // With fewer than 128 tiles half of the CUs or more stand idle and the two-launch plan is ahead (tuned: 512 columns
  // 20.0 against 17.1 us; 1024 columns 23.4 against 23.3).
  if (dev.rulesOfThumb && (uint64_t)(p.M / 8) * p.batch < 128) return false;
  return dev.ldsPerBlock >= (8 * 64 * 65 + 32) * 4;
}
// The two-phase form: M a multiple of 256.  By rule only from 2048 columns on (one column block per XCD), where it
// is 1.4 times faster than the whole-column kernel; with fewer columns part of the XCDs would work on blocks whose
// intermediate lives in another XCD's L2.
static bool kmm4x6TwoPhaseCanRun(const KernelInfo&, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                                 const DeviceInfo& dev) {
  if (p.dt != DType::F32 || p.mm != MMType::KMM || hi - lo + 1 != 6 || p.forward) return false;
  for (uint32_t i = lo; i <= hi; i++) if (p.P[i] != 4 || p.Q[i] != 4) return false;
  if (p.colsBefore(hi) != 4096 || p.M % 256) return false;
  if (first && p.opX == 2) return false;
  if ((uint64_t)(p.M / 256) * p.batch > 248) return false;          // counters per column block in a 4 KB area
  if (!dev.xcdRoundRobin) return false;                              // its blocks synchronise through one XCD's L2
  if (dev.rulesOfThumb && (p.M % 2048 || dev.cus < 256)) return false;
  return true;
}
static hipError_t kmm4x6TwoPhaseLaunch(const KernelInfo&, const StepArgs& a, hipStream_t s) { return launchKmm4x6TwoPhase(a, s); }
static bool kmm4x6TwoPhaseCheck(const KernelInfo&, const StepArgs& a) { return kmm4x6TwoPhaseSupported(a); }
static hipError_t kmm4x6Launch(const KernelInfo&, const StepArgs& a, hipStream_t s) { return launchKmm4x6(a, s); }
static bool kmm4x6Check(const KernelInfo&, const StepArgs& a) { return kmm4x6Supported(a); }

// ---- KMM-layout register kernel: NF fused PxP fp32 factors with P^NF = 64 ----
static bool kmmRegCanRun(const KernelInfo& k, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                         const DeviceInfo& dev) {
  if (p.dt != DType::F32 || p.mm != MMType::KMM || hi - lo + 1 != k.fused || p.forward) return false;
  for (uint32_t i = lo; i <= hi; i++) if (p.P[i] != k.P || p.Q[i] != k.Q) return false;
  if (first && p.opX == 2) return false;
  // lanes run along M: with 16 columns a quarter of each wave works, and one plain launch per factor is 1.3 times
  // faster than half as many launches here (sgekmm 16 x 8^8; three fused factors still pay)
  if (dev.rulesOfThumb && p.M < 32 && k.fused <= 2) return false;
  return p.colsBefore(hi) % k.tileK == 0 && p.M >= 16;
}
static hipError_t kmmRegLaunch(const KernelInfo&, const StepArgs& a, hipStream_t s) { return launchKmmReg(a, s); }

// ---- KMM layout: three fused 8x8 fp32 factors, 512 rows by 64 columns per workgroup ----
static bool kmm8x3CanRun(const KernelInfo&, const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool,
                         const DeviceInfo&) {
  if (p.dt != DType::F32 || p.mm != MMType::KMM || hi - lo + 1 != 3 || p.forward) return false;
  for (uint32_t i = lo; i <= hi; i++) if (p.P[i] != 8 || p.Q[i] != 8) return false;
  if (first && p.opX == 2) return false;
  return p.colsBefore(hi) % 512 == 0 && p.M % 64 == 0;
}
static hipError_t kmm8x3Launch(const KernelInfo&, const StepArgs& a, hipStream_t s) { return launchKmm8x3(a, s); }
static bool kmm8x3Check(const KernelInfo&, const StepArgs& a) { return kmm8x3Supported(a); }
static bool kmmRegCheck(const KernelInfo&, const StepArgs& a) { return kmmRegSupported(a); }

void registerRowKernels(std::vector<KernelInfo>& out) {
  // grammar: <mm>_<backend>_<arch>_<threads>_<type>_<PxQ>_<TilePxTileQ>_<fused>_<TileMxTileK>_<regs>_<ops>_<batch>_<p2p>_<opt>
  // two or three 16x16 factors: one wave per 4096-element block (measured faster than the workgroup kernel below on
  // three factors, 4.6 against 4.1 TB/s in fp32, and free of its row-count conditions); 9x9 ... 15x15 zero-padded
  for (DType dt : {DType::F64, DType::F32}) {
    KernelInfo kd3{};
    kd3.name = std::string("mkm_hip_gfx950_256_") + (dt == DType::F64 ? "d" : "f") +
               "_16x16_16x16_3_1x4096_mfma16x16x4_NN_strided_0_3";      // also 9x9 ... 15x15, padded to this tile
    kd3.dt = dt; kd3.P = 16; kd3.Q = 16; kd3.fused = 3; kd3.tileM = 1; kd3.tileK = 4096; kd3.threads = 256;
    kd3.variant = 0; kd3.canRun = row16x3CanRun; kd3.launch = row16x3Launch; kd3.check = row16x3Check;
    out.push_back(kd3);
  }

  // two builds of the 16x16 whole-block kernel: 16 waves (preferred online), 8 waves with the whole next block
  // prefetched (a candidate for the tuner)
  for (uint32_t threads : {1024u, 512u}) {
    KernelInfo k{};
    k.name = "mkm_hip_gfx950_" + std::to_string(threads) + "_f_16x16_16x16_4_1x65536_mfma16x16x4_NN_strided_0_3";
    k.dt = DType::F32; k.P = 16; k.Q = 16; k.fused = 4; k.tileM = 1; k.tileK = 65536; k.threads = threads; k.variant = 0;
    k.canRun = row16CanRun; k.launch = row16Launch; k.check = row16Check;
    out.push_back(k);
    if (threads == 1024) {
      // for the tuner: all workgroups started at once ("ns" in the tile field) instead of in groups
      KernelInfo v = k;
      v.name = "mkm_hip_gfx950_1024_f_16x16_16x16_4_1x65536ns_mfma16x16x4_NN_strided_0_3";
      v.variant = 1; v.tunerOnly = true;
      out.push_back(v);
    }
  }

  KernelInfo k8{};
  k8.name = "mkm_hip_gfx950_512_f_8x8_8x8_5_1x32768_mfma4x4x1_NN_strided_0_3";
  k8.dt = DType::F32; k8.P = 8; k8.Q = 8; k8.fused = 5; k8.tileM = 1; k8.tileK = 32768; k8.threads = 512; k8.variant = 0;
  k8.canRun = row8CanRun; k8.launch = row8Launch; k8.check = row8Check;
  out.push_back(k8);
  // the same kernel under other schedules, for the tuner: one workgroup per CU ("wg1"), two without the start delay
  // of the later one ("wg2nd"); the tile field of the name carries the schedule
  for (uint32_t schedule : {1u, 2u}) {
    KernelInfo v = k8;
    v.name = std::string("mkm_hip_gfx950_512_f_8x8_8x8_5_1x32768") + (schedule == 1 ? "wg1" : "wg2nd") + "_mfma4x4x1_NN_strided_0_3";
    v.variant = schedule; v.tunerOnly = true;
    out.push_back(v);
  }

  KernelInfo k8d{};
  k8d.name = "mkm_hip_gfx950_512_d_8x8_8x8_5_1x32768_valu_NN_strided_0_3";
  k8d.dt = DType::F64; k8d.P = 8; k8d.Q = 8; k8d.fused = 5; k8d.tileM = 1; k8d.tileK = 32768; k8d.threads = 512; k8d.variant = 0;
  k8d.canRun = row8dCanRun; k8d.launch = row8dLaunch; k8d.check = row8dCheck;
  out.push_back(k8d);

  KernelInfo k32{};
  k32.name = "mkm_hip_gfx950_512_f_32x16_32x16_3_1x32768_mfma16x16x4_NN_strided_0_3";
  k32.dt = DType::F32; k32.P = 32; k32.Q = 16; k32.fused = 3; k32.tileM = 1; k32.tileK = 32768; k32.threads = 512;
  k32.variant = 0; k32.canRun = row32CanRun; k32.launch = row32Launch; k32.check = row32Check;
  out.push_back(k32);

  {
    // ahead of the kernel with two workgroups of 8 waves per CU: chosen first where both apply
    KernelInfo kp{};
    kp.name = "mkm_hip_gfx950_1024_f_32x32_32x32_3_1x32768_mfma16x16x4_NN_strided_0_3";
    kp.dt = DType::F32; kp.P = 32; kp.Q = 32; kp.fused = 3; kp.tileM = 1; kp.tileK = 32768; kp.threads = 1024;
    kp.variant = 0; kp.canRun = row32x3CanRun; kp.launch = row32x3Launch; kp.check = row32x3Check;
    out.push_back(kp);
  }
  KernelInfo k323{};
  k323.name = "mkm_hip_gfx950_512_f_32x32_32x32_3_1x32768_mfma16x16x4_NN_strided_0_3";
  k323.dt = DType::F32; k323.P = 32; k323.Q = 32; k323.fused = 3; k323.tileM = 1; k323.tileK = 32768; k323.threads = 512;
  k323.variant = 0; k323.canRun = row32x3CanRun; k323.launch = row32x3Launch; k323.check = row32x3Check;
  out.push_back(k323);

  for (DType dt : {DType::F32, DType::F64}) {
    KernelInfo k2{};
    k2.name = std::string("kmm_hip_gfx950_256_") + (dt == DType::F32 ? "f" : "d") +
              "_16x16_16x16_2_16x256_mfma16x16x4_NN_strided_0_3";
    k2.dt = dt; k2.P = 16; k2.Q = 16; k2.fused = 2; k2.tileM = 16; k2.tileK = 256; k2.threads = 256; k2.variant = 0;
    k2.canRun = kmm16x2CanRun; k2.launch = kmm16x2Launch; k2.check = kmm16x2Check;
    out.push_back(k2);
  }

  {
    // ahead of the whole-column kernel: chosen first where both apply
    KernelInfo k6{};
    k6.name = "kmm_hip_gfx950_256_f_4x4_4x4_6_256x4096_mfma4x4x1_NN_strided_0_3";
    k6.dt = DType::F32; k6.P = 4; k6.Q = 4; k6.fused = 6; k6.tileM = 256; k6.tileK = 4096; k6.threads = 256; k6.variant = 0;
    k6.canRun = kmm4x6TwoPhaseCanRun; k6.launch = kmm4x6TwoPhaseLaunch; k6.check = kmm4x6TwoPhaseCheck;
    k6.usesSync = true;
    out.push_back(k6);
  }
  {
    KernelInfo k6{};
    k6.name = "kmm_hip_gfx950_512_f_4x4_4x4_6_8x4096_mfma4x4x1_NN_strided_0_3";
    k6.dt = DType::F32; k6.P = 4; k6.Q = 4; k6.fused = 6; k6.tileM = 8; k6.tileK = 4096; k6.threads = 512; k6.variant = 0;
    k6.canRun = kmm4x6CanRun; k6.launch = kmm4x6Launch; k6.check = kmm4x6Check;
    out.push_back(k6);
  }

  {
    KernelInfo k3{};
    k3.name = "kmm_hip_gfx950_512_f_8x8_8x8_3_64x512_mfma4x4x1_NN_strided_0_3";
    k3.dt = DType::F32; k3.P = 8; k3.Q = 8; k3.fused = 3; k3.tileM = 64; k3.tileK = 512; k3.threads = 512; k3.variant = 0;
    k3.canRun = kmm8x3CanRun; k3.launch = kmm8x3Launch; k3.check = kmm8x3Check;
    out.push_back(k3);
  }

  // deepest fusion first: the online selection takes the first kernel that fits at a given depth
  // (online, single 4x4 / 8x8 / 16x16 factors are left to the plain kernel, which is faster in this layout on large
  // problems: lanes along M, about 5 TB/s per launch against 2.5 for the one-factor register kernel)
  for (auto pn : {std::pair<uint32_t, uint32_t>{4, 3}, {8, 2}, {4, 2}, {4, 1}, {8, 1}, {16, 1}}) {
    KernelInfo kk{};
    const std::string ps = std::to_string(pn.first);
    uint32_t G = 1;
    for (uint32_t i = 0; i < pn.second; i++) G *= pn.first;
    kk.fused = pn.second;
    kk.name = "kmm_hip_gfx950_256_f_" + ps + "x" + ps + "_" + ps + "x" + ps + "_" + std::to_string(kk.fused) +
              "_64x" + std::to_string(G) + "_mfma4x4x1_NN_strided_0_3";
    kk.dt = DType::F32; kk.P = pn.first; kk.Q = pn.first; kk.tileM = 64; kk.tileK = G; kk.threads = 256; kk.variant = 0;
    kk.canRun = kmmRegCanRun; kk.launch = kmmRegLaunch; kk.check = kmmRegCheck;
    kk.tunerOnly = (pn.second == 1);
    out.push_back(kk);
  }

  for (DType dt : {DType::F64, DType::F32})
  for (uint32_t P : {64u, 32u}) {
    KernelInfo kp{};
    const std::string ps = std::to_string(P);
    const bool f64 = dt == DType::F64;
    kp.name = std::string("mkm_hip_gfx950_") + (f64 && P == 64 ? "512" : "256") + (f64 ? "_d_" : "_f_") + ps + "x" + ps + "_" +
              ps + "x" + ps + "_2_1x" + std::to_string(P * P) + (f64 && P == 64 ? "_mfma4x4x4" : "_mfma16x16x4") +
              "_NN_strided_0_3";
    kp.dt = dt; kp.P = P; kp.Q = P; kp.fused = 2; kp.tileM = 1; kp.tileK = P * P; kp.threads = (f64 && P == 64) ? 512 : 256;
    kp.variant = 0;
    kp.canRun = pairCanRun; kp.launch = pairLaunch; kp.check = pairCheck;
    out.push_back(kp);
  }

  // rectangular pairs on exact tiles (fp64 only 32x64: see pair_mfma.hip)
  for (DType dt : {DType::F32, DType::F64})
  for (auto pq : {std::pair<uint32_t, uint32_t>{32, 64}, {64, 32}}) {
    if (dt == DType::F64 && pq.first == 64) continue;
    KernelInfo kp{};
    const std::string ps = std::to_string(pq.first) + "x" + std::to_string(pq.second);
    kp.name = std::string("mkm_hip_gfx950_256") + (dt == DType::F64 ? "_d_" : "_f_") + ps + "_" + ps + "_2_1x" +
              std::to_string(pq.first * pq.first) + "_mfma16x16x4_NN_strided_0_3";
    kp.dt = dt; kp.P = pq.first; kp.Q = pq.second; kp.fused = 2; kp.tileM = 1; kp.tileK = pq.first * pq.first; kp.threads = 256;
    kp.variant = 0;
    kp.canRun = pairCanRun; kp.launch = pairLaunch; kp.check = pairCheck;
    out.push_back(kp);
  }

  {
    KernelInfo kk{};
    kk.name = "kmm_hip_gfx950_256_d_64x64_64x64_1_64x64_mfma4x4x4_NN_strided_0_3";
    kk.dt = DType::F64; kk.P = 64; kk.Q = 64; kk.fused = 1; kk.tileM = 64; kk.tileK = 64; kk.threads = 256; kk.variant = 2;
    kk.canRun = kmm64CanRun; kk.launch = kmm64Launch; kk.check = kmm64Check;
    out.push_back(kk);
  }

  for (uint32_t variant : {3u, 4u})
  for (DType dt : {DType::F32, DType::F64})
  for (uint32_t P : {32u, 64u, 128u}) {
    KernelInfo kw{};
    const uint32_t E = 16384 / (uint32_t)dtypeSize(dt);
    const std::string ps = std::to_string(P), ts = std::to_string(E / P);
    kw.name = std::string(variant == 4 ? "kmm" : "mkm") + "_hip_gfx950_256_" + (dt == DType::F32 ? "f_" : "d_") + ps + "x" + ps +
              "_" + ps + "x" + ps + "_1_" + (variant == 4 ? ts + "x" + ps : "1x" + std::to_string(E)) + "_mfma16x16x4lds_NN_strided_0_3";
    kw.dt = dt; kw.P = P; kw.Q = P; kw.fused = 1; kw.tileM = variant == 4 ? E / P : 1;
    kw.tileK = variant == 4 ? P : E; kw.threads = 256; kw.variant = variant;
    kw.canRun = stepWideCanRun; kw.launch = stepWideLaunch; kw.check = stepWideCheck;
    out.push_back(kw);
    // for the tuner: the same kernel with at most one / two persistent workgroups per CU ("wg1", "wg2" in the tile field)
    for (uint32_t cap : {1u, 2u}) {
      KernelInfo v = kw;
      const size_t at = v.name.find("_mfma16x16x4lds");
      v.name.insert(at, "wg" + std::to_string(cap));
      v.variant = variant | (cap << 8); v.tunerOnly = true;
      out.push_back(v);
    }
  }

  // variant 1 = the same kernel on the KMM layout (tiles of 16 consecutive m)
  for (uint32_t variant : {0u, 1u})
  for (DType dt : {DType::F64, DType::F32})
  for (uint32_t P : {16u, 32u, 64u, 128u}) {
    KernelInfo kd{};
    const std::string ps = std::to_string(P);
    kd.name = std::string(variant ? "kmm" : "mkm") + "_hip_gfx950_256_" + (dt == DType::F64 ? "d_" : "f_") + ps + "x" + ps +
              "_" + ps + "x" + ps + "_1_" + (variant ? "16x" + ps : "1x" + std::to_string(16 * P)) +
              "_mfma16x16x4_NN_strided_0_3";
    kd.dt = dt; kd.P = P; kd.Q = P; kd.fused = 1; kd.tileM = variant ? 16 : 1; kd.tileK = variant ? P : 16 * P;
    kd.threads = 256; kd.variant = variant;
    kd.canRun = stepF64CanRun; kd.launch = stepF64Launch; kd.check = stepF64Check;
    // fp32 16x16 in the KMM layout: the plain kernel's 256-byte accesses along M beat the 64-byte tile rows
    // and for 128x128 the padded step (factor in LDS instead of split over wave tasks) is a third faster
    // ... fp32 64x64 in that layout likewise (1.15 times), 16x16 in either type, and fp64 128x128 in both layouts (the
    // padded step with the factor in LDS is 1.5 times faster than the factor split over eight wave tasks): all measured
    // by tuning the reference's published shape table
    kd.tunerOnly = (variant == 1 && P == 16) || (variant == 1 && dt == DType::F32 && (P == 64 || P == 128)) ||
                   (dt == DType::F64 && P == 128);
    out.push_back(kd);
  }
}

KernelDB::KernelDB() {
  registerRowKernels(kernels_);
  registerGenericKernels(kernels_);
}

int KernelDB::findByName(const std::string& name) const {
  for (size_t i = 0; i < kernels_.size(); i++) if (kernels_[i].name == name) return (int)i;
  return -1;
}

int KernelDB::genericKernel(DType dt) const {
  for (size_t i = 0; i < kernels_.size(); i++)
    if (kernels_[i].P == 0 && kernels_[i].dt == dt) return (int)i;
  return -1;
}

std::vector<int> KernelDB::candidates(const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool last,
                                      const DeviceInfo& dev) const {
  std::vector<int> r;
  for (size_t i = 0; i < kernels_.size(); i++)
    if (kernels_[i].canRun(kernels_[i], p, lo, hi, first, last, dev)) r.push_back((int)i);
  return r;
}

Plan KernelDB::selectOnline(const KronProblem& p, const DeviceInfo& dev, bool allowFusion,
                            const std::vector<int>* excluded) const {
  auto barred = [&](int k) {
    if (excluded) for (int x : *excluded) if (x == k) return true;
    return false;
  };
  Plan plan;
  int hi = (int)p.N - 1;
  while (hi >= 0) {
    int bestLo = hi, bestK = genericKernel(p.dt);
    {
      const uint32_t maxDepth = (allowFusion && !p.forward) ? kMaxFused : 1;   // forward keeps every step's output
      for (int lo = (hi + 1 >= (int)maxDepth) ? hi + 1 - (int)maxDepth : 0; lo <= hi; lo++) {
        auto c = candidates(p, (uint32_t)lo, (uint32_t)hi, hi == (int)p.N - 1, lo == 0, dev);
        int pick = -1;
        for (int k : c) if (kernels_[k].P != 0 && !kernels_[k].tunerOnly && !barred(k)) { pick = k; break; }   // first registered = preferred
        if (pick >= 0) { bestLo = lo; bestK = pick; break; }           // deepest fusion wins
      }
      // The LDS-fused kernel taken as deep as it goes can leave one or two factors, which then run one plain launch
      // each (or a shallow group): two groups of about equal depth are faster (tuned plans: sgemkm 1024 x (2x4)^7 as
      // 4 + 3 instead of 6 + 1: 1.34 times, sgekmm 1024 x 3^7 as 4 + 3 instead of 5 + 1 + 1: 1.3 times).
      const int total = hi + 1, depth = hi - bestLo + 1;
      if (kernels_[bestK].canRun == fusedSmallCanRun && bestLo > 0 && bestLo < depth - 1 && total <= 2 * (int)maxDepth) {
        auto fusedPick = [&](int lo, int h) {
          for (int k : candidates(p, (uint32_t)lo, (uint32_t)h, h == (int)p.N - 1, lo == 0, dev))
            if (kernels_[k].P != 0 && !kernels_[k].tunerOnly && !barred(k)) return kernels_[k].canRun == fusedSmallCanRun ? k : -1;
          return -1;
        };
        const int lo2 = hi + 1 - (total + 1) / 2;
        const int upper = fusedPick(lo2, hi);
        if (upper >= 0 && fusedPick(0, lo2 - 1) >= 0) { bestLo = lo2; bestK = upper; }
      }
    }
    plan.push_back(PlanStep{(uint32_t)bestLo, (uint32_t)hi, bestK});
    hi = bestLo - 1;
  }
  return plan;
}

bool KernelDB::validPlan(const KronProblem& p, const Plan& plan, const DeviceInfo& dev) const {
  if (plan.empty() || p.N == 0) return false;
  int64_t expectHi = (int64_t)p.N - 1;
  for (size_t l = 0; l < plan.size(); l++) {
    const PlanStep& s = plan[l];
    if (s.kernel < 0 || (size_t)s.kernel >= kernels_.size()) return false;
    if ((int64_t)s.hi != expectHi || s.lo > s.hi || s.hi - s.lo + 1 > kMaxFused) return false;
    const KernelInfo& k = kernels_[s.kernel];
    DeviceInfo able = dev;
    able.rulesOfThumb = false;
    if (!k.canRun(k, p, s.lo, s.hi, l == 0, s.lo == 0, able)) return false;
    expectHi = (int64_t)s.lo - 1;
  }
  return expectHi == -1;
}

bool KernelDB::lookupTuned(const std::string& key, Plan* plan, int* merge, uint32_t* split, int* transposeX) const {
  auto it = tuned_.find(key);
  if (it == tuned_.end()) return false;
  if (merge) *merge = it->second.merge;
  if (split) *split = it->second.split;
  if (transposeX) *transposeX = it->second.transposeX;
  Plan pl;
  for (auto& s : it->second.steps) {
    int k = findByName(s.second);
    if (k < 0) return false;
    pl.push_back(PlanStep{s.first.first, s.first.second, k});
  }
  *plan = pl;
  return true;
}

void KernelDB::storeTuned(const std::string& key, const Plan& plan, float ms, int merge, uint32_t split, int transposeX) {
  Tuned t;
  t.ms = ms; t.merge = merge; t.split = split; t.transposeX = transposeX;
  for (auto& s : plan) t.steps.push_back({{s.lo, s.hi}, kernels_[s.kernel].name});
  tuned_[key] = t;
}

// File format, one problem per line:
//   <problem string> <ms> [M<merge> S<split> [X<transposeX>]] <nsteps> {<lo> <hi> <kernel name>}...
// (lines without the M / S fields leave both to the online selection)
bool KernelDB::loadFile(const std::string& path, bool shipped) {
  std::ifstream f(path);
  if (!f) return false;
  std::string line;
  while (std::getline(f, line)) {
    if (line.empty() || line[0] == '#') continue;
    std::istringstream is(line);
    std::string key, tok; float ms; size_t n = 0;
    if (!(is >> key >> ms >> tok)) continue;
    Tuned t; t.ms = ms; t.shipped = shipped;
    if (!tok.empty() && tok[0] == 'M') {
      std::string stok, ntok;
      if (!(is >> stok >> ntok) || stok.empty() || stok[0] != 'S') continue;
      t.merge = atoi(tok.c_str() + 1) ? 1 : 0;
      t.split = (uint32_t)strtoul(stok.c_str() + 1, nullptr, 10);
      if (!ntok.empty() && ntok[0] == 'X') {
        t.transposeX = atoi(ntok.c_str() + 1) ? 1 : 0;
        if (!(is >> ntok)) continue;
      }
      char* end = nullptr;
      n = strtoul(ntok.c_str(), &end, 10);
      if (end == ntok.c_str() || *end) continue;
    } else {
      char* end = nullptr;
      n = strtoul(tok.c_str(), &end, 10);
      if (end == tok.c_str() || *end) continue;
    }
    if (n == 0 || n > kMaxFactors) continue;
    bool ok = true;
    for (size_t i = 0; i < n; i++) {
      uint32_t lo, hi; std::string name;
      if (!(is >> lo >> hi >> name)) { ok = false; break; }
      t.steps.push_back({{lo, hi}, name});
    }
    if (ok) tuned_[key] = t;
  }
  return true;
}

bool KernelDB::saveFile(const std::string& path) const {
  std::ofstream f(path);
  if (!f) return false;
  f << "# fastkron gfx950 tuned launch plans: problem ms nsteps {lo hi kernel}\n";
  for (auto& kv : tuned_) {
    if (kv.second.shipped) continue;       // the library's own records stay in its own file
    f << kv.first << " " << kv.second.ms;
    if (kv.second.merge >= 0) {
      f << " M" << kv.second.merge << " S" << kv.second.split;
      if (kv.second.transposeX) f << " X1";
    }
    f << " " << kv.second.steps.size();
    for (auto& s : kv.second.steps) f << " " << s.first.first << " " << s.first.second << " " << s.second;
    f << "\n";
  }
  return (bool)f;
}

std::string KernelDB::defaultPath() {
  if (const char* e = getenv("FASTKRON_TUNED_DB")) return e;
  return "";
}

// The plans tuned on an MI355X that ship with the library: gfx950_plans.txt in the directory above the one that
// holds libFastKron.so (found through the address of this function).  FASTKRON_SHIPPED_PLANS=0 switches them off.
std::string KernelDB::shippedPath() {
  const char* e = getenv("FASTKRON_SHIPPED_PLANS");
  if (e && !strcmp(e, "0")) return "";
  Dl_info info;
  if (!dladdr((const void*)&KernelDB::shippedPath, &info) || !info.dli_fname) return "";
  std::string lib = info.dli_fname;
  const size_t slash = lib.rfind('/');
  if (slash == std::string::npos) return "";
  return lib.substr(0, slash) + "/../gfx950_plans.txt";
}

}  // namespace fk
