// Launch entry points of the kernel translation units (one per .hip file).
#pragma once
#include <hip/hip_runtime.h>
#include <atomic>
#include "../problem.h"

// Non-temporal global accesses, chosen at compile time by a kernel's NT mode: 0 = ordinary loads and stores,
// 1 = non-temporal stores, 2 = non-temporal loads and stores.  On a streaming copy of 268 MB (operands that no cache
// holds) ordinary accesses reach 5.5 TB/s, non-temporal stores 5.7; the whole-row kernels gain 2.5 to 4 %.  Partial
// lines must not be written this way (the kernel that writes 32-byte pieces of lines shared between workgroups loses
// 40 %), and an intermediate that the next launch reads back from the 256 MB memory-side cache should stay ordinary.
#define FK_LD(NT, p) ((NT) >= 2 ? __builtin_nontemporal_load(p) : *(p))
#define FK_ST(NT, v, p) do { if ((NT) >= 1) __builtin_nontemporal_store((v), (p)); else *(p) = (v); } while (0)

namespace fk {

// 16-byte stores of results that nothing reads back soon, at system scope and non-temporal ("sc0 sc1 nt"): a copy of
// 268 MB runs at 6.30 TB/s with them against 6.06 with non-temporal stores and 5.68 with ordinary ones (sgemkm
// 1024 x 16^4: 103.1 -> 100.5 us).  The compiler has no such store for a plain pointer, so they go through a buffer
// descriptor: a wave-uniform base and a 32-bit byte offset per lane below `bytes` (stores beyond it are dropped).
// 4-byte stores lose with this policy (sgemkm 1024 x 8^5: 52.6 -> 53.8 us).
typedef unsigned int StreamU4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ __amdgpu_buffer_rsrc_t streamTarget(void* uniformBase, uint32_t bytes) {
  return __builtin_amdgcn_make_buffer_rsrc(uniformBase, 0, (int)bytes, 0x00020000);
}
template <typename V>
__device__ __forceinline__ void streamStore16(V v, __amdgpu_buffer_rsrc_t target, uint32_t byteOffset) {
  static_assert(sizeof(V) == 16, "16-byte elements");
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(StreamU4, v), target, (int)byteOffset, 0, 19);
}


// Function attributes and the number of compute units belong to a device, not to the process: the launchers
// keep both per device, so that handles on different GPUs of one process (and threads) do not share them.
constexpr int kMaxDevices = 64;
inline int launchDeviceIndex() {
  int d = 0;
  if (hipGetDevice(&d) != hipSuccess || d < 0 || d >= kMaxDevices) d = 0;
  return d;
}
inline int deviceCUs() {
  static std::atomic<int> cus[kMaxDevices];
  const int d = launchDeviceIndex();
  int c = cus[d].load(std::memory_order_relaxed);
  if (c == 0) {
    hipDeviceProp_t prop;
    c = (hipGetDeviceProperties(&prop, d) == hipSuccess && prop.multiProcessorCount > 0) ? prop.multiProcessorCount : 256;
    cus[d].store(c, std::memory_order_relaxed);
  }
  return c;
}
inline int streamMode(const StepArgs& a) { return a.stream_out ? (a.stream_in ? 2 : 1) : 0; }
struct PerDeviceOnce {               // "done once on this device" for set-up such as hipFuncSetAttribute
  std::atomic<uint64_t> mask{0};
  bool done(int dev) const { return (mask.load(std::memory_order_acquire) >> dev) & 1; }
  void mark(int dev) { mask.fetch_or(1ull << dev, std::memory_order_release); }
};

// Workgroups that share a CU and start together move through their load, compute and store phases in lockstep, so
// that one's arithmetic never hides the other's memory traffic.  In the first round of a launch (the workgroups the
// device starts before any has finished) the workgroup that got a later LDS allocation of its CU, i.e. one whose LDS
// base is not 0, therefore waits `ticks` of the 100 MHz clock before its first load; workgroups of later rounds
// start whenever a predecessor ends and need no delay.  Every wave of a workgroup takes the same branch.
__device__ __forceinline__ void delayLaterWorkgroupOfCU(uint32_t firstRound, uint32_t ticks) {
  if (ticks && blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z) < firstRound) {
    const uint32_t ldsBase = __builtin_amdgcn_s_getreg((7 << 11) | (0 << 6) | 6);      // HW_REG_LDS_ALLOC, LDS_BASE
    if (ldsBase) {
      const unsigned long long t0 = __builtin_amdgcn_s_memrealtime();
      while (__builtin_amdgcn_s_memrealtime() - t0 < (unsigned long long)ticks) __builtin_amdgcn_s_sleep(16);
    }
  }
}

// Any shape, one factor per launch.
hipError_t launchGenericStep(const StepArgs& a, DType dt, hipStream_t stream);

// Four fused 16x16 fp32 factors on rows of exactly 16^4 columns, one workgroup per row.
bool row16x4Supported(const StepArgs& a);
hipError_t launchRow16x4(const StepArgs& a, hipStream_t stream, bool staggered = true);

// The same with 8 waves of 128 values per lane and the whole next block prefetched.
bool row16x4W8Supported(const StepArgs& a);
hipError_t launchRow16x4W8(const StepArgs& a, hipStream_t stream);

// Five fused 8x8 fp64 factors on rows of exactly 8^5 columns, one workgroup per row and CU, on the vector ALU.
bool row8x5F64Supported(const StepArgs& a);
hipError_t launchRow8x5F64(const StepArgs& a, hipStream_t stream);

// Five fused 8x8 fp32 factors on rows of exactly 8^5 columns, one workgroup per row, two per CU.
bool row8x5Supported(const StepArgs& a);
hipError_t launchRow8x5(const StepArgs& a, hipStream_t stream, int schedule = 0);

// Three fused 32x16 fp32 factors on rows of exactly 32^3 columns, one workgroup per row, two per CU.
bool row32x16x3Supported(const StepArgs& a);
hipError_t launchRow32x16x3(const StepArgs& a, hipStream_t stream);
bool row32x3Supported(const StepArgs& a);
hipError_t launchRow32x3(const StepArgs& a, hipStream_t stream);
// The same as one persistent workgroup of 16 waves per CU with the next row's loads in flight.
bool row32x3pSupported(const StepArgs& a);
hipError_t launchRow32x3p(const StepArgs& a, hipStream_t stream);

// Two fused 32x32 or 64x64 factors (fp64 or fp32) on rows of exactly P*P columns (MKM layout), one wave per row.
bool pairMfmaSupported(const StepArgs& a, DType dt);
hipError_t launchPairMfma(const StepArgs& a, DType dt, hipStream_t stream);

// Three fused 8x8 fp32 factors in the KMM layout, 512 rows by 64 columns per workgroup.
bool kmm8x3Supported(const StepArgs& a);
hipError_t launchKmm8x3(const StepArgs& a, hipStream_t stream);

// One step with a 64x64 or 128x128 factor, either type and layout, tiles of 16 KB passed through LDS.
bool stepWideSupported(const StepArgs& a, DType dt);
hipError_t launchStepWide(const StepArgs& a, DType dt, hipStream_t stream, int maxWorkgroupsPerCU = 0);

// One step with a 16x16 ... 128x128 factor on the matrix cores, fp64 or fp32, MKM or KMM layout.
bool stepMfmaSupported(const StepArgs& a, DType dt);
hipError_t launchStepMfma(const StepArgs& a, DType dt, hipStream_t stream);

// Two or three fused 16x16 factors on blocks of 4096 elements (MKM layout), fp64 or fp32, one wave per block.
bool row16x3Supported(const StepArgs& a, DType dt);
hipError_t launchRow16x3(const StepArgs& a, DType dt, hipStream_t stream);

// One step with a factor of any shape up to 256x512 on the matrix cores (zero padded), fp64 or fp32, any layout.
bool stepAnyMfmaSupported(const StepArgs& a, DType dt);
hipError_t launchStepAnyMfma(const StepArgs& a, DType dt, hipStream_t stream);

// Two fused 16x16 factors on the KMM layout, fp32 or fp64: matrix cores for one digit, vector FMAs over the
// register index for the other; 256 x 16 tiles in registers.
bool kmm16x2Supported(const StepArgs& a, DType dt);
hipError_t launchKmm16x2(const StepArgs& a, DType dt, hipStream_t stream);

// One step with a 64x64 fp64 factor on the KMM layout (4x4x4 matrix-core instruction, 64-column tiles).
bool kmm64F64Supported(const StepArgs& a);
hipError_t launchKmm64F64(const StepArgs& a, hipStream_t stream);

// KMM layout, fp32: six fused 4x4 factors on all 4096 rows of 8 columns per workgroup (one launch for 4x4^6).
bool kmm4x6Supported(const StepArgs& a);
hipError_t launchKmm4x6(const StepArgs& a, hipStream_t stream);

// The same problem in two phases with an intermediate in a temporary of the call: every access a full 256-byte piece.
bool kmm4x6TwoPhaseSupported(const StepArgs& a);
hipError_t launchKmm4x6TwoPhase(const StepArgs& a, hipStream_t stream);
constexpr size_t kSyncAreaBytes = 4096;     // zero-initialised counter area such kernels need (StepArgs::sync)
// Whether workgroups i and i + 8 k of a launch share an XCD on this device (checked with a small launch and a
// synchronisation, at set-up); the kernel above is only offered where that holds.
bool kmm4x6TwoPhasePlacementHolds(uint32_t* scratchWords, hipStream_t stream);
// Polls after which a waiting workgroup of that kernel runs missing jobs itself (tests set 0).
void setKmm4x6TwoPhaseHelpAfter(uint32_t polls);

// Copy kernels with the access patterns of the two kernels above (0 contiguous, 1 strips, 2 two phases): Z = 1.5 X + 0.5 Y
// on 4096 x M fp32.  Measurement only (bench.py --pattern-ceilings).
hipError_t launchPatternProbe(int pattern, const float* X, const float* Y, float* Z, float* T, void* sync, uint32_t M,
                              hipStream_t stream);

// KMM layout, fp32: three fused 4x4 or two fused 8x8 factors held in registers, lanes along M.
bool kmmRegSupported(const StepArgs& a);
hipError_t launchKmmReg(const StepArgs& a, hipStream_t stream);

// Several small factors of any shape (P <= 8) fused through LDS, MKM or KMM layout, fp32 or fp64.
// fusedSmallFits: whether a group of factors (p[0], q[0] applied first) on Kin input columns has a tile.
bool fusedSmallFits(uint32_t nf, const uint32_t* p, const uint32_t* q, uint64_t Kin, uint32_t M, bool kmm, DType dt);
bool fusedSmallSupported(const StepArgs& a, DType dt);
hipError_t launchFusedSmall(const StepArgs& a, DType dt, hipStream_t stream);

// Kronecker products of adjacent small factors into the handle's workspace, one workgroup per product.
hipError_t launchMergeFactors(const MergeArgs& a, DType dt, hipStream_t stream);
// Transposed copy: in is R x C row-major per batch entry, out is C x R.
hipError_t launchTranspose(const void* in, void* out, uint32_t R, uint32_t C, uint32_t batch, uint64_t inBatch,
                           uint64_t outBatch, DType dt, hipStream_t stream);
hipError_t launchTransposeAdd(const void* in, void* out, uint32_t R, uint32_t C, uint32_t batch, uint64_t inBatch,
                              uint64_t outBatch, const void* y, uint64_t yBatch, double beta, DType dt, hipStream_t stream,
                              bool streamOut);
// Fills `elems` elements with values spread over [-1, 1] (data for the tuner's timing runs).
hipError_t launchFill(void* dst, size_t elems, DType dt, hipStream_t stream);

}  // namespace fk
