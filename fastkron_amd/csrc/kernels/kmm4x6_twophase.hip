// Six fused 4x4 fp32 factors in the KMM layout (X is 4096 x M row-major, the M columns are contiguous), one launch in
// which every global access is a full 256-byte piece of a row per wave instruction.
//
//   Z[(q1..q6), m] = alpha * sum_{k1..k6} F1[q1,k1] ... F6[q6,k6] * X[(k1..k6), m]  (+ beta * Y)
//
// A workgroup that owns whole columns can hold only 8 of them (4096 rows x 8 columns = 128 KB), so it touches 32 bytes
// of each of 4096 rows 8 KB apart; measured on an MI355X, a compute unit sustains no more line fills per microsecond
// on such strips than on a contiguous sweep, which leaves a quarter of the bandwidth (kmm4x6_mfma.hip is that kernel).
// Here the six digits of the row index are contracted in two phases by different workgroups instead:
//   phase 1  tile = 128 consecutive rows x 256 columns: a lane holds the 64 rows (digits k4 k5 k6) of one column in
//            registers and contracts them with V_MFMA_F32_4X4X1_16B_F32 (16 independent 4x4 outer products per
//            instruction: every lane gets its own outputs); the result goes to an intermediate T in the caller's
//            temporary, laid out [column block][unit][s = row bits 0-5][c = row bits 6-11][128 columns];
//   phase 2  tile = the 64 rows s + 64 c of two values of s x 256 columns: T is read back (contiguous 32 KB per s and
//            unit), the digits k1 k2 k3 are contracted the same way, alpha / beta * Y applied, Z written.
// A column block (256 columns, 1 KB of every row) has 32 jobs of each phase; phase 2 of a block needs phase 1 of the
// whole block, i.e. of 31 other workgroups.  The device hands workgroup i to XCD i % (number of XCDs), so the 32
// workgroups i = q mod 8 of block q share one XCD and its L2: T (4 MB per block, written and read once) travels
// through that L2, and so do the words the workgroups synchronise with, which are only ever touched by L2 atomics
// and loads that bypass the first-level cache.  (Synchronising through memory-side atomics instead costs 6 to 14 us
// per launch: the polls queue up behind the 64 MB of X and Y that are on their way.)  T itself is written and read
// with agent-scope accesses (sc1), coherent across the XCDs' L2 caches, at no cost in time.  fastKronInitHIP checks
// the placement once (a small launch that records the XCD each workgroup ran on); without it the kernel is not offered.
//
// Each workgroup of four waves works on the block's two halves of 128 columns (units A and B) one behind the other:
// X of both is requested at the start; as A arrives it is contracted and stored to T, Y of A is requested (it is not
// needed before the end, but the memory system must not run dry meanwhile), then the same for B; then T of A and B
// are read back, contracted and Z stored, unit A before unit B is waited for.  Loads and stores of a wave complete in issue order, so "T is stored" is
// known when at most as many younger operations are outstanding as were issued behind the stores.
//
// Synchronisation without assuming that all workgroups are resident at once.  Per block and unit a bit mask of the
// phase-1 jobs that are done: a workgroup sets its bit (an atomic OR: idempotent, no answer needed) when its T is
// stored and polls the mask until it is full.  If that takes more than `helpAfter` polls it looks for a job whose
// bit is missing (its workgroup may not have been started yet, e.g. because another kernel holds compute units), runs
// it as well and sets that bit itself.  Both workgroups then store the same values; a workgroup thus only ever waits
// for work that it can also do itself, so the launch cannot deadlock whatever the device schedules.  Waits are
// bounded as well; a wait that runs out sets an error word.  The last of a block's 32 workgroups to be through with
// the block's words zeroes them, so every launch finds them zero (launches that share a counter area must be ordered
// on one stream, as all calls on one handle are).
//
// The reference runs this shape as several launches of at most as many fused factors as fit its shared-memory tile
// (reference src/kernel_db/kernel_db.cpp:152-290).
// Algorithmic traffic per launch: read 4096*M, write 4096*M elements (+ 4096*M for Y); T adds the same again through L2.
#include <hip/hip_runtime.h>
#include "../problem.h"
#include "launch.h"

namespace fk {

typedef float t6f4 __attribute__((ext_vector_type(4)));
#define T6MFMA(a, b, c) __builtin_amdgcn_mfma_f32_4x4x1f32((a), (b), (c), 0, 0, 0)

constexpr int kT6Rows = 4096;                 // 4^6
constexpr int kT6BlockCols = 256;             // columns per block: 1 KB of every row
constexpr int kT6Jobs = 32;                   // jobs per block and phase
constexpr uint32_t kT6SpinLimit = 1u << 22;   // bounded waits: seconds
// counter area: word 1 = error, then four words per block from word 16 on ([0], [1]: masks of the phase-1 jobs of
// unit A, B that are done, [2]: workgroups that are through with the block's words)
constexpr int kT6Header = 16;
constexpr uint32_t kT6MaxBlocks = (kSyncAreaBytes / 4 - kT6Header) / 4;

// Contract the three digits held in the registers of x (digit j has register stride 4^j) with the factors whose
// operands are fa[j][p] = F_j[q = lane & 3][p].
__device__ __forceinline__ void t6Contract3(float (&x)[64], const float (&fa)[3][4]) {
#pragma unroll
  for (int j = 0; j < 3; j++) {
    const int st = (j == 0) ? 1 : (j == 1) ? 4 : 16;
#pragma unroll
    for (int s = 0; s < 16; s++) {
      const int base = (s / st) * st * 4 + (s % st);
      t6f4 d = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int p = 0; p < 4; p++) d = T6MFMA(fa[j][p], x[base + p * st], d);
#pragma unroll
      for (int i = 0; i < 4; i++) x[base + i * st] = d[i];
    }
  }
}

// The synchronisation words live in the L2 of the XCD that runs the block: read-modify-write operations without the
// agent-scope bit are carried out there.  They are also read with one (OR with a zero that the compiler cannot see,
// or it would make a load of it): a load at this scope may be served by the compute unit's first-level cache, which
// never sees the other workgroups' updates.
__device__ __forceinline__ void t6L2Or(uint32_t* p, uint32_t v) {
  (void)__hip_atomic_fetch_or(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ uint32_t t6L2Add(uint32_t* p, uint32_t v) {
  return __hip_atomic_fetch_add(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}
__device__ __forceinline__ uint32_t t6L2Load(uint32_t* p, uint32_t zero) {
  return __hip_atomic_fetch_or(p, zero, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

// at most `n` vector memory operations outstanding (n <= 63); other counters are not waited for
#define T6_WAIT_VM(n) __builtin_amdgcn_s_waitcnt(0x0F70 | ((n) & 15) | (((n) >> 4) << 14))

template <bool HAS_Y>
__global__ __launch_bounds__(256) void kron_kmm4x6_twophase_kernel(const StepArgs a, const uint32_t blocksPerEntry,
                                                                   const uint32_t totalBlocks, const uint32_t helpAfter,
                                                                   const uint32_t zero) {
  __shared__ int shared[2];
  const int tid = threadIdx.x;
  const int l = tid & 63;
  const int w = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int g = w >> 1, h = w & 1;                  // row group of the tile, 64-column half of the unit
  // workgroup i: block (i % 8) + 8 * (i / 256), job (i / 8) % 32: the 32 jobs of a block on one XCD
  const uint32_t q = (blockIdx.x & 7) + 8 * (blockIdx.x >> 8);
  const int j = (blockIdx.x >> 3) & 31;
  if (q >= totalBlocks) return;
  uint32_t* const sync = (uint32_t*)a.sync;
  uint32_t* const words = sync + kT6Header + 4 * q;

  const uint32_t bt = q / blocksPerEntry, cb = q % blocksPerEntry;
  // Every access goes through a buffer descriptor with a wave-uniform base, the lane's 4 bytes as the vector offset
  // and everything else (row, unit) as the scalar offset: no per-lane address arithmetic.  Policy bits: 2 = non-temporal
  // (X, Y, Z: used once), 16 = agent scope (T).  Offsets stay below 4 GB (4096 rows of at most 2^18 elements).
  const uint32_t ldi = (uint32_t)a.in_ldc * 4, ldo = (uint32_t)a.out_ldc * 4, ldy = (uint32_t)a.y_ldc * 4;   // bytes
  const size_t colOff = (size_t)cb * kT6BlockCols + h * 64;
  const float* const xBase = (const float*)a.in + (size_t)bt * a.in_batch + colOff;
  const float* const yBase = HAS_Y ? (const float*)a.y + (size_t)bt * a.y_batch + colOff : xBase;
  float* const zBase = (float*)a.out + (size_t)bt * a.out_batch + colOff;
  const __amdgpu_buffer_rsrc_t xRes = __builtin_amdgcn_make_buffer_rsrc((void*)xBase, 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t yRes = __builtin_amdgcn_make_buffer_rsrc((void*)yBase, 0, -1, 0x00020000);
  const __amdgpu_buffer_rsrc_t zRes = __builtin_amdgcn_make_buffer_rsrc((void*)zBase, 0, -1, 0x00020000);
  const uint32_t lane4 = (uint32_t)l * 4;
  // T of this block: [unit][s][c][128]
  float* const tBlock = (float*)a.scratch + (size_t)q * (kT6Rows * kT6BlockCols) + h * 64;
  const __amdgpu_buffer_rsrc_t tRes = __builtin_amdgcn_make_buffer_rsrc(tBlock, 0, kT6Rows * kT6BlockCols * 4, 0x00020000);

  // factor operands: fa[d][p] = F_d[q = l & 3][p]; a.f[0] is the factor of the fastest digit (k6).  Element (p, q)
  // of a factor lives at p*f_sp + q*f_sq.
  float fa[6][4];
#pragma unroll
  for (int d = 0; d < 6; d++) {
    const float* F = (const float*)a.f[d] + (size_t)bt * a.f_batch[d];
#pragma unroll
    for (int p = 0; p < 4; p++) fa[d][p] = F[(int64_t)p * a.f_sp[d] + (int64_t)(l & 3) * a.f_sq[d]];
  }
  const float fLo[3][4] = {{fa[0][0], fa[0][1], fa[0][2], fa[0][3]}, {fa[1][0], fa[1][1], fa[1][2], fa[1][3]},
                           {fa[2][0], fa[2][1], fa[2][2], fa[2][3]}};
  const float fHi[3][4] = {{fa[3][0], fa[3][1], fa[3][2], fa[3][3]}, {fa[4][0], fa[4][1], fa[4][2], fa[4][3]},
                           {fa[5][0], fa[5][1], fa[5][2], fa[5][3]}};

  float xa[64], xb[64];
  float ya[HAS_Y ? 64 : 1], yb[HAS_Y ? 64 : 1];
  const int s = 2 * j + g;                          // the row residue of this wave's phase-2 tile

  // (every lambda here is inlined: a call would take the arrays they capture out of the registers)
  auto loadX = [&](int job, int unit, float (&x)[64]) __attribute__((always_inline)) {
    const uint32_t off = (uint32_t)(128 * job + 64 * g) * ldi + unit * 512;
#pragma unroll
    for (int r = 0; r < 64; r++)
      x[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(xRes, lane4, off + r * ldi, 2));
  };
  // phase 1 of one unit: contract the low digits, store to T rows c = 2 job + g
  auto storeT = [&](int job, int unit, float (&x)[64]) __attribute__((always_inline)) {
    t6Contract3(x, fLo);
    const uint32_t off = (uint32_t)(unit * (64 * 64 * 128) + (2 * job + g) * 128) * 4;
#pragma unroll
    for (int r = 0; r < 64; r++)
      __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, x[r]), tRes, lane4, off + r * (64 * 128 * 4), 16);
  };
  // Y of the wave's phase-2 tile, requested behind the stores to T; returns once those stores are complete
  auto loadYBehindT = [&](int unit, float (&y)[HAS_Y ? 64 : 1]) __attribute__((always_inline)) {
    if (HAS_Y) {
      const uint32_t off = (uint32_t)s * ldy + unit * 512;
#pragma unroll
      for (int r = 0; r < 63; r++)
        y[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(yRes, lane4, off + (r * 64) * ldy, 2));
      __builtin_amdgcn_sched_barrier(0);
      T6_WAIT_VM(63);                                // 63 younger operations: the stores to T are complete
      __builtin_amdgcn_sched_barrier(0);
      y[63] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(yRes, lane4, off + (63 * 64) * ldy, 2));
    } else {
      T6_WAIT_VM(0);
    }
  };
  auto markDone = [&](int job, int unit) __attribute__((always_inline)) {
    __syncthreads();                                 // every wave's T stores of the unit are complete
    if (tid == 0) t6L2Or(words + unit, 1u << job);
  };

  loadX(j, 0, xa);
  loadX(j, 1, xb);
  __builtin_amdgcn_sched_barrier(0);
  storeT(j, 0, xa);
  __builtin_amdgcn_sched_barrier(0);
  loadYBehindT(0, ya);
  __builtin_amdgcn_sched_barrier(0);
  markDone(j, 0);
  __builtin_amdgcn_sched_barrier(0);
  storeT(j, 1, xb);
  __builtin_amdgcn_sched_barrier(0);
  loadYBehindT(1, yb);
  __builtin_amdgcn_sched_barrier(0);
  markDone(j, 1);
  __builtin_amdgcn_sched_barrier(0);

  // phase 2: wait until the block's 32 phase-1 jobs of unit A are done, running missing ones after a long wait
  for (uint32_t spins = 0;; spins++) {
    if (tid == 0) {
      int what = 0;                                  // 0: go on, 1: keep waiting, 2 + job: run that phase-1 job
      const uint32_t mask = t6L2Load(words + 0, zero);
      if (mask != ~0u) {
        what = 1;
        if (spins >= kT6SpinLimit) {
          (void)__hip_atomic_fetch_or(sync + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);   // results not valid
          what = 0;
        } else if (spins >= helpAfter) {
          what = 2 + __builtin_ctz(~mask);
        } else {
          __builtin_amdgcn_s_sleep(4);
        }
      }
      shared[0] = what;
    }
    __syncthreads();
    const int what = __builtin_amdgcn_readfirstlane(shared[0]);
    __syncthreads();
    if (what == 0) break;
    if (what >= 2) {
      // (rare) another workgroup's phase-1 job, both units, in the registers that are free at this point
      const int job = what - 2;
      loadX(job, 0, xa);
      storeT(job, 0, xa);
      T6_WAIT_VM(0);
      markDone(job, 0);
      loadX(job, 1, xa);
      storeT(job, 1, xa);
      T6_WAIT_VM(0);
      markDone(job, 1);
    }
  }
  auto loadT = [&](int unit, float (&x)[64]) __attribute__((always_inline)) {
    const uint32_t off = (uint32_t)(unit * (64 * 64 * 128) + s * (64 * 128)) * 4;
#pragma unroll
    for (int r = 0; r < 64; r++)
      x[r] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(tRes, lane4, off + r * (128 * 4), 16));
  };
  const float alpha = a.epilogue ? (float)a.alpha : 1.f, beta = (float)a.beta;
  auto storeZ = [&](int unit, float (&x)[64], float (&y)[HAS_Y ? 64 : 1]) __attribute__((always_inline)) {
    t6Contract3(x, fHi);
    const uint32_t off = (uint32_t)s * ldo + unit * 512;
#pragma unroll
    for (int r = 0; r < 64; r++) {
      float v = x[r] * alpha;
      if (HAS_Y) v += beta * y[r];
      __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), zRes, lane4, off + (r * 64) * ldo, 2);
    }
  };
  // Unit A is finished before unit B is waited for (measured: 29.2 us against 31.0 with the intermediates of both
  // units read back first).
  loadT(0, xa);
  storeZ(0, xa, ya);
  // (a full mask of unit A means that every job has at least started its unit B, which nothing holds up: only wait)
  for (uint32_t spins = 0; tid == 0 && t6L2Load(words + 1, zero) != ~0u; spins++) {
    if (spins >= kT6SpinLimit) { (void)__hip_atomic_fetch_or(sync + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT); break; }
    __builtin_amdgcn_s_sleep(4);
  }
  // this workgroup is through with the block's words: said now, the answer (am I the last?) is looked at at the end
  uint32_t through = 0;
  if (tid == 0) through = t6L2Add(words + 2, 1u);
  __syncthreads();
  __builtin_amdgcn_sched_barrier(0);
  loadT(1, xb);
  storeZ(1, xb, yb);
  // the last of the block's workgroups to be through zeroes the words for the next launch (the same L2 serves it)
  if (tid == 0 && through + 1 == (uint32_t)kT6Jobs) {
    (void)__hip_atomic_exchange(words + 0, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    (void)__hip_atomic_exchange(words + 1, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    (void)__hip_atomic_exchange(words + 2, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
  }
}

// Records the XCD (HW_REG_XCC_ID) each workgroup of a 256-workgroup launch ran on.
__global__ void kron_record_xcc_kernel(uint32_t* out) {
  if (threadIdx.x == 0) out[blockIdx.x] = __builtin_amdgcn_s_getreg((3 << 11) | (0 << 6) | 20) & 15;
}

// True when workgroups i and i + 8 k of a launch run on the same XCD, which is what lets the two-phase kernel keep a
// block's intermediate and synchronisation words in one L2.  `scratchWords`: 256 words of device memory.  Synchronises
// the device: called at set-up, not from a gemkm / gekmm call.
bool kmm4x6TwoPhasePlacementHolds(uint32_t* scratchWords, hipStream_t stream) {
  uint32_t host[256];
  for (int rep = 0; rep < 3; rep++) {
    hipLaunchKernelGGL(kron_record_xcc_kernel, dim3(256), dim3(64), 0, stream, scratchWords);
    if (hipGetLastError() != hipSuccess) return false;
    if (hipMemcpyAsync(host, scratchWords, sizeof(host), hipMemcpyDeviceToHost, stream) != hipSuccess) return false;
    if (hipStreamSynchronize(stream) != hipSuccess) return false;
    for (int i = 8; i < 256; i++) if (host[i] != host[i % 8]) return false;
  }
  return true;
}

bool kmm4x6TwoPhaseSupported(const StepArgs& a) {
  if (a.nf != 6 || a.Kin != kT6Rows || a.Kout != kT6Rows) return false;
  for (uint32_t d = 0; d < 6; d++) if (a.p[d] != 4 || a.q[d] != 4) return false;
  if (a.in_ldm != 1 || a.out_ldm != 1 || (a.y && a.y_ldm != 1)) return false;
  if (a.M % kT6BlockCols || a.M == 0) return false;
  // 32-bit byte offsets within an operand
  if ((uint64_t)a.in_ldc * kT6Rows * 4 >= (1ull << 32) || (uint64_t)a.out_ldc * kT6Rows * 4 >= (1ull << 32) ||
      (a.y && (uint64_t)a.y_ldc * kT6Rows * 4 >= (1ull << 32))) return false;
  const uint64_t blocks = (uint64_t)(a.M / kT6BlockCols) * a.batch;
  if (blocks > kT6MaxBlocks) return false;
  // the intermediate lives in a temporary of the call that this launch neither reads nor writes
  if (!a.scratch || !a.sync || a.scratch_elems < blocks * (uint64_t)(kT6Rows * kT6BlockCols)) return false;
  if (a.scratch == a.in || a.scratch == a.out || a.scratch == a.y) return false;
  return true;
}

// Polls of a waiting workgroup before it runs jobs that are still missing itself: far more than a launch ever needs
// when its workgroups all run (a poll takes a fraction of a microsecond).  Tests lower it to 0.
static std::atomic<uint32_t> t6HelpAfter{100000};
void setKmm4x6TwoPhaseHelpAfter(uint32_t polls) { t6HelpAfter.store(polls, std::memory_order_relaxed); }

hipError_t launchKmm4x6TwoPhase(const StepArgs& a, hipStream_t stream) {
  if (!kmm4x6TwoPhaseSupported(a)) return hipErrorInvalidValue;
  const uint32_t blocksPerEntry = a.M / kT6BlockCols;
  const uint32_t totalBlocks = blocksPerEntry * a.batch;
  const uint32_t helpAfter = t6HelpAfter.load(std::memory_order_relaxed);
  dim3 grid(256 * ((totalBlocks + 7) / 8)), block(256);
  if (a.y && a.epilogue)
    hipLaunchKernelGGL(kron_kmm4x6_twophase_kernel<true>, grid, block, 0, stream, a, blocksPerEntry, totalBlocks, helpAfter, 0u);
  else
    hipLaunchKernelGGL(kron_kmm4x6_twophase_kernel<false>, grid, block, 0, stream, a, blocksPerEntry, totalBlocks, helpAfter, 0u);
  return hipGetLastError();
}

}  // namespace fk
