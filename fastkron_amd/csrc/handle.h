// The object behind fastKronHandle: backends, options, the HIP stream, the gfx950 kernel database and
// the tuner.  Role of reference src/handle/handle.{h,cpp} (FastKronHandle, xgemm, gekmmSizes).
#pragma once
#include <hip/hip_runtime.h>
#include <string>
#include <unordered_map>
#include "../../include/fastkron.h"
#include "kernel_db.h"
#include "problem.h"

namespace fk {

struct BufferPlan {          // where each launch reads and writes
  const void* in;  void* out;
  uint64_t in_batch, out_batch;
};

// Address of the library's static scratch array on the current GPU (static_scratch.hip).
hipError_t staticScratchForCurrentDevice(void** out);

StepArgs makeStepArgs(const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool last);

class Handle {
 public:
  explicit Handle(uint32_t backends);
  ~Handle();

  bool hasBackend(uint32_t b) const { return (backends_ & b) == b; }
  void setOptions(uint32_t o) { options_ = o; }
  bool canTune() const { return (options_ & fastKronOptionsTune) != 0; }
  bool useFusion() const { return (options_ & fastKronOptionsUseFusion) != 0; }

  fastKronError initHIP(void* ptrToStream);
  fastKronError setStream(fastKronBackend backend, void* ptrToStream);

  static fastKronError sizes(uint32_t M, uint32_t N, const uint32_t* Ps, const uint32_t* Qs,
                             size_t* yElems, size_t* tmpElems);
  static fastKronError sizesForward(uint32_t M, uint32_t N, const uint32_t* Ps, const uint32_t* Qs,
                                    size_t* yElems, size_t* interElems);

  // Entry point of every gemkm/gekmm/forward call (reference src/handle/handle.cpp:114-286).
  // With `ws` the call takes its merged-factor workspace from the caller instead of the handle's own, and neither
  // tunes nor allocates anything on the device.
  struct CallWorkspace { void* merge; size_t mergeBytes; };
  fastKronError xgemm(KronProblem p, fastKronBackend backend, void* temp1, void* temp2, const CallWorkspace* ws = nullptr);

  // Runs `plan` on the stream; temps may be null when the plan has a single launch.
  // dryRun: only the kernels' checks of the concrete buffers run; *refused then names the kernel that said no
  fastKronError execute(const KronProblem& p, const Plan& plan, void* temp1, void* temp2, bool dryRun = false,
                        int* refused = nullptr);
  // What a tuned record prescribes for a problem: merge small factors or not, two-part plan with `split` leading
  // factors or one chain (0), and the launches (numbered in the chain after merging; for a two-part plan the
  // trailing part's steps, on factors >= split, come first).
  struct Choice { bool transposeX = false; bool merge = false; uint32_t split = 0; Plan plan; };
  // Times the alternatives for `p` (merged or not, every two-part split, every kernel on every sub-chain), stores the
  // fastest under the problem's own string and returns it.
  fastKronError tune(const KronProblem& p, bool haveTemp2, Choice* best);
  // The online selection: merge by rule, tuned records of the older kind, the two-part plan by rule, greedy choice.
  fastKronError runOnline(KronProblem p, void* temp1, void* temp2, const CallWorkspace* ws);
  // op(X) = T handled by a transposed copy of X ahead of the launches (into temp2, or temp1 for a single launch)
  bool transposedProblem(const KronProblem& p, void* temp1, void* temp2, KronProblem* pn, void** xt) const;
  bool transposeFirstOnline(const KronProblem& p, const KronProblem& pn, void* temp1, void* temp2, const CallWorkspace* ws);
  hipError_t launchTransposeX(const KronProblem& p, void* xt, uint64_t xtStride);
  void noteTranspose(const KronProblem& p);
  // GeKMM with op(X) = T as the GeMKM of the same buffer and a transposition of the result
  bool viaMKMOnline(const KronProblem& p) const;
  fastKronError runViaMKM(const KronProblem& p, fastKronBackend backend, void* temp1, void* temp2, const CallWorkspace* ws);
  bool lookupChoice(const KronProblem& p, Choice* c) const;
  fastKronError runChoice(const KronProblem& p, const Choice& c, void* temp1, void* temp2, const CallWorkspace* ws);
  bool buildSplit(const KronProblem& p, uint32_t g, void* temp1, void* temp2, KronProblem* q1, KronProblem* q2) const;
  fastKronError runSplit(const KronProblem& p, uint32_t g, const KronProblem& q1, const Plan& plan1,
                         const KronProblem& q2, const Plan& plan2, void* temp2);
  uint32_t chunkRowsForCache(const KronProblem& p, const KronProblem& q2) const;
  // MKM chains longer than a whole-row kernel can take: trailing factors by the row kernel on
  // M * prod(leading P) virtual rows, leading factors as a batched KMM over the row blocks.
  // Returns fastKronKernelNotFound when the problem does not have that form.
  fastKronError trySplitLeadingTrailing(const KronProblem& p, void* temp1, void* temp2);
  // Chains of 2x2 / 4x4 (fp64: also 8x8) factors: adjacent factors are replaced by their Kronecker product
  // (16x16; 64x64 in fp64 when the chain holds 8x8 or 32x32 factors), computed into the handle's workspace by one small launch, so that the
  // kernels for those sizes apply.  Returns false when nothing is merged; on true `out` is the merged problem.
  bool mergeSmallFactors(const KronProblem& p, KronProblem* out, const CallWorkspace* ws = nullptr);

  const std::string& lastPlan() const { return lastPlan_; }
  void setTunedDB(const char* path);

  // Plan-only mode: calls go through every check, the planner and the kernels' argument checks, but nothing is
  // launched and no device is needed (an MI355X is assumed); lastLaunches() then lists the launches the call
  // would have made, one per line, with their buffers, strides and batch counts.
  void setPlanOnly(bool on);
  bool planOnly() const { return planOnly_; }
  const std::string& lastLaunches() const { return launchLog_; }

  KernelDB& db() { return db_; }
  const DeviceInfo& device() const { return dev_; }
  hipStream_t stream() const { return stream_; }
  // the zero-initialised counter area behind the merged-factor workspace (null before fastKronInitHIP)
  // Reads and clears the error word of the counter area (synchronises the stream).
  fastKronError syncError(uint32_t* word);
  void* syncArea() const { return mergeWs_ ? (char*)mergeWs_ + mergeWsBytes_ : nullptr; }

 private:
  fastKronError ensureDevice();
  void orderWorkspaceBehind(hipStream_t next);

  uint32_t backends_;
  uint32_t options_ = fastKronOptionsNone;
  hipStream_t stream_ = nullptr;
  bool hipInit_ = false;
  DeviceInfo dev_;
  KernelDB db_;
  std::unordered_map<std::string, Plan> planCache_;   // online selections, per problem string
  std::unordered_map<std::string, bool> transposeCache_;   // op(X) = T: transpose first or not, per problem string
  std::string dbPath_;
  std::string lastPlan_;
  void* mergeWs_ = nullptr;                           // device memory for merged factors, allocated by initHIP
  size_t mergeWsBytes_ = 0;
  bool mergeWsOwned_ = false;
  hipStream_t mergeWsStream_ = nullptr;               // stream of the last call that wrote the workspace
  bool mergeWsUsed_ = false;
  hipEvent_t mergeWsEvent_ = nullptr;                 // orders a new stream behind the last user of the workspace
  bool planOnly_ = false;
  long chunkMB_ = 0;                                  // FASTKRON_CHUNK_MB: two-part plans run in row chunks of this size (0: whole)
  bool callWs_ = false;                               // the running call brought its own workspace (touches none of the handle's)
  std::string launchLog_;
};

}  // namespace fk
