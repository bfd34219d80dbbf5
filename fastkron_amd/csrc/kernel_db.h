// Registry of compiled gfx950 kernels, launch-plan selection and the persisted tuning database.
//
// Role of reference src/kernel_db/kernel_db.{h,cpp} (abstract database + online selection,
// :152-290) with a gfx950 subclass in place of the reference's CUDA one (cuda_kernel_db.cu); unlike
// the reference, whose tuner keeps results only in memory (src/autotuner/autotuner.h:101-116), tuned
// plans are written to a text file and reloaded by later processes.
#pragma once
#include <hip/hip_runtime.h>
#include <map>
#include <string>
#include <vector>
#include "problem.h"

namespace fk {

struct DeviceInfo {
  int  device = -1;
  int  cus = 256;
  int  ldsPerBlock = 65536;      // bytes a workgroup may allocate
  int  waveSize = 64;
  int  clockKHz = 2400000;
  char arch[64] = "gfx950";
  bool valid = false;
  // Selection without timing: a kernel's canRun then also refuses where a measured rule of thumb says another plan
  // is faster (few rows, small factors ...).  The tuner and the check of a tuned plan switch this off and ask only
  // what a kernel is able to run.
  bool rulesOfThumb = true;
  // Workgroups i and i + 8 k of a launch run on one XCD and share its L2 (checked once by fastKronInitHIP).
  bool xcdRoundRobin = false;
};

struct KernelInfo;
using CanRunFn = bool (*)(const KernelInfo&, const KronProblem&, uint32_t lo, uint32_t hi,
                          bool firstLaunch, bool lastLaunch, const DeviceInfo&);
using LaunchFn = hipError_t (*)(const KernelInfo&, const StepArgs&, hipStream_t);
// Final check on the concrete launch arguments (pointer alignment, strides); null = always fine.
using CheckFn  = bool (*)(const KernelInfo&, const StepArgs&);

// One compiled kernel variant.  `name` follows the reference kernel-string grammar
// (src/kernels/kmmkernel.cpp:128-136 with the backend/arch prefix of src/kernels/gpu_kmmkernel.cu:3-8).
struct KernelInfo {
  std::string name;
  DType    dt;
  uint32_t P, Q;          // 0: any factor shape
  uint32_t fused;         // factors applied per launch
  uint32_t tileM, tileK;  // rows and input columns per workgroup (0: not tiled that way)
  uint32_t threads;
  uint32_t variant;       // kernel-family specific
  bool     tunerOnly;     // a candidate for the tuner, never chosen by the online selection
  bool     usesSync;      // synchronises its workgroups through the handle's counter area (StepArgs::sync)
  CanRunFn canRun;
  LaunchFn launch;
  CheckFn  check;
};

struct PlanStep { uint32_t lo, hi; int kernel; };   // factors [lo, hi], hi applied first
using Plan = std::vector<PlanStep>;

class KernelDB {
 public:
  KernelDB();
  const std::vector<KernelInfo>& kernels() const { return kernels_; }
  int findByName(const std::string& name) const;
  int genericKernel(DType dt) const;

  // Online selection (no timing): greedy over the chain, deepest fusion first.
  // `excluded`: kernels (indices) that must not be chosen, e.g. because they refused the call's buffers
  Plan selectOnline(const KronProblem& p, const DeviceInfo& dev, bool allowFusion,
                    const std::vector<int>* excluded = nullptr) const;
  // All kernels able to run factors [lo, hi] as one launch.
  std::vector<int> candidates(const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool last,
                              const DeviceInfo& dev) const;

  // True when `plan` applies every factor of `p` exactly once, last factor first, and every step's kernel
  // accepts its factor range (a plan read from a file is not trusted before it passes this).
  bool validPlan(const KronProblem& p, const Plan& plan, const DeviceInfo& dev) const;

  // Tuned plans, keyed by the problem string.  A record may also say how the chain is to be rewritten before the plan
  // applies: `merge` (1: adjacent small factors replaced by their Kronecker products, 0: not, -1: unspecified, as the
  // online selection decides) and `split` (g > 0: the plan's steps on factors >= g are the trailing part of a two-part
  // plan, run on the contiguous blocks of the rows, the steps on factors < g the leading part, run across the blocks).
  // `transposeX` (1: op(X) = T is handled by a transposed copy of X ahead of the launches, which then see op(X) = N).
  bool lookupTuned(const std::string& key, Plan* plan, int* merge = nullptr, uint32_t* split = nullptr,
                   int* transposeX = nullptr) const;
  void storeTuned(const std::string& key, const Plan& plan, float ms, int merge = -1, uint32_t split = 0,
                  int transposeX = 0);
  // `shipped`: the records come from the file that ships with the library; saveFile leaves those out, so that a
  // user's file never holds stale copies that would override later versions of them
  bool loadFile(const std::string& path, bool shipped = false);
  bool saveFile(const std::string& path) const;
  static std::string defaultPath();
  static std::string shippedPath();

 private:
  std::vector<KernelInfo> kernels_;
  struct Tuned {
    std::vector<std::pair<std::pair<uint32_t, uint32_t>, std::string>> steps;
    float ms;
    int merge = -1;
    uint32_t split = 0;
    int transposeX = 0;
    bool shipped = false;
  };
  std::map<std::string, Tuned> tuned_;
};

// Filled in by each kernel family's translation unit.
void registerGenericKernels(std::vector<KernelInfo>& out);
void registerRowKernels(std::vector<KernelInfo>& out);

}  // namespace fk
