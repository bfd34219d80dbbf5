// Fast tuning: time every compiled kernel on every contiguous sub-chain of the problem, then pick the
// cheapest split of the chain with a dynamic program.  Same search as reference
// src/autotuner/autotuner.cpp:24-150 (minExecTimeOfSeries over all sub-chains) with hipEvent timing
// in place of the reference's cudaEvent timing (src/kernel_db/cuda_kernel_db.cu:426-483: 5 warm-up
// and 5 timed runs per candidate); the winner is also written to the tuning file when one is set.
#include <cfloat>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "handle.h"

namespace fk {

static float timeLaunch(const KernelInfo& k, const StepArgs& a, hipStream_t stream, hipEvent_t e0, hipEvent_t e1) {
  const int warm = 3, runs = 5;
  for (int i = 0; i < warm; i++) if (k.launch(k, a, stream) != hipSuccess) return FLT_MAX;
  if (hipStreamSynchronize(stream) != hipSuccess) return FLT_MAX;
  hipEventRecord(e0, stream);
  for (int i = 0; i < runs; i++) if (k.launch(k, a, stream) != hipSuccess) return FLT_MAX;
  hipEventRecord(e1, stream);
  if (hipEventSynchronize(e1) != hipSuccess) return FLT_MAX;
  float ms = 0;
  hipEventElapsedTime(&ms, e0, e1);
  return ms / runs;
}

fastKronError Handle::tune(const KronProblem& p, Plan* best) {
  const bool verbose = getenv("FASTKRON_LOG") != nullptr;
  const uint32_t N = p.N;
  size_t yElems = 0, tmpElems = 0;
  fastKronError e = sizes(p.M, N, p.P, p.Q, &yElems, &tmpElems);
  if (e != fastKronSuccess) return e;
  const size_t elems = std::max<size_t>(std::max(tmpElems, yElems), (size_t)p.M * p.K()) * p.batch;
  const size_t bytes = elems * dtypeSize(p.dt);
  void *bufA = nullptr, *bufB = nullptr;
  if (hipMalloc(&bufA, bytes) != hipSuccess) return fastKronInvalidMemoryAccess;
  if (hipMalloc(&bufB, bytes) != hipSuccess) { hipFree(bufA); return fastKronInvalidMemoryAccess; }
  hipMemsetAsync(bufA, 0, bytes, stream_);
  hipMemsetAsync(bufB, 0, bytes, stream_);
  hipEvent_t e0, e1;
  hipEventCreate(&e0); hipEventCreate(&e1);

  // bestT[lo][hi]: fastest single launch for factors [lo, hi]
  std::vector<std::vector<float>> bestT(N, std::vector<float>(N, FLT_MAX));
  std::vector<std::vector<int>> bestK(N, std::vector<int>(N, -1));
  for (int hi = (int)N - 1; hi >= 0; hi--) {
    for (int lo = hi; lo >= 0 && hi - lo < (int)kMaxFused; lo--) {
      if (!useFusion() && lo != hi) break;
      const bool first = (hi == (int)N - 1), last = (lo == 0);
      DeviceInfo able = dev_;
      able.rulesOfThumb = false;      // every kernel able to run the group is timed
      auto cands = db_.candidates(p, lo, hi, first, last, able);
      for (int ki : cands) {
        const KernelInfo& k = db_.kernels()[ki];
        StepArgs a = makeStepArgs(p, lo, hi, first, last);
        a.in = bufA; a.in_batch = (uint64_t)p.M * a.Kin;
        a.out = bufB; a.out_batch = (uint64_t)p.M * a.Kout;
        if (a.y) { a.y = bufA; a.y_batch = (uint64_t)p.M * a.Kout; }
        for (uint32_t j = 0; j < a.nf; j++) a.f_batch[j] = p.strideF[hi - j];
        const float ms = timeLaunch(k, a, stream_, e0, e1);
        if (verbose) printf("[fastkron] tune [%d,%d] %s: %.4f ms\n", lo, hi, k.name.c_str(), ms);
        if (ms < bestT[lo][hi]) { bestT[lo][hi] = ms; bestK[lo][hi] = ki; }
      }
    }
  }
  hipEventDestroy(e0); hipEventDestroy(e1);
  hipFree(bufA); hipFree(bufB);

  // cost[h]: cheapest way to apply factors h .. 0 (h applied first); split[h]: lo of its first launch
  std::vector<float> cost(N, FLT_MAX);
  std::vector<int> split(N, -1);
  for (int h = 0; h < (int)N; h++) {
    for (int lo = 0; lo <= h; lo++) {
      if (bestK[lo][h] < 0) continue;
      const float rest = (lo == 0) ? 0.f : cost[lo - 1];
      if (rest == FLT_MAX) continue;
      if (bestT[lo][h] + rest < cost[h]) { cost[h] = bestT[lo][h] + rest; split[h] = lo; }
    }
  }
  if (split[N - 1] < 0) return fastKronKernelNotFound;
  Plan plan;
  for (int h = (int)N - 1; h >= 0;) {
    const int lo = split[h];
    plan.push_back(PlanStep{(uint32_t)lo, (uint32_t)h, bestK[lo][h]});
    h = lo - 1;
  }
  *best = plan;
  db_.storeTuned(p.str(), plan, cost[N - 1]);
  if (!dbPath_.empty()) db_.saveFile(dbPath_);
  if (verbose) {
    printf("[fastkron] tuned %s: %.4f ms", p.str().c_str(), cost[N - 1]);
    for (auto& s : plan) printf(" [%u,%u] %s", s.lo, s.hi, db_.kernels()[s.kernel].name.c_str());
    printf("\n");
  }
  return fastKronSuccess;
}

}  // namespace fk
