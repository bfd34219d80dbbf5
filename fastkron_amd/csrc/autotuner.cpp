// Fast tuning: time every compiled kernel on every contiguous sub-chain of the problem, pick the cheapest split of
// the chain with a dynamic program (the search of reference src/autotuner/autotuner.cpp:24-150,
// minExecTimeOfSeries over all sub-chains, with hipEvent timing in place of the reference's cudaEvent timing,
// src/kernel_db/cuda_kernel_db.cu:426-483) -- and, beyond the reference, do so for every way this library can
// rewrite the chain first: small factors merged into their Kronecker products or not, and every two-part plan
// (trailing factors on the contiguous blocks of the rows, leading factors across the blocks).  The candidates that
// survive are then timed end to end and the fastest is kept, also in the tuning file when one is set.
//
// Timing runs on buffers of the tuner's own, filled with values spread over [-1, 1], and rotates through enough
// operand sets that the 256 MB memory-side cache serves none of them: a candidate is timed as it will run on
// operands coming from HBM.
#include <algorithm>
#include <cfloat>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "handle.h"
#include "kernels/launch.h"

namespace fk {

namespace {

struct TuneBuffers {
  std::vector<void*> in, out;        // rotated operand sets
  void* t1 = nullptr;
  void* t2 = nullptr;
  size_t elems = 0;
  hipEvent_t e0 = nullptr, e1 = nullptr;
  ~TuneBuffers() {
    for (void* p : in) if (p) (void)hipFree(p);
    for (void* p : out) if (p) (void)hipFree(p);
    if (t1) (void)hipFree(t1);
    if (t2) (void)hipFree(t2);
    if (e0) (void)hipEventDestroy(e0);
    if (e1) (void)hipEventDestroy(e1);
  }
};

constexpr int kWarm = 2, kRuns = 6;

// One launch of `k` per run, each run on the next operand set.
float timeLaunch(const KernelInfo& k, StepArgs a, const TuneBuffers& B, hipStream_t stream) {
  if (k.check && !k.check(k, a)) return FLT_MAX;
  const size_t n = B.in.size();
  auto launch = [&](int i) {
    a.in = B.in[i % n]; a.out = B.out[i % n];
    if (a.y) a.y = B.out[(i + 1) % n];
    return k.launch(k, a, stream);
  };
  for (int i = 0; i < kWarm; i++) if (launch(i) != hipSuccess) return FLT_MAX;
  if (hipStreamSynchronize(stream) != hipSuccess) return FLT_MAX;
  (void)hipEventRecord(B.e0, stream);
  for (int i = 0; i < kRuns; i++) if (launch(kWarm + i) != hipSuccess) return FLT_MAX;
  (void)hipEventRecord(B.e1, stream);
  if (hipEventSynchronize(B.e1) != hipSuccess) return FLT_MAX;
  float ms = 0;
  (void)hipEventElapsedTime(&ms, B.e0, B.e1);
  return ms / kRuns;
}

}  // namespace

// Fastest series of launches for `q` as one chain: every kernel able to run a group is timed on it, then the
// dynamic program of the reference picks the groups.  Returns false when some factor has no kernel.
static bool tuneChain(Handle& h, const KronProblem& q, const TuneBuffers& B, bool fusion, bool verbose, Plan* plan,
                      float* total) {
  const uint32_t N = q.N;
  KernelDB& db = h.db();
  DeviceInfo able = h.device();
  able.rulesOfThumb = false;             // every kernel able to run a group is timed, whatever the online rules say
  std::vector<std::vector<float>> bestT(N, std::vector<float>(N, FLT_MAX));
  std::vector<std::vector<int>> bestK(N, std::vector<int>(N, -1));
  for (int hi = (int)N - 1; hi >= 0; hi--) {
    for (int lo = hi; lo >= 0 && hi - lo < (int)kMaxFused; lo--) {
      if (!fusion && lo != hi) break;
      const bool first = (hi == (int)N - 1), last = (lo == 0);
      for (int ki : db.candidates(q, lo, hi, first, last, able)) {
        const KernelInfo& k = db.kernels()[ki];
        StepArgs a = makeStepArgs(q, lo, hi, first, last);
        a.in = B.in[0]; a.in_batch = (uint64_t)q.M * a.Kin;
        a.out = B.out[0]; a.out_batch = (uint64_t)q.M * a.Kout;
        if (a.y) { a.y = B.out[0]; a.y_batch = (uint64_t)q.M * a.Kout; }
        a.scratch = B.t1; a.scratch_elems = B.elems; a.sync = h.syncArea();
        const float ms = timeLaunch(k, a, B, h.stream());
        if (verbose) printf("[fastkron] tune %s [%d,%d] %s: %.4f ms\n", q.str().c_str(), lo, hi, k.name.c_str(), ms);
        if (ms < bestT[lo][hi]) { bestT[lo][hi] = ms; bestK[lo][hi] = ki; }
      }
    }
  }
  // cost[h]: cheapest way to apply factors h .. 0 (h applied first); split[h]: lo of its first launch
  std::vector<float> cost(N, FLT_MAX);
  std::vector<int> split(N, -1);
  for (int hh = 0; hh < (int)N; hh++) {
    for (int lo = 0; lo <= hh; lo++) {
      if (bestK[lo][hh] < 0) continue;
      const float rest = (lo == 0) ? 0.f : cost[lo - 1];
      if (rest == FLT_MAX) continue;
      if (bestT[lo][hh] + rest < cost[hh]) { cost[hh] = bestT[lo][hh] + rest; split[hh] = lo; }
    }
  }
  if (split[N - 1] < 0) return false;
  plan->clear();
  for (int hh = (int)N - 1; hh >= 0;) {
    const int lo = split[hh];
    plan->push_back(PlanStep{(uint32_t)lo, (uint32_t)hh, bestK[lo][hh]});
    hh = lo - 1;
  }
  *total = cost[N - 1];
  return true;
}

// Fastest single launch for all of `q` (the trailing part of a two-part plan has no scratch for more).
static bool tuneSingle(Handle& h, const KronProblem& q, const TuneBuffers& B, bool verbose, Plan* plan, float* ms) {
  KernelDB& db = h.db();
  DeviceInfo able = h.device();
  able.rulesOfThumb = false;
  if (q.N > kMaxFused) return false;
  float best = FLT_MAX;
  int bestK = -1;
  for (int ki : db.candidates(q, 0, q.N - 1, true, true, able)) {
    const KernelInfo& k = db.kernels()[ki];
    StepArgs a = makeStepArgs(q, 0, q.N - 1, true, true);
    a.in = B.in[0]; a.in_batch = (uint64_t)q.M * a.Kin;
    a.out = B.out[0]; a.out_batch = (uint64_t)q.M * a.Kout;
    if (a.y) { a.y = B.out[0]; a.y_batch = (uint64_t)q.M * a.Kout; }
    a.scratch = B.t2; a.scratch_elems = B.elems; a.sync = h.syncArea();
    const float t = timeLaunch(k, a, B, h.stream());
    if (verbose) printf("[fastkron] tune %s [0,%u] %s: %.4f ms\n", q.str().c_str(), q.N - 1, k.name.c_str(), t);
    if (t < best) { best = t; bestK = ki; }
  }
  if (bestK < 0 || best == FLT_MAX) return false;
  plan->assign(1, PlanStep{0, q.N - 1, bestK});
  *ms = best;
  return true;
}

fastKronError Handle::tune(const KronProblem& p0, bool haveTemp2, Choice* best) {
  const bool verbose = getenv("FASTKRON_LOG") != nullptr;
  size_t yElems = 0, tmpElems = 0;
  fastKronError e = sizes(p0.M, p0.N, p0.P, p0.Q, &yElems, &tmpElems);
  if (e != fastKronSuccess) return e;
  TuneBuffers B;
  B.elems = std::max<size_t>(std::max(tmpElems, yElems), (size_t)p0.M * p0.K()) * p0.batch;
  const size_t bytes = B.elems * dtypeSize(p0.dt);
  // enough operand sets that a pass over them moves more than twice what the memory-side cache holds
  size_t nsets = (size_t)((640ull << 20) / (2 * bytes)) + 1;
  nsets = std::min<size_t>(std::max<size_t>(nsets, 1), 12);
  for (size_t i = 0; i < nsets; i++) {
    void *a = nullptr, *b = nullptr;
    if (hipMalloc(&a, bytes) != hipSuccess) { if (i == 0) return fastKronInvalidMemoryAccess; break; }
    if (hipMalloc(&b, bytes) != hipSuccess) { (void)hipFree(a); if (i == 0) return fastKronInvalidMemoryAccess; break; }
    B.in.push_back(a); B.out.push_back(b);
  }
  if (hipMalloc(&B.t1, bytes) != hipSuccess || hipMalloc(&B.t2, bytes) != hipSuccess) return fastKronInvalidMemoryAccess;
  for (size_t i = 0; i < B.in.size(); i++) {
    (void)launchFill(B.in[i], B.elems, p0.dt, stream_);
    (void)launchFill(B.out[i], B.elems, p0.dt, stream_);
  }
  (void)launchFill(B.t1, B.elems, p0.dt, stream_);
  (void)launchFill(B.t2, B.elems, p0.dt, stream_);
  if (hipEventCreate(&B.e0) != hipSuccess || hipEventCreate(&B.e1) != hipSuccess) return fastKronOtherError;
  // the device raises its clocks over the first tens of milliseconds of load: the fills above are repeated for that long
  {
    (void)hipEventRecord(B.e0, stream_);
    float ms = 0;
    for (int rounds = 0; rounds < 200 && ms < 40.f; rounds++) {
      (void)launchFill(B.t1, B.elems, p0.dt, stream_);
      (void)hipEventRecord(B.e1, stream_);
      (void)hipEventSynchronize(B.e1);
      (void)hipEventElapsedTime(&ms, B.e0, B.e1);
    }
  }

  // the problem on the tuner's buffers (compact strides), the factors are the caller's
  auto onBuffers = [&](KronProblem q) {
    q.X = B.in[0]; q.Z = B.out[0];
    q.strideX = (uint64_t)q.M * q.K(); q.strideZ = (uint64_t)q.M * q.L(); q.strideY = q.strideZ;
    if (q.Y && q.beta != 0.0) q.Y = (p0.Y == p0.Z) ? q.Z : B.out[B.out.size() > 1 ? 1 : 0];
    else q.Y = nullptr;
    return q;
  };

  struct Variant { Choice c; float estimate; float measured; };
  std::vector<Variant> variants;
  // op(X) = T: also everything the untransposed problem offers, behind a transposed copy of X (timed by itself here)
  float transposeMs = 0.f;
  KronProblem pT = p0;
  bool canTranspose = false;
  if (p0.opX == fastKronOp_T && useFusion()) {
    void* xt = nullptr;
    KronProblem src = onBuffers(p0);
    canTranspose = transposedProblem(src, B.t1, haveTemp2 ? B.t2 : nullptr, &pT, &xt);
    if (canTranspose) {
      for (int i = 0; i < kWarm; i++) (void)launchTransposeX(src, xt, pT.strideX);
      (void)hipStreamSynchronize(stream_);
      (void)hipEventRecord(B.e0, stream_);
      for (int i = 0; i < kRuns; i++) {
        src.X = B.in[i % B.in.size()];
        (void)launchTransposeX(src, xt, pT.strideX);
      }
      (void)hipEventRecord(B.e1, stream_);
      (void)hipEventSynchronize(B.e1);
      (void)hipEventElapsedTime(&transposeMs, B.e0, B.e1);
      transposeMs /= kRuns;
    }
  }
  for (int tx = 0; tx < (canTranspose ? 2 : 1); tx++)
  for (int merge = 0; merge < 2; merge++) {
    KronProblem base = p0;
    if (tx) { base.opX = fastKronOp_N; }
    KronProblem q = base;
    if (merge) {
      KronProblem m;
      if (!useFusion() || !mergeSmallFactors(base, &m)) continue;
      q = m;
    }
    q = onBuffers(q);
    const float extra = tx ? transposeMs : 0.f;
    Plan plan;
    float ms = 0;
    if (tuneChain(*this, q, B, useFusion(), verbose, &plan, &ms)) {
      Variant v; v.c.merge = merge != 0; v.c.split = 0; v.c.plan = plan; v.estimate = ms + extra; v.measured = FLT_MAX;
      v.c.transposeX = tx != 0;
      if (!(tx && !haveTemp2 && plan.size() != 1)) variants.push_back(v);
    }
    if (!useFusion() || !haveTemp2) continue;
    for (uint32_t g = 1; g < q.N; g++) {
      KronProblem q1, q2;
      if (!buildSplit(q, g, B.t1, B.t2, &q1, &q2)) continue;
      Plan plan1, plan2;
      float ms1 = 0, ms2 = 0;
      if (!tuneSingle(*this, q1, B, verbose, &plan1, &ms1)) continue;
      if (!tuneChain(*this, q2, B, true, verbose, &plan2, &ms2)) continue;
      if (plan2.size() > 2 && p0.Y == p0.Z && p0.beta != 0.0) continue;
      Variant v; v.c.merge = merge != 0; v.c.split = g; v.estimate = ms1 + ms2 + extra; v.measured = FLT_MAX;
      v.c.transposeX = tx != 0;
      for (auto& s : plan1) v.c.plan.push_back(PlanStep{s.lo + g, s.hi + g, s.kernel});
      for (auto& s : plan2) v.c.plan.push_back(s);
      variants.push_back(v);
    }
  }
  if (variants.empty()) return fastKronKernelNotFound;

  // The estimates are sums of launches timed alone; the best few are run end to end, as the call will run them.
  std::sort(variants.begin(), variants.end(), [](const Variant& a, const Variant& b) { return a.estimate < b.estimate; });
  const size_t finalists = std::min<size_t>(variants.size(), 4);
  const std::string savedPlan = lastPlan_;
  for (size_t vi = 0; vi < finalists; vi++) {
    Variant& v = variants[vi];
    auto run = [&](int i) {
      KronProblem q = p0;
      const size_t n = B.in.size();
      q.X = B.in[i % n]; q.Z = B.out[i % n];
      q.strideX = (uint64_t)q.M * q.K(); q.strideZ = (uint64_t)q.M * q.L(); q.strideY = q.strideZ;
      if (q.Y && q.beta != 0.0) q.Y = (p0.Y == p0.Z) ? q.Z : B.out[(i + 1) % n];
      else q.Y = nullptr;
      return runChoice(q, v.c, B.t1, haveTemp2 ? B.t2 : nullptr, nullptr);
    };
    bool ok = true;
    for (int i = 0; i < kWarm && ok; i++) ok = run(i) == fastKronSuccess;
    if (!ok || hipStreamSynchronize(stream_) != hipSuccess) continue;
    (void)hipEventRecord(B.e0, stream_);
    for (int i = 0; i < kRuns && ok; i++) ok = run(kWarm + i) == fastKronSuccess;
    (void)hipEventRecord(B.e1, stream_);
    if (hipEventSynchronize(B.e1) != hipSuccess || !ok) continue;
    float ms = 0;
    (void)hipEventElapsedTime(&ms, B.e0, B.e1);
    v.measured = ms / kRuns;
    if (verbose) {
      printf("[fastkron] tune %s: transposeX=%d merge=%d split=%u estimate %.4f ms, end to end %.4f ms:", p0.str().c_str(),
             (int)v.c.transposeX, (int)v.c.merge, v.c.split, v.estimate, v.measured);
      for (auto& s : v.c.plan) printf(" [%u,%u] %s", s.lo, s.hi, db_.kernels()[s.kernel].name.c_str());
      printf("\n");
    }
  }
  lastPlan_ = savedPlan;
  const Variant* win = nullptr;
  for (size_t vi = 0; vi < finalists; vi++)
    if (variants[vi].measured != FLT_MAX && (!win || variants[vi].measured < win->measured)) win = &variants[vi];
  if (!win) return fastKronKernelNotFound;
  *best = win->c;
  db_.storeTuned(p0.str(), win->c.plan, win->measured, win->c.merge ? 1 : 0, win->c.split, win->c.transposeX ? 1 : 0);
  if (!dbPath_.empty()) db_.saveFile(dbPath_);
  return fastKronSuccess;
}

}  // namespace fk
