#include "handle.h"
#include "kernels/launch.h"

#include <algorithm>
#include <cstdio>
#include <cstdlib>
#include <cstring>

namespace fk {

static int logLevel() {
  static int lvl = -1;
  if (lvl < 0) {
    const char* e = getenv("FASTKRON_LOG");          // reference src/env/env.cpp:57-65
    lvl = 0;
    if (e && (!strcmp(e, "INFO") || !strcmp(e, "info"))) lvl = 1;
    if (e && (!strcmp(e, "DEBUG") || !strcmp(e, "debug"))) lvl = 2;
  }
  return lvl;
}

Handle::Handle(uint32_t backends) : backends_(backends) {
  // the plans that ship with the library first, then the user's own file on top of them
  const std::string shipped = KernelDB::shippedPath();
  if (!shipped.empty()) db_.loadFile(shipped, true);
  if (const char* e = getenv("FASTKRON_CHUNK_MB")) chunkMB_ = atol(e);          // read when the handle is created
  dbPath_ = KernelDB::defaultPath();
  if (!dbPath_.empty()) db_.loadFile(dbPath_);
}

Handle::~Handle() {
  if (mergeWs_ && mergeWsOwned_) (void)hipFree(mergeWs_);
  if (mergeWsEvent_) (void)hipEventDestroy(mergeWsEvent_);
}

void Handle::setPlanOnly(bool on) {
  planOnly_ = on;
  if (!on && mergeWs_ && !mergeWsOwned_) {
    // the stand-in address of plan-only mode must never reach a launch: without it initHIP allocates the real one
    mergeWs_ = nullptr; mergeWsBytes_ = 0;
  }
  if (on && !dev_.valid) {
    // the device the library is written for: 256 compute units, 160 KB of LDS per workgroup
    dev_.cus = 256; dev_.ldsPerBlock = 160 * 1024; dev_.waveSize = 64; dev_.xcdRoundRobin = true;
  }
  if (on && !mergeWs_) {
    // never dereferenced: in this mode no launch is made
    mergeWs_ = (void*)(uintptr_t)0x7f0000000000ull;
    mergeWsBytes_ = (size_t)kMaxMergeGroups * 64 * 64 * sizeof(double);
    mergeWsOwned_ = false;
  }
}

void Handle::setTunedDB(const char* path) {
  dbPath_ = path ? path : "";
  if (!dbPath_.empty()) db_.loadFile(dbPath_);
}

fastKronError Handle::ensureDevice() {
  if (dev_.valid) return fastKronSuccess;
  int d = 0;
  if (hipGetDevice(&d) != hipSuccess) return fastKronBackendNotAvailable;
  hipDeviceProp_t prop;
  if (hipGetDeviceProperties(&prop, d) != hipSuccess) return fastKronBackendNotAvailable;
  dev_.device = d;
  dev_.cus = prop.multiProcessorCount;
  dev_.ldsPerBlock = (int)prop.sharedMemPerBlock;
  dev_.waveSize = prop.warpSize;
  dev_.clockKHz = prop.clockRate;
  strncpy(dev_.arch, prop.gcnArchName, sizeof(dev_.arch) - 1);
  dev_.valid = true;
  if (logLevel() >= 1)
    printf("[fastkron] device %d %s: %d CUs, %d B LDS per workgroup, wave %d, %d kHz\n", d, dev_.arch,
           dev_.cus, dev_.ldsPerBlock, dev_.waveSize, dev_.clockKHz);
  return fastKronSuccess;
}

fastKronError Handle::initHIP(void* ptrToStream) {
  if (!hasBackend(fastKronBackend_HIP)) return fastKronBackendNotAvailable;
  stream_ = ptrToStream ? *(hipStream_t*)ptrToStream : nullptr;
  hipInit_ = true;
  fastKronError e = ensureDevice();
  if (e != fastKronSuccess) return e;
  // the static scratch array of the calls that must not allocate: its address on this GPU is looked up here, once
  { void* p = nullptr; (void)staticScratchForCurrentDevice(&p); }
  // workspace for merged factors (kMaxMergeGroups products of at most 64x64 doubles); allocated here so that
  // the gemkm / gekmm calls themselves never allocate
  if (mergeWs_ && !mergeWsOwned_) { mergeWs_ = nullptr; mergeWsBytes_ = 0; }       // plan-only stand-in
  if (!mergeWs_) {
    mergeWsBytes_ = (size_t)kMaxMergeGroups * 64 * 64 * sizeof(double);
    // (behind the merged factors: the counter area of the kernels that synchronise their workgroups, zero once and
    // left zero by every launch that uses it)
    if (hipMalloc(&mergeWs_, mergeWsBytes_ + kSyncAreaBytes) != hipSuccess ||
        hipMemset((char*)mergeWs_ + mergeWsBytes_, 0, kSyncAreaBytes) != hipSuccess) {
      if (mergeWs_) (void)hipFree(mergeWs_);
      mergeWs_ = nullptr; mergeWsBytes_ = 0;
    }
    mergeWsOwned_ = mergeWs_ != nullptr;
    // how the device places workgroups on its XCDs, recorded once (the counter area serves as the 1 KB this needs
    // and is zeroed again afterwards)
    if (mergeWs_) {
      uint32_t* area = (uint32_t*)((char*)mergeWs_ + mergeWsBytes_);
      dev_.xcdRoundRobin = kmm4x6TwoPhasePlacementHolds(area, stream_);
      if (hipMemsetAsync(area, 0, kSyncAreaBytes, stream_) != hipSuccess || hipStreamSynchronize(stream_) != hipSuccess)
        dev_.xcdRoundRobin = false;
    }
    if (mergeWs_ && hipEventCreateWithFlags(&mergeWsEvent_, hipEventDisableTiming) != hipSuccess) mergeWsEvent_ = nullptr;
  }
  return fastKronSuccess;
}

fastKronError Handle::syncError(uint32_t* word) {
  *word = 0;
  if (planOnly_ || !mergeWs_ || !mergeWsOwned_) return fastKronSuccess;
  uint32_t* dev = (uint32_t*)syncArea() + 1;
  if (hipMemcpyAsync(word, dev, sizeof(uint32_t), hipMemcpyDeviceToHost, stream_) != hipSuccess ||
      hipMemsetAsync(dev, 0, sizeof(uint32_t), stream_) != hipSuccess || hipStreamSynchronize(stream_) != hipSuccess)
    return fastKronOtherError;
  return fastKronSuccess;
}

// The merged-factor workspace is the one piece of device state the handle owns.  A call on a new stream may
// overwrite it while launches of an earlier call on another stream still read it; the new stream is therefore made
// to wait for everything the old stream has been given so far.  (Nothing is recorded while either stream is being
// captured into a graph: a handle that is used under capture stays on one stream.)
void Handle::orderWorkspaceBehind(hipStream_t next) {
  if (!mergeWsUsed_ || !mergeWsEvent_ || next == mergeWsStream_) return;
  hipStreamCaptureStatus c0 = hipStreamCaptureStatusNone, c1 = hipStreamCaptureStatusNone;
  (void)hipStreamIsCapturing(mergeWsStream_, &c0);
  (void)hipStreamIsCapturing(next, &c1);
  if (c0 == hipStreamCaptureStatusNone && c1 == hipStreamCaptureStatusNone &&
      hipEventRecord(mergeWsEvent_, mergeWsStream_) == hipSuccess)
    (void)hipStreamWaitEvent(next, mergeWsEvent_, 0);
  mergeWsUsed_ = false;
}

fastKronError Handle::setStream(fastKronBackend backend, void* ptrToStream) {
  if (!ptrToStream) return fastKronInvalidArgument;                    // reference handle.cpp:94
  if (!hasBackend(backend)) return fastKronBackendNotAvailable;        // reference handle.cpp:95
  if (backend != fastKronBackend_HIP) return fastKronBackendNotAvailable;
  hipStream_t next = *(hipStream_t*)ptrToStream;
  if (next != stream_ && !planOnly_) orderWorkspaceBehind(next);
  stream_ = next;
  return fastKronSuccess;
}

// Columns of every step's output, widths[i] for the step of factor i.
static void stepWidths(uint32_t N, const uint32_t* Ps, const uint32_t* Qs, uint64_t* widths) {
  uint64_t w = 1;
  for (uint32_t i = 0; i < N; i++) w *= Ps[i];
  for (int i = (int)N - 1; i >= 0; i--) { w = (w / Ps[i]) * Qs[i]; widths[i] = w; }
}

// reference src/handle/handle.cpp:305-342,375-388: the temporary holds the widest step output
// (X itself is not counted), except for N == 1 where it is max(K, L) columns.
fastKronError Handle::sizes(uint32_t M, uint32_t N, const uint32_t* Ps, const uint32_t* Qs,
                            size_t* yElems, size_t* tmpElems) {
  if (!yElems || !tmpElems) return fastKronInvalidArgument;
  if (N == 0 || N > kMaxFactors || !Ps || !Qs) return fastKronInvalidKMMProblem;
  uint64_t K = 1, L = 1;
  for (uint32_t i = 0; i < N; i++) { K *= Ps[i]; L *= Qs[i]; }
  *yElems = (size_t)M * L;
  if (N == 1) { *tmpElems = (size_t)M * std::max(K, L); return fastKronSuccess; }
  uint64_t w[kMaxFactors];
  stepWidths(N, Ps, Qs, w);
  *tmpElems = (size_t)M * *std::max_element(w, w + N);
  return fastKronSuccess;
}

// reference src/handle/handle.cpp:390-408
fastKronError Handle::sizesForward(uint32_t M, uint32_t N, const uint32_t* Ps, const uint32_t* Qs,
                                   size_t* yElems, size_t* interElems) {
  if (!yElems || !interElems) return fastKronInvalidArgument;
  if (N == 0 || N > kMaxFactors || !Ps || !Qs) return fastKronInvalidKMMProblem;
  uint64_t w[kMaxFactors];
  stepWidths(N, Ps, Qs, w);
  for (uint32_t i = 1; i < N; i++) interElems[i - 1] = (size_t)M * w[i];
  *yElems = (size_t)M * w[0];
  return fastKronSuccess;
}

fastKronError Handle::xgemm(KronProblem p, fastKronBackend backend, void* temp1, void* temp2, const CallWorkspace* ws) {
  callWs_ = ws != nullptr;
  // argument checks in the order of reference src/handle/handle.cpp:116-122
  if (!p.forward) {
    if (p.Z == nullptr || temp1 == nullptr || !hasBackend(backend)) return fastKronInvalidArgument;
    if (p.Z == p.Y && temp2 == nullptr) return fastKronInvalidArgument;
  } else {
    if (p.Z == nullptr || !hasBackend(backend)) return fastKronInvalidArgument;
  }
  if (backend != fastKronBackend_HIP) return fastKronInvalidArgument;
  if (p.N == 0 || p.N > kMaxFactors || p.M == 0 || p.batch == 0) return fastKronInvalidKMMProblem;
  for (uint32_t i = 0; i < p.N; i++)
    if (p.P[i] == 0 || p.Q[i] == 0 || p.F[i] == nullptr) return fastKronInvalidKMMProblem;
  if (p.X == nullptr) return fastKronInvalidArgument;
  if (p.forward && p.N > 1)
    for (uint32_t i = 0; i + 1 < p.N; i++) if (!p.inter[i]) return fastKronInvalidArgument;

  // A KMM with a single column is the MKM of the same vector with transposed factors
  // (reference src/handle/handle.cpp:134-138).
  if (p.mm == MMType::KMM && p.M == 1) {
    p.mm = MMType::MKM;
    p.opF = (p.opF == fastKronOp_N) ? fastKronOp_T : fastKronOp_N;
    p.opX = fastKronOp_N;
  }

  fastKronError e = planOnly_ ? fastKronSuccess : ensureDevice();
  if (e != fastKronSuccess) return e;
  launchLog_.clear();

  // 1. A tuned record under the call's own problem string says everything: whether small factors are merged,
  //    whether the chain runs as a two-part plan, and which kernel runs which factors.  With tuning switched on a
  //    problem without a record is tuned here, once.  A record that does not fit the call's buffers falls through
  //    to the online selection.
  if (!p.forward) {
    Choice c;
    bool have = lookupChoice(p, &c);
    // (a GeKMM that runs as a GeMKM is tuned as that GeMKM, below)
    const bool asMKM = p.mm == MMType::KMM && useFusion() && temp2 && viaMKMOnline(p);
    if (!have && canTune() && !planOnly_ && !ws && !asMKM) {
      // a tuner that cannot run (no memory for its operand sets, no events) leaves the problem without a record:
      // the call then runs on the online selection, as it would untuned
      have = tune(p, temp2 != nullptr, &c) == fastKronSuccess;
    }
    if (have) {
      e = runChoice(p, c, temp1, temp2, ws);
      if (e != fastKronKernelNotFound) return e;
    }
  }

  // 2. Online selection.  A GeKMM whose X is stored transposed is the GeMKM of that buffer with a transposed result:
  //    the whole-row GeMKM kernels then apply, and one transposition at the end writes Z.
  //    With few columns that pays even when X has to be transposed first.
  if (p.mm == MMType::KMM && !p.forward && useFusion() && temp2 && viaMKMOnline(p)) {
    e = runViaMKM(p, backend, temp1, temp2, ws);
    if (e != fastKronKernelNotFound) return e;
  }
  //    With op(X) = T otherwise the question whether to transpose X ahead of the launches.
  if (p.opX == fastKronOp_T && !p.forward && useFusion()) {
    KronProblem pn;
    void* xt = nullptr;
    if (transposedProblem(p, temp1, temp2, &pn, &xt) && transposeFirstOnline(p, pn, temp1, temp2, ws)) {
      if (!planOnly_) {
        hipError_t he = launchTransposeX(p, xt, pn.strideX);
        if (he != hipSuccess) return fastKronInvalidArgument;
      }
      e = runOnline(pn, temp1, temp2, ws);
      if (e == fastKronSuccess) noteTranspose(p);
      return e;
    }
  }
  return runOnline(p, temp1, temp2, ws);
}

// Online rule for a GeKMM with op(X) = T: as the GeMKM of the same buffer plus a transposition of the result.
// FASTKRON_KMM_VIA_MKM=0 / 1 forces the answer.
bool Handle::viaMKMOnline(const KronProblem& p) const {
  static const int forced = [] { const char* e = getenv("FASTKRON_KMM_VIA_MKM"); return e ? atoi(e) : -1; }();
  if (p.L() >= (1ull << 32) || p.M < 2) return false;
  if (forced >= 0) return forced != 0;
  if (p.opX != fastKronOp_T) {
    // X has to be transposed as well, two more passes over the data: fp32 with fewer than 64 columns, square factors up
    // to 32x32 and at least 64 MB of X (sgekmm 16 x 8^8 2.91 -> 1.55 ms, 16 x 16^6 1.86 -> 1.55, 16 x 32^5 5.67 -> 4.36;
    // 32 x 8^6, 33 MB: no difference, 48 x 16^4, 13 MB: 23 -> 37 us; fp64 loses 1.1 to 1.6 times)
    if (p.dt != DType::F32 || p.M >= 64 || (uint64_t)p.M * p.K() * 4 < (64ull << 20)) return false;
    for (uint32_t i = 0; i < p.N; i++) if (p.P[i] != p.Q[i] || p.P[i] > 32) return false;
    return true;
  }
  // Measured on the reference's published shapes with both operands transposed.  Square factors up to 32x32 gain 1.3
  // to 2.8 times in fp32 (sgekmm 1024 x 8^5 171 -> 112 us, 16 x 8^8 3.34 -> 1.20 ms) and up to 1.2 times in fp64.  With
  // fewer than 64 columns the GeKMM kernels move short pieces and larger factors gain as well (sgekmm 16 x 64^4 and
  // 16 x 128^3 1.27 times, fp64 up to 1.12 times); from 64 columns on, 64x64 and 128x128 factors are within 3 % in
  // fp32 or lose up to 10 % (320 x 128^3), fp64 chains of three 64x64 factors gain 1.1 times.
  uint32_t maxP = 0;
  for (uint32_t i = 0; i < p.N; i++) {
    if (p.P[i] != p.Q[i]) return false;
    if (p.P[i] > maxP) maxP = p.P[i];
  }
  return maxP <= 32 || p.M < 64 || (p.dt == DType::F64 && maxP == 64 && p.N >= 3);
}

// Z (L x M) = transpose(R) + beta * Y with R (M x L) = alpha * X^T (F_1 (x) ... (x) F_N) computed by the GeMKM path
// into temp1; the GeMKM uses temp2 and, when Z is free to be overwritten and large enough, Z as its temporaries.
fastKronError Handle::runViaMKM(const KronProblem& p, fastKronBackend backend, void* temp1, void* temp2, const CallWorkspace* ws) {
  size_t yElems = 0, tmpElems = 0;
  if (sizes(p.M, p.N, p.P, p.Q, &yElems, &tmpElems) != fastKronSuccess) return fastKronKernelNotFound;
  const uint64_t ML = (uint64_t)p.M * p.L();
  KronProblem q = p;
  q.mm = MMType::MKM;
  q.opF = (p.opF == fastKronOp_N) ? fastKronOp_T : fastKronOp_N;      // KMM factors are stored Q x P
  q.opX = fastKronOp_N;
  q.Z = temp1; q.strideZ = p.batch > 1 ? ML : 0;
  q.Y = nullptr; q.strideY = 0; q.beta = 0.0;
  q.zReadNext = true;
  const bool zFree = !(p.Y == p.Z && p.beta != 0.0);
  void* zTemp = (zFree && tmpElems <= ML && (p.batch == 1 || p.strideZ >= ML)) ? p.Z : nullptr;
  fastKronError e;
  const bool copyX = p.opX != fastKronOp_T;
  if (copyX) {
    // X (K x M) goes to temp2 as M x K first; the GeMKM then has Z and, once its first launch has read it, temp2
    const uint64_t MK = (uint64_t)p.M * p.K();
    if (!zTemp || MK > tmpElems || p.K() >= (1ull << 32)) return fastKronKernelNotFound;
    const uint32_t nb = (p.batch > 1 && p.strideX != 0) ? p.batch : 1;         // a shared X is transposed once
    q.X = temp2; q.strideX = nb > 1 ? MK : 0; q.xJustWritten = true;
    if (!planOnly_) {
      constexpr uint32_t kMaxGridBatch = 65535;
      const size_t es = dtypeSize(p.dt);
      for (uint32_t b0 = 0; b0 < nb; b0 += kMaxGridBatch) {
        const uint32_t n = nb - b0 < kMaxGridBatch ? nb - b0 : kMaxGridBatch;
        if (launchTranspose((const char*)p.X + (size_t)b0 * p.strideX * es, (char*)temp2 + (size_t)b0 * MK * es, (uint32_t)p.K(), p.M, n,
                            p.strideX, MK, p.dt, stream_) != hipSuccess) return fastKronInvalidArgument;
      }
    }
    e = xgemm(q, backend, zTemp, temp2, ws);
  } else {
    e = xgemm(q, backend, temp2, zTemp, ws);
  }
  if (e != fastKronSuccess) return e;
  const size_t semi = lastPlan_.find(';');
  const std::string ty = p.dt == DType::F32 ? "f" : "d";
  lastPlan_ = p.str() + (copyX ? ";" + std::to_string(p.N - 1) + "-" + std::to_string(p.N - 1) + ":transpose_hip_gfx950_256_" + ty + "_x" : "") +
              (semi == std::string::npos ? "" : lastPlan_.substr(semi)) + ";0-0:transpose_hip_gfx950_256_" + ty + "_z";
  if (planOnly_) return fastKronSuccess;
  constexpr uint32_t kMaxGridBatch = 65535;
  const size_t es = dtypeSize(p.dt);
  const void* y = (p.beta != 0.0) ? p.Y : nullptr;
  // Z goes to the caller: streamed from the size on at which the kernels stream their results (Handle::execute)
  const bool streamZ = !p.zReadNext && (uint64_t)(y ? 3 : 2) * ML * p.batch * es >= (96ull << 20);
  for (uint32_t b0 = 0; b0 < p.batch; b0 += kMaxGridBatch) {
    const uint32_t n = p.batch - b0 < kMaxGridBatch ? p.batch - b0 : kMaxGridBatch;
    hipError_t he = launchTransposeAdd((const char*)temp1 + (size_t)b0 * ML * es, (char*)p.Z + (size_t)b0 * p.strideZ * es, p.M,
                                       (uint32_t)p.L(), n, ML, p.strideZ, y ? (const char*)y + (size_t)b0 * p.strideY * es : nullptr,
                                       p.strideY, p.beta, p.dt, stream_, streamZ);
    if (he != hipSuccess) return fastKronInvalidArgument;
  }
  return fastKronSuccess;
}

// How many launches the last planned call makes (entries of lastPlan_).
static size_t countLaunches(const std::string& plan) {
  size_t n = 0;
  for (char ch : plan) if (ch == ';') n++;
  return n;
}

// The problem with X already transposed into `xt` (temp2, or temp1 when there is no temp2): false when X does not
// fit there.  The transposed copy has the compact layout, batch entries one after the other.
bool Handle::transposedProblem(const KronProblem& p, void* temp1, void* temp2, KronProblem* pn, void** xt) const {
  if (p.opX != fastKronOp_T) return false;
  size_t yElems = 0, tmpElems = 0;
  if (sizes(p.M, p.N, p.P, p.Q, &yElems, &tmpElems) != fastKronSuccess) return false;
  if ((size_t)p.M * p.K() > tmpElems) return false;                  // shrinking chains: X is larger than a temporary
  *xt = temp2 ? temp2 : temp1;
  if (!*xt) return false;
  *pn = p;
  pn->opX = fastKronOp_N;
  pn->X = *xt;
  pn->xJustWritten = true;
  pn->strideX = (p.batch > 1 && p.strideX != 0) ? (uint64_t)p.M * p.K() : 0;
  return true;
}

hipError_t Handle::launchTransposeX(const KronProblem& p, void* xt, uint64_t xtStride) {
  // MKM: op(X) = T means the buffer holds K x M; KMM: it holds M x K (reference tests/testBase.h:272-273,303-304)
  const uint32_t R = p.mm == MMType::MKM ? (uint32_t)p.K() : p.M;
  const uint32_t C = p.mm == MMType::MKM ? p.M : (uint32_t)p.K();
  const uint32_t nb = (p.batch > 1 && p.strideX != 0) ? p.batch : 1;       // a shared X is transposed once
  constexpr uint32_t kMaxGridBatch = 65535;
  for (uint32_t b0 = 0; b0 < nb; b0 += kMaxGridBatch) {
    const uint32_t n = nb - b0 < kMaxGridBatch ? nb - b0 : kMaxGridBatch;
    const size_t es = dtypeSize(p.dt);
    hipError_t he = launchTranspose((const char*)p.X + (size_t)b0 * p.strideX * es, (char*)xt + (size_t)b0 * xtStride * es, R, C, n,
                                    p.strideX, xtStride, p.dt, stream_);
    if (he != hipSuccess) return he;
  }
  return hipSuccess;
}

// lastPlan_ of a call that transposed X first: the call's own problem string, the transposition as a launch ahead
// of the last factor, then the launches of the untransposed problem.
void Handle::noteTranspose(const KronProblem& p) {
  const size_t semi = lastPlan_.find(';');
  const std::string rest = semi == std::string::npos ? "" : lastPlan_.substr(semi);
  lastPlan_ = p.str() + ";" + std::to_string(p.N - 1) + "-" + std::to_string(p.N - 1) + ":transpose_hip_gfx950_256_" +
              (p.dt == DType::F32 ? "f" : "d") + "_x" + rest;
}

// Online rule for op(X) = T: transpose first when that plus the launches of the untransposed problem are no more
// launches (passes over the data) than the kernels that read a transposed X need.  Both plans are laid out in
// plan-only mode on the call's own buffers; the answer is kept per problem.
bool Handle::transposeFirstOnline(const KronProblem& p, const KronProblem& pn, void* temp1, void* temp2,
                                  const CallWorkspace* ws) {
  // Lays a problem out in plan-only mode on the call's own buffers and counts its launches.
  auto plannedLaunches = [&](const KronProblem& q, bool* ok) {
    const bool wasPlanOnly = planOnly_;
    const std::string savedPlan = lastPlan_, savedLog = launchLog_;
    planOnly_ = true;
    *ok = runOnline(q, temp1, temp2, ws) == fastKronSuccess;
    const size_t n = countLaunches(lastPlan_);
    const std::string plan = lastPlan_;
    planOnly_ = wasPlanOnly;
    lastPlan_ = savedPlan; launchLog_ = savedLog;
    return std::make_pair(n, plan);
  };
  const std::string ck = p.str() + (temp2 ? "_t2" : "_t1");
  auto it = transposeCache_.find(ck);
  bool yes;
  if (it != transposeCache_.end()) yes = it->second;
  else {
    bool okT = false, okN = false;
    auto planT = plannedLaunches(p, &okT);
    size_t nT = planT.first;
    // a first launch that reads a transposed X through the padded step with a large factor counts twice: in the MKM layout
    // always (tuned plans: 128x128 chains run 1.3 to 3.3 times faster behind a transposed copy, pairs of single 64x64
    // steps 1.3 to 1.4 times); in the KMM layout, where that step reads the transposed X along its rows, only while X
    // stays in the caches (up to 64 MB the copy is ahead by 8 to 14 %, beyond that behind by 5 to 30 %)
    const uint64_t xBytes = p.M * p.K() * (p.dt == DType::F32 ? 4 : 8) * (uint64_t)(p.batch ? p.batch : 1);
    if (okT && p.P[p.N - 1] >= 64 && (p.mm == MMType::MKM || xBytes <= (64ull << 20))) {
      const std::string& pl = planT.second;
      const size_t s0 = pl.find(':');
      if (s0 != std::string::npos && pl.compare(s0 + 1, 6, "gekmm_") == 0 && pl.find("anyxany", s0) < pl.find(';', s0)) nT++;
    }
    const size_t nN = plannedLaunches(pn, &okN).first;
    // with equal counts the copy goes first, except in the KMM layout with fewer than 64 columns, where the copy cannot
    // run on whole 64-wide tiles with 16-byte accesses (sgekmm 16x16^4 with 256 and 1024 columns: 1.26 times faster
    // behind the copy; 16 columns, 16x16^6: 1.16 times slower; factors below 16x16 read a transposed X too slowly in any
    // case)
    const bool copyOnTie = p.mm == MMType::MKM || p.M >= 64 || p.P[p.N - 1] < 16;
    yes = okN && (!okT || (copyOnTie ? 1 + nN <= nT : 1 + nN < nT));
    transposeCache_[ck] = yes;           // the preference of the shape; the buffers of each call are checked below
  }
  if (!yes) return false;
  // Without a second temporary the transposed copy sits in temp1, which a plan of several launches writes while its
  // first launch still reads the copy.  How many launches the untransposed problem takes depends on the call's own
  // buffers (a misaligned operand moves it off the whole-row kernels), so this is asked on every call.
  if (!temp2) {
    bool okN = false;
    if (plannedLaunches(pn, &okN).first != 1 || !okN) return false;
  }
  return true;
}

fastKronError Handle::runOnline(KronProblem p, void* temp1, void* temp2, const CallWorkspace* ws) {
  fastKronError e;
  {
    KronProblem merged;
    if (useFusion() && mergeSmallFactors(p, &merged, ws)) p = merged;
  }

  Plan plan;
  const std::string key = p.str();
  bool have = false;
  // (records without the merge / split fields are keyed by the chain as the online rules rewrite it)
  if (!p.forward) {
    int merge = -1;
    have = db_.lookupTuned(key, &plan, &merge) && merge < 0 && db_.validPlan(p, plan, dev_);
  }
  // chains longer than one whole-block kernel: the two-part plan, when the problem and the buffers allow it
  if (!have && useFusion()) {
    e = trySplitLeadingTrailing(p, temp1, temp2);
    if (e != fastKronKernelNotFound) return e;
  }
  if (!have) {
    const std::string ck = key + (p.forward ? "_fwd" : "") + (useFusion() ? "" : "_nofuse");
    auto it = planCache_.find(ck);
    if (it != planCache_.end()) plan = it->second;
    else {
      plan = db_.selectOnline(p, dev_, useFusion());
      planCache_[ck] = plan;
      if (logLevel() >= 1) {
        printf("[fastkron] %s ->", key.c_str());
        for (auto& s : plan) printf(" [%u,%u] %s", s.lo, s.hi, db_.kernels()[s.kernel].name.c_str());
        printf("\n");
      }
    }
  }
  // Kernel-specific requirements on the actual buffers (alignment, strides): a kernel that refuses them is left out
  // and the selection repeated (the 16-byte accesses of the whole-row and wide kernels need aligned operands, the
  // streaming kernels behind them in the list do not); one generic launch per factor is the last resort.
  std::vector<int> refusedKernels;
  for (int attempt = 0;; attempt++) {
    int refused = -1;
    e = execute(p, plan, temp1, temp2, true, &refused);
    if (e != fastKronKernelNotFound) break;
    if (refused < 0 || attempt >= 8 || db_.kernels()[refused].P == 0) {
      plan.clear();
      for (int i = (int)p.N - 1; i >= 0; i--) plan.push_back(PlanStep{(uint32_t)i, (uint32_t)i, db_.genericKernel(p.dt)});
      e = fastKronSuccess;
      break;
    }
    refusedKernels.push_back(refused);
    // (cached like the first selection, under the problem and the kernels left out)
    std::string rk = key + (p.forward ? "_fwd" : "") + (useFusion() ? "" : "_nofuse") + "|without";
    for (int k : refusedKernels) rk += ":" + std::to_string(k);
    auto it = planCache_.find(rk);
    if (it != planCache_.end()) plan = it->second;
    else { plan = db_.selectOnline(p, dev_, useFusion(), &refusedKernels); planCache_[rk] = plan; }
  }
  if (e != fastKronSuccess) return e;
  lastPlan_ = key;
  for (auto& s : plan)
    lastPlan_ += ";" + std::to_string(s.lo) + "-" + std::to_string(s.hi) + ":" + db_.kernels()[s.kernel].name;
  if (planOnly_) { launchLog_.clear(); return execute(p, plan, temp1, temp2, true); }
  return execute(p, plan, temp1, temp2);
}

static bool isPow2(uint32_t v) { return v && !(v & (v - 1)); }

bool Handle::mergeSmallFactors(const KronProblem& p, KronProblem* out, const CallWorkspace* ws) {
  void* const wsBase = ws ? ws->merge : mergeWs_;
  const size_t wsBytes = ws ? ws->mergeBytes : mergeWsBytes_;
  if (!wsBase || p.forward || p.N < 2) return false;
  // fp32 GeKMM already fuses small factors in registers; everything else gains from merging
  if (p.mm == MMType::KMM && p.dt == DType::F32) return false;
  if (p.batch > 1) for (uint32_t i = 0; i < p.N; i++) if (p.strideF[i] != 0) return false;
  // fp32: 16x16 products.  fp64: 64x64 products when the chain holds 8x8 (or 32x32) factors, which do not pack into
  // 16x16 ones; chains of 2x2 and 4x4 factors alone run faster as 16x16 products (a quarter of the multiplications,
  // and the wave-per-block kernel for three 16x16 factors: dgemkm 1024x4^8 0.57 -> 0.47 ms, 1024x4^6 60 -> 20 us).
  uint32_t target = 16;
  // fp64 rows of five 8x8 factors have a whole-row kernel of their own (one launch, one pass, an eighth of the
  // multiplications of 64x64 products): the chain stays as it is where that kernel is the online choice
  if (p.dt == DType::F64 && p.mm == MMType::MKM && p.N == 5) {
    bool all8 = true;
    for (uint32_t i = 0; i < p.N; i++) all8 = all8 && p.P[i] == 8 && p.Q[i] == 8;
    if (all8) {
      const Plan whole = db_.selectOnline(p, dev_, true);
      if (whole.size() == 1 && whole[0].lo == 0 && whole[0].hi == 4) return false;
    }
  }
  if (p.dt == DType::F64) {
    for (uint32_t i = 0; i < p.N; i++)
      if (p.P[i] == p.Q[i] && (p.P[i] == 8 || p.P[i] == 32)) target = 64;
  }
  // groups of adjacent square power-of-two factors, formed from the last factor towards the first, each as
  // large as fits the target size
  // fp64 chains of six or seven 8x8 factors: the trailing five stay as they are, for the whole-row kernel on the
  // blocks of 32768 columns (a two-part plan), and only the leading ones are merged (tuned: dgemkm 1024 x 8^6 1.95 ->
  // 1.79 ms, 256 x 8^6 0.52 -> 0.45 ms; with eight factors the merged chain takes as many launches and stays)
  int keepFrom = (int)p.N;
  if (p.dt == DType::F64 && p.mm == MMType::MKM && (p.N == 6 || p.N == 7) && p.opX == fastKronOp_N && dev_.rulesOfThumb) {
    bool all8 = true;
    for (uint32_t i = 0; i < p.N; i++) all8 = all8 && p.P[i] == 8 && p.Q[i] == 8;
    // (from 32 blocks on, as the kernel's own rule has it)
    const uint64_t blocks = (uint64_t)p.M * (p.N == 6 ? 8 : 64) * p.batch;
    if (all8 && blocks >= 32) keepFrom = (int)p.N - 5;
  }
  struct Grp { uint32_t lo, hi, size; };
  Grp grp[kMaxFactors];
  uint32_t ng = 0, mergedGroups = 0;
  for (int hi = (int)p.N - 1; hi >= 0;) {
    uint32_t size = p.P[hi];
    int lo = hi;
    const bool small = p.P[hi] == p.Q[hi] && isPow2(p.P[hi]) && p.P[hi] < target && hi < keepFrom;
    if (small)
      while (lo > 0 && p.P[lo - 1] == p.Q[lo - 1] && isPow2(p.P[lo - 1]) && size * p.P[lo - 1] <= target &&
             (uint32_t)(hi - lo + 1) < kMaxMergeSources) {
        lo--; size *= p.P[lo];
      }
    // a product smaller than 8 is not worth a kernel of its own size class: leave such factors alone
    if (lo < hi && size < 8) lo = hi, size = p.P[hi];
    grp[ng++] = Grp{(uint32_t)lo, (uint32_t)hi, size};
    if (lo < hi) mergedGroups++;
    hi = lo - 1;
  }
  if (mergedGroups == 0 || mergedGroups > kMaxMergeGroups) return false;

  const bool pMajor = (p.mm == MMType::MKM) == (p.opF == fastKronOp_N);   // as in makeStepArgs
  MergeArgs ma{};
  KronProblem q = p;
  q.N = ng;
  size_t wsOff = 0;
  for (uint32_t g = 0; g < ng; g++) {
    const Grp& G = grp[ng - 1 - g];                    // groups were collected last to first
    q.strideF[g] = 0;
    if (G.lo == G.hi) {
      q.P[g] = p.P[G.lo]; q.Q[g] = p.Q[G.lo]; q.F[g] = p.F[G.lo]; q.strideF[g] = p.strideF[G.lo];
      continue;
    }
    MergeGroup& mg = ma.g[ma.groups++];
    mg.count = G.hi - G.lo + 1;
    for (uint32_t j = 0; j < mg.count; j++) {
      const uint32_t fi = G.lo + j;
      mg.src[j] = p.F[fi]; mg.p[j] = p.P[fi]; mg.q[j] = p.Q[fi];
      mg.sp[j] = pMajor ? (int64_t)p.Q[fi] : 1;
      mg.sq[j] = pMajor ? 1 : (int64_t)p.P[fi];
    }
    const size_t bytes = (size_t)G.size * G.size * dtypeSize(p.dt);
    if (wsOff + bytes > wsBytes) return false;
    mg.dst = (char*)wsBase + wsOff;
    mg.dsp = pMajor ? (int64_t)G.size : 1;
    mg.dsq = pMajor ? 1 : (int64_t)G.size;
    wsOff += (bytes + 255) & ~(size_t)255;
    q.P[g] = G.size; q.Q[g] = G.size; q.F[g] = mg.dst;
  }
  if (!planOnly_) {
    if (!ws && mergeWsUsed_ && mergeWsStream_ != stream_) orderWorkspaceBehind(stream_);
    if (launchMergeFactors(ma, p.dt, stream_) != hipSuccess) return false;
    if (!ws) { mergeWsStream_ = stream_; mergeWsUsed_ = true; }
  }
  *out = q;
  return true;
}

// X (F_0 x ... x F_{N-1}) = first apply the trailing factors B = F_g x ... x F_{N-1} to every contiguous
// block of prod(P_g..) columns (an MKM problem on M * K_A "virtual rows", K_A = prod of the leading P), then
// apply the leading factors A = F_0 x ... x F_{g-1} across the blocks: for every row that is a KMM problem
// on a K_A x T matrix whose T columns are contiguous.  Two or three launches instead of N.  The layout
// between the two parts is [row][k_A][q_B] (digits in place), which only these two sub-problems see.
//
// buildSplit sets up the two sub-problems for g leading factors (q1: trailing factors, X -> temp1; q2: leading
// factors, temp1 -> Z with the call's epilogue) and returns false when the problem does not have that form.
bool Handle::buildSplit(const KronProblem& p, uint32_t g, void* temp1, void* temp2, KronProblem* q1out,
                        KronProblem* q2out) const {
  if (p.mm != MMType::MKM || p.forward || p.opX != fastKronOp_N) return false;
  if (!temp1 || !temp2 || p.N < 3 || g == 0 || g >= p.N) return false;
  const uint32_t nT = p.N - g;
  // KA x Tin columns come in; the trailing factors make Tout of every Tin, the leading ones LA of the KA blocks
  uint64_t KA = 1, LA = 1, Tin = 1, Tout = 1;
  for (uint32_t i = 0; i < g; i++) { KA *= p.P[i]; LA *= p.Q[i]; }
  for (uint32_t i = g; i < p.N; i++) { Tin *= p.P[i]; Tout *= p.Q[i]; }
  const uint64_t K = KA * Tin, L = LA * Tout, mid = KA * Tout;
  if (Tin >= (1ull << 32) || Tout >= (1ull << 32)) return false;
  {
    // the intermediate (M x KA x Tout) is one of the step outputs the temporaries are sized for; the second part uses
    // temp2 for the outputs of all but its last launch, each at most as wide as the widest step of the call
    size_t yElems = 0, tmpElems = 0;
    if (const_cast<Handle*>(this)->sizes(p.M, p.N, p.P, p.Q, &yElems, &tmpElems) != fastKronSuccess) return false;
    if ((uint64_t)p.M * mid > tmpElems) return false;
  }
  if (p.batch > 1) {
    if (p.strideX != (uint64_t)p.M * K || p.strideZ != (uint64_t)p.M * L) return false;
    if (p.Y && p.beta != 0.0 && p.strideY != (uint64_t)p.M * L) return false;
  }
  // the leading factors are read by a problem whose batch entries are the rows of this one: shared factors only
  for (uint32_t i = 0; i < g; i++) if (p.strideF[i] != 0) return false;
  if ((uint64_t)p.M * p.batch > 65535 || (uint64_t)p.M * KA >= (1ull << 31)) return false;

  // part 1: trailing factors, X -> temp1, no epilogue
  KronProblem q1 = p;
  q1.M = (uint32_t)(p.M * KA); q1.N = nT;
  for (uint32_t i = 0; i < nT; i++) {
    q1.P[i] = p.P[g + i]; q1.Q[i] = p.Q[g + i]; q1.F[i] = p.F[g + i]; q1.strideF[i] = p.strideF[g + i];
  }
  q1.Z = temp1; q1.strideZ = (uint64_t)p.M * mid;
  q1.Y = nullptr; q1.strideY = 0; q1.alpha = 1.0; q1.beta = 0.0;
  q1.zReadNext = true;

  // part 2: leading factors as a KMM over every row block; P x Q storage is the transpose of KMM's Q x P
  KronProblem q2 = p;
  q2.mm = MMType::KMM; q2.M = (uint32_t)Tout; q2.N = g;
  q2.opF = (p.opF == fastKronOp_N) ? fastKronOp_T : fastKronOp_N;
  q2.opX = fastKronOp_N;
  q2.X = temp1; q2.strideX = mid;
  q2.xJustWritten = true;
  q2.strideZ = L; q2.strideY = L;
  q2.batch = p.batch * p.M; q2.strided = true;
  for (uint32_t i = 0; i < g; i++) q2.strideF[i] = 0;
  *q1out = q1; *q2out = q2;
  return true;
}

// Validates (on the concrete buffers) and runs a two-part plan: plan1 on q1, plan2 on q2 with temp2 as its scratch.
fastKronError Handle::runSplit(const KronProblem& p, uint32_t g, const KronProblem& q1, const Plan& plan1,
                               const KronProblem& q2, const Plan& plan2, void* temp2) {
  if (plan1.size() != 1) return fastKronKernelNotFound;                    // q1 has no scratch of its own
  // more than two leading launches ping-pong between temp2 and Z, which must then not be Y
  if (plan2.size() > 2 && p.Y == p.Z && p.beta != 0.0) return fastKronKernelNotFound;
  if (execute(q1, plan1, nullptr, nullptr, true) != fastKronSuccess) return fastKronKernelNotFound;
  if (execute(q2, plan2, temp2, nullptr, true) != fastKronSuccess) return fastKronKernelNotFound;
  lastPlan_ = p.str();
  for (auto& s : plan1)
    lastPlan_ += ";" + std::to_string(g + s.lo) + "-" + std::to_string(g + s.hi) + ":" + db_.kernels()[s.kernel].name;
  for (auto& s : plan2)
    lastPlan_ += ";" + std::to_string(s.lo) + "-" + std::to_string(s.hi) + ":" + db_.kernels()[s.kernel].name;
  // Rows are independent, and the intermediate between the two parts is written once and read once.  With
  // FASTKRON_CHUNK_MB set, the rows go through the two parts in chunks whose intermediate has that size, every chunk
  // through the same stretch of temp1, so that the second part reads what the first wrote from the 256 MB memory-side
  // cache and the stretch is overwritten before most of it has to go out to HBM.  Off by default: measured on an
  // MI355X it loses (dgemkm 256 x 64^3: 496 us unchunked, 548 / 569 / 601 us with chunks of 192 / 128 / 64 MB; sgemkm
  // 1024 x 16^5: 2.98 ms against 3.33 ms at 128 MB; 1024 x 8^6, 1024 x 32^4, dgemkm 1024 x 16^4, sgemkm 16 x 16^6 likewise):
  // each chunk's launches start and drain on their own, which costs more than the cache returns.
  // (reference src/kmm/kmmalgo.cpp:72-115 plans whole-problem intermediates.)
  const uint32_t chunkRows = chunkRowsForCache(p, q2);
  auto forChunks = [&](bool dry) -> fastKronError {
    const size_t es = dtypeSize(p.dt);
    const uint64_t K = q2.strideX;                              // elements of one row of the problem
    const uint64_t KA = q1.M / p.M;                             // blocks of a row
    for (uint32_t m0 = 0; m0 < p.M; m0 += chunkRows) {
      const uint32_t rows = p.M - m0 < chunkRows ? p.M - m0 : chunkRows;
      KronProblem c1 = q1, c2 = q2;
      c1.M = (uint32_t)(rows * KA);
      c1.X = (const char*)q1.X + (size_t)m0 * K * es;
      c2.batch = rows;
      c2.Z = (char*)q2.Z + (size_t)m0 * K * es;
      if (q2.Y) c2.Y = (const char*)q2.Y + (size_t)m0 * K * es;
      fastKronError e = execute(c1, plan1, nullptr, nullptr, dry);
      if (e != fastKronSuccess) return e;
      e = execute(c2, plan2, temp2, nullptr, dry);
      if (e != fastKronSuccess) return e;
    }
    return fastKronSuccess;
  };
  if (chunkRows < p.M) {
    if (planOnly_) { launchLog_.clear(); return forChunks(true); }
    if (forChunks(true) != fastKronSuccess) return fastKronKernelNotFound;      // every chunk's buffers checked first
    return forChunks(false);
  }
  if (planOnly_) {
    launchLog_.clear();
    (void)execute(q1, plan1, nullptr, nullptr, true);
    return execute(q2, plan2, temp2, nullptr, true);
  }
  fastKronError e = execute(q1, plan1, nullptr, nullptr);
  if (e != fastKronSuccess) return e;
  return execute(q2, plan2, temp2, nullptr);
}

// Rows per chunk of a two-part plan (p.M: no chunking, the default).  FASTKRON_CHUNK_MB=<n> sets the size of a
// chunk's intermediate.
uint32_t Handle::chunkRowsForCache(const KronProblem& p, const KronProblem& q2) const {
  const long forcedMB = chunkMB_;
  if (forcedMB <= 0 || p.batch != 1 || p.M < 2 || p.forward || p.K() != p.L()) return p.M;
  const uint64_t rowBytes = q2.strideX * dtypeSize(p.dt);
  uint64_t rows = ((uint64_t)forcedMB << 20) / rowBytes;
  if (rows < 1) rows = 1;
  return rows >= p.M ? p.M : (uint32_t)rows;
}

// The online rule for the two-part plan: how many trailing factors one whole-block kernel takes.
fastKronError Handle::trySplitLeadingTrailing(const KronProblem& p, void* temp1, void* temp2) {
  if (p.mm != MMType::MKM || p.forward || p.opX != fastKronOp_N) return fastKronKernelNotFound;
  if (!temp1 || !temp2 || p.N < 3) return fastKronKernelNotFound;
  // trailing run of identical square factors that one whole-row kernel fuses:
  // fp32 8x8 (five), 16x16 (four), 32x32 (three), 64x64 (two); fp64 16x16 (three), 32x32 or 64x64 (two);
  // 9x9 ... 15x15 (three, either type)
  const uint32_t tp = p.P[p.N - 1], tq = p.Q[p.N - 1];
  if (tq != tp) {
    // two trailing rectangular factors of a shape the pair kernel has exact tiles for (32x64, 64x32)
    if (p.P[p.N - 2] != tp || p.Q[p.N - 2] != tq) return fastKronKernelNotFound;
    const uint32_t g2 = p.N - 2;
    KronProblem r1, r2;
    if (!buildSplit(p, g2, temp1, temp2, &r1, &r2)) return fastKronKernelNotFound;
    Plan rp1 = db_.selectOnline(r1, dev_, true);
    if (rp1.size() != 1 || db_.kernels()[rp1[0].kernel].fused != 2 || db_.kernels()[rp1[0].kernel].P == 0)
      return fastKronKernelNotFound;
    Plan rp2 = db_.selectOnline(r2, dev_, true);
    return runSplit(p, g2, r1, rp1, r2, rp2, temp2);
  }
  uint32_t maxT = 0;
  if (tp == 32 && p.dt == DType::F32) maxT = 3;      // three 32x32 fp32 factors fused per 32768-column block
  else if (tp == 32 || tp == 64)      maxT = 2;
  else if (p.dt == DType::F32) maxT = (tp == 8) ? 5 : (tp == 16) ? 4 : 0;
  else if (tp == 16)           maxT = 3;
  else if (tp == 8)            maxT = 5;              // fp64: the whole-row kernel for five 8x8 factors
  // (few rows of 32^3, fp32: the pair kernel spreads them over more CUs than one workgroup per row does)
  if (p.dt == DType::F32 && tp == 32 && (uint64_t)p.M * (p.K() / 32768) * p.batch < 96) maxT = 2;
  // (few blocks of 16^4: the wave-per-block kernel for three factors spreads them over more CUs)
  if (p.dt == DType::F32 && tp == 16 && p.N >= 4 && (uint64_t)p.M * (p.K() / 65536) * p.batch < 96) maxT = 3;
  if (maxT == 0 && tp >= 9 && tp <= 15) maxT = 3;       // zero-padded form of the 16x16x3 wave-per-block kernel
  if (maxT == 0 && tp >= 17 && tp <= 31) maxT = 2;      // zero-padded form of the 32x32 pair kernel
  if (maxT == 0) return fastKronKernelNotFound;
  uint32_t nT = 0;
  while (nT < maxT && nT < p.N && p.P[p.N - 1 - nT] == tp && p.Q[p.N - 1 - nT] == tp) nT++;
  if (nT < 2 || nT == p.N) return fastKronKernelNotFound;         // a chain of nT factors alone is a whole-row problem
  if (p.dt == DType::F64 && tp == 8 && nT != 5) return fastKronKernelNotFound;   // (that kernel takes exactly five)
  const uint32_t g = p.N - nT;
  KronProblem q1, q2;
  if (!buildSplit(p, g, temp1, temp2, &q1, &q2)) return fastKronKernelNotFound;
  Plan plan1 = db_.selectOnline(q1, dev_, true);
  if (plan1.size() != 1 || db_.kernels()[plan1[0].kernel].P == 0) return fastKronKernelNotFound;
  Plan plan2 = db_.selectOnline(q2, dev_, true);
  return runSplit(p, g, q1, plan1, q2, plan2, temp2);
}

// A tuned record with explicit merge / split fields for this problem, if the file has one.
bool Handle::lookupChoice(const KronProblem& p, Choice* c) const {
  int merge = -1, transposeX = 0;
  uint32_t split = 0;
  Plan plan;
  if (!db_.lookupTuned(p.str(), &plan, &merge, &split, &transposeX) || merge < 0) return false;
  c->merge = merge != 0; c->split = split; c->plan = plan; c->transposeX = transposeX != 0;
  return true;
}

// Runs a tuned choice; fastKronKernelNotFound when it does not fit this call (the caller then selects online).
fastKronError Handle::runChoice(const KronProblem& p0, const Choice& c, void* temp1, void* temp2, const CallWorkspace* ws) {
  if (c.transposeX) {
    KronProblem pn;
    void* xt = nullptr;
    if (!transposedProblem(p0, temp1, temp2, &pn, &xt)) return fastKronKernelNotFound;
    if (!temp2 && (c.split || c.plan.size() != 1)) return fastKronKernelNotFound;      // the copy sits in temp1 then
    Choice rest = c;
    rest.transposeX = false;
    if (!planOnly_ && launchTransposeX(p0, xt, pn.strideX) != hipSuccess) return fastKronInvalidArgument;
    fastKronError e = runChoice(pn, rest, temp1, temp2, ws);
    if (e == fastKronSuccess) noteTranspose(p0);
    return e;
  }
  KronProblem p = p0;
  if (c.merge) {
    KronProblem merged;
    if (!mergeSmallFactors(p0, &merged, ws)) return fastKronKernelNotFound;
    p = merged;
  }
  if (c.split) {
    KronProblem q1, q2;
    if (!buildSplit(p, c.split, temp1, temp2, &q1, &q2)) return fastKronKernelNotFound;
    Plan plan1, plan2;
    for (auto& s : c.plan) {
      if (s.lo >= c.split) plan1.push_back(PlanStep{s.lo - c.split, s.hi - c.split, s.kernel});
      else if (s.hi < c.split) plan2.push_back(s);
      else return fastKronKernelNotFound;
    }
    if (!db_.validPlan(q1, plan1, dev_) || !db_.validPlan(q2, plan2, dev_)) return fastKronKernelNotFound;
    return runSplit(p, c.split, q1, plan1, q2, plan2, temp2);
  }
  if (!db_.validPlan(p, c.plan, dev_)) return fastKronKernelNotFound;
  fastKronError e = execute(p, c.plan, temp1, temp2, true);
  if (e != fastKronSuccess) return e;
  lastPlan_ = p.str();
  for (auto& s : c.plan)
    lastPlan_ += ";" + std::to_string(s.lo) + "-" + std::to_string(s.hi) + ":" + db_.kernels()[s.kernel].name;
  if (planOnly_) { launchLog_.clear(); return execute(p, c.plan, temp1, temp2, true); }
  return execute(p, c.plan, temp1, temp2);
}

// Everything of a launch's arguments that follows from the problem and the factor range; the caller
// fills in the input/output buffers.
StepArgs makeStepArgs(const KronProblem& p, uint32_t lo, uint32_t hi, bool first, bool last) {
  StepArgs a{};
  a.nf = hi - lo + 1;
  a.M = p.M; a.batch = p.batch;
  a.Kin = p.colsBefore(hi);
  a.Kout = p.colsAfter(lo);
  for (uint32_t j = 0; j < a.nf && j < kMaxFused; j++) {
    const uint32_t fi = hi - j;
    a.f[j] = p.F[fi]; a.f_batch[j] = p.strideF[fi];
    a.p[j] = p.P[fi]; a.q[j] = p.Q[fi];
    // Storage of op(F): MKM factors are P x Q, KMM factors are Q x P; opF = T stores the transpose
    // (reference tests/testBase.h:264-268,295-299).
    const bool pMajor = (p.mm == MMType::MKM) == (p.opF == fastKronOp_N);
    a.f_sp[j] = pMajor ? (int64_t)p.Q[fi] : 1;
    a.f_sq[j] = pMajor ? 1 : (int64_t)p.P[fi];
  }
  const bool rowMajor = (p.mm == MMType::MKM);      // rows contiguous along the columns
  auto setLd = [&](int64_t& ldm, int64_t& ldc, uint64_t cols, bool transposed) {
    const bool rm = transposed ? !rowMajor : rowMajor;
    if (rm) { ldm = (int64_t)cols; ldc = 1; } else { ldm = 1; ldc = (int64_t)p.M; }
  };
  setLd(a.in_ldm, a.in_ldc, a.Kin, first && p.opX == fastKronOp_T);
  setLd(a.out_ldm, a.out_ldc, a.Kout, false);
  if (last) {
    a.epilogue = 1; a.alpha = p.alpha; a.beta = p.beta;
    a.y = (p.beta != 0.0) ? p.Y : nullptr;          // beta is skipped when Y is null, reference kernel.h:158-159
    a.y_batch = p.strideY;
    setLd(a.y_ldm, a.y_ldc, p.L(), false);
  }
  return a;
}

// With dryRun the launches are only validated (kernel-specific checks on the concrete buffers);
// fastKronKernelNotFound then means "this plan cannot run on these buffers".
fastKronError Handle::execute(const KronProblem& p, const Plan& plan, void* temp1, void* temp2, bool dryRun,
                              int* refused) {
  const size_t n = plan.size();
  if (n == 0) return fastKronKernelNotFound;
  const uint64_t L = p.L();

  // Ping-pong plan of reference src/kmm/kmmalgo.cpp:82-110: launch l < n-1 writes tmps[l % 2]; when
  // only one temporary is given, Z is the other one, placed so that the last intermediate is not Z.
  void* tmps[2] = {temp1, temp2};
  bool zIsTmp[2] = {false, false};
  if (!p.forward && n > 1 && temp2 == nullptr) {
    if (n % 2 == 1) { tmps[1] = temp1; tmps[0] = p.Z; zIsTmp[0] = true; }
    else            { tmps[1] = p.Z; zIsTmp[1] = true; }
    if (n == 2) { tmps[1] = nullptr; zIsTmp[1] = false; }     // a 2-launch plan never touches the second one
  }

  // capacity of a temporary by the API's contract: the widest step output of every batch entry
  uint64_t tempElems = 0;
  if (!p.forward) {
    size_t ye = 0, te = 0;
    if (sizes(p.M, p.N, p.P, p.Q, &ye, &te) == fastKronSuccess) tempElems = (uint64_t)te * p.batch;
  }
  const void* in = p.X;
  uint64_t inBatch = p.strideX;
  for (size_t l = 0; l < n; l++) {
    const PlanStep& s = plan[l];
    const KernelInfo& k = db_.kernels()[s.kernel];
    const bool first = (l == 0), last = (l + 1 == n);
    if (s.hi - s.lo + 1 > kMaxFused) return fastKronKernelNotFound;
    StepArgs a = makeStepArgs(p, s.lo, s.hi, first, last);
    a.in = in; a.in_batch = inBatch;
    if (last) {
      a.out = p.Z; a.out_batch = p.strideZ;
    } else if (p.forward) {
      a.out = p.inter[s.lo - 1];
      a.out_batch = p.haveStrideInter ? p.strideInter[s.lo - 1] : (uint64_t)p.M * a.Kout;
    } else {
      const int t = (int)(l % 2);
      a.out = tmps[t];
      a.out_batch = (uint64_t)p.M * a.Kout;
      if (zIsTmp[t]) {
        // Z doubles as scratch: the intermediate has to fit the per-batch Z region.
        if (a.Kout > L || (p.batch > 1 && p.strideZ < (uint64_t)p.M * L)) return fastKronInvalidArgument;
        if (p.batch > 1) a.out_batch = p.strideZ;
      }
      if (a.out == nullptr) return fastKronInvalidArgument;
    }
    {
      // Non-temporal hints (StepArgs::stream_in / stream_out).  Measured: an intermediate of 134 MB is read back
      // from the memory-side cache by the next launch (non-temporal stores cost 4 % there), one of 268 MB is not
      // (they gain 2 %); X and Z of a launch that moves 268 MB or more with nothing cached gain 2.5 to 4 %, also
      // when Z itself is small (8 x 512 x (32x16)^3: 67 MB of Z behind 537 MB of X, 126.2 -> 121.9 us).
      constexpr uint64_t kStreamFrom = 96ull << 20, kBeyondCache = 192ull << 20;
      const uint64_t es8 = dtypeSize(p.dt);
      const uint64_t inBytes = (uint64_t)p.M * a.Kin * p.batch * es8, outBytes = (uint64_t)p.M * a.Kout * p.batch * es8;
      const uint64_t moved = inBytes + outBytes + (a.y ? outBytes : 0);
      const bool inFromCaller = first && !p.xJustWritten, outToCaller = (last || p.forward) && !p.zReadNext;
      a.stream_in = inFromCaller ? (moved >= kStreamFrom && inBytes >= kStreamFrom / 2) : inBytes > kBeyondCache;
      a.stream_out = outToCaller ? moved >= kStreamFrom : outBytes > kBeyondCache;
    }
    {
      // A temporary that this launch neither reads nor writes, for kernels that keep an intermediate of their own:
      // the first launch reads X and the last writes Z, so one of the two temporaries is idle then.
      void* idle = nullptr;
      if (!p.forward && (first || last)) {
        for (void* t : {temp1, temp2})
          if (t && t != a.in && t != a.out && t != (const void*)p.Z && t != p.X && t != p.Y && !idle) idle = t;
      }
      a.scratch = idle; a.scratch_elems = idle ? tempElems : 0;
      a.sync = callWs_ ? nullptr : syncArea();
    }
    if (logLevel() >= 2)
      printf("[fastkron]   launch %zu: factors [%u,%u] Kin=%llu Kout=%llu kernel %s\n", l, s.lo, s.hi,
             (unsigned long long)a.Kin, (unsigned long long)a.Kout, k.name.c_str());
    // The batch index is a grid dimension (at most 65535): larger batches go out in chunks of that many.
    constexpr uint32_t kMaxGridBatch = 65535;
    const size_t es = dtypeSize(p.dt);
    for (uint32_t b0 = 0; b0 < a.batch; b0 += kMaxGridBatch) {
      StepArgs c = a;
      c.batch = a.batch - b0 < kMaxGridBatch ? a.batch - b0 : kMaxGridBatch;
      c.in = (const char*)a.in + (size_t)b0 * a.in_batch * es;
      c.out = (char*)a.out + (size_t)b0 * a.out_batch * es;
      if (a.y) c.y = (const char*)a.y + (size_t)b0 * a.y_batch * es;
      for (uint32_t j = 0; j < a.nf && j < kMaxFused; j++)
        c.f[j] = (const char*)a.f[j] + (size_t)b0 * a.f_batch[j] * es;
      if (dryRun) {
        if (k.check && !k.check(k, c)) {                                // every chunk: its base pointers differ
          if (refused) *refused = s.kernel;
          return fastKronKernelNotFound;
        }
        if (planOnly_) {
          char line[768];
          int n = snprintf(line, sizeof(line), "kernel=%s lo=%u hi=%u M=%u batch=%u Kin=%llu Kout=%llu in=%p out=%p y=%p "
                           "in_batch=%llu out_batch=%llu y_batch=%llu stream_in=%u stream_out=%u f_batch=", k.name.c_str(), s.lo, s.hi, c.M, c.batch,
                           (unsigned long long)c.Kin, (unsigned long long)c.Kout, c.in, c.out, c.y,
                           (unsigned long long)c.in_batch, (unsigned long long)c.out_batch, (unsigned long long)c.y_batch,
                           c.stream_in, c.stream_out);
          launchLog_.append(line, n > 0 ? (size_t)n : 0);
          for (uint32_t j = 0; j < c.nf && j < kMaxFused; j++)
            launchLog_ += (j ? "," : "") + std::to_string(c.f_batch[j]);
          launchLog_ += "\n";
        }
        continue;
      }
      if (k.usesSync) {
        // the counter area is one more piece of device state of the handle: a later call on another stream is
        // ordered behind this launch (orderWorkspaceBehind)
        if (mergeWsUsed_ && mergeWsStream_ != stream_) orderWorkspaceBehind(stream_);
        mergeWsStream_ = stream_; mergeWsUsed_ = true;
      }
      hipError_t he = k.launch(k, c, stream_);
      if (he != hipSuccess) {
        fprintf(stderr, "[fastkron] launch of %s failed: %s\n", k.name.c_str(), hipGetErrorString(he));
        return fastKronInvalidArgument;               // reference cuda_kernel_db.cu:296-301
      }
    }
    in = a.out; inBatch = a.out_batch;
  }
  return fastKronSuccess;
}

}  // namespace fk
