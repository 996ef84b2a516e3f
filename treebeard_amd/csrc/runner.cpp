#include "runner.h"

#include <algorithm>
#include <mutex>
#include <sstream>
#include <vector>

namespace tbamd {

bool gMeasureGpuKernelTime = false;
int32_t gNumberOfKernelRuns = 1;
bool gPeeledWalks = false;

namespace {

void Check(hipError_t e, const char *what) {
  if (e != hipSuccess) throw Error(std::string(what) + ": " + hipGetErrorString(e));
}

// Scratch memory of the entry point that allocates nothing (RunDeviceNoAlloc): partial sums and
// rank-quantised rows of one call.  Every GPU the library runs on holds its own copy of the array
// until the process ends.  In host code the array's name is only a handle for the runtime: the
// address kernels can use is looked up once per device and kept in gScratchAddress.
constexpr size_t kNoAllocScratchBytes = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
constexpr int kMaxDevices = 64;
unsigned char *gScratchAddress[kMaxDevices] = {};
std::mutex gScratchMutex;

// Device address of `scratch` on the current device (looked up on first use, then cached).
unsigned char *ScratchOfCurrentDevice() {
  int device = -1;
  Check(hipGetDevice(&device), "hipGetDevice");
  if (device < 0 || device >= kMaxDevices) throw Error("device index out of range for the fixed scratch array");
  std::lock_guard<std::mutex> lock(gScratchMutex);
  if (!gScratchAddress[device]) {
    void *address = nullptr;
    Check(hipGetSymbolAddress(&address, HIP_SYMBOL(scratch)), "hipGetSymbolAddress");
    if (!address) throw Error("hipGetSymbolAddress returned no address for the fixed scratch array");
    gScratchAddress[device] = static_cast<unsigned char *>(address);
  }
  return gScratchAddress[device];
}

template <typename T> T *Upload(const std::vector<T> &host, const char *what) {
  T *ptr = nullptr;
  const size_t bytes = std::max<size_t>(host.size(), 1) * sizeof(T);
  Check(hipMalloc(reinterpret_cast<void **>(&ptr), bytes), what);
  if (!host.empty()) Check(hipMemcpy(ptr, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice), what);
  return ptr;
}

} // namespace

InferenceRunner::InferenceRunner(Forest forest, const CompilerOptions &options,
                                 const GPUAutoScheduleOptions *gpuOptions, std::unique_ptr<HitCountProfile> profile)
    : m_forest(std::move(forest)), m_profile(std::move(profile)), m_options(options) {
  try {
    InitDevice();
    m_walk.tileSize = m_options.tileSize;
    m_walk.tiling = m_profile ? (int32_t)m_options.tilingType : 0;
    m_walk.peelWalks = m_profile && gPeeledWalks;
    m_model = PackForest(m_forest, ChoosePlan(m_forest, m_options.batchSize, gpuOptions, m_limits, m_walk), m_profile.get());
    UploadModel();
  } catch (...) { // a constructor that throws gets no destructor call: give back what was created
    Release();
    throw;
  }
}

InferenceRunner::InferenceRunner(Forest forest, const CompilerOptions &options, const LaunchPlan &plan,
                                 std::unique_ptr<HitCountProfile> profile)
    : m_forest(std::move(forest)), m_profile(std::move(profile)), m_options(options) {
  try {
    m_options.tileSize = plan.tileSize;
    InitDevice();
    m_walk.tileSize = plan.tileSize;
    m_walk.tiling = plan.tiling;
    m_walk.peelWalks = plan.peelWalks;
    m_model = PackForest(m_forest, plan, m_profile.get());
    UploadModel();
  } catch (...) {
    Release();
    throw;
  }
}

void InferenceRunner::InitDevice() {
  if (m_options.batchSize <= 0) throw Error("batchSize must be positive");
  if (m_options.inputElementTypeWidth != 32) throw Error("only 32-bit float inputs are supported");
  if (m_options.thresholdTypeWidth != 32) throw Error("only 32-bit float thresholds are supported");
  const bool floatResults = m_options.returnTypeWidth == 32 && m_options.returnTypeFloatType;
  const bool int8Results = m_options.returnTypeWidth == 8 && !m_options.returnTypeFloatType;
  if (m_forest.numClasses == 0 && !floatResults) throw Error("only 32-bit float predictions are supported");
  if (m_forest.numClasses > 0 && !floatResults && !int8Results)
    throw Error("class ids are returned as 8-bit integers or 32-bit floats");
  m_forest.Validate();

  int deviceCount = 0;
  if (hipGetDeviceCount(&deviceCount) != hipSuccess || deviceCount == 0)
    throw Error("no HIP device available: this library has no CPU fallback");
  // A runner belongs to the device that is current when it is made: its limits, model and workspace are that
  // device's, and its calls must be made with the same device current.
  Check(hipGetDevice(&m_device), "hipGetDevice");
  hipDeviceProp_t prop;
  Check(hipGetDeviceProperties(&prop, m_device), "hipGetDeviceProperties");
  m_limits.computeUnits = prop.multiProcessorCount;
  m_limits.ldsBytesPerBlock = (int32_t)std::min<size_t>(prop.sharedMemPerBlock, 160 * 1024);
  // Set-up: the no-allocation entry point finds its array's address ready.  A failure here is that entry
  // point's business only (it looks the address up again and reports the error): other callers never need it.
  try {
    (void)ScratchOfCurrentDevice();
  } catch (const Error &) {
    (void)hipGetLastError();
  }
  Check(hipStreamCreateWithFlags(&m_stream, hipStreamNonBlocking), "hipStreamCreate");
  Check(hipEventCreate(&m_evStart), "hipEventCreate");
  Check(hipEventCreate(&m_evStop), "hipEventCreate");
  Check(hipEventCreateWithFlags(&m_asyncDone, hipEventDisableTiming), "hipEventCreate");
}

void InferenceRunner::OrderAfterAsyncCall(hipStream_t stream) {
  if (!m_asyncPending || stream == m_asyncStream) return; // (calls on one stream are ordered by the stream)
  Check(hipStreamWaitEvent(stream, m_asyncDone, 0), "hipStreamWaitEvent");
}

void InferenceRunner::WaitForAsyncCall() {
  if (!m_asyncPending) return;
  Check(hipEventSynchronize(m_asyncDone), "hipEventSynchronize");
  m_asyncPending = false;
}

InferenceRunner::~InferenceRunner() { Release(); }

void InferenceRunner::Release() noexcept {
  if (m_asyncPending) (void)hipEventSynchronize(m_asyncDone); // kernels of an asynchronous call still read the model
  if (m_stream) (void)hipStreamSynchronize(m_stream);
  FreeModel();
  (void)hipFree(m_dPartial);
  (void)hipFree(m_dRanks);
  (void)hipFree(m_dStageIn);
  (void)hipFree(m_dStageOut);
  for (void *buf : m_pinned)
    if (buf) (void)hipHostFree(buf);
  for (auto &ev : m_pieceReady)
    if (ev) (void)hipEventDestroy(ev);
  if (m_copyStream) (void)hipStreamDestroy(m_copyStream);
  if (m_evStart) (void)hipEventDestroy(m_evStart);
  if (m_evStop) (void)hipEventDestroy(m_evStop);
  if (m_asyncDone) (void)hipEventDestroy(m_asyncDone);

  if (m_stream) (void)hipStreamDestroy(m_stream);
}

void InferenceRunner::FreeModel() {
  (void)hipFree(m_dNodes);
  (void)hipFree(m_dBundles);
  (void)hipFree(m_dBundleRoots);
  (void)hipFree(m_dGroups);
  (void)hipFree(m_dNodeOrigin);
  (void)hipFree(m_dSlotTree);
  (void)hipFree(m_dBinTable);
  (void)hipFree(m_dRankFeatures);
  (void)hipFree(m_dRankChunks);
  (void)hipFree(m_dTailNodes);
  (void)hipFree(m_dTailOrigin);
  m_dTailNodes = nullptr;
  m_dTailOrigin = nullptr;
  m_dRankFeatures = nullptr;
  m_dRankChunks = nullptr;
  (void)hipFree(m_dGlobalNodes);
  (void)hipFree(m_dGlobalTrees);
  m_dBinTable = nullptr;
  m_dGlobalNodes = nullptr;
  m_dGlobalTrees = nullptr;
  m_dNodes = nullptr;
  m_dBundles = nullptr;
  m_dBundleRoots = nullptr;
  m_dGroups = nullptr;
  m_dNodeOrigin = nullptr;
  m_dSlotTree = nullptr;
}

void InferenceRunner::UploadModel() {
  if (m_model.plan.kernel == LaunchPlan::Kernel::kGlobalWalk) {
    m_model.plan.treeSlices = std::max(1, std::min<int32_t>(m_model.plan.treeSlices, (int32_t)m_model.globalTrees.size()));
    m_dGlobalNodes = Upload(m_model.globalNodes, "upload nodes");
    m_dGlobalTrees = Upload(m_model.globalTrees, "upload trees");
    return;
  }
  // treeSlices never exceeds the number of groups the packer produced
  m_model.plan.treeSlices = std::max(1, std::min<int32_t>(m_model.plan.treeSlices, (int32_t)m_model.groups.size()));
  if (m_model.LdsBytes() > (size_t)m_limits.ldsBytesPerBlock) throw Error("launch plan exceeds the LDS of one workgroup");
  m_dNodes = Upload(m_model.nodes, "upload nodes");
  m_dBundles = Upload(m_model.bundles, "upload bundles");
  m_dBundleRoots = Upload(m_model.bundleRoots, "upload bundle roots");
  m_dGroups = Upload(m_model.groups, "upload groups");
  m_dNodeOrigin = Upload(m_model.nodeOrigin, "upload node origins");
  m_dSlotTree = Upload(m_model.slotTree, "upload slot table");
  if (m_model.plan.quantizedRows) m_dBinTable = Upload(m_model.binThresholds, "upload threshold table");
  if (m_model.plan.deferTails) {
    m_dTailNodes = Upload(m_model.tailNodes, "upload tail nodes");
    m_dTailOrigin = Upload(m_model.tailOrigin, "upload tail node origins");
  }
  if (m_model.plan.rankRows16) {
    m_dBinTable = Upload(m_model.rankTables, "upload threshold tables");
    m_dRankFeatures = Upload(m_model.rankFeatures, "upload rank table index");
    m_dRankChunks = Upload(m_model.rankChunks, "upload rank chunk index");
    m_rankChunkEntries = m_rankChunkFeatures = 0;
    for (const RankChunkDesc &c : m_model.rankChunks) {
      m_rankChunkEntries = std::max(m_rankChunkEntries, c.tableEntries);
      m_rankChunkFeatures = std::max(m_rankChunkFeatures, c.numFeatures);
    }
  }
}

void InferenceRunner::Repack(const LaunchPlan &plan) {
  PackedModel next = PackForest(m_forest, plan, m_profile.get());
  // refuse before anything is freed: a plan that fails leaves the runner as it was
  if (next.LdsBytes() > (size_t)m_limits.ldsBytesPerBlock) throw Error("launch plan exceeds the LDS of one workgroup");
  WaitForAsyncCall();
  Check(hipStreamSynchronize(m_stream), "hipStreamSynchronize");
  FreeModel();
  m_model = std::move(next);
  UploadModel();
}

size_t InferenceRunner::PartialBytes(int64_t rows) const {
  if (!NeedsFinalize()) return 0;
  // (+ the spare slot the wide finalize of a classifier leaves its class sums in)
  const size_t slots = (size_t)m_model.PartialCount() +
                       (m_forest.numClasses > 0 && m_model.PartialCount() >= kWideFinalizeSlices ? 1 : 0);
  return slots * (size_t)rows * (size_t)std::max(1, m_forest.numClasses) * sizeof(double);
}

size_t InferenceRunner::RanksBytes(int64_t rows) const {
  if (m_model.plan.rankRows16) { // whole row blocks of [feature pair][row][2] two-byte ranks
    // (the ranking kernel works in tiles of 1024 rows: smaller row blocks are rounded up once more)
    const size_t rb = (size_t)m_model.plan.rowsPerBlock;
    const size_t padded = (((size_t)rows + rb - 1) / rb * rb + 1023) / 1024 * 1024;
    return (padded + rb - 1) / rb * m_model.RowTileBytes();
  }
  if (!m_model.plan.quantizedRows) return 0;
  return (size_t)((rows + 63) / 64) * 64 * (size_t)m_forest.numFeatures;
}

void InferenceRunner::EnsurePartial(int64_t rows) {
  const size_t need = PartialBytes(rows);
  if (need <= m_partialBytes) return;
  WaitForAsyncCall();
  Check(hipStreamSynchronize(m_stream), "hipStreamSynchronize");
  (void)hipFree(m_dPartial);
  m_dPartial = nullptr;
  m_partialBytes = 0;
  Check(hipMalloc(reinterpret_cast<void **>(&m_dPartial), need), "allocate partial sums");
  m_partialBytes = need;
}

void InferenceRunner::EnsureRanks(int64_t rows) {
  const size_t need = RanksBytes(rows);
  if (need <= m_ranksBytes) return;
  WaitForAsyncCall();
  Check(hipStreamSynchronize(m_stream), "hipStreamSynchronize");
  (void)hipFree(m_dRanks);
  m_dRanks = nullptr;
  m_ranksBytes = 0;
  Check(hipMalloc(reinterpret_cast<void **>(&m_dRanks), need), "allocate rank-quantised rows");
  m_ranksBytes = need;
}

InferenceRunner::Workspace InferenceRunner::OwnWorkspace(int64_t rows, hipStream_t stream) {
  EnsurePartial(rows);
  EnsureRanks(rows);
  // An asynchronous call on another stream may still use these buffers: `stream` waits for it on the device.
  OrderAfterAsyncCall(stream);
  Workspace ws;
  ws.partial = m_dPartial;
  ws.ranks = m_dRanks;
  return ws;
}

const float *InferenceRunner::PrepareRows(const float *deviceInputs, int64_t rows, uint8_t *ranks, hipStream_t stream) {
  if (m_model.plan.rankRows16) {
    Check(LaunchRankRows16(deviceInputs, m_dBinTable, m_dRankFeatures, m_dRankChunks, (int)m_model.rankChunks.size(),
                           m_rankChunkEntries, m_rankChunkFeatures, reinterpret_cast<uint16_t *>(ranks), rows, m_forest.numFeatures,
                           m_model.plan.rowsPerBlock, stream),
          "launch ranking kernel");
    return reinterpret_cast<const float *>(ranks);
  }
  if (!m_model.plan.quantizedRows) return deviceInputs;
  Check(LaunchBinRows(deviceInputs, m_dBinTable, ranks, rows, m_forest.numFeatures, m_model.binTableDepth,
                      m_model.binChunkFeatures, stream),
        "launch rank-quantisation kernel");
  return reinterpret_cast<const float *>(ranks);
}

void InferenceRunner::EnsureStaging(int64_t rows) {
  if (rows <= m_stageRows) return;
  Check(hipStreamSynchronize(m_stream), "hipStreamSynchronize");
  (void)hipFree(m_dStageIn);
  (void)hipFree(m_dStageOut);
  m_dStageIn = nullptr;
  m_dStageOut = nullptr;
  m_stageRows = 0;
  Check(hipMalloc(reinterpret_cast<void **>(&m_dStageIn), (size_t)rows * m_forest.numFeatures * sizeof(float)), "allocate input staging");
  Check(hipMalloc(&m_dStageOut, (size_t)rows * sizeof(float)), "allocate output staging");
  m_stageRows = rows;
}

void InferenceRunner::SetGroupStaging(int32_t mode) {
  if (mode < 0 || mode > 2) throw Error("group staging mode must be 0 (by rule), 1 (registers) or 2 (direct)");
  m_groupStaging = mode;
}

bool InferenceRunner::DirectStaging() const {
  const LaunchPlan &plan = m_model.plan;
  if (plan.kernel != LaunchPlan::Kernel::kRowParallelLds) return false; // (only the row-parallel walks have the form)
  if (plan.tileSize > 1 || plan.rankRows16) return true;                 // (the tiled walk and the walk on two-byte ranks have no other)
  if (m_groupStaging != 0) return m_groupStaging == 2;
  // Measured on MI355X (28 to 520 features, 600 to 1000 trees): 5 to 15 % faster with two blocks per CU,
  // 2 to 4 % slower with one, whose wait for the copy nothing covers.  (LDS is handed out in coarse pieces.)
  return 2 * (m_model.LdsBytes() + 512) <= (size_t)m_limits.ldsBytesPerBlock;
}

hipError_t InferenceRunner::LaunchWalk(const WalkParams &p, hipStream_t stream) const {
  const LaunchPlan &plan = m_model.plan;
  if (plan.kernel == LaunchPlan::Kernel::kGlobalWalk) return LaunchWalkGlobal(p, plan.interleave, stream);
  if (plan.kernel == LaunchPlan::Kernel::kTreeParallel)
    return LaunchWalkTreeParallel(p, plan.interleave, m_model.LdsBytes(), stream);
  if (plan.tileSize > 1) return LaunchWalkRowsTiled(p, plan.tileSize, plan.interleave, m_model.LdsBytes(), stream);
  const int tileMode = plan.rankRows16 ? 3 : plan.quantizedRows ? 2 : (plan.featureOffsetInWords ? 1 : 0);
  return LaunchWalkRowsLds(p, plan.interleave, tileMode, m_model.LdsBytes(), stream);
}

WalkParams InferenceRunner::MakeWalkParams(const float *deviceInputs, int64_t rows) const {
  WalkParams p;
  p.s.rows = rows;
  p.s.numFeatures = m_forest.numFeatures;
  p.s.numClasses = m_forest.numClasses;
  p.s.numGroups = (int32_t)m_model.groups.size();
  p.s.treeSlices = m_model.plan.treeSlices;
  p.s.groupRegionBytes = m_model.GroupRegionBytes();
  p.s.treeThreads = m_model.plan.treeThreads;
  p.s.transform = m_forest.transform == Transform::kSigmoid ? 1 : 0;
  p.s.numTrees = (int32_t)m_forest.trees.size();
  p.s.rowsPerBlock = m_model.plan.rowsPerBlock;
  p.s.treeLanes = m_model.plan.treeLanes;
  p.s.initialValue = m_forest.initialValue;
  p.peelWalks = m_model.plan.peelWalks;
  p.s.deferTails = m_model.plan.deferTails ? 1 : 0;
  p.s.tailDepth = (int32_t)m_model.maxTailDepth;
  p.s.tileHops = m_model.maxTileHops;
  p.tailNodes = m_dTailNodes;
  p.tailOrigin = m_dTailOrigin;
  p.directStaging = DirectStaging();
  p.x = deviceInputs;
  p.globalNodes = m_dGlobalNodes;
  p.globalTrees = m_dGlobalTrees;
  p.nodes16 = reinterpret_cast<const uint4 *>(m_dNodes);
  p.bundles = m_dBundles;
  p.bundleRoots = m_dBundleRoots;
  p.groups = m_dGroups;
  return p;
}

void InferenceRunner::Launch(const float *deviceInputs, int64_t rows, float *out, int8_t *classOut, float *margins,
                             float *probabilities, int32_t *leafIds, hipStream_t stream, const Workspace &ws) {
  if (rows <= 0) return;
  WalkParams p = MakeWalkParams(PrepareRows(deviceInputs, rows, ws.ranks, stream), rows);
  // A classifier whose trees all sit in one slice needs no second kernel when only the class id is wanted:
  // the row-parallel kernels keep the running arg-max themselves.
  const bool fused = FusesArgmax() && !margins && !probabilities && !leafIds;
  const bool finalize = NeedsFinalize() && !fused;
  p.s.fuseArgmax = fused ? 1 : 0;
  p.out = finalize ? nullptr : out;
  p.classOut = fused ? classOut : nullptr;
  p.partial = finalize ? ws.partial : nullptr;
  if (leafIds) {
    p.leafIds = leafIds;
    p.nodeOrigin = m_dNodeOrigin;
    p.slotTree = m_dSlotTree;
  }
  Check(LaunchWalk(p, stream), "launch walk kernel");
  if (finalize) {
    FinalizeParams f;
    f.partial = ws.partial;
    f.rows = rows;
    f.numClasses = m_forest.numClasses;
    f.treeSlices = m_model.PartialCount();
    f.initialValue = m_forest.initialValue;
    f.transform = p.s.transform;
    f.out = out;
    f.classOut = classOut;
    f.margins = margins;
    f.probabilities = probabilities;
    Check(LaunchFinalize(f, stream), "launch finalize kernel");
  }
}

void InferenceRunner::RunDevice(const float *deviceInputs, void *deviceResults, int64_t rows) {
  const int runs = gMeasureGpuKernelTime ? std::max(1, gNumberOfKernelRuns) : 1;
  const Workspace ws = OwnWorkspace(rows, m_stream);
  if (gMeasureGpuKernelTime) Check(hipEventRecord(m_evStart, m_stream), "hipEventRecord");
  for (int i = 0; i < runs; ++i) {
    if (ClassIdsAsInt8())
      Launch(deviceInputs, rows, nullptr, static_cast<int8_t *>(deviceResults), nullptr, nullptr, nullptr, m_stream, ws);
    else
      Launch(deviceInputs, rows, static_cast<float *>(deviceResults), nullptr, nullptr, nullptr, nullptr, m_stream, ws);
  }
  if (gMeasureGpuKernelTime) Check(hipEventRecord(m_evStop, m_stream), "hipEventRecord");
  Check(hipStreamSynchronize(m_stream), "inference kernels");
  if (gMeasureGpuKernelTime) {
    float ms = 0.f;
    Check(hipEventElapsedTime(&ms, m_evStart, m_evStop), "hipEventElapsedTime");
    m_lastKernelMicros = (int64_t)(ms * 1000.0);
  }
}

void InferenceRunner::RunDeviceOnStream(const float *deviceInputs, void *deviceResults, int64_t rows, hipStream_t stream) {
  if (rows < 0) throw Error("negative row count");
  if (rows > 0 && (!deviceInputs || !deviceResults)) throw Error("null device buffer");
  if (rows == 0) return;
  // The runner's own stream is idle here (every entry point that uses it waits for it before returning); an
  // earlier asynchronous call may still be running on another stream and uses the same buffers.
  const Workspace ws = OwnWorkspace(rows, stream);
  if (ClassIdsAsInt8())
    Launch(deviceInputs, rows, nullptr, static_cast<int8_t *>(deviceResults), nullptr, nullptr, nullptr, stream, ws);
  else
    Launch(deviceInputs, rows, static_cast<float *>(deviceResults), nullptr, nullptr, nullptr, nullptr, stream, ws);
  Check(hipEventRecord(m_asyncDone, stream), "hipEventRecord");
  m_asyncStream = stream;
  m_asyncPending = true;
}

size_t InferenceRunner::NoAllocScratchBytes() { return kNoAllocScratchBytes; }

void InferenceRunner::RunDeviceNoAlloc(const float *deviceInputs, void *deviceResults, int64_t rows, hipStream_t stream) {
  if (rows < 0) throw Error("negative row count");
  if (rows == 0) return;
  if (!deviceInputs || !deviceResults) throw Error("null device buffer");
  const size_t partialBytes = FusesArgmax() ? 0 : (PartialBytes(rows) + 255) & ~(size_t)255; // (no partial sums when the walk keeps the arg-max)
  const size_t ranksBytes = RanksBytes(rows);
  if (partialBytes + ranksBytes > kNoAllocScratchBytes)
    throw Error("this launch plan needs " + std::to_string(partialBytes + ranksBytes) + " bytes of scratch memory for " +
                std::to_string(rows) + " rows; the fixed array of the no-allocation entry point holds " +
                std::to_string(kNoAllocScratchBytes) + ": pass fewer rows per call or use tbmi_run_device_async");
  unsigned char *base = ScratchOfCurrentDevice();
  Workspace ws;
  ws.partial = reinterpret_cast<double *>(base);
  ws.ranks = base + partialBytes;
  // Every partial sum the finalize kernel reads and every rank the walk reads is written earlier in
  // this same call, so nothing has to be cleared between calls.
  if (ClassIdsAsInt8())
    Launch(deviceInputs, rows, nullptr, static_cast<int8_t *>(deviceResults), nullptr, nullptr, nullptr, stream, ws);
  else
    Launch(deviceInputs, rows, static_cast<float *>(deviceResults), nullptr, nullptr, nullptr, nullptr, stream, ws);
}

void InferenceRunner::RunDeviceMulticlass(const float *deviceInputs, int64_t rows, int8_t *classIds, float *margins,
                                          float *probabilities) {
  if (m_forest.numClasses == 0) throw Error("model is not a multiclass classifier");
  Launch(deviceInputs, rows, nullptr, classIds, margins, probabilities, nullptr, m_stream, OwnWorkspace(rows, m_stream));
  Check(hipStreamSynchronize(m_stream), "inference kernels");
}

void InferenceRunner::DumpLeafIds(const float *deviceInputs, int32_t *deviceLeafIds, int64_t rows) {
  // results of the prediction itself are discarded
  const Workspace ws = OwnWorkspace(rows, m_stream);
  float *scratch = nullptr;
  Check(hipMalloc(reinterpret_cast<void **>(&scratch), std::max<int64_t>(rows, 1) * sizeof(float)), "allocate scratch");
  try {
    Launch(deviceInputs, rows, scratch, reinterpret_cast<int8_t *>(scratch), nullptr, nullptr, deviceLeafIds, m_stream, ws);
    Check(hipStreamSynchronize(m_stream), "leaf-id kernels");
  } catch (...) {
    (void)hipFree(scratch);
    throw;
  }
  (void)hipFree(scratch);
}

void InferenceRunner::RunInference(const void *hostInputs, void *hostResults) {
  RunHostChunk(hostInputs, hostResults, m_options.batchSize);
}

void InferenceRunner::RunHost(const void *hostInputs, void *hostResults, int64_t rows) {
  if (rows < 0) throw Error("negative row count");
  if (rows > 0 && (!hostInputs || !hostResults)) throw Error("null host buffer");
  // Windows of at least one compiled batch and at most about 256 MB of rows (the staging buffers grow
  // to the window): a long input of small batches is not walked one small batch at a time.
  const size_t rowBytes = (size_t)m_forest.numFeatures * sizeof(float);
  const int64_t cap = std::max<int64_t>(m_options.batchSize, (int64_t)(((size_t)256 << 20) / rowBytes));
  const int64_t window = std::min<int64_t>(cap, std::max<int64_t>(rows, 1));
  for (int64_t first = 0; first < rows; first += window)
    RunHostChunk(static_cast<const char *>(hostInputs) + (size_t)first * rowBytes,
                 static_cast<char *>(hostResults) + (size_t)first * ReturnTypeBytes(), std::min(window, rows - first));
}

namespace {

// True when the runtime knows the address as pinned (or registered) host memory, which DMA reads
// directly; pageable memory makes the query fail, and that error must not linger.
bool IsPinnedHost(const void *ptr) {
  hipPointerAttribute_t attr;
  if (hipPointerGetAttributes(&attr, ptr) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return attr.type == hipMemoryTypeHost;
}

} // namespace

void InferenceRunner::RunHostChunk(const void *hostInputs, void *hostResults, int64_t rows) {
  if (rows <= 0) return;
  EnsureStaging(rows);
  const size_t rowBytes = (size_t)m_forest.numFeatures * sizeof(float);
  const size_t totalBytes = (size_t)rows * rowBytes;
  // Large batches go through in pieces: the copy of piece i+1 (on its own stream) overlaps the kernels
  // of piece i.  Rows are independent, so the pieces give the same results as one launch.
  if (gMeasureGpuKernelTime || totalBytes < ((size_t)16 << 20) || rows < 2 * 4096) {
    Check(hipMemcpyAsync(m_dStageIn, hostInputs, totalBytes, hipMemcpyHostToDevice, m_stream), "copy inputs");
    RunDevice(m_dStageIn, m_dStageOut, rows);
  } else {
    if (!m_copyStream) {
      Check(hipStreamCreateWithFlags(&m_copyStream, hipStreamNonBlocking), "hipStreamCreate");
      for (auto &ev : m_pieceReady) Check(hipEventCreateWithFlags(&ev, hipEventDisableTiming), "hipEventCreate");
    }
    // Pinned inputs are read by DMA where they lie, in 8 pieces.  Pageable inputs are first moved into
    // one of two pinned buffers by a few host threads (one core copies slower than the link carries):
    // pieces of about 16 MB, the host copy of piece i+1 overlapping the DMA of piece i.
    const bool staged = !IsPinnedHost(hostInputs);
    int64_t pieces = staged ? (int64_t)((totalBytes + ((size_t)16 << 20) - 1) >> 24) : 8;
    pieces = std::max<int64_t>(2, std::min<int64_t>({pieces, (int64_t)kMaxPieces, rows / 4096}));
    const int64_t perPiece = ((rows + pieces - 1) / pieces + 1023) / 1024 * 1024;
    if (staged) {
      const size_t pieceBytes = (size_t)perPiece * rowBytes;
      if (pieceBytes > m_pinnedBytes) {
        for (void *&buf : m_pinned) {
          if (buf) (void)hipHostFree(buf);
          buf = nullptr;
        }
        m_pinnedBytes = 0;
        for (void *&buf : m_pinned) Check(hipHostMalloc(&buf, pieceBytes, hipHostMallocDefault), "allocate pinned staging");
        m_pinnedBytes = pieceBytes;
      }
      if (!m_copier) m_copier.reset(new ParallelCopier((int)std::min(8u, std::max(1u, std::thread::hardware_concurrency()))));
    }
    const Workspace ws = OwnWorkspace(perPiece, m_stream); // the pieces run one after the other on the runner's stream
    int p = 0;
    for (int64_t first = 0; first < rows; first += perPiece, ++p) {
      const int64_t count = std::min(perPiece, rows - first);
      float *dIn = m_dStageIn + first * m_forest.numFeatures;
      const char *src = static_cast<const char *>(hostInputs) + (size_t)first * rowBytes;
      if (staged) {
        if (p >= 2) Check(hipEventSynchronize(m_pieceReady[p - 2]), "hipEventSynchronize"); // its buffer is free again
        m_copier->Copy(m_pinned[p & 1], src, (size_t)count * rowBytes);
        src = static_cast<const char *>(m_pinned[p & 1]);
      }
      Check(hipMemcpyAsync(dIn, src, (size_t)count * rowBytes, hipMemcpyHostToDevice, m_copyStream), "copy inputs");
      Check(hipEventRecord(m_pieceReady[p], m_copyStream), "hipEventRecord");
      Check(hipStreamWaitEvent(m_stream, m_pieceReady[p], 0), "hipStreamWaitEvent");
      if (ClassIdsAsInt8())
        Launch(dIn, count, nullptr, static_cast<int8_t *>(m_dStageOut) + first, nullptr, nullptr, nullptr, m_stream, ws);
      else
        Launch(dIn, count, static_cast<float *>(m_dStageOut) + first, nullptr, nullptr, nullptr, nullptr, m_stream, ws);
    }
    Check(hipStreamSynchronize(m_stream), "inference kernels");
  }
  Check(hipMemcpy(hostResults, m_dStageOut, (size_t)rows * ReturnTypeBytes(), hipMemcpyDeviceToHost), "copy results");
}

void InferenceRunner::TimeKernels(const float *deviceInputs, void *deviceResults, int64_t rows, int32_t runs,
                                  double *walkMs, double *finalizeMs, double *binMs) {
  runs = std::max(1, runs);
  const Workspace ws = OwnWorkspace(rows, m_stream);
  const bool fused = FusesArgmax();
  const bool finalize = NeedsFinalize() && !fused;
  float ms = 0.f;
  if (binMs) *binMs = 0.0;
  const float *walkInputs = deviceInputs;
  if (m_model.plan.quantizedRows || m_model.plan.rankRows16) {
    Check(hipEventRecord(m_evStart, m_stream), "hipEventRecord");
    for (int i = 0; i < runs; ++i) walkInputs = PrepareRows(deviceInputs, rows, ws.ranks, m_stream);
    Check(hipEventRecord(m_evStop, m_stream), "hipEventRecord");
    Check(hipStreamSynchronize(m_stream), "rank-quantisation kernel");
    Check(hipEventElapsedTime(&ms, m_evStart, m_evStop), "hipEventElapsedTime");
    if (binMs) *binMs = ms / runs;
  }
  WalkParams p = MakeWalkParams(walkInputs, rows);
  p.s.fuseArgmax = fused ? 1 : 0;
  p.out = finalize || (fused && ClassIdsAsInt8()) ? nullptr : static_cast<float *>(deviceResults);
  p.classOut = fused && ClassIdsAsInt8() ? static_cast<int8_t *>(deviceResults) : nullptr;
  p.partial = finalize ? ws.partial : nullptr;
  Check(hipEventRecord(m_evStart, m_stream), "hipEventRecord");
  for (int i = 0; i < runs; ++i) Check(LaunchWalk(p, m_stream), "launch walk kernel");
  Check(hipEventRecord(m_evStop, m_stream), "hipEventRecord");
  Check(hipStreamSynchronize(m_stream), "walk kernel");
  Check(hipEventElapsedTime(&ms, m_evStart, m_evStop), "hipEventElapsedTime");
  if (walkMs) *walkMs = ms / runs;
  if (finalizeMs) *finalizeMs = 0.0;
  if (finalize) {
    FinalizeParams f;
    f.partial = ws.partial;
    f.rows = rows;
    f.numClasses = m_forest.numClasses;
    f.treeSlices = m_model.PartialCount();
    f.initialValue = m_forest.initialValue;
    f.transform = p.s.transform;
    if (ClassIdsAsInt8()) f.classOut = static_cast<int8_t *>(deviceResults);
    else f.out = static_cast<float *>(deviceResults);
    Check(hipEventRecord(m_evStart, m_stream), "hipEventRecord");
    for (int i = 0; i < runs; ++i) Check(LaunchFinalize(f, m_stream), "launch finalize kernel");
    Check(hipEventRecord(m_evStop, m_stream), "hipEventRecord");
    Check(hipStreamSynchronize(m_stream), "finalize kernel");
    Check(hipEventElapsedTime(&ms, m_evStart, m_evStop), "hipEventElapsedTime");
    if (finalizeMs) *finalizeMs = ms / runs;
  }
}

std::unique_ptr<HitCountProfile> InferenceRunner::CollectProfile(const float *deviceInputs, int64_t rows) {
  std::unique_ptr<HitCountProfile> profile(new HitCountProfile());
  const size_t T = m_forest.trees.size();
  profile->numRows = rows;
  profile->hits.resize(T);
  for (size_t t = 0; t < T; ++t) profile->hits[t].assign(m_forest.trees[t].NumNodes(), 0);
  if (rows <= 0 || T == 0) return profile;
  int32_t *dIds = nullptr;
  Check(hipMalloc(reinterpret_cast<void **>(&dIds), (size_t)rows * T * sizeof(int32_t)), "allocate leaf ids");
  std::vector<int32_t> ids((size_t)rows * T);
  try {
    DumpLeafIds(deviceInputs, dIds, rows);
    Check(hipMemcpy(ids.data(), dIds, ids.size() * sizeof(int32_t), hipMemcpyDeviceToHost), "copy leaf ids");
  } catch (...) {
    (void)hipFree(dIds);
    throw;
  }
  (void)hipFree(dIds);
  for (int64_t r = 0; r < rows; ++r)
    for (size_t t = 0; t < T; ++t) {
      const int32_t leaf = ids[(size_t)r * T + t];
      if (leaf < 0 || (size_t)leaf >= profile->hits[t].size()) throw Error("internal error: leaf id outside its tree");
      ++profile->hits[t][(size_t)leaf];
    }
  // internal nodes: the rows that pass through (children before parents in reverse breadth-first order)
  for (size_t t = 0; t < T; ++t) {
    const Tree &tree = m_forest.trees[t];
    std::vector<int32_t> order{0};
    for (size_t head = 0; head < order.size(); ++head) {
      const int32_t n = order[head];
      if (!tree.IsLeaf(n)) { order.push_back(tree.left[n]); order.push_back(tree.right[n]); }
    }
    for (size_t k = order.size(); k-- > 0;) {
      const int32_t n = order[k];
      if (!tree.IsLeaf(n)) profile->hits[t][(size_t)n] = profile->hits[t][(size_t)tree.left[n]] + profile->hits[t][(size_t)tree.right[n]];
    }
  }
  return profile;
}

void InferenceRunner::EnablePeeledWalks(const float *deviceInputs, int64_t rows) {
  if (rows <= 0 || !deviceInputs) throw Error("peeled walks need rows to profile");
  if (!m_profile) m_profile = CollectProfile(deviceInputs, std::min<int64_t>(rows, 4096));
  LaunchPlan plan = m_model.plan;
  plan.peelWalks = true;
  if (!plan.deferTails && DeferTailsFit(m_forest, &plan)) plan.deferTails = true;
  Repack(plan);
  m_walk.peelWalks = true;
}

double InferenceRunner::AutoTune(const float *deviceInputs, int64_t rows) {
  void *out = nullptr;
  Check(hipMalloc(&out, std::max<int64_t>(rows, 1) * sizeof(float)), "allocate tuning output");
  const LaunchPlan original = m_model.plan;
  // Two rounds: every candidate with a few launches, then the best few (and the analytic plan the runner started
  // with) again with more launches, so that the plan kept is not one that merely had a lucky first timing.
  struct Timed { LaunchPlan plan; double ms; };
  std::vector<Timed> timed;
  auto timePlan = [&](const LaunchPlan &cand, int runs, double *ms) {
    try {
      Repack(cand);
    } catch (const Error &) {
      return false; // plan cannot hold this model
    }
    double w = 0, f = 0, b = 0;
    try {
      TimeKernels(deviceInputs, out, rows, 1, &w, &f, &b); // warm-up
      TimeKernels(deviceInputs, out, rows, runs, &w, &f, &b);
    } catch (const Error &) {
      (void)hipGetLastError(); // plan the launcher rejects (e.g. too few lanes to prefetch a group)
      return false;
    }
    *ms = w + f + b;
    return true;
  };
  LaunchPlan best = original;
  double bestMs = 1e300;
  try {
    for (const LaunchPlan &cand : CandidatePlans(m_forest, rows, m_limits, m_walk)) {
      double ms = 0;
      if (timePlan(cand, 3, &ms)) timed.push_back(Timed{m_model.plan, ms});
    }
    std::stable_sort(timed.begin(), timed.end(), [](const Timed &a, const Timed &b) { return a.ms < b.ms; });
    if (timed.size() > 6) timed.resize(6);
    timed.push_back(Timed{original, 0.0});
    // Peeled walks (deferred tails) of the same shapes: they need a hit-count profile; without one from the caller
    // the rows of this batch are profiled (leaf ids of up to 4096 rows, counted on the host).
    if (!original.deferTails && m_forest.numClasses == 0 && original.tileSize == 1) {
      if (!m_profile) m_profile = CollectProfile(deviceInputs, std::min<int64_t>(rows, 4096));
      const size_t shapes = timed.size();
      for (size_t i = 0; i < shapes; ++i) {
        LaunchPlan p = timed[i].plan;
        p.peelWalks = true;
        if (DeferTailsFit(m_forest, &p)) {
          p.deferTails = true;
          timed.push_back(Timed{p, 0.0});
        }
      }
    }
    // The finalists take turns, three passes of eight launches each, and a plan is judged by its best pass: the
    // clock of the device drifts while it warms up, and a plan timed once, early, would be judged by that.
    std::vector<double> bestPass(timed.size(), 1e300);
    for (int pass = 0; pass < 3; ++pass)
      for (size_t i = 0; i < timed.size(); ++i) {
        double ms = 0;
        if (bestPass[i] < 0 || !timePlan(timed[i].plan, 8, &ms)) {
          bestPass[i] = -1; // a plan that failed once is out
          continue;
        }
        bestPass[i] = std::min(bestPass[i], ms);
        timed[i].plan = m_model.plan;
      }
    for (size_t i = 0; i < timed.size(); ++i)
      if (bestPass[i] >= 0 && bestPass[i] < bestMs) {
        bestMs = bestPass[i];
        best = timed[i].plan;
      }
    m_walk.peelWalks = best.peelWalks;
    Repack(best);
  } catch (...) {
    (void)hipFree(out);
    throw;
  }
  (void)hipFree(out);
  return bestMs;
}

std::string InferenceRunner::DescribePlan() const {
  std::ostringstream os;
  const LaunchPlan &p = m_model.plan;
  // Walk peeling as the launch will apply it: the tiled walk and the scalar row-parallel walk on an f32 tile
  // with byte offsets have the peeled form; the other walks take every bundle to its full depth.
  std::string peel = "0";
  if (p.peelWalks) {
    if (p.kernel == LaunchPlan::Kernel::kTreeParallel) peel = "ignored(tree_parallel)";
    else if (p.kernel == LaunchPlan::Kernel::kGlobalWalk) peel = "ignored(global_walk)";
    else if (p.tileSize > 1 || p.deferTails) peel = "1";
    else if (m_forest.numClasses > 0) peel = "ignored(classes)";
    else if (p.quantizedRows || p.rankRows16) peel = "ignored(ranks)";
    else if (p.featureOffsetInWords) peel = "ignored(words)";
    else peel = "ignored(lds)"; // the stub column and the queues do not fit beside this plan's tree groups
  }
  os << "kernel="
     << (p.kernel == LaunchPlan::Kernel::kTreeParallel ? "tree_parallel"
         : p.kernel == LaunchPlan::Kernel::kGlobalWalk ? "global_walk"
                                                       : "rows_lds")
     << " rowsPerBlock=" << p.rowsPerBlock << " treeThreads=" << p.treeThreads << " treeLanes=" << p.treeLanes
     << " interleave=" << p.interleave
     << " groupBytes=" << p.groupBytes << " treeSlices=" << p.treeSlices
     << " offsetsInWords=" << (p.featureOffsetInWords ? 1 : 0) << " quantizedRows=" << (p.quantizedRows ? 1 : 0) << " rankRows16=" << (p.rankRows16 ? 1 : 0)
     << " groups=" << m_model.groups.size()
     << " bundles=" << m_model.bundles.size() << " nodes=" << m_model.nodes.size()
     << " ldsBytes=" << m_model.LdsBytes() << " tileSize=" << p.tileSize << " tiling=" << p.tiling
     << " staging=" << (DirectStaging() ? "direct" : "registers")
     << " peelWalks=" << peel << " treesTiledByProfile=" << m_model.treesTiledByProfile
     << " lockStepSteps=" << m_model.lockStepSteps << " profiledSteps=" << m_model.profiledSteps
     << " treesDeferred=" << m_model.treesDeferred << " deferredEntriesPerRow=" << m_model.deferredEntriesPerRow;
  return os.str();
}

} // namespace tbamd
