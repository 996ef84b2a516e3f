// Compiled model + device buffers + the RunInference entry points.
//
// Stands where the reference has InferenceRunnerBase / GPUInferenceRunner
// (src/mlir/ExecutionHelpers.h:42-111, src/gpu/GPUExecutionHelper.h:34-60) and
// the generated Prediction_Function's per-call alloc + H2D + kernel + D2H
// (src/gpu/GPUSupportUtils.cpp:150-343).  Here the staging buffers are
// allocated once per runner.
#pragma once

#include "forest.h"
#include "kernels.h"
#include "options.h"
#include "host_copy.h"
#include "packer.h"
#include "tuner.h"

#include <hip/hip_runtime.h>

#include <memory>
#include <string>

namespace tbamd {

// Process-wide switches of the reference's kernel-time shim
// (src/gpu/GPUSupportUtils.cpp:52-104, :389-390).
extern bool gMeasureGpuKernelTime;
extern int32_t gNumberOfKernelRuns;
// The reference's switch for peeled walks under probability-based tiling
// (SetPeeledCodeGenForProbabilityBasedTiling, src/runtime/runtime.cpp:309-315); read when a runner is made.
extern bool gPeeledWalks;

class InferenceRunner {
public:
  // `profile` (may be null): leaf hit counts for probability-based tiling and walk peeling, used when the
  // options ask for a non-uniform tiling type.
  InferenceRunner(Forest forest, const CompilerOptions &options, const GPUAutoScheduleOptions *gpuOptions,
                  std::unique_ptr<HitCountProfile> profile = nullptr);
  // Reopens a compiled model: the plan is taken as saved instead of asking the tuner.
  InferenceRunner(Forest forest, const CompilerOptions &options, const LaunchPlan &plan,
                  std::unique_ptr<HitCountProfile> profile = nullptr);
  ~InferenceRunner();
  InferenceRunner(const InferenceRunner &) = delete;
  InferenceRunner &operator=(const InferenceRunner &) = delete;

  // Host buffers, exactly batchSize rows (src/runtime/runtime.cpp:58-67).
  void RunInference(const void *hostInputs, void *hostResults);
  // Host buffers, any number of rows: batch-sized windows, each copied and computed in overlapping pieces.
  void RunHost(const void *hostInputs, void *hostResults, int64_t rows);
  // Device-resident rows; `out` holds ReturnTypeBytes() per row.
  void RunDevice(const float *deviceInputs, void *deviceResults, int64_t rows);
  // The same kernels enqueued on the caller's stream; returns without waiting for them.  Work the caller
  // queued on that stream before the call is seen by the kernels, work queued after it sees their results.
  // The runner's buffers (model, partial sums, rank-quantised rows) are shared by all calls: an event recorded
  // behind the kernels orders the next call after them when it comes on another stream (or on the runner's
  // own), and re-packing, growing the buffers and deleting the runner wait for it on the host.
  void RunDeviceOnStream(const float *deviceInputs, void *deviceResults, int64_t rows, hipStream_t stream);
  // As RunDeviceOnStream, but the partial sums and rank-quantised rows go into the library's fixed
  // device array instead of allocated buffers: no allocation, no free, no synchronisation.  Throws when
  // the plan needs more than NoAllocScratchBytes() for `rows` rows.
  void RunDeviceNoAlloc(const float *deviceInputs, void *deviceResults, int64_t rows, hipStream_t stream);
  // Bytes of the fixed device array the no-allocation entry point may use.
  static size_t NoAllocScratchBytes();
  // Multiclass extras: any of the outputs may be null.
  void RunDeviceMulticlass(const float *deviceInputs, int64_t rows, int8_t *classIds, float *margins,
                           float *probabilities);
  // Parity check: original leaf node id reached by every (row, tree), int32[rows][numTrees].
  void DumpLeafIds(const float *deviceInputs, int32_t *deviceLeafIds, int64_t rows);
  // Average duration in milliseconds of the walk kernel, of the finalize kernel and of the
  // rank-quantisation kernel (0 when the plan does not use them) over `runs` launches each,
  // HIP events on the runner's stream.
  void TimeKernels(const float *deviceInputs, void *deviceResults, int64_t rows, int32_t runs, double *walkMs,
                   double *finalizeMs, double *binMs);
  // Re-packs the model for another launch plan (used by the timed search).
  void Repack(const LaunchPlan &plan);
  // Timed search over CandidatePlans(); keeps the fastest.  Returns its time in ms.  A runner without a hit-count
  // profile profiles up to 4096 of the rows itself, so that peeled walks can be among the candidates.
  double AutoTune(const float *deviceInputs, int64_t rows);
  // Peeled walks without a profile file: profiles up to 4096 of the given rows on the device (unless the runner
  // has a profile already) and re-packs the current plan with peeled walks where the plan has the form.
  void EnablePeeledWalks(const float *deviceInputs, int64_t rows);
  // Leaf hit counts of `rows` device-resident rows (the reference's probability profile, src/utils/StatsUtils.cpp:10-52).
  std::unique_ptr<HitCountProfile> CollectProfile(const float *deviceInputs, int64_t rows);

  int32_t BatchSize() const { return m_options.batchSize; }
  int32_t RowSize() const { return m_forest.numFeatures; }
  int32_t NumTrees() const { return (int32_t)m_forest.trees.size(); }
  int32_t NumClasses() const { return m_forest.numClasses; }
  // Regressors and binary classifiers return float32; multiclass models return the class id as int8
  // (returnTypeWidth 8, the reference's multiclass setting) or as float32 (its default options).
  bool ClassIdsAsInt8() const { return m_forest.numClasses > 0 && m_options.returnTypeWidth == 8; }
  int32_t ReturnTypeBytes() const { return ClassIdsAsInt8() ? 1 : 4; }
  const CompilerOptions &Options() const { return m_options; }
  int64_t LastKernelMicros() const { return m_lastKernelMicros; }
  // How the row-parallel scalar walk brings tree groups into LDS: 0 by rule (direct global -> LDS copies when two
  // blocks fit a CU, so that one walks while the other waits for its copy; through prefetch registers
  // otherwise), 1 always through registers, 2 always direct.
  void SetGroupStaging(int32_t mode);
  bool DirectStaging() const;
  const PackedModel &Model() const { return m_model; }
  const Forest &GetForest() const { return m_forest; }
  const HitCountProfile *Profile() const { return m_profile.get(); }
  std::string DescribePlan() const;
  hipStream_t Stream() const { return m_stream; }

private:
  void Release() noexcept;
  void RunHostChunk(const void *hostInputs, void *hostResults, int64_t rows);
  void InitDevice();
  // Ordering of calls that share the runner's buffers (see RunDeviceOnStream).
  void OrderAfterAsyncCall(hipStream_t stream); // device-side: `stream` waits for the last asynchronous call
  void WaitForAsyncCall();                       // host-side: returns when the last asynchronous call has finished
  void UploadModel();
  void FreeModel();
  void EnsurePartial(int64_t rows);
  void EnsureStaging(int64_t rows);
  void EnsureRanks(int64_t rows);
  // Device memory the kernels of one call use beyond inputs and outputs.
  struct Workspace {
    double *partial = nullptr; // [PartialCount()][rows][max(1, classes)] when NeedsFinalize()
    uint8_t *ranks = nullptr;  // rank-quantised rows when the plan uses them
  };
  // Allocating callers: grows the runner's own buffers to hold `rows` rows and orders `stream`, on which the
  // caller is about to launch, behind an asynchronous call that may still use them.
  Workspace OwnWorkspace(int64_t rows, hipStream_t stream);
  size_t PartialBytes(int64_t rows) const;
  size_t RanksBytes(int64_t rows) const;
  // Rank-quantised plans: runs the binning kernel and returns the buffer the walk kernel reads.
  const float *PrepareRows(const float *deviceInputs, int64_t rows, uint8_t *ranks, hipStream_t stream);
  bool NeedsFinalize() const { return m_model.plan.treeSlices > 1 || m_forest.numClasses > 0; }
  // Classifier, one tree slice, row-parallel LDS kernel: the walk kernel can store the class id itself.
  bool FusesArgmax() const {
    return m_forest.numClasses > 0 && m_model.plan.treeSlices == 1 && m_model.plan.kernel == LaunchPlan::Kernel::kRowParallelLds;
  }
  WalkParams MakeWalkParams(const float *deviceInputs, int64_t rows) const;
  hipError_t LaunchWalk(const WalkParams &p, hipStream_t stream) const;
  void Launch(const float *deviceInputs, int64_t rows, float *out, int8_t *classOut, float *margins,
              float *probabilities, int32_t *leafIds, hipStream_t stream, const Workspace &ws);

  Forest m_forest;
  std::unique_ptr<HitCountProfile> m_profile;
  WalkOptions m_walk;
  CompilerOptions m_options;
  DeviceLimits m_limits;
  PackedModel m_model;
  int m_device = 0; // the device that was current at construction
  hipStream_t m_stream = nullptr;
  hipStream_t m_copyStream = nullptr; // host-buffer entry point: copies of the next piece overlap the kernels
  static constexpr int kMaxPieces = 64;
  hipEvent_t m_pieceReady[kMaxPieces] = {};
  // pageable inputs pass through two pinned buffers, filled by a few host threads
  void *m_pinned[2] = {nullptr, nullptr};
  size_t m_pinnedBytes = 0;
  std::unique_ptr<ParallelCopier> m_copier;
  hipEvent_t m_evStart = nullptr, m_evStop = nullptr;
  hipEvent_t m_asyncDone = nullptr; // recorded behind the kernels of the last RunDeviceOnStream call
  hipStream_t m_asyncStream = nullptr;
  bool m_asyncPending = false;

  DeviceGlobalNode *m_dGlobalNodes = nullptr;
  DeviceGlobalTree *m_dGlobalTrees = nullptr;
  DeviceNode *m_dNodes = nullptr;
  DeviceBundle *m_dBundles = nullptr;
  DeviceNode *m_dBundleRoots = nullptr;
  DeviceGroup *m_dGroups = nullptr;
  int32_t *m_dNodeOrigin = nullptr;
  int32_t *m_dSlotTree = nullptr;
  double *m_dPartial = nullptr;
  size_t m_partialBytes = 0;
  float *m_dBinTable = nullptr;                 // threshold tables of the rank-quantising kernels (one- or two-byte ranks)
  DeviceNode *m_dTailNodes = nullptr;           // deferred tails: the subtrees below the stubs
  int32_t *m_dTailOrigin = nullptr;
  RankFeatureDesc *m_dRankFeatures = nullptr;   // two-byte ranks: per-feature table index
  RankChunkDesc *m_dRankChunks = nullptr;
  uint32_t m_rankChunkEntries = 0, m_rankChunkFeatures = 0; // the largest chunk: the ranking kernel's LDS need
  uint8_t *m_dRanks = nullptr;
  size_t m_ranksBytes = 0;
  float *m_dStageIn = nullptr;
  void *m_dStageOut = nullptr;
  int64_t m_stageRows = 0;
  int64_t m_lastKernelMicros = 0;
  int32_t m_groupStaging = 0;
};

} // namespace tbamd
