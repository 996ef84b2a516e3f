// extern "C" surface (include/tbruntime_amd.h).  Nothing throws across it.
#include "../../include/tbruntime_amd.h"

#include "model_file.h"
#include "runner.h"

#include <cstring>
#include <fstream>
#include <memory>
#include <random>
#include <sstream>

using namespace tbamd;

namespace {

thread_local std::string gLastError;
int32_t gSparseRepresentation = 0;
int32_t gPeeledCodeGen = 0;

struct Context {
  std::string modelPath, globalsPath;
  CompilerOptions options;
  bool hasGpuOptions = false;
  GPUAutoScheduleOptions gpuOptions;
  std::string creatorType = "xgboost_json";
  std::string representation;
  std::unique_ptr<Forest> forest;
};

template <typename Fn> auto Guard(Fn &&fn, decltype(fn()) onError) -> decltype(fn()) {
  try {
    gLastError.clear();
    return fn();
  } catch (const std::exception &e) {
    gLastError = e.what();
  } catch (...) {
    gLastError = "unknown error";
  }
  return onError;
}

template <typename Fn> void GuardVoid(Fn &&fn) {
  try {
    gLastError.clear();
    fn();
  } catch (const std::exception &e) {
    gLastError = e.what();
  } catch (...) {
    gLastError = "unknown error";
  }
}

CompilerOptions *Opts(intptr_t h) {
  if (!h) throw Error("null CompilerOptions handle");
  return reinterpret_cast<CompilerOptions *>(h);
}
GPUAutoScheduleOptions *GpuOpts(intptr_t h) {
  if (!h) throw Error("null GPUAutoScheduleOptions handle");
  return reinterpret_cast<GPUAutoScheduleOptions *>(h);
}
InferenceRunner *Runner(intptr_t h) {
  if (!h) throw Error("null inference runner handle");
  return reinterpret_cast<InferenceRunner *>(h);
}
Context *Ctx(intptr_t h) {
  if (!h) throw Error("null TreebeardContext handle");
  return reinterpret_cast<Context *>(h);
}

Forest LoadByType(const std::string &path, const std::string &type, int32_t numFeatures) {
  if (type == "xgboost_json") return LoadXGBoostJSON(path);
  if (type == "onnx_file") return LoadONNX(path, numFeatures);
  throw Error("unknown forest creator type " + type);
}

// The leaf hit-count profile the options name, when they ask for a tiling type that uses one
// (src/mlir/ProbabilityBasedTilingTransform.cpp:124-198 reads the same counts from the model's nodes).
std::unique_ptr<HitCountProfile> ProfileFor(const Forest &forest, const CompilerOptions &options) {
  if (options.statsProfileCSVPath.empty() || options.tilingType == TilingType::kUniform) return nullptr;
  return std::make_unique<HitCountProfile>(LoadHitCountProfile(forest, options.statsProfileCSVPath));
}

InferenceRunner *RunnerFromContext(Context *ctx) {
  Forest forest = ctx->forest ? *ctx->forest : LoadByType(ctx->modelPath, ctx->creatorType, ctx->options.numberOfFeatures);
  std::unique_ptr<HitCountProfile> profile = ProfileFor(forest, ctx->options);
  return new InferenceRunner(std::move(forest), ctx->options, ctx->hasGpuOptions ? &ctx->gpuOptions : nullptr,
                             std::move(profile));
}

// Rows for the timed plan search: `<model>.test.sampled.csv` next to the model
// when it exists (what the reference's tuner reads,
// src/test/GPUBenchmarkUtils.h:58-80, :172-202), repeated to fill the batch;
// otherwise seeded standard-normal values.
std::vector<float> TuningRows(const std::string &modelPath, int32_t rowSize, int64_t rows) {
  std::vector<float> sample;
  std::ifstream in(modelPath + ".test.sampled.csv");
  std::string line;
  while (in && std::getline(in, line)) {
    std::vector<float> vals;
    std::stringstream ss(line);
    std::string cell;
    while (std::getline(ss, cell, ',')) vals.push_back(std::strtof(cell.c_str(), nullptr));
    if ((int32_t)vals.size() >= rowSize) sample.insert(sample.end(), vals.begin(), vals.begin() + rowSize);
  }
  std::vector<float> out((size_t)rows * rowSize);
  if (!sample.empty()) {
    for (size_t i = 0; i < out.size(); ++i) out[i] = sample[i % sample.size()];
  } else {
    std::mt19937 rng(12345);
    std::normal_distribution<float> dist(0.f, 1.f);
    for (auto &v : out) v = dist(rng);
  }
  return out;
}

} // namespace

extern "C" {

// ---- execution ----
void RunInference(intptr_t h, void *inputs, void *results) {
  GuardVoid([&] { Runner(h)->RunInference(inputs, results); });
}

void RunInferenceOnMultipleBatches(intptr_t h, void *inputs, void *results, int32_t numRows) {
  GuardVoid([&] {
    InferenceRunner *r = Runner(h);
    if (numRows % r->BatchSize() != 0) throw Error("numRows must be a multiple of the batch size");
    // rows are independent: the batches go through together (same results as one RunInference per batch)
    r->RunHost(inputs, results, numRows);
  });
}

int32_t GetBatchSize(intptr_t h) { return Guard([&] { return Runner(h)->BatchSize(); }, -1); }
int32_t GetRowSize(intptr_t h) { return Guard([&] { return Runner(h)->RowSize(); }, -1); }
void DeleteInferenceRunner(intptr_t h) { GuardVoid([&] { delete reinterpret_cast<InferenceRunner *>(h); }); }

// ---- compiler options ----
intptr_t CreateCompilerOptions(void) { return reinterpret_cast<intptr_t>(new CompilerOptions); }
void DeleteCompilerOptions(intptr_t h) { delete reinterpret_cast<CompilerOptions *>(h); }

#define TBAMD_OPTION_SETTER(name)                                                                                      \
  void Set_##name(intptr_t h, int32_t val) { GuardVoid([&] { Opts(h)->name = val; }); }
TBAMD_OPTION_SETTER(numberOfFeatures)
TBAMD_OPTION_SETTER(batchSize)
TBAMD_OPTION_SETTER(tileSize)
TBAMD_OPTION_SETTER(thresholdTypeWidth)
TBAMD_OPTION_SETTER(returnTypeWidth)
TBAMD_OPTION_SETTER(returnTypeFloatType)
TBAMD_OPTION_SETTER(featureIndexTypeWidth)
TBAMD_OPTION_SETTER(nodeIndexTypeWidth)
TBAMD_OPTION_SETTER(inputElementTypeWidth)
TBAMD_OPTION_SETTER(tileShapeBitWidth)
TBAMD_OPTION_SETTER(childIndexBitWidth)
TBAMD_OPTION_SETTER(makeAllLeavesSameDepth)
TBAMD_OPTION_SETTER(reorderTreesByDepth)
TBAMD_OPTION_SETTER(pipelineSize)
TBAMD_OPTION_SETTER(numberOfCores)
TBAMD_OPTION_SETTER(numParallelTreeBatches)
#undef TBAMD_OPTION_SETTER

void Set_statsProfileCSVPath(intptr_t h, const char *val) {
  GuardVoid([&] { Opts(h)->statsProfileCSVPath = val ? val : ""; });
}

void Set_tilingType(intptr_t h, int32_t val) {
  GuardVoid([&] {
    if (val < 0 || val > 2) throw Error("Invalid tiling type value");
    Opts(h)->tilingType = static_cast<TilingType>(val);
  });
}

// ---- GPU auto-schedule options ----
intptr_t CreateGPUAutoScheduleOptions(void) { return reinterpret_cast<intptr_t>(new GPUAutoScheduleOptions); }
void DeleteGPUAutoScheduleOptions(intptr_t h) { delete reinterpret_cast<GPUAutoScheduleOptions *>(h); }

#define TBAMD_GPU_OPTION_SETTER(name)                                                                                  \
  void Set_##name(intptr_t h, int32_t val) { GuardVoid([&] { GpuOpts(h)->name = val; }); }
TBAMD_GPU_OPTION_SETTER(numRowsPerTB)
TBAMD_GPU_OPTION_SETTER(numRowsPerThread)
TBAMD_GPU_OPTION_SETTER(rowTileSize)
TBAMD_GPU_OPTION_SETTER(numTreeThreads)
TBAMD_GPU_OPTION_SETTER(numTreesAtATime)
TBAMD_GPU_OPTION_SETTER(cacheRows)
TBAMD_GPU_OPTION_SETTER(cacheTrees)
TBAMD_GPU_OPTION_SETTER(unrollTreeWalks)
TBAMD_GPU_OPTION_SETTER(treeWalkInterleaveFactor)
TBAMD_GPU_OPTION_SETTER(sharedMemoryReduce)
#undef TBAMD_GPU_OPTION_SETTER

// ---- compile ----
intptr_t CreateInferenceRunner(const char *modelJSONPath, const char *profileCSVPath, intptr_t options) {
  return Guard(
      [&]() -> intptr_t {
        CompilerOptions opts = *Opts(options);
        if (profileCSVPath && *profileCSVPath) opts.statsProfileCSVPath = profileCSVPath;
        Forest forest = LoadXGBoostJSON(modelJSONPath);
        std::unique_ptr<HitCountProfile> profile = ProfileFor(forest, opts);
        return reinterpret_cast<intptr_t>(new InferenceRunner(std::move(forest), opts, nullptr, std::move(profile)));
      },
      0);
}

intptr_t CreateInferenceRunnerForONNXModel(const char *modelPath, intptr_t options) {
  return Guard(
      [&]() -> intptr_t {
        CompilerOptions opts = *Opts(options);
        Forest forest = LoadONNX(modelPath, opts.numberOfFeatures);
        std::unique_ptr<HitCountProfile> profile = ProfileFor(forest, opts);
        return reinterpret_cast<intptr_t>(new InferenceRunner(std::move(forest), opts, nullptr, std::move(profile)));
      },
      0);
}

// ---- process-wide switches ----
void SetEnableSparseRepresentation(int32_t val) { gSparseRepresentation = val; }
int32_t IsSparseRepresentationEnabled(void) { return gSparseRepresentation; }
void SetPeeledCodeGenForProbabilityBasedTiling(int32_t val) {
  gPeeledCodeGen = val;
  gPeeledWalks = val != 0;
}
int32_t IsPeeledCodeGenForProbabilityBasedTilingEnabled(void) { return gPeeledCodeGen; }
void SetEnableMeasureGpuKernelTime(bool val) { gMeasureGpuKernelTime = val; }
void SetNumberOfKernelRuns(int32_t val) { gNumberOfKernelRuns = val < 1 ? 1 : val; }
int64_t GetGPUKernelExecutionTime(intptr_t h) {
  return Guard([&]() -> int64_t { return Runner(h)->LastKernelMicros(); }, -1);
}

// ---- context API ----
intptr_t ConstructTreebeardContext(const char *modelPath, const char *globalsPath, intptr_t options) {
  return Guard(
      [&]() -> intptr_t {
        auto *ctx = new Context;
        ctx->modelPath = modelPath ? modelPath : "";
        ctx->globalsPath = globalsPath ? globalsPath : "";
        ctx->options = *Opts(options);
        return reinterpret_cast<intptr_t>(ctx);
      },
      0);
}

intptr_t ConstructTreebeardContextFromGPUAutoscheduleOptions(const char *modelPath, const char *globalsPath,
                                                             intptr_t options, intptr_t gpuOptions) {
  return Guard(
      [&]() -> intptr_t {
        auto *ctx = new Context;
        ctx->modelPath = modelPath ? modelPath : "";
        ctx->globalsPath = globalsPath ? globalsPath : "";
        ctx->options = *Opts(options);
        ctx->gpuOptions = *GpuOpts(gpuOptions);
        ctx->hasGpuOptions = true;
        return reinterpret_cast<intptr_t>(ctx);
      },
      0);
}

void DestroyTreebeardContext(intptr_t h) { delete reinterpret_cast<Context *>(h); }

void SetForestCreatorType(intptr_t h, const char *creatorType) {
  GuardVoid([&] {
    std::string type = creatorType ? creatorType : "";
    if (type != "xgboost_json" && type != "onnx_file") throw Error("unknown forest creator type " + type);
    Ctx(h)->creatorType = type;
  });
}

void SetRepresentationAndSerializer(intptr_t h, const char *repType) {
  GuardVoid([&] {
    std::string rep = repType ? repType : "";
    // The reference's layouts (array, sparse, gpu_array, gpu_sparse, gpu_reorg) all
    // map onto the one LDS-staged device layout here; the name is validated only.
    if (rep != "array" && rep != "sparse" && rep != "gpu_array" && rep != "gpu_sparse" && rep != "gpu_reorg")
      throw Error("unknown representation " + rep);
    Ctx(h)->representation = rep;
  });
}

void BuildHIRRepresentation(void *h) {
  GuardVoid([&] {
    Context *ctx = Ctx(reinterpret_cast<intptr_t>(h));
    ctx->forest = std::make_unique<Forest>(LoadByType(ctx->modelPath, ctx->creatorType, ctx->options.numberOfFeatures));
  });
}

void *ConstructGPUInferenceRunnerFromTBContext(void *h) {
  return Guard([&]() -> void * { return RunnerFromContext(Ctx(reinterpret_cast<intptr_t>(h))); }, nullptr);
}
void *ConstructInferenceRunnerFromHIR(void *h) { return ConstructGPUInferenceRunnerFromTBContext(h); }
void *ConstructGPUInferenceRunnerFromHIR(void *h) { return ConstructGPUInferenceRunnerFromTBContext(h); }

void *findBestGPUScheduleAndCompileModel(void *h) {
  return Guard(
      [&]() -> void * {
        Context *ctx = Ctx(reinterpret_cast<intptr_t>(h));
        std::unique_ptr<InferenceRunner> runner(RunnerFromContext(ctx));
        const int64_t rows = runner->BatchSize();
        std::vector<float> host = TuningRows(ctx->modelPath, runner->RowSize(), rows);
        float *dev = nullptr;
        if (hipMalloc(reinterpret_cast<void **>(&dev), host.size() * sizeof(float)) != hipSuccess)
          throw Error("cannot allocate tuning rows");
        hipError_t e = hipMemcpy(dev, host.data(), host.size() * sizeof(float), hipMemcpyHostToDevice);
        try {
          if (e != hipSuccess) throw Error("cannot copy tuning rows");
          runner->AutoTune(dev, rows);
        } catch (...) {
          (void)hipFree(dev);
          throw;
        }
        (void)hipFree(dev);
        return runner.release();
      },
      nullptr);
}

// ---- additions ----
const char *tbmi_last_error(void) { return gLastError.c_str(); }

int32_t tbmi_device_count(void) {
  int n = 0;
  if (hipGetDeviceCount(&n) != hipSuccess) return 0;
  return n;
}

int32_t tbmi_run_device(intptr_t h, const float *in, void *out, int64_t rows) {
  return Guard([&] { Runner(h)->RunDevice(in, out, rows); return 0; }, -1);
}

int32_t tbmi_run_device_async(intptr_t h, const float *in, void *out, int64_t rows, void *stream) {
  return Guard([&] { Runner(h)->RunDeviceOnStream(in, out, rows, static_cast<hipStream_t>(stream)); return 0; }, -1);
}

int32_t tbmi_run_device_noalloc(intptr_t h, const float *in, void *out, int64_t rows, void *stream) {
  return Guard([&] { Runner(h)->RunDeviceNoAlloc(in, out, rows, static_cast<hipStream_t>(stream)); return 0; }, -1);
}

int64_t tbmi_noalloc_scratch_bytes(void) { return (int64_t)InferenceRunner::NoAllocScratchBytes(); }

int32_t tbmi_run_host(intptr_t h, const void *in, void *out, int64_t rows) {
  return Guard(
      [&] {
        Runner(h)->RunHost(in, out, rows);
        return 0;
      },
      -1);
}

int32_t tbmi_result_bytes(intptr_t h) { return Guard([&] { return Runner(h)->ReturnTypeBytes(); }, -1); }

int32_t tbmi_run_device_multiclass(intptr_t h, const float *in, int64_t rows, int8_t *cls, float *margins,
                                   float *probs) {
  return Guard([&] { Runner(h)->RunDeviceMulticlass(in, rows, cls, margins, probs); return 0; }, -1);
}

int32_t tbmi_dump_leaf_ids(intptr_t h, const float *in, int32_t *ids, int64_t rows) {
  return Guard([&] { Runner(h)->DumpLeafIds(in, ids, rows); return 0; }, -1);
}

int32_t tbmi_time_kernels(intptr_t h, const float *in, void *out, int64_t rows, int32_t runs, double *walkMs,
                          double *finalizeMs, double *binMs) {
  return Guard([&] { Runner(h)->TimeKernels(in, out, rows, runs, walkMs, finalizeMs, binMs); return 0; }, -1);
}

int32_t tbmi_autotune(intptr_t h, const float *in, int64_t rows, double *bestMs) {
  return Guard([&] { double ms = Runner(h)->AutoTune(in, rows); if (bestMs) *bestMs = ms; return 0; }, -1);
}

int32_t tbmi_enable_peeled_walks(intptr_t h, const float *in, int64_t rows) {
  return Guard([&] { Runner(h)->EnablePeeledWalks(in, rows); return 0; }, -1);
}

int32_t tbmi_set_plan(intptr_t h, int32_t rowsPerBlock, int32_t treeThreads, int32_t interleave, int32_t groupBytes,
                      int32_t treeSlices) {
  return Guard(
      [&] {
        InferenceRunner *r = Runner(h);
        LaunchPlan plan = r->Model().plan;
        plan.kernel = LaunchPlan::Kernel::kRowParallelLds;
        plan.treeLanes = 1;
        plan.quantizedRows = false;
        plan.rankRows16 = false;
        if (rowsPerBlock > 0) plan.rowsPerBlock = rowsPerBlock;
        plan.treeThreads = treeThreads > 0 ? treeThreads : 1;
        if (interleave > 0) plan.interleave = interleave;
        if (groupBytes > 0) plan.groupBytes = groupBytes;
        if (treeSlices > 0) plan.treeSlices = treeSlices;
        const int64_t words = (int64_t)(r->RowSize() + 1) * plan.rowsPerBlock;
        plan.featureOffsetInWords = words * 4 > 0xFFFF;
        // peeled walks keep their form where the new shape has room for it (the caller's group size gives up the
        // stub column's and the queues' share)
        plan.deferTails = false;
        if (plan.peelWalks && r->Profile() && plan.tileSize == 1 && DeferTailsFit(r->GetForest(), &plan)) plan.deferTails = true;
        r->Repack(plan);
        return 0;
      },
      -1);
}

int32_t tbmi_set_tree_parallel_plan(intptr_t h, int32_t rowsPerBlock, int32_t treeLanes, int32_t interleave,
                                    int32_t groupBytes, int32_t treeSlices) {
  return Guard(
      [&] {
        InferenceRunner *r = Runner(h);
        LaunchPlan plan = r->Model().plan;
        plan.kernel = LaunchPlan::Kernel::kTreeParallel;
        plan.deferTails = false;
        plan.featureOffsetInWords = false;
        plan.quantizedRows = false;
        plan.rankRows16 = false;
        plan.treeThreads = 1;
        plan.rowsPerBlock = rowsPerBlock;
        plan.treeLanes = treeLanes;
        plan.interleave = interleave > 0 ? interleave : 1;
        if (groupBytes > 0) plan.groupBytes = groupBytes;
        else plan.groupBytes = std::min(plan.groupBytes, 256 * plan.ThreadsPerBlock());
        if (treeSlices > 0) plan.treeSlices = treeSlices;
        r->Repack(plan);
        return 0;
      },
      -1);
}

int32_t tbmi_set_global_walk_plan(intptr_t h, int32_t rowsPerBlock, int32_t interleave, int32_t treeSlices) {
  return Guard(
      [&] {
        InferenceRunner *r = Runner(h);
        LaunchPlan plan;
        plan.kernel = LaunchPlan::Kernel::kGlobalWalk;
        // what the options asked of the walk stays in the plan: a tiled runner is refused by the packer (the
        // global-memory walk has scalar nodes only) instead of quietly turning into a scalar walk
        plan.tileSize = r->Model().plan.tileSize;
        plan.tiling = r->Model().plan.tiling;
        plan.peelWalks = r->Model().plan.peelWalks;
        plan.rowsPerBlock = rowsPerBlock > 0 ? rowsPerBlock : 256;
        plan.interleave = interleave > 0 ? interleave : 4;
        plan.treeSlices = treeSlices > 0 ? treeSlices : 1;
        plan.groupBytes = 0;
        r->Repack(plan);
        return 0;
      },
      -1);
}

int32_t tbmi_set_quantized_plan(intptr_t h, int32_t treeThreads, int32_t interleave, int32_t groupBytes,
                                int32_t treeSlices) {
  return Guard(
      [&] {
        InferenceRunner *r = Runner(h);
        LaunchPlan plan = r->Model().plan;
        plan.kernel = LaunchPlan::Kernel::kRowParallelLds;
        plan.quantizedRows = true;
        plan.rankRows16 = false;
        plan.deferTails = false;
        plan.featureOffsetInWords = false;
        plan.rowsPerBlock = 64;
        plan.treeLanes = 1;
        plan.treeThreads = treeThreads > 0 ? treeThreads : 8;
        plan.interleave = interleave > 0 ? interleave : 4;
        if (groupBytes > 0) plan.groupBytes = groupBytes;
        else plan.groupBytes = std::min(plan.groupBytes, 256 * plan.ThreadsPerBlock());
        plan.treeSlices = treeSlices > 0 ? treeSlices : 1;
        r->Repack(plan);
        return 0;
      },
      -1);
}

int32_t tbmi_set_rank16_plan(intptr_t h, int32_t rowsPerBlock, int32_t treeThreads, int32_t interleave, int32_t groupBytes,
                             int32_t treeSlices) {
  return Guard(
      [&] {
        InferenceRunner *r = Runner(h);
        LaunchPlan plan = r->Model().plan;
        plan.kernel = LaunchPlan::Kernel::kRowParallelLds;
        plan.rankRows16 = true;
        plan.quantizedRows = false;
        plan.deferTails = false;
        plan.featureOffsetInWords = false;
        plan.treeLanes = 1;
        plan.rowsPerBlock = rowsPerBlock > 0 ? rowsPerBlock : 256;
        plan.treeThreads = treeThreads > 0 ? treeThreads : std::max(1, 1024 / plan.rowsPerBlock);
        plan.interleave = interleave > 0 ? interleave : 4;
        if (groupBytes > 0) plan.groupBytes = groupBytes;
        else plan.groupBytes = std::min(plan.groupBytes, 256 * plan.ThreadsPerBlock());
        plan.treeSlices = treeSlices > 0 ? treeSlices : 1;
        r->Repack(plan);
        return 0;
      },
      -1);
}

int32_t tbmi_set_group_staging(intptr_t h, int32_t mode) {
  return Guard(
      [&] {
        Runner(h)->SetGroupStaging(mode);
        return 0;
      },
      -1);
}

int32_t tbmi_describe_plan(intptr_t h, char *buffer, int32_t length) {
  return Guard(
      [&] {
        std::string s = Runner(h)->DescribePlan();
        if (buffer && length > 0) {
          std::strncpy(buffer, s.c_str(), (size_t)length - 1);
          buffer[length - 1] = 0;
        }
        return (int32_t)s.size();
      },
      -1);
}

int32_t tbmi_save_compiled_model(intptr_t h, const char *path) {
  return Guard(
      [&] {
        InferenceRunner *r = Runner(h);
        SaveCompiledModel(path ? path : "", r->GetForest(), r->Model().plan, r->BatchSize(),
                          r->Options().returnTypeWidth, r->Options().returnTypeFloatType, r->Profile());
        return 0;
      },
      -1);
}

intptr_t tbmi_load_compiled_model(const char *path, int32_t batchSize) {
  return Guard(
      [&]() -> intptr_t {
        CompiledModel m = LoadCompiledModel(path ? path : "");
        CompilerOptions options;
        options.batchSize = batchSize > 0 ? batchSize : m.batchSize;
        options.returnTypeWidth = m.returnTypeWidth;
        options.returnTypeFloatType = m.returnTypeFloatType;
        return reinterpret_cast<intptr_t>(new InferenceRunner(std::move(m.forest), options, m.plan, std::move(m.profile)));
      },
      0);
}

// src/runtime/runtime.cpp:35-54.  The reference reopens a compiled shared object together with the JSON of its
// model buffers; here the compiled model is the one file tbmi_save_compiled_model writes, named by `soPath`, and
// it holds everything the reference reads from the JSON (tile size, type widths, the model), so the second
// path is not opened.
intptr_t InitializeInferenceRunner(const char *soPath, const char *modelGlobalsJSONPath) {
  (void)modelGlobalsJSONPath;
  return tbmi_load_compiled_model(soPath, 0);
}

int32_t tbmi_forest_load_profile(intptr_t h, const char *profileCSVPath, int64_t *numRows, double *expectedSteps) {
  return Guard(
      [&] {
        if (!h) throw Error("null forest handle");
        const Forest *f = reinterpret_cast<const Forest *>(h);
        HitCountProfile profile = LoadHitCountProfile(*f, profileCSVPath ? profileCSVPath : "");
        for (size_t t = 0; t < f->trees.size(); ++t)
          if (profile.hits[t][0] != profile.numRows)
            throw Error("hit-count profile: the leaf hits of tree " + std::to_string(t) + " do not add up to numRows");
        if (numRows) *numRows = profile.numRows;
        if (expectedSteps) *expectedSteps = ExpectedWalkSteps(*f, profile);
        return 0;
      },
      -1);
}

int32_t tbmi_num_trees(intptr_t h) { return Guard([&] { return Runner(h)->NumTrees(); }, -1); }
int32_t tbmi_num_classes(intptr_t h) { return Guard([&] { return Runner(h)->NumClasses(); }, -1); }

intptr_t tbmi_load_forest(const char *modelPath, const char *creatorType, int32_t numberOfFeatures) {
  return Guard(
      [&]() -> intptr_t {
        return reinterpret_cast<intptr_t>(
            new Forest(LoadByType(modelPath ? modelPath : "", creatorType ? creatorType : "xgboost_json", numberOfFeatures)));
      },
      0);
}

void tbmi_delete_forest(intptr_t h) { delete reinterpret_cast<Forest *>(h); }

int32_t tbmi_forest_info(intptr_t h, int64_t *info, double *initialValue) {
  return Guard(
      [&] {
        if (!h) throw Error("null forest handle");
        const Forest *f = reinterpret_cast<const Forest *>(h);
        info[0] = (int64_t)f->trees.size();
        info[1] = f->numFeatures;
        info[2] = f->numClasses;
        info[3] = (int64_t)f->transform;
        info[4] = (int64_t)f->predicate;
        info[5] = (int64_t)f->NumNodes();
        if (initialValue) *initialValue = f->initialValue;
        return 0;
      },
      -1);
}

int32_t tbmi_forest_tree_size(intptr_t h, int32_t tree) {
  return Guard(
      [&] {
        if (!h) throw Error("null forest handle");
        return (int32_t) reinterpret_cast<const Forest *>(h)->trees.at((size_t)tree).NumNodes();
      },
      -1);
}

int32_t tbmi_forest_tree(intptr_t h, int32_t tree, float *value, int32_t *feature, int32_t *left, int32_t *right,
                         int32_t *classId) {
  return Guard(
      [&] {
        if (!h) throw Error("null forest handle");
        const Tree &t = reinterpret_cast<const Forest *>(h)->trees.at((size_t)tree);
        std::memcpy(value, t.value.data(), t.NumNodes() * sizeof(float));
        std::memcpy(feature, t.feature.data(), t.NumNodes() * sizeof(int32_t));
        std::memcpy(left, t.left.data(), t.NumNodes() * sizeof(int32_t));
        std::memcpy(right, t.right.data(), t.NumNodes() * sizeof(int32_t));
        if (classId) *classId = t.classId;
        return 0;
      },
      -1);
}

int32_t tbmi_pack_roundtrip(intptr_t h, int32_t rowsPerBlock, int32_t interleave, int32_t groupBytes, int64_t *stats) {
  return Guard(
      [&] {
        if (!h) throw Error("null forest handle");
        const Forest *f = reinterpret_cast<const Forest *>(h);
        LaunchPlan plan;
        plan.rowsPerBlock = rowsPerBlock;
        plan.interleave = interleave;
        plan.groupBytes = groupBytes;
        plan.featureOffsetInWords = (int64_t)(f->numFeatures + 1) * rowsPerBlock * 4 > 0xFFFF;
        if (groupBytes == 0) plan.kernel = LaunchPlan::Kernel::kGlobalWalk; // the layout without tree groups
        PackedModel pm = PackForest(*f, plan);
        const Forest norm = NormalizeToLessThan(*f);
        int32_t mismatches = 0;
        for (size_t t = 0; t < norm.trees.size(); ++t) {
          Tree u = UnpackTree(pm, (int32_t)t);
          const Tree &o = norm.trees[t];
          bool same = u.value == o.value && u.left == o.left && u.right == o.right;
          for (size_t i = 0; same && i < o.NumNodes(); ++i)
            if (!o.IsLeaf((int32_t)i) && u.feature[i] != o.feature[i]) same = false;
          if (f->numClasses > 0 && u.classId != o.classId) same = false;
          if (!same) ++mismatches;
        }
        if (stats) {
          int64_t padding = 0;
          for (int32_t s : pm.slotTree) padding += s < 0;
          stats[0] = (int64_t)pm.groups.size();
          stats[1] = (int64_t)pm.bundles.size();
          stats[2] = (int64_t)(pm.nodes.size() + pm.globalNodes.size());
          stats[3] = (int64_t)pm.LdsBytes();
          stats[4] = padding;
        }
        return mismatches;
      },
      -1);
}

} // extern "C"
