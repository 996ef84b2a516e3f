/*
 * C ABI of the MI355X decision-forest inference runtime.
 *
 * Every entry point in the first part keeps the name, argument list and
 * meaning of the reference runtime it stands in for
 * (src/runtime/tbruntime.h:10-48 and src/runtime/runtime.cpp in the reference
 * checkout; the line given with each declaration is the definition it
 * replaces).  Handles are pointers passed as intptr_t / void*, created by the
 * Create / Construct functions and released by the matching Delete / Destroy.
 * The reference aborts on errors; here a failing call returns 0 / does nothing
 * and leaves a message for tbmi_last_error().  Not thread-safe (neither is the
 * reference: process-wide singletons and flags).
 *
 * Buffers of the reference entry points are caller-owned HOST memory:
 * inputs  = batchSize x rowSize float32, row-major, contiguous;
 * results = batchSize float32; a multiclass model returns class ids, as int8
 *           when the options say returnTypeWidth 8 / returnTypeFloatType 0 (what
 *           the reference's multiclass tests set), as float32 with the default options.
 *
 * The tbmi_ entry points in the second part have no counterpart in the
 * reference: device-resident inference, parity dumps, timing and tuning.
 */
#ifndef TBRUNTIME_AMD_H
#define TBRUNTIME_AMD_H

#include <stdbool.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define TBAMD_EXPORT __attribute__((visibility("default")))

/* ---- execution (runtime.cpp:58, :69, :94, :103, :112) ---- */
TBAMD_EXPORT void RunInference(intptr_t inferenceRunner, void *inputs, void *results);
TBAMD_EXPORT void RunInferenceOnMultipleBatches(intptr_t inferenceRunner, void *inputs, void *results,
                                                int32_t numRows);
TBAMD_EXPORT int32_t GetBatchSize(intptr_t inferenceRunner);
TBAMD_EXPORT int32_t GetRowSize(intptr_t inferenceRunner);
TBAMD_EXPORT void DeleteInferenceRunner(intptr_t inferenceRunner);

/* ---- compiler options (runtime.cpp:123-174) ---- */
TBAMD_EXPORT intptr_t CreateCompilerOptions(void);
TBAMD_EXPORT void DeleteCompilerOptions(intptr_t options);
TBAMD_EXPORT void Set_numberOfFeatures(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_batchSize(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_tileSize(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_thresholdTypeWidth(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_returnTypeWidth(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_returnTypeFloatType(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_featureIndexTypeWidth(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_nodeIndexTypeWidth(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_inputElementTypeWidth(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_tileShapeBitWidth(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_childIndexBitWidth(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_makeAllLeavesSameDepth(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_reorderTreesByDepth(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_statsProfileCSVPath(intptr_t options, const char *val);
TBAMD_EXPORT void Set_pipelineSize(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_numberOfCores(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_numParallelTreeBatches(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_tilingType(intptr_t options, int32_t val); /* 0 uniform, 1 probabilistic, 2 hybrid */

/* ---- GPU auto-schedule options (runtime.cpp:181-208) ---- */
TBAMD_EXPORT intptr_t CreateGPUAutoScheduleOptions(void);
TBAMD_EXPORT void DeleteGPUAutoScheduleOptions(intptr_t options);
TBAMD_EXPORT void Set_numRowsPerTB(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_numRowsPerThread(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_rowTileSize(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_numTreeThreads(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_numTreesAtATime(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_cacheRows(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_cacheTrees(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_unrollTreeWalks(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_treeWalkInterleaveFactor(intptr_t options, int32_t val);
TBAMD_EXPORT void Set_sharedMemoryReduce(intptr_t options, int32_t val);

/* ---- compile (runtime.cpp:231, :283) ---- */
TBAMD_EXPORT intptr_t CreateInferenceRunner(const char *modelJSONPath, const char *profileCSVPath,
                                            intptr_t options);
TBAMD_EXPORT intptr_t CreateInferenceRunnerForONNXModel(const char *modelPath, intptr_t options);

/* ---- process-wide switches (runtime.cpp:301-325, :753) ---- */
TBAMD_EXPORT void SetEnableSparseRepresentation(int32_t val);
TBAMD_EXPORT int32_t IsSparseRepresentationEnabled(void);
TBAMD_EXPORT void SetPeeledCodeGenForProbabilityBasedTiling(int32_t val);
TBAMD_EXPORT int32_t IsPeeledCodeGenForProbabilityBasedTilingEnabled(void);
TBAMD_EXPORT void SetEnableMeasureGpuKernelTime(bool val);
TBAMD_EXPORT void SetNumberOfKernelRuns(int32_t val);
TBAMD_EXPORT int64_t GetGPUKernelExecutionTime(intptr_t inferenceRunner); /* microseconds */

/* ---- context API used by the GPU path (runtime.cpp:363-412, :468, :769) ---- */
TBAMD_EXPORT intptr_t ConstructTreebeardContext(const char *modelPath, const char *modelGlobalsJSONPath,
                                                intptr_t options);
TBAMD_EXPORT intptr_t ConstructTreebeardContextFromGPUAutoscheduleOptions(const char *modelPath,
                                                                          const char *modelGlobalsJSONPath,
                                                                          intptr_t options,
                                                                          intptr_t gpuScheduleOptions);
TBAMD_EXPORT void DestroyTreebeardContext(intptr_t tbContext);
TBAMD_EXPORT void SetForestCreatorType(intptr_t tbContext, const char *creatorType); /* "xgboost_json" | "onnx_file" */
TBAMD_EXPORT void SetRepresentationAndSerializer(intptr_t tbContext, const char *repType);
TBAMD_EXPORT void *ConstructGPUInferenceRunnerFromTBContext(void *tbContext);
TBAMD_EXPORT void *ConstructInferenceRunnerFromHIR(void *tbContext);    /* runtime.cpp:442 */
TBAMD_EXPORT void *ConstructGPUInferenceRunnerFromHIR(void *tbContext); /* runtime.cpp:455 */
TBAMD_EXPORT void BuildHIRRepresentation(void *tbContext);              /* runtime.cpp:418; loads the model */
TBAMD_EXPORT void *findBestGPUScheduleAndCompileModel(void *tbContext);

/* ------------------------------------------------------------------------ */
/* Additions without a counterpart in the reference.  Functions returning    */
/* int32_t return 0 on success and -1 on failure (see tbmi_last_error).      */
/* ------------------------------------------------------------------------ */
TBAMD_EXPORT const char *tbmi_last_error(void);
TBAMD_EXPORT int32_t tbmi_device_count(void);

/* Inference on rows already resident in device memory (any row count); results as RunInference writes them.
 * The kernels run on a stream of the runner that does not order itself with any other stream: whatever
 * produced the buffers (a fill, a copy, a kernel on the caller's stream) must have completed before the
 * call - synchronise that stream first.  The call returns after the results are written. */
TBAMD_EXPORT int32_t tbmi_run_device(intptr_t runner, const float *deviceInputs, void *deviceResults, int64_t rows);
/* The same kernels enqueued on the caller's stream (a hipStream_t; null is the default stream); the call
 * returns without waiting for them.  Work queued on that stream before the call is seen by the kernels,
 * work queued after it sees their results: no synchronisation is needed on either side.  All calls on one
 * runner share its device buffers (the packed model, partial sums, rank-quantised rows); the library records
 * an event behind the kernels of every call made here, and the next call on this runner - on another stream,
 * or through an entry point that uses the runner's own stream - waits for it on the device, while calls that
 * re-pack the model (tbmi_set_*_plan, tbmi_autotune), grow the buffers (the first call, and a call with more
 * rows than any before it, allocates) or delete the runner wait for it on the host.  Calls on one runner are
 * therefore ordered, never concurrent; use one runner per stream for kernels that should overlap.  One caller
 * thread per runner, as in the reference. */
TBAMD_EXPORT int32_t tbmi_run_device_async(intptr_t runner, const float *deviceInputs, void *deviceResults,
                                           int64_t rows, void *stream);
/* No counterpart in the reference.  For callers that cannot allocate device memory (code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc): tbmi_run_device_async with the kernels'
 * scratch memory (partial sums of classifiers and of plans that split the trees over several blocks, the
 * rank-quantised rows of wide models) taken from one fixed device array of tbmi_noalloc_scratch_bytes()
 * bytes (32 MiB) that the library holds on every GPU it runs on.  It allocates, frees and synchronises
 * nothing.  A call whose plan needs more scratch memory than that for `rows` rows fails with a message
 * naming both sizes (pass fewer rows per call).  All calls on one GPU share the array: calls that overlap
 * in time on one GPU, from any runner or stream, race on it.  Because it may be captured into a graph this
 * entry point records no event either: the caller keeps the runner alive and un-repacked (no tbmi_set_*_plan,
 * tbmi_autotune, DeleteInferenceRunner) until the kernels of its calls have finished.  The array costs every
 * process that loads the library 32 MiB of device memory per GPU it touches. */
TBAMD_EXPORT int32_t tbmi_run_device_noalloc(intptr_t runner, const float *deviceInputs, void *deviceResults,
                                             int64_t rows, void *stream);
TBAMD_EXPORT int64_t tbmi_noalloc_scratch_bytes(void);
/* Host buffers like RunInference, but any number of rows (the reference fixes the batch at compile time,
 * src/runtime/runtime.cpp:58-67): batch-sized windows, copies overlapped with the kernels. */
TBAMD_EXPORT int32_t tbmi_run_host(intptr_t runner, const void *hostInputs, void *hostResults, int64_t rows);
/* Bytes per row that RunInference / tbmi_run_device write: 4 (float32) or 1 (int8 class ids). */
TBAMD_EXPORT int32_t tbmi_result_bytes(intptr_t runner);
/* Multiclass: arg-max class ids (int8), per-class sums and softmax (float32 [rows][classes]); any may be null. */
TBAMD_EXPORT int32_t tbmi_run_device_multiclass(intptr_t runner, const float *deviceInputs, int64_t rows,
                                                int8_t *deviceClassIds, float *deviceMargins,
                                                float *deviceProbabilities);
/* Parity check: id (in the model file's numbering) of the leaf each row reaches in each tree,
 * int32 [rows][numTrees] in device memory. */
TBAMD_EXPORT int32_t tbmi_dump_leaf_ids(intptr_t runner, const float *deviceInputs, int32_t *deviceLeafIds,
                                        int64_t rows);
/* Average kernel durations (ms) over `runs` launches each, measured with HIP events on the runner's stream:
 * the walk kernel, the finalize kernel and the rank-quantisation kernel (0 when the plan has none). */
TBAMD_EXPORT int32_t tbmi_time_kernels(intptr_t runner, const float *deviceInputs, void *deviceResults,
                                       int64_t rows, int32_t runs, double *walkMs, double *finalizeMs,
                                       double *binMs);
/* Timed search over launch plans on the given rows; keeps the fastest plan. */
TBAMD_EXPORT int32_t tbmi_autotune(intptr_t runner, const float *deviceInputs, int64_t rows, double *bestMs);
/* Pins the row-parallel kernel: rowsPerBlock rows per block, treeThreads lanes per row (in different
 * waves), interleave trees walked at once per lane, groupBytes of LDS per tree group, treeSlices blocks
 * per row block (values <= 0 keep the current choice; treeThreads <= 0 means 1). */
TBAMD_EXPORT int32_t tbmi_set_plan(intptr_t runner, int32_t rowsPerBlock, int32_t treeThreads, int32_t interleave,
                                   int32_t groupBytes, int32_t treeSlices);
/* Pins the tree-parallel kernel: rowsPerBlock rows per block, treeLanes lanes per row. */
TBAMD_EXPORT int32_t tbmi_set_tree_parallel_plan(intptr_t runner, int32_t rowsPerBlock, int32_t treeLanes,
                                                 int32_t interleave, int32_t groupBytes, int32_t treeSlices);
/* Pins the global-memory walk (the fallback for trees too big for LDS): one lane per row. */
TBAMD_EXPORT int32_t tbmi_set_global_walk_plan(intptr_t runner, int32_t rowsPerBlock, int32_t interleave,
                                               int32_t treeSlices);
/* Pins the row-parallel kernel on rank-quantised rows (64 rows per block, one byte per feature value). */
TBAMD_EXPORT int32_t tbmi_set_quantized_plan(intptr_t runner, int32_t treeThreads, int32_t interleave,
                                             int32_t groupBytes, int32_t treeSlices);
/* Peeled walks (SetPeeledCodeGenForProbabilityBasedTiling, src/runtime/runtime.cpp:309-315) without a profile
 * file: the library profiles up to 4096 of the given device-resident rows itself (leaf hit counts, as
 * src/utils/StatsUtils.cpp:10-52 writes them) unless the runner was made with a profile, and re-packs the current
 * launch plan with peeled walks where the plan has the form (tbmi_describe_plan says `peelWalks=1` or why not). */
TBAMD_EXPORT int32_t tbmi_enable_peeled_walks(intptr_t runner, const float *deviceInputs, int64_t rows);
/* Pins the row-parallel kernel on two-byte rank rows: a ranking kernel first replaces every value by the number
 * of its feature's distinct split thresholds that are <= it (exact: every comparison keeps its outcome), laid
 * out so that the walk's row tile takes half the LDS of float32 rows.  For models of up to about 120 features
 * (the tile of `rowsPerBlock` rows must stay below 64 KB) with at most 65534 distinct thresholds per feature.
 * No counterpart in the reference. */
TBAMD_EXPORT int32_t tbmi_set_rank16_plan(intptr_t runner, int32_t rowsPerBlock, int32_t treeThreads, int32_t interleave,
                                          int32_t groupBytes, int32_t treeSlices);
/* How the row-parallel scalar walk brings tree groups into LDS: 0 by rule (direct global-to-LDS copies when two
 * blocks fit a compute unit, through prefetch registers otherwise), 1 always through registers, 2 always direct.
 * Results do not depend on it.  No counterpart in the reference (its GPU schedules cache trees with cooperative
 * loads, src/gpu/GPURepresentations.cpp:279-399). */
TBAMD_EXPORT int32_t tbmi_set_group_staging(intptr_t runner, int32_t mode);
TBAMD_EXPORT int32_t tbmi_describe_plan(intptr_t runner, char *buffer, int32_t length);
/* Compile once, reload: saves the compiled model (forest + launch plan) of a runner to one file and
 * reopens it without the source model (batchSize <= 0 keeps the saved batch size).  Stands in for
 * InitializeInferenceRunner(soPath, globalsJSON), runtime.cpp:35-54. */
TBAMD_EXPORT int32_t tbmi_save_compiled_model(intptr_t runner, const char *path);
TBAMD_EXPORT intptr_t tbmi_load_compiled_model(const char *path, int32_t batchSize);
/* src/runtime/runtime.cpp:35-54 (`InitializeInferenceRunner(soPath, modelGlobalsJSONPath)`, bound by
 * src/python/treebeard.py:314-319 FromSOFile): reopens a compiled model with the saved batch size.  `soPath` names
 * a file written by tbmi_save_compiled_model, which also holds what the reference keeps in its model-globals
 * JSON (tile size, type widths, the model buffers' contents); `modelGlobalsJSONPath` is accepted and not opened.
 * Returns 0 on failure (message in tbmi_last_error). */
TBAMD_EXPORT intptr_t InitializeInferenceRunner(const char *soPath, const char *modelGlobalsJSONPath);
TBAMD_EXPORT int32_t tbmi_num_trees(intptr_t runner);
TBAMD_EXPORT int32_t tbmi_num_classes(intptr_t runner);

/* Host-only model inspection (works without a GPU): loader and packer checks. */
TBAMD_EXPORT intptr_t tbmi_load_forest(const char *modelPath, const char *creatorType, int32_t numberOfFeatures);
TBAMD_EXPORT void tbmi_delete_forest(intptr_t forest);
/* info[0..5] = numTrees, numFeatures, numClasses, transform, predicate, totalNodes; *initialValue */
TBAMD_EXPORT int32_t tbmi_forest_info(intptr_t forest, int64_t *info, double *initialValue);
TBAMD_EXPORT int32_t tbmi_forest_tree_size(intptr_t forest, int32_t tree);
TBAMD_EXPORT int32_t tbmi_forest_tree(intptr_t forest, int32_t tree, float *value, int32_t *feature, int32_t *left,
                                      int32_t *right, int32_t *classId);
/* Reads a leaf hit-count profile (the reference's probability profile: `numTrees, numRows`, then per tree
 * `hitCount, depth` for every leaf in node order) and checks it against the forest; returns the row count
 * and the average number of internal nodes a profiled row visits. */
TBAMD_EXPORT int32_t tbmi_forest_load_profile(intptr_t forest, const char *profileCSVPath, int64_t *numRows,
                                              double *expectedSteps);
/* Packs the forest for the given plan and unpacks it again; returns the number of trees that differ
 * from the (comparison-normalised) input, or -1 when the plan cannot hold the model.  groupBytes 0 packs
 * the global-memory layout (no tree groups) instead.
 * stats[0..4] = groups, bundles, nodes, ldsBytes, paddingTrees. */
TBAMD_EXPORT int32_t tbmi_pack_roundtrip(intptr_t forest, int32_t rowsPerBlock, int32_t interleave,
                                         int32_t groupBytes, int64_t *stats);

#ifdef __cplusplus
}
#endif
#endif /* TBRUNTIME_AMD_H */
