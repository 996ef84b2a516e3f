"""Python front end over the C ABI, with the class and method names of the
reference's wrapper (src/python/treebeard.py) so that scripts written against
it keep working: GPUAutoScheduleOptions (:11-67), CompilerOptions (:72-139),
TreebeardContext (:255-303), TreebeardInferenceRunner (:306-383) and the
module-level switches (:391-411).  The schedule-manipulation classes of the
reference steer its code generator and have no counterpart here.
"""
import ctypes

import numpy

from .runtime_api import api


def _lib():
    return api().runtime_lib


def _check(handle, what):
    if not handle:
        raise RuntimeError("%s failed: %s" % (what, api().last_error()))
    return handle


class GPUAutoScheduleOptions:
    def __init__(self):
        self.optionsPtr = _lib().CreateGPUAutoScheduleOptions()
        self.unrollTreeWalks = False

    def __del__(self):
        try:
            _lib().DeleteGPUAutoScheduleOptions(self.optionsPtr)
        except Exception:
            pass

    def NumberOfRowsPerThreadBlock(self, val):
        _lib().Set_numRowsPerTB(self.optionsPtr, val)

    def NumberOfRowsPerThread(self, val):
        _lib().Set_numRowsPerThread(self.optionsPtr, val)

    def RowTileSize(self, val):
        _lib().Set_rowTileSize(self.optionsPtr, val)

    def NumberOfTreeThreads(self, val):
        _lib().Set_numTreeThreads(self.optionsPtr, val)

    def NumberOfTreesAtATime(self, val):
        _lib().Set_numTreesAtATime(self.optionsPtr, val)

    def CacheRows(self, val):
        _lib().Set_cacheRows(self.optionsPtr, 1 if val else 0)

    def CacheTrees(self, val):
        _lib().Set_cacheTrees(self.optionsPtr, 1 if val else 0)

    def UnrollTreeWalks(self, val):
        self.unrollTreeWalks = val
        _lib().Set_unrollTreeWalks(self.optionsPtr, 1 if val else 0)

    def TreeWalkInterleaveFactor(self, val):
        _lib().Set_treeWalkInterleaveFactor(self.optionsPtr, val)

    def SharedReduce(self, val):
        _lib().Set_sharedMemoryReduce(self.optionsPtr, 1 if val else 0)

    @classmethod
    def Construct(cls, num_rows_per_TB, num_rows_per_thread=1, num_tree_threads=1, cache_rows=False,
                  cache_trees=False, unroll_tree_walks=False, tree_walk_interleave_factor=-1, shared_reduce=False):
        options = GPUAutoScheduleOptions()
        options.NumberOfRowsPerThreadBlock(num_rows_per_TB)
        options.NumberOfRowsPerThread(num_rows_per_thread)
        options.RowTileSize(1)
        options.NumberOfTreeThreads(num_tree_threads)
        options.NumberOfTreesAtATime(1)
        options.CacheRows(cache_rows)
        options.CacheTrees(cache_trees)
        options.UnrollTreeWalks(unroll_tree_walks)
        options.TreeWalkInterleaveFactor(tree_walk_interleave_factor)
        options.SharedReduce(shared_reduce)
        return options


class CompilerOptions:
    def __init__(self, batchSize, tileSize):
        self.optionsPtr = _lib().CreateCompilerOptions()
        _lib().Set_batchSize(self.optionsPtr, batchSize)
        _lib().Set_tileSize(self.optionsPtr, tileSize)

    def __del__(self):
        try:
            _lib().DeleteCompilerOptions(self.optionsPtr)
        except Exception:
            pass

    def SetThresholdTypeWidth(self, val):
        _lib().Set_thresholdTypeWidth(self.optionsPtr, val)

    def SetReturnTypeWidth(self, val):
        _lib().Set_returnTypeWidth(self.optionsPtr, val)

    def SetReturnTypeIsFloatType(self, val):
        _lib().Set_returnTypeFloatType(self.optionsPtr, 1 if val else 0)

    def SetFeatureIndexTypeWidth(self, val):
        _lib().Set_featureIndexTypeWidth(self.optionsPtr, val)

    def SetNodeIndexTypeWidth(self, val):
        _lib().Set_nodeIndexTypeWidth(self.optionsPtr, val)

    def SetInputElementTypeWidth(self, val):
        _lib().Set_inputElementTypeWidth(self.optionsPtr, val)

    def SetTileShapeBitWidth(self, val):
        _lib().Set_tileShapeBitWidth(self.optionsPtr, val)

    def SetChildIndexBitWidth(self, val):
        _lib().Set_childIndexBitWidth(self.optionsPtr, val)

    def SetMakeAllLeavesSameDepth(self, val):
        _lib().Set_makeAllLeavesSameDepth(self.optionsPtr, val)

    def SetReorderTreesByDepth(self, val):
        _lib().Set_reorderTreesByDepth(self.optionsPtr, 1 if val else 0)

    def SetTilingType(self, val):
        _lib().Set_tilingType(self.optionsPtr, val)

    def SetPipelineWidth(self, val):
        _lib().Set_pipelineSize(self.optionsPtr, val)

    def SetNumberOfFeatures(self, val):
        _lib().Set_numberOfFeatures(self.optionsPtr, val)

    def SetNumberOfCores(self, val):
        _lib().Set_numberOfCores(self.optionsPtr, val)

    def SetStatsProfileCSVPath(self, val):
        _lib().Set_statsProfileCSVPath(self.optionsPtr, val.encode("ascii"))

    def SetNumberOfParallelTreeBatches(self, val):
        _lib().Set_numParallelTreeBatches(self.optionsPtr, val)


class TreebeardContext:
    def __init__(self, model_filepath, globals_file_path, options, gpuAutoScheduleOptions=None):
        self.options = options
        self.gpuAutoScheduleOptions = gpuAutoScheduleOptions
        if gpuAutoScheduleOptions is None:
            self.tbContext = _lib().ConstructTreebeardContext(model_filepath.encode("ascii"),
                                                              globals_file_path.encode("ascii"), options.optionsPtr)
        else:
            self.tbContext = _lib().ConstructTreebeardContextFromGPUAutoscheduleOptions(
                model_filepath.encode("ascii"), globals_file_path.encode("ascii"), options.optionsPtr,
                gpuAutoScheduleOptions.optionsPtr)
        _check(self.tbContext, "ConstructTreebeardContext")

    def __del__(self):
        try:
            _lib().DestroyTreebeardContext(self.tbContext)
        except Exception:
            pass

    def SetInputFiletype(self, file_type):
        _lib().SetForestCreatorType(self.tbContext, file_type.encode("ascii"))
        if api().last_error():
            raise ValueError(api().last_error())

    def SetRepresentationType(self, rep_type):
        _lib().SetRepresentationAndSerializer(self.tbContext, rep_type.encode("ascii"))
        if api().last_error():
            raise ValueError(api().last_error())

    def BuildHIRRepresentation(self):
        _lib().BuildHIRRepresentation(self.tbContext)
        if api().last_error():
            raise RuntimeError(api().last_error())

    def ConstructInferenceRunnerFromHIR(self):
        return TreebeardInferenceRunner._from_handle(
            _check(_lib().ConstructInferenceRunnerFromHIR(self.tbContext), "ConstructInferenceRunnerFromHIR"))

    def ConstructGPUInferenceRunnerFromHIR(self):
        return TreebeardInferenceRunner._from_handle(
            _check(_lib().ConstructGPUInferenceRunnerFromHIR(self.tbContext), "ConstructGPUInferenceRunnerFromHIR"))

    def ConstructGPUInferenceRunnerAutoSchedule(self):
        return TreebeardInferenceRunner._from_handle(
            _check(_lib().findBestGPUScheduleAndCompileModel(self.tbContext), "findBestGPUScheduleAndCompileModel"))


class TreebeardInferenceRunner:
    def __init__(self):
        self.inferenceRunner = 0
        self.batchSize = 0
        self.rowSize = 0

    @classmethod
    def _from_handle(cls, handle):
        self = cls()
        self.inferenceRunner = handle
        self.batchSize = _lib().GetBatchSize(handle)
        self.rowSize = _lib().GetRowSize(handle)
        return self

    @classmethod
    def FromModelFile(cls, modelJSONPathStr, profileCSVPathStr, options):
        return cls._from_handle(_check(_lib().CreateInferenceRunner(
            modelJSONPathStr.encode("ascii"), (profileCSVPathStr or "").encode("ascii"), options.optionsPtr),
            "CreateInferenceRunner"))

    @classmethod
    def FromONNXModelFile(cls, onnx_model_path, options):
        return cls._from_handle(_check(_lib().CreateInferenceRunnerForONNXModel(
            onnx_model_path.encode("ascii"), options.optionsPtr), "CreateInferenceRunnerForONNXModel"))

    @classmethod
    def FromSOFile(cls, modelSOPath, modelGlobalsJSONPath=""):
        """src/python/treebeard.py:314-319: reopens a compiled model through InitializeInferenceRunner.  Here
        `modelSOPath` names a file written by save_compiled_model; the globals path is accepted and not opened."""
        return cls._from_handle(_check(_lib().InitializeInferenceRunner(
            modelSOPath.encode("ascii"), (modelGlobalsJSONPath or "").encode("ascii")), "InitializeInferenceRunner"))

    @classmethod
    def FromCompiledModelFile(cls, path, batchSize=0):
        """Reopens a model saved with save_compiled_model (the counterpart of the reference's FromSOFile)."""
        return cls._from_handle(_check(_lib().tbmi_load_compiled_model(path.encode("ascii"), batchSize),
                                       "tbmi_load_compiled_model"))

    def save_compiled_model(self, path):
        self._rc(_lib().tbmi_save_compiled_model(self.inferenceRunner, path.encode("ascii")), "tbmi_save_compiled_model")

    @classmethod
    def FromTBContext(cls, tbContext):
        return tbContext.ConstructInferenceRunnerFromHIR()

    @classmethod
    def GPUInferenceRunnerFromTBContext(cls, tbContext):
        return cls._from_handle(_check(_lib().ConstructGPUInferenceRunnerFromTBContext(tbContext.tbContext),
                                       "ConstructGPUInferenceRunnerFromTBContext"))

    @classmethod
    def AutoScheduleGPUInferenceRunnerFromTBContext(cls, tbContext):
        return tbContext.ConstructGPUInferenceRunnerAutoSchedule()

    def __del__(self):
        try:
            if self.inferenceRunner:
                _lib().DeleteInferenceRunner(self.inferenceRunner)
        except Exception:
            pass

    def _host_inputs(self, inputs):
        return numpy.ascontiguousarray(inputs, dtype=numpy.float32)

    def RunInference(self, inputs, resultType=numpy.float32):
        inputs = self._host_inputs(inputs)
        assert inputs.size == self.batchSize * self.rowSize, "RunInference takes exactly one batch"
        self._check_result_type(resultType)
        results = numpy.zeros((self.batchSize,), resultType)
        _lib().RunInference(self.inferenceRunner, inputs.ctypes.data, results.ctypes.data)
        if api().last_error():
            raise RuntimeError(api().last_error())
        return results

    def RunInferenceOnMultipleBatches(self, inputs, resultType=numpy.float32):
        inputs = self._host_inputs(inputs)
        numRows = inputs.shape[0]
        assert numRows % self.batchSize == 0
        self._check_result_type(resultType)
        results = numpy.zeros((numRows,), resultType)
        _lib().RunInferenceOnMultipleBatches(self.inferenceRunner, inputs.ctypes.data, results.ctypes.data, numRows)
        if api().last_error():
            raise RuntimeError(api().last_error())
        return results

    # ---- additions over the reference wrapper: device-resident tensors ----
    def describe_plan(self):
        buf = ctypes.create_string_buffer(1024)
        _lib().tbmi_describe_plan(self.inferenceRunner, buf, 1024)
        return buf.value.decode()

    def num_trees(self):
        return _lib().tbmi_num_trees(self.inferenceRunner)

    def num_classes(self):
        return _lib().tbmi_num_classes(self.inferenceRunner)

    def _rc(self, rc, what):
        if rc != 0:
            raise RuntimeError("%s failed: %s" % (what, api().last_error()))

    def run_device(self, device_inputs_ptr, device_results_ptr, rows):
        self._rc(_lib().tbmi_run_device(self.inferenceRunner, device_inputs_ptr, device_results_ptr, rows),
                 "tbmi_run_device")

    def run_device_async(self, device_inputs_ptr, device_results_ptr, rows, stream=None):
        """Enqueues the kernels on `stream` (a hipStream_t address, None = the default stream) and returns."""
        self._rc(_lib().tbmi_run_device_async(self.inferenceRunner, device_inputs_ptr, device_results_ptr, rows,
                                              stream), "tbmi_run_device_async")

    def run_device_noalloc(self, device_inputs_ptr, device_results_ptr, rows, stream=None):
        """run_device_async without any allocation: scratch memory comes from the library's fixed device array."""
        self._rc(_lib().tbmi_run_device_noalloc(self.inferenceRunner, device_inputs_ptr, device_results_ptr, rows,
                                                stream), "tbmi_run_device_noalloc")

    def run_device_multiclass(self, device_inputs_ptr, rows, class_ids_ptr=None, margins_ptr=None, probs_ptr=None):
        self._rc(_lib().tbmi_run_device_multiclass(self.inferenceRunner, device_inputs_ptr, rows, class_ids_ptr,
                                                   margins_ptr, probs_ptr), "tbmi_run_device_multiclass")

    def dump_leaf_ids(self, device_inputs_ptr, device_leaf_ids_ptr, rows):
        self._rc(_lib().tbmi_dump_leaf_ids(self.inferenceRunner, device_inputs_ptr, device_leaf_ids_ptr, rows),
                 "tbmi_dump_leaf_ids")

    def time_kernels(self, device_inputs_ptr, device_results_ptr, rows, runs):
        """(walk ms, finalize + rank-quantisation ms) per launch."""
        walk, fin, pre = self.time_kernels3(device_inputs_ptr, device_results_ptr, rows, runs)
        return walk, fin + pre

    def time_kernels3(self, device_inputs_ptr, device_results_ptr, rows, runs):
        """(walk ms, finalize ms, rank-quantisation ms) per launch."""
        walk, fin, pre = ctypes.c_double(), ctypes.c_double(), ctypes.c_double()
        self._rc(_lib().tbmi_time_kernels(self.inferenceRunner, device_inputs_ptr, device_results_ptr, rows, runs,
                                          ctypes.byref(walk), ctypes.byref(fin), ctypes.byref(pre)),
                 "tbmi_time_kernels")
        return walk.value, fin.value, pre.value

    def run_host(self, inputs):
        """Any number of host rows (numpy in, numpy out); the batch size only sizes the staging buffers."""
        inputs = self._host_inputs(inputs)
        rows = inputs.size // self.rowSize
        assert rows * self.rowSize == inputs.size
        results = numpy.zeros((rows,), self.result_dtype())
        self._rc(_lib().tbmi_run_host(self.inferenceRunner, inputs.ctypes.data, results.ctypes.data, rows), "tbmi_run_host")
        return results

    def _check_result_type(self, resultType):
        # the library writes result_dtype() elements: a narrower numpy buffer would be overrun
        if numpy.dtype(resultType).itemsize != numpy.dtype(self.result_dtype()).itemsize:
            raise ValueError("this runner returns %s results (see CompilerOptions.SetReturnTypeWidth), not %s"
                             % (numpy.dtype(self.result_dtype()).name, numpy.dtype(resultType).name))

    def result_dtype(self):
        """numpy dtype of the results RunInference / run_device write for this runner."""
        return numpy.int8 if _lib().tbmi_result_bytes(self.inferenceRunner) == 1 else numpy.float32

    def set_global_walk_plan(self, rows_per_block=256, interleave=4, tree_slices=1):
        self._rc(_lib().tbmi_set_global_walk_plan(self.inferenceRunner, rows_per_block, interleave, tree_slices),
                 "tbmi_set_global_walk_plan")

    def set_group_staging(self, mode):
        """0 by rule, 1 tree groups through prefetch registers, 2 direct global-to-LDS copies."""
        self._rc(_lib().tbmi_set_group_staging(self.inferenceRunner, mode), "tbmi_set_group_staging")

    def enable_peeled_walks(self, device_inputs_ptr, rows):
        """Profiles up to 4096 of the device-resident rows and re-packs the current plan with peeled walks."""
        self._rc(_lib().tbmi_enable_peeled_walks(self.inferenceRunner, device_inputs_ptr, rows), "tbmi_enable_peeled_walks")

    def set_rank16_plan(self, rows_per_block=256, tree_threads=0, interleave=4, group_bytes=0, tree_slices=1):
        self._rc(_lib().tbmi_set_rank16_plan(self.inferenceRunner, rows_per_block, tree_threads, interleave, group_bytes,
                                             tree_slices), "tbmi_set_rank16_plan")

    def set_quantized_plan(self, tree_threads=8, interleave=4, group_bytes=0, tree_slices=1):
        self._rc(_lib().tbmi_set_quantized_plan(self.inferenceRunner, tree_threads, interleave, group_bytes,
                                                tree_slices), "tbmi_set_quantized_plan")

    def autotune(self, device_inputs_ptr, rows):
        best = ctypes.c_double()
        self._rc(_lib().tbmi_autotune(self.inferenceRunner, device_inputs_ptr, rows, ctypes.byref(best)),
                 "tbmi_autotune")
        return best.value

    def set_plan(self, rows_per_block=0, tree_threads=1, interleave=0, group_bytes=0, tree_slices=0):
        self._rc(_lib().tbmi_set_plan(self.inferenceRunner, rows_per_block, tree_threads, interleave, group_bytes,
                                      tree_slices), "tbmi_set_plan")

    def set_tree_parallel_plan(self, rows_per_block, tree_lanes, interleave=1, group_bytes=0, tree_slices=0):
        self._rc(_lib().tbmi_set_tree_parallel_plan(self.inferenceRunner, rows_per_block, tree_lanes, interleave,
                                                    group_bytes, tree_slices), "tbmi_set_tree_parallel_plan")


def SetEnableSparseRepresentation(val):
    _lib().SetEnableSparseRepresentation(1 if val else 0)


def IsSparseRepresentationEnabled():
    return _lib().IsSparseRepresentationEnabled() != 0


def SetPeeledCodeGenForProbabilityBasedTiling(val):
    _lib().SetPeeledCodeGenForProbabilityBasedTiling(1 if val else 0)


def IsPeeledCodeGenForProbabilityBasedTilingEnabled():
    return _lib().IsPeeledCodeGenForProbabilityBasedTilingEnabled() != 0


def SetEnableMeasureGpuKernelTime(val):
    _lib().SetEnableMeasureGpuKernelTime(bool(val))


def SetNumberOfKernelRuns(val):
    _lib().SetNumberOfKernelRuns(val)


def GetGPUKernelExecutionTime(inferenceRunner):
    return _lib().GetGPUKernelExecutionTime(inferenceRunner.inferenceRunner)
