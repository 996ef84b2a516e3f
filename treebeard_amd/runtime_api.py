"""ctypes declarations for libtreebeard_amd.so (include/tbruntime_amd.h).

Counterpart of the reference's `TreebeardAPI` (src/python/treebeard_runtime_api.py:12-…):
loads the runtime library that sits next to this file and declares argument and
return types of every entry point.  There is no fallback: a missing library is
an error.

In a process that also uses PyTorch-ROCm, import torch before the first call that
loads this library.  The library links against the system's libamdhip64; a torch
wheel brings a HIP runtime of its own.  With torch loaded first the dynamic linker
gives this library torch's copy and the process holds one runtime; loaded the other
way round the process holds two, and torch then reports that no GPU is available
(measured on MI355X with ROCm 7.2 beside a ROCm 7.0 torch wheel).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libtreebeard_amd.so")

c_i32, c_i64, c_ip, c_vp, c_cp = ctypes.c_int32, ctypes.c_int64, ctypes.c_ssize_t, ctypes.c_void_p, ctypes.c_char_p

OPTION_SETTERS = ["numberOfFeatures", "batchSize", "tileSize", "thresholdTypeWidth", "returnTypeWidth",
                  "returnTypeFloatType", "featureIndexTypeWidth", "nodeIndexTypeWidth", "inputElementTypeWidth",
                  "tileShapeBitWidth", "childIndexBitWidth", "makeAllLeavesSameDepth", "reorderTreesByDepth",
                  "pipelineSize", "numberOfCores", "numParallelTreeBatches", "tilingType"]
GPU_OPTION_SETTERS = ["numRowsPerTB", "numRowsPerThread", "rowTileSize", "numTreeThreads", "numTreesAtATime",
                      "cacheRows", "cacheTrees", "unrollTreeWalks", "treeWalkInterleaveFactor", "sharedMemoryReduce"]

SIGNATURES = {
    "RunInference": (None, [c_ip, c_vp, c_vp]),
    "RunInferenceOnMultipleBatches": (None, [c_ip, c_vp, c_vp, c_i32]),
    "GetBatchSize": (c_i32, [c_ip]),
    "GetRowSize": (c_i32, [c_ip]),
    "DeleteInferenceRunner": (None, [c_ip]),
    "CreateCompilerOptions": (c_ip, []),
    "DeleteCompilerOptions": (None, [c_ip]),
    "Set_statsProfileCSVPath": (None, [c_ip, c_cp]),
    "CreateGPUAutoScheduleOptions": (c_ip, []),
    "DeleteGPUAutoScheduleOptions": (None, [c_ip]),
    "CreateInferenceRunner": (c_ip, [c_cp, c_cp, c_ip]),
    "CreateInferenceRunnerForONNXModel": (c_ip, [c_cp, c_ip]),
    "SetEnableSparseRepresentation": (None, [c_i32]),
    "IsSparseRepresentationEnabled": (c_i32, []),
    "SetPeeledCodeGenForProbabilityBasedTiling": (None, [c_i32]),
    "IsPeeledCodeGenForProbabilityBasedTilingEnabled": (c_i32, []),
    "SetEnableMeasureGpuKernelTime": (None, [ctypes.c_bool]),
    "SetNumberOfKernelRuns": (None, [c_i32]),
    "GetGPUKernelExecutionTime": (c_i64, [c_ip]),
    "ConstructTreebeardContext": (c_ip, [c_cp, c_cp, c_ip]),
    "ConstructTreebeardContextFromGPUAutoscheduleOptions": (c_ip, [c_cp, c_cp, c_ip, c_ip]),
    "DestroyTreebeardContext": (None, [c_ip]),
    "SetForestCreatorType": (None, [c_ip, c_cp]),
    "SetRepresentationAndSerializer": (None, [c_ip, c_cp]),
    "ConstructGPUInferenceRunnerFromTBContext": (c_vp, [c_vp]),
    "ConstructInferenceRunnerFromHIR": (c_vp, [c_vp]),
    "ConstructGPUInferenceRunnerFromHIR": (c_vp, [c_vp]),
    "BuildHIRRepresentation": (None, [c_vp]),
    "findBestGPUScheduleAndCompileModel": (c_vp, [c_vp]),
    "tbmi_last_error": (c_cp, []),
    "tbmi_device_count": (c_i32, []),
    "tbmi_run_device": (c_i32, [c_ip, c_vp, c_vp, c_i64]),
    "tbmi_run_device_async": (c_i32, [c_ip, c_vp, c_vp, c_i64, c_vp]),
    "tbmi_run_device_noalloc": (c_i32, [c_ip, c_vp, c_vp, c_i64, c_vp]),
    "tbmi_noalloc_scratch_bytes": (c_i64, []),
    "tbmi_run_device_multiclass": (c_i32, [c_ip, c_vp, c_i64, c_vp, c_vp, c_vp]),
    "tbmi_dump_leaf_ids": (c_i32, [c_ip, c_vp, c_vp, c_i64]),
    "tbmi_time_kernels": (c_i32, [c_ip, c_vp, c_vp, c_i64, c_i32, ctypes.POINTER(ctypes.c_double),
                                  ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]),
    "tbmi_result_bytes": (c_i32, [c_ip]),
    "tbmi_run_host": (c_i32, [c_ip, c_vp, c_vp, c_i64]),
    "tbmi_set_global_walk_plan": (c_i32, [c_ip, c_i32, c_i32, c_i32]),
    "tbmi_set_quantized_plan": (c_i32, [c_ip, c_i32, c_i32, c_i32, c_i32]),
    "tbmi_set_rank16_plan": (c_i32, [c_ip, c_i32, c_i32, c_i32, c_i32, c_i32]),
    "tbmi_enable_peeled_walks": (c_i32, [c_ip, c_vp, c_i64]),
    "tbmi_set_group_staging": (c_i32, [c_ip, c_i32]),
    "tbmi_autotune": (c_i32, [c_ip, c_vp, c_i64, ctypes.POINTER(ctypes.c_double)]),
    "tbmi_set_plan": (c_i32, [c_ip, c_i32, c_i32, c_i32, c_i32, c_i32]),
    "tbmi_set_tree_parallel_plan": (c_i32, [c_ip, c_i32, c_i32, c_i32, c_i32, c_i32]),
    "tbmi_describe_plan": (c_i32, [c_ip, c_cp, c_i32]),
    "tbmi_save_compiled_model": (c_i32, [c_ip, c_cp]),
    "tbmi_load_compiled_model": (c_ip, [c_cp, c_i32]),
    "InitializeInferenceRunner": (c_ip, [c_cp, c_cp]),
    "tbmi_forest_load_profile": (c_i32, [c_ip, c_cp, ctypes.POINTER(c_i64), ctypes.POINTER(ctypes.c_double)]),
    "tbmi_num_trees": (c_i32, [c_ip]),
    "tbmi_num_classes": (c_i32, [c_ip]),
    "tbmi_load_forest": (c_ip, [c_cp, c_cp, c_i32]),
    "tbmi_delete_forest": (None, [c_ip]),
    "tbmi_forest_info": (c_i32, [c_ip, ctypes.POINTER(c_i64), ctypes.POINTER(ctypes.c_double)]),
    "tbmi_forest_tree_size": (c_i32, [c_ip, c_i32]),
    "tbmi_forest_tree": (c_i32, [c_ip, c_i32, c_vp, c_vp, c_vp, c_vp, ctypes.POINTER(c_i32)]),
    "tbmi_pack_roundtrip": (c_i32, [c_ip, c_i32, c_i32, c_i32, ctypes.POINTER(c_i64)]),
}
for _name in OPTION_SETTERS + GPU_OPTION_SETTERS:
    SIGNATURES["Set_" + _name] = (None, [c_ip, c_i32])


class TreebeardAPI:
    def __init__(self, lib_path=LIB_PATH):
        if not os.path.exists(lib_path):
            raise FileNotFoundError(
                "%s is missing: build it with `python -m treebeard_amd.build` (there is no fallback path)" % lib_path)
        self.runtime_lib = ctypes.CDLL(lib_path)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(self.runtime_lib, name)
            fn.restype = restype
            fn.argtypes = argtypes

    def last_error(self):
        msg = self.runtime_lib.tbmi_last_error()
        return msg.decode() if msg else ""


BENCH_LIB_PATH = os.path.join(_HERE, "libtbamd_bench.so")


def lds_read_bandwidth(width_bytes):
    """Bytes per second of conflict-free LDS reads (4, 8 or 16 bytes per lane) measured by the bench-only
    library libtbamd_bench.so; raises when that library is missing or the measurement fails."""
    if not os.path.exists(BENCH_LIB_PATH):
        raise FileNotFoundError("%s is missing: build it with `python -m treebeard_amd.build`" % BENCH_LIB_PATH)
    lib = ctypes.CDLL(BENCH_LIB_PATH)
    lib.tbbench_lds_read_bandwidth.restype = c_i32
    lib.tbbench_lds_read_bandwidth.argtypes = [c_i32, ctypes.POINTER(ctypes.c_double)]
    rate = ctypes.c_double()
    rc = lib.tbbench_lds_read_bandwidth(width_bytes, ctypes.byref(rate))
    if rc != 0:
        raise RuntimeError("LDS micro-benchmark failed with HIP error %d" % rc)
    return rate.value


LDS_READ_OPS = ("ds_read_b32", "ds_read_b64", "ds_read_b128", "ds_read2_b32", "ds_read_u16", "ds_read_u8", "ds_read_b96")


def lds_read_cost(op, pattern=0, mask=0):
    """Cycles (nominal shader clock) a compute unit spends per wave-level LDS read, measured by the bench-only
    library.  op indexes LDS_READ_OPS; pattern 0 = lane i reads element i, 1 = random over 48 KB, 2 = random over
    1 KB, 5..7 = random among 2**pattern consecutive elements; mask 0 = all lanes, 1 = lanes 0-31, 2 = even lanes,
    3 = a random half, 4 = a random quarter."""
    if not os.path.exists(BENCH_LIB_PATH):
        raise FileNotFoundError("%s is missing: build it with `python -m treebeard_amd.build`" % BENCH_LIB_PATH)
    lib = ctypes.CDLL(BENCH_LIB_PATH)
    lib.tbbench_lds_read_cost.restype = c_i32
    lib.tbbench_lds_read_cost.argtypes = [c_i32, c_i32, c_i32, ctypes.POINTER(ctypes.c_double)]
    cycles = ctypes.c_double()
    rc = lib.tbbench_lds_read_cost(op, pattern, mask, ctypes.byref(cycles))
    if rc != 0:
        raise RuntimeError("LDS read-cost measurement failed with HIP error %d" % rc)
    return cycles.value


_api = None


def api():
    global _api
    if _api is None:
        _api = TreebeardAPI()
    return _api
