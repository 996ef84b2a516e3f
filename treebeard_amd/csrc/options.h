// Option structs behind the C-ABI handles.  Field names, defaults and meaning
// follow the reference (src/include/TreebeardContext.h:64-162) so that the
// Set_* entry points keep their semantics; fields that only steer the
// reference's MLIR code generation are accepted and recorded but do not change
// the kernels chosen here.
#pragma once

#include <cstdint>
#include <string>

namespace tbamd {

enum class TilingType : int32_t { kUniform = 0, kProbabilistic = 1, kHybrid = 2 };

struct CompilerOptions {
  int32_t numberOfFeatures = -1; // used by the ONNX front end only
  int32_t batchSize = 0;
  int32_t tileSize = 1;
  int32_t thresholdTypeWidth = 32;
  int32_t returnTypeWidth = 32;
  bool returnTypeFloatType = true;
  int32_t featureIndexTypeWidth = 16;
  int32_t nodeIndexTypeWidth = 16;
  int32_t inputElementTypeWidth = 32;
  int32_t tileShapeBitWidth = 16;
  int32_t childIndexBitWidth = 16;
  TilingType tilingType = TilingType::kUniform;
  bool makeAllLeavesSameDepth = false;
  bool reorderTreesByDepth = false;
  int32_t pipelineSize = -1;
  std::string statsProfileCSVPath;
  int32_t numberOfCores = -1;
  int32_t numParallelTreeBatches = -1;
};

// src/include/TreebeardContext.h:138-162.  A value <= 0 leaves the choice to
// the launch-parameter tuner.
struct GPUAutoScheduleOptions {
  int32_t numRowsPerTB = 0;
  int32_t numRowsPerThread = 0;
  int32_t rowTileSize = 0;
  int32_t numTreeThreads = 0;
  int32_t numTreesAtATime = 0;
  bool cacheRows = false;
  bool cacheTrees = false;
  bool unrollTreeWalks = false;
  int32_t treeWalkInterleaveFactor = -1;
  bool sharedMemoryReduce = false;
};

} // namespace tbamd
