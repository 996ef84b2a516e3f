#pragma once

#include "forest.h"
#include "packer.h"

#include <string>
#include <vector>

namespace tbamd {

struct CompiledModel {
  Forest forest;
  LaunchPlan plan;
  int32_t batchSize = 0;
  int32_t returnTypeWidth = 32;
  bool returnTypeFloatType = true;
};

void SaveCompiledModel(const std::string &path, const Forest &forest, const LaunchPlan &plan, int32_t batchSize,
                       int32_t returnTypeWidth, bool returnTypeFloatType);
CompiledModel LoadCompiledModel(const std::string &path);

// Leaf hit counts of a profiling run (the reference's probability profile), with the counts of the
// internal nodes filled in from their subtrees.
struct HitCountProfile {
  int64_t numRows = 0;
  std::vector<std::vector<int64_t>> hits; // per tree, per node
};

HitCountProfile LoadHitCountProfile(const Forest &forest, const std::string &path);
// Average number of internal nodes a profiled row visits over the whole forest.
double ExpectedWalkSteps(const Forest &forest, const HitCountProfile &profile);

} // namespace tbamd
