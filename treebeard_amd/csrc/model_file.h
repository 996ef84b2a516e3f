#pragma once

#include "forest.h"
#include "packer.h"

#include <memory>
#include <string>
#include <vector>

namespace tbamd {

struct CompiledModel {
  Forest forest;
  LaunchPlan plan;
  int32_t batchSize = 0;
  int32_t returnTypeWidth = 32;
  bool returnTypeFloatType = true;
  std::unique_ptr<HitCountProfile> profile; // the hit counts the model was tiled with, if any
};

void SaveCompiledModel(const std::string &path, const Forest &forest, const LaunchPlan &plan, int32_t batchSize,
                       int32_t returnTypeWidth, bool returnTypeFloatType, const HitCountProfile *profile = nullptr);
CompiledModel LoadCompiledModel(const std::string &path);

HitCountProfile LoadHitCountProfile(const Forest &forest, const std::string &path);
// Average number of internal nodes a profiled row visits over the whole forest.
double ExpectedWalkSteps(const Forest &forest, const HitCountProfile &profile);

} // namespace tbamd
