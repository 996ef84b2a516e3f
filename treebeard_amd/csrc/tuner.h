// Launch-parameter tuner: picks the kernel and its shape from the model's
// statistics and the batch size.  It stands where the reference has its
// scheduling language and GPU auto-tuner (src/schedule/schedule.h,
// src/mlir/GPUAutoSchedule.cpp:597-624 heuristic subset, :799-934 timed search).
#pragma once

#include "forest.h"
#include "options.h"
#include "packer.h"

#include <vector>

namespace tbamd {

struct DeviceLimits {
  int32_t computeUnits = 256;
  int32_t ldsBytesPerBlock = 160 * 1024;
};

// Analytic choice; `overrides` (may be null) pins what the caller set.
LaunchPlan ChoosePlan(const Forest &forest, int64_t batchSize, const GPUAutoScheduleOptions *overrides,
                      const DeviceLimits &limits);

// Candidate plans for the timed search (the analytic choice comes first).
std::vector<LaunchPlan> CandidatePlans(const Forest &forest, int64_t batchSize, const DeviceLimits &limits);

} // namespace tbamd
