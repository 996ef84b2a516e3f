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

// What the compiler options ask of the walk itself (CompilerOptions::tileSize, tilingType and the peeled
// code generation switch); copied into the plan.
struct WalkOptions {
  int32_t tileSize = 1;
  int32_t tiling = 0;     // 0 uniform, 1 probabilistic, 2 hybrid
  bool peelWalks = false;
};

// Analytic choice; `overrides` (may be null) pins what the caller set.  Tile sizes above 1 always get the
// row-parallel kernel on f32 rows (the only one that walks tiles) and fail when its row tile does not fit.
LaunchPlan ChoosePlan(const Forest &forest, int64_t batchSize, const GPUAutoScheduleOptions *overrides,
                      const DeviceLimits &limits, const WalkOptions &walk = WalkOptions());

// Whether `plan` can defer the tails of its walks (LaunchPlan::deferTails: the scalar row-parallel kernel on an f32
// tile with byte offsets, a model without classes); when it can, the plan's tree groups give up the LDS the stub
// feature's column and the waves' queues take.  The caller sets the flag.
bool DeferTailsFit(const Forest &forest, LaunchPlan *plan);

// Candidate plans for the timed search (the analytic choice comes first).
std::vector<LaunchPlan> CandidatePlans(const Forest &forest, int64_t batchSize, const DeviceLimits &limits,
                                       const WalkOptions &walk = WalkOptions());

} // namespace tbamd
