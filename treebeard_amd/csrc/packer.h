// Re-packs a Forest into the device layout described in device_model.h.
#pragma once

#include "device_model.h"
#include "forest.h"

#include <vector>

namespace tbamd {

// How the row-parallel LDS kernel is launched; chosen by the tuner.
struct LaunchPlan {
  enum class Kernel : int32_t { kRowParallelLds = 0, kTreeParallel = 1 };
  Kernel kernel = Kernel::kRowParallelLds;
  int32_t rowsPerBlock = 256;   // = threads per block (one row per lane), power of two
  int32_t interleave = 4;       // K: trees walked concurrently by one lane (1, 2, 4, 8)
  int32_t groupBytes = 48 * 1024; // LDS bytes for one tree group's nodes (<= 65536)
  int32_t treeSlices = 1;       // grid.y: how many blocks share one row block's trees
  bool featureOffsetInWords = false;
};

struct PackedModel {
  LaunchPlan plan;
  int32_t numFeatures = 0;
  int32_t numClasses = 0;
  int32_t numTrees = 0;
  std::vector<DeviceNode> nodes;
  std::vector<DeviceBundle> bundles;
  std::vector<DeviceGroup> groups;
  // Parity/debug side tables (not touched by the timed kernels):
  std::vector<int32_t> nodeOrigin; // per packed node: original node id inside its tree (-1: null leaf)
  std::vector<int32_t> slotTree;   // per bundle slot: original tree index, -1 for a padding tree
  uint32_t maxGroupNodes = 0;

  uint32_t PadFeatureOffset() const;
  size_t LdsBytes() const; // transposed row tile + the largest group
};

// Throws tbamd::Error when the plan cannot hold the model (tree larger than a
// group, feature offsets that do not fit 16 bits, ...).
PackedModel PackForest(const Forest &forest, const LaunchPlan &plan);

// Inverse of PackForest for tests: rebuilds (value, feature, left, right) of
// original tree `tree` from the packed arrays.
Tree UnpackTree(const PackedModel &model, int32_t tree);

// Children-swapped / threshold-adjusted copy in which "x < value -> left" holds
// for every comparison mode the loaders accept.
Forest NormalizeToLessThan(const Forest &forest);

} // namespace tbamd
