// Re-packs a Forest into the device layout described in device_model.h.
#pragma once

#include "device_model.h"
#include "forest.h"

#include <vector>

namespace tbamd {

// How the kernels are launched; chosen by the tuner.
//
//  kRowParallelLds: one lane per row, rowsPerBlock lanes per block, the block's
//    rows transposed in LDS, every lane walks all trees (K at a time).
//  kGlobalWalk:     one lane per row, rows and nodes read from global memory (through L1/L2); the
//    fallback for forests with a tree that does not fit one 64 KB LDS group.
//  kTreeParallel:   rowsPerBlock rows per block kept row-major in LDS and
//    treeLanes lanes per row that split the trees between them; per-row sums are
//    reduced across lanes (wave shuffles, then LDS across waves).  For models
//    whose rows are too wide to transpose into LDS and for batches too small to
//    fill the chip with one lane per row.
struct LaunchPlan {
  enum class Kernel : int32_t { kRowParallelLds = 0, kTreeParallel = 1, kGlobalWalk = 2 };
  Kernel kernel = Kernel::kRowParallelLds;
  int32_t rowsPerBlock = 256;   // row-parallel: rows (= lanes per tree thread) per block, power of two
  int32_t treeThreads = 1;      // row-parallel: lanes in different waves that share a row; block = rowsPerBlock * treeThreads
  int32_t treeLanes = 1;        // tree-parallel: lanes per row, power of two; block = rowsPerBlock * treeLanes
  int32_t interleave = 4;       // K: trees walked concurrently by one lane (1, 2, 4, 8)
  int32_t groupBytes = 48 * 1024; // LDS bytes for one tree group's nodes (<= 65536)
  int32_t treeSlices = 1;       // grid.y: how many blocks share one row block's trees
  bool featureOffsetInWords = false;
  // Row-parallel kernel on rank-quantised rows: a separate kernel first replaces every feature value
  // by the number of that feature's split thresholds that are <= it (one byte), which preserves the
  // outcome of every comparison; 64 rows of 1 byte per feature then fit LDS where 64 f32 rows do not.
  bool quantizedRows = false;
  // The same idea for narrow models whose features have up to 65534 distinct thresholds: two-byte ranks, made by
  // a separate kernel and laid out as [row block][feature pair][row][2], so that a row's LDS column keeps one bank
  // of its own and the tile takes half the bytes of f32 rows (more rows per block, bigger tree groups).
  bool rankRows16 = false;
  // Tiled walk (row-parallel kernel on f32 rows only): nodes per tile (up to 8), 1 = scalar nodes.  How the members of a
  // tile are chosen follows the reference: 0 breadth first (src/mlir/UniformTilingTransformation.cpp:148-195),
  // 1 most-visited child first on trees whose profile is skewed, 2 the same but breadth first below nodes that
  // fewer than 20 % of the rows reach (src/mlir/ProbabilityBasedTilingTransform.cpp:124-198, :243-262); 1 and
  // 2 need a hit-count profile and fall back to 0 without one.
  int32_t tileSize = 1;
  int32_t tiling = 0;
  // Walk peeling (src/mlir/ProbabilityBasedTilingTransform.cpp:66-73): with a profile, a bundle first takes the
  // steps that bring 90 % of the profiled rows to their leaves without looking, then steps on only while some
  // lane of the wave still moves.
  bool peelWalks = false;
  // How the scalar row-parallel walk on f32 rows (byte offsets, regressors and binary classifiers) peels: the
  // walk of a tree stops at the level up to which lock step pays; the internal nodes of that level become
  // stubs, the rows that reach one are queued per wave as (row, node) and walked on densely, 64 queue entries
  // at a time, whatever trees they come from.  Needs a profile; set by ChoosePlan where the kernel has the form.
  bool deferTails = false;

  int32_t ThreadsPerBlock() const {
    if (kernel == Kernel::kGlobalWalk) return rowsPerBlock;
    return kernel == Kernel::kTreeParallel ? rowsPerBlock * treeLanes : rowsPerBlock * treeThreads;
  }
  // Distance in LDS between feature f and f+1 of one row, in the units node offsets use.
  uint32_t FeatureStride() const {
    if (kernel == Kernel::kTreeParallel) return 4u;
    if (quantizedRows) return (uint32_t)rowsPerBlock / 4u; // byte tile, offsets in units of 4 bytes
    return featureOffsetInWords ? (uint32_t)rowsPerBlock : (uint32_t)rowsPerBlock * 4u;
  }
  // What a node stores for feature f (f = numFeatures: the pad feature).
  uint32_t FeatureOffset(uint32_t f) const {
    if (rankRows16) return (f >> 1) * (uint32_t)rowsPerBlock * 4u + (f & 1u) * 2u; // byte offset in the [pair][row][2] tile
    return f * FeatureStride();
  }
  uint32_t FeatureOfOffset(uint32_t offset) const {
    if (rankRows16) return offset / ((uint32_t)rowsPerBlock * 4u) * 2u + ((offset >> 1) & 1u);
    return offset / FeatureStride();
  }
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
  // Copies of the root nodes, plan.interleave per bundle: every lane of a wave starts a tree at its root, so
  // the f32 row-parallel walk takes level 0 from scalar registers instead of an LDS node read.
  std::vector<DeviceNode> bundleRoots;
  uint32_t maxGroupNodes = 0;
  // Tiled plans: how many trees were tiled by visit counts (the others breadth first), and the tile steps
  // one row takes over the whole forest: lock-step (deepest leaf of every tree) and, when a profile was
  // given, what the profiled rows need on average.
  int32_t treesTiledByProfile = 0;
  int32_t maxTileHops = 1;   // eight-slot tiles: the most levels of nodes any tile holds (links a tile step follows)
  int64_t lockStepSteps = 0;
  double profiledSteps = 0.0;
  // plan.deferTails: trees whose walks stop early, and what the profile says a row's deferred walks cost
  // The subtrees below the stubs: nodes { value; (left child index << kTailFeatureBits) | feature index } with
  // indices into this array (right = left + 1; a leaf points at itself and tests the pad feature); entry 0 is a
  // leaf of value 0.  tailOrigin: original node id of every entry (parity side table).
  std::vector<DeviceNode> tailNodes;
  std::vector<int32_t> tailOrigin;
  uint32_t maxTailDepth = 0; // steps the deepest deferred walk takes below its stub
  int32_t treesDeferred = 0;
  double deferredEntriesPerRow = 0.0; // queue entries a profiled row makes over the whole forest
  // kGlobalWalk only:
  std::vector<DeviceGlobalNode> globalNodes;
  std::vector<DeviceGlobalTree> globalTrees; // ordered by (class, depth)
  // Rank quantisation (plan.quantizedRows): per feature the sorted distinct thresholds, stored for the
  // binning kernel as [featureChunk][k][binChunkFeatures] with +inf behind a feature's last threshold;
  // binTableDepth = 2^n - 1 entries per feature.
  std::vector<float> binThresholds;
  int32_t binTableDepth = 0;
  int32_t binChunkFeatures = 0;
  // Two-byte ranks (plan.rankRows16): the thresholds of every feature as a complete search tree in breadth-first
  // order (root, its two children, ...; 2^levels - 1 entries, +inf behind the feature's last threshold), feature
  // after feature; the ranking kernel's blocks each take one chunk of whole feature pairs whose tables fit LDS.
  // RankFeatureDesc: the feature's first table entry relative to its chunk's first entry, and its search steps
  // (0: no threshold); RankChunkDesc: whole pairs (firstFeature is even) and the chunk's tables in rankTables.
  std::vector<float> rankTables;
  std::vector<std::vector<float>> rankThresholds; // per feature, sorted (host side only: unpacking and checks)
  std::vector<RankFeatureDesc> rankFeatures;      // one per slot of the tile: (numFeatures + 2) / 2 pairs
  std::vector<RankChunkDesc> rankChunks;

  uint32_t PadFeatureOffset() const;
  // LDS bytes of the tree-group region (regressors reuse it for the tree threads' cross-wave pass).
  uint32_t GroupRegionBytes() const {
    uint32_t bytes = maxGroupNodes * kNodeBytes;
    if (plan.kernel == LaunchPlan::Kernel::kRowParallelLds && plan.treeThreads > 1 && numClasses == 0)
      bytes = bytes > (uint32_t)plan.ThreadsPerBlock() * 8u ? bytes : (uint32_t)plan.ThreadsPerBlock() * 8u;
    return (bytes + 15u) & ~15u;
  }
  // How many partial sums per (row, class) the walk kernel leaves for the finalize kernel.
  int32_t PartialCount() const { return plan.treeSlices; }
  size_t RowTileBytes() const;
  size_t LdsBytes() const; // row tile + the largest group (+ reduction scratch)
};

// Largest number of distinct split thresholds any one feature has (after comparison normalisation).
int32_t MaxThresholdsPerFeature(const Forest &forest);

// Bytes of the biggest tree once tiled breadth first with `tileSize` (2..8) nodes per tile, leaf tiles included.
// (Tiling by hit counts picks other members but much the same number of tiles.)
int64_t BiggestTiledTreeBytes(const Forest &forest, int tileSize);

// Throws tbamd::Error when the plan cannot hold the model (tree larger than a
// group, feature offsets that do not fit 16 bits, ...).  `profile` (may be null) feeds the plan's
// probability-based tiling and walk peeling.
PackedModel PackForest(const Forest &forest, const LaunchPlan &plan, const HitCountProfile *profile = nullptr);

// Inverse of PackForest for tests: rebuilds (value, feature, left, right) of
// original tree `tree` from the packed arrays.
Tree UnpackTree(const PackedModel &model, int32_t tree);

// Children-swapped / threshold-adjusted copy in which "x < value -> left" holds
// for every comparison mode the loaders accept.
Forest NormalizeToLessThan(const Forest &forest);

} // namespace tbamd
