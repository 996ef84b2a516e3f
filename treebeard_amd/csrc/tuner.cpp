#include "tuner.h"

#include <algorithm>

namespace tbamd {

namespace {

int32_t FloorPow2(int64_t v) {
  int32_t p = 1;
  while ((int64_t)p * 2 <= v) p *= 2;
  return p;
}

// Largest rows-per-block (power of two, >= 64) whose transposed row tile keeps
// 16-bit feature offsets and leaves room for a tree group.
bool RowTileFits(int32_t numFeatures, int32_t rowsPerBlock, int32_t ldsBytes, bool *offsetsInWords) {
  const int64_t words = (int64_t)(numFeatures + 1) * rowsPerBlock;
  if (words > 0xFFFF) return false;
  if (words * 4 + 16 * 1024 > ldsBytes) return false; // keep at least 16 KB for trees
  *offsetsInWords = words * 4 > 0xFFFF;
  return true;
}


int64_t BiggestTreeNodes(const Forest &forest) {
  int64_t biggest = 0;
  for (auto &t : forest.trees) biggest = std::max<int64_t>(biggest, (int64_t)t.NumNodes());
  return biggest;
}

// Rows row-major in LDS, several lanes per row.
LaunchPlan ChooseTreeParallelPlan(const Forest &forest, int64_t batchSize, const GPUAutoScheduleOptions *ov,
                                  const DeviceLimits &limits) {
  LaunchPlan plan;
  plan.kernel = LaunchPlan::Kernel::kTreeParallel;
  plan.interleave = 1;
  if (ov && ov->treeWalkInterleaveFactor > 0)
    plan.interleave = std::min(kMaxInterleave, FloorPow2(ov->treeWalkInterleaveFactor));
  const int64_t rowBytes = (int64_t)(forest.numFeatures + 1) * 4;
  const int64_t need = (BiggestTreeNodes(forest) + 2) * kNodeBytes;
  if (need > 65536) throw Error("a tree does not fit one LDS tree group");
  int64_t group = std::max<int64_t>(need, 24 * 1024);
  const int64_t reserve = 4096; // reduction scratch and class sums
  if (rowBytes + group + reserve > limits.ldsBytesPerBlock) group = need;
  if (rowBytes + group + reserve > limits.ldsBytesPerBlock)
    throw Error("a row of " + std::to_string(forest.numFeatures) + " features does not fit LDS next to a tree group");
  int64_t rows = FloorPow2((limits.ldsBytesPerBlock - group - reserve) / rowBytes);
  rows = std::min<int64_t>(rows, 16);
  if (ov && ov->numRowsPerTB > 0) rows = std::min<int64_t>(rows, FloorPow2(ov->numRowsPerTB));
  if (batchSize > 0) rows = std::min<int64_t>(rows, FloorPow2(std::max<int64_t>(batchSize, 1) * 2 - 1));
  plan.rowsPerBlock = (int32_t)std::max<int64_t>(rows, 1);
  plan.treeLanes = std::max(1, 256 / plan.rowsPerBlock);
  // narrow rows leave LDS for bigger groups
  const int64_t rowTile = rowBytes * plan.rowsPerBlock;
  group = std::max<int64_t>(group, std::min<int64_t>(65536, (limits.ldsBytesPerBlock / 2 - rowTile - reserve)));
  group = std::min<int64_t>(group, 256LL * plan.ThreadsPerBlock()); // 16 prefetch registers of 16 bytes per lane
  if (group < need) throw Error("the biggest tree does not fit the group prefetch registers of this block shape");
  plan.groupBytes = (int32_t)(std::min<int64_t>(group, 65536) & ~15);

  const int64_t rowBlocks = std::max<int64_t>(1, (batchSize + plan.rowsPerBlock - 1) / plan.rowsPerBlock);
  const int64_t totalBytes = (int64_t)forest.NumNodes() * kNodeBytes;
  int64_t groups = std::max<int64_t>(1, (totalBytes + plan.groupBytes - 1) / plan.groupBytes);
  int64_t slices = 1;
  const int64_t wantBlocks = 2LL * limits.computeUnits;
  if (rowBlocks < wantBlocks) slices = (wantBlocks + rowBlocks - 1) / rowBlocks;
  if (ov && ov->numTreeThreads > 0) slices = ov->numTreeThreads;
  slices = std::min<int64_t>(slices, std::max<int64_t>(1, totalBytes / 8192)); // at least 8 KB of trees per slice
  if (slices > groups) {
    int64_t perSlice = std::max<int64_t>((totalBytes + slices - 1) / slices + 2048, need);
    plan.groupBytes = (int32_t)(std::min<int64_t>(perSlice, 65536) & ~15);
  }
  plan.treeSlices = (int32_t)std::max<int64_t>(1, slices);
  return plan;
}

} // namespace

namespace {
LaunchPlan ChooseScalarPlan(const Forest &forest, int64_t batchSize, const GPUAutoScheduleOptions *ov,
                            const DeviceLimits &limits, int tileSize);
// LDS bytes a tree group must offer the biggest tree of a tiled forest (the null leaf tile and the alignment
// pad of a group included).
int64_t TiledGroupNeed(const Forest &forest, int tileSize) {
  return BiggestTiledTreeBytes(forest, tileSize) + 2 * (int64_t)TileBytes(tileSize) + 16;
}
}

LaunchPlan ChoosePlan(const Forest &forest, int64_t batchSize, const GPUAutoScheduleOptions *ov,
                      const DeviceLimits &limits, const WalkOptions &walk) {
  if (walk.tileSize < 1 || walk.tileSize > kMaxTileSize)
    throw Error("tile size " + std::to_string(walk.tileSize) + " is not supported: the device kernels walk tiles of 1 to " +
                std::to_string(kMaxTileSize) + " nodes");
  LaunchPlan plan = ChooseScalarPlan(forest, batchSize, ov, limits, walk.tileSize);
  plan.tileSize = walk.tileSize;
  plan.tiling = walk.tiling;
  plan.peelWalks = walk.peelWalks;
  plan.deferTails = false;
  if (walk.peelWalks && DeferTailsFit(forest, &plan)) plan.deferTails = true;
  return plan;
}

bool DeferTailsFit(const Forest &forest, LaunchPlan *plan) {
  if (plan->kernel != LaunchPlan::Kernel::kRowParallelLds || plan->tileSize != 1 || plan->quantizedRows || plan->rankRows16 ||
      plan->featureOffsetInWords || forest.numClasses > 0)
    return false;
  // every wave's queue comes out of the tree group's share of LDS
  const int64_t extra = (int64_t)(plan->ThreadsPerBlock() / 64) * kDeferBytesPerWave + 32;
  if (forest.numFeatures + 1 >= (1 << kTailFeatureBits)) return false;
  const int64_t need = (BiggestTreeNodes(forest) + 2) * kNodeBytes;
  if (plan->groupBytes - extra < std::max<int64_t>(need, 8192)) return false;
  plan->groupBytes = (int32_t)((plan->groupBytes - extra) & ~15);
  return true;
}

namespace {

// tileSize > 1: the plan must be the row-parallel kernel on f32 rows with byte offsets (tiles hold byte offsets
// into a row tile below 64 KB), and groups are sized for tiles, which take three to eight times the bytes of
// scalar nodes.
LaunchPlan ChooseScalarPlan(const Forest &forest, int64_t batchSize, const GPUAutoScheduleOptions *ov,
                            const DeviceLimits &limits, int tileSize) {
  if (tileSize > 1) {
    const int64_t need = TiledGroupNeed(forest, tileSize);
    if (need > 65536)
      throw Error("tile sizes above 1 need every tree to fit one LDS tree group; this forest has a tree that does not");
    LaunchPlan plan;
    plan.kernel = LaunchPlan::Kernel::kRowParallelLds;
    int32_t rb = 256;
    if (ov && ov->numRowsPerTB > 0) rb = std::max(64, std::min(256, FloorPow2(ov->numRowsPerTB)));
    // two blocks per CU while 24 KB remain for a group, byte offsets below 64 KB
    auto tileBytes = [&](int32_t r) { return (int64_t)(forest.numFeatures + 1) * r * 4; };
    while (rb > 64 && (tileBytes(rb) > 0xFFFF || limits.ldsBytesPerBlock / 2 - tileBytes(rb) < 24 * 1024)) rb /= 2;
    if (tileBytes(rb) > 0xFFFF)
      throw Error("tile sizes above 1 need a row tile below 64 KB: " + std::to_string(forest.numFeatures) + " features are too many");
    plan.rowsPerBlock = rb;
    plan.treeThreads = std::max(1, 1024 / rb);
    if (ov && ov->numTreeThreads > 0) plan.treeThreads = std::max(1, std::min(ov->numTreeThreads, 1024 / rb));
    plan.interleave = 2;
    if (ov && ov->treeWalkInterleaveFactor > 0) plan.interleave = std::min(4, FloorPow2(ov->treeWalkInterleaveFactor));
    const int64_t meet = forest.numClasses > 0 ? (int64_t)rb * plan.treeThreads * 8 : 0;
    int64_t budget = limits.ldsBytesPerBlock / 2;
    int64_t group = std::min<int64_t>(65536, budget - tileBytes(rb) - meet - 512);
    if (group < need) group = std::min<int64_t>(65536, limits.ldsBytesPerBlock - tileBytes(rb) - meet - 512);
    group = std::min<int64_t>(group, 256LL * rb * plan.treeThreads);
    if (group < need) throw Error("the biggest tree does not fit LDS next to the row tile when tiled");
    plan.groupBytes = (int32_t)(group & ~15);
    const int64_t rowBlocks = std::max<int64_t>(1, (batchSize + rb - 1) / rb);
    const int64_t totalBytes = (int64_t)forest.NumNodes() * (tileSize > kMaxSelectTile ? 40 : 24);
    int64_t slices = 1;
    const int64_t wantBlocks = 2LL * limits.computeUnits;
    if (rowBlocks < wantBlocks) slices = (wantBlocks + rowBlocks - 1) / rowBlocks;
    slices = std::min<int64_t>(slices, std::max<int64_t>(1, totalBytes / plan.groupBytes));
    plan.treeSlices = (int32_t)std::max<int64_t>(1, slices);
    return plan;
  }
  // A tree that cannot sit in one LDS group walks from global memory; so do rows that neither LDS form can
  // hold (below): more than 16383 features have no 16-bit byte offset inside one row-major LDS row.
  auto globalPlan = [&]() {
    LaunchPlan plan;
    plan.kernel = LaunchPlan::Kernel::kGlobalWalk;
    plan.rowsPerBlock = 256;
    plan.interleave = 4;
    if (ov && ov->treeWalkInterleaveFactor > 0)
      plan.interleave = std::min(kMaxInterleave, FloorPow2(ov->treeWalkInterleaveFactor));
    const int64_t rowBlocks = std::max<int64_t>(1, (batchSize + 255) / 256);
    int64_t slices = 1;
    if (rowBlocks < 4LL * limits.computeUnits) slices = (4LL * limits.computeUnits + rowBlocks - 1) / rowBlocks;
    plan.treeSlices = (int32_t)std::max<int64_t>(1, std::min<int64_t>(slices, (int64_t)forest.trees.size()));
    plan.groupBytes = 0;
    return plan;
  };
  if ((BiggestTreeNodes(forest) + 2) * kNodeBytes > 65536) return globalPlan();
  const bool rowMajorFits = (int64_t)(forest.numFeatures + 1) * 4 <= 0xFFFF &&
                            (int64_t)(forest.numFeatures + 1) * 4 + (BiggestTreeNodes(forest) + 2) * kNodeBytes + 4096 <=
                                limits.ldsBytesPerBlock;
  bool fitsTransposed = false;
  {
    bool words = false;
    fitsTransposed = RowTileFits(forest.numFeatures, 64, limits.ldsBytesPerBlock, &words);
  }
  if (batchSize > 0 && batchSize <= 128 && rowMajorFits) return ChooseTreeParallelPlan(forest, batchSize, ov, limits);
  if (!fitsTransposed) {
    // Rows too wide for 64 f32 rows in LDS: one-byte ranks (exact) if every feature has few enough
    // distinct thresholds and 64 rank rows fit; otherwise a few f32 rows with several lanes each.
    const int64_t tile = (int64_t)(forest.numFeatures + 1) * 64;
    const int64_t need = (BiggestTreeNodes(forest) + 2) * kNodeBytes;
    const int64_t room = limits.ldsBytesPerBlock - tile - 2048 - (forest.numClasses > 0 ? 1024 * 8 : 0);
    if (room >= std::max<int64_t>(need, 8192) && forest.numFeatures * 16 <= 0xFFFF &&
        MaxThresholdsPerFeature(forest) <= 254) {
      LaunchPlan plan;
      plan.kernel = LaunchPlan::Kernel::kRowParallelLds;
      plan.quantizedRows = true;
      plan.rowsPerBlock = 64;
      plan.treeThreads = 16;
      if (ov && ov->numTreeThreads > 0) plan.treeThreads = std::max(1, std::min(ov->numTreeThreads, 16));
      plan.interleave = 2;
      if (ov && ov->treeWalkInterleaveFactor > 0)
        plan.interleave = std::min(kMaxInterleave, FloorPow2(ov->treeWalkInterleaveFactor));
      plan.groupBytes = (int32_t)(std::min<int64_t>({room, 65536, 256LL * plan.ThreadsPerBlock()}) & ~15);
      const int64_t rowBlocks = std::max<int64_t>(1, (batchSize + 63) / 64);
      const int64_t totalBytes = (int64_t)forest.NumNodes() * kNodeBytes;
      int64_t slices = 1;
      if (rowBlocks < limits.computeUnits) slices = (limits.computeUnits + rowBlocks - 1) / rowBlocks;
      slices = std::min<int64_t>(slices, std::max<int64_t>(1, totalBytes / plan.groupBytes));
      plan.treeSlices = (int32_t)std::max<int64_t>(1, slices);
      return plan;
    }
    return rowMajorFits ? ChooseTreeParallelPlan(forest, batchSize, ov, limits) : globalPlan();
  }

  LaunchPlan plan;
  plan.kernel = LaunchPlan::Kernel::kRowParallelLds;

  // Block shape, from timings on MI355X (blocks of 1024 lanes; 600-1000 trees of depth 6-8; 28..520 features).
  // Two blocks per CU hide each other's group loads and barriers, but only while enough LDS is left for
  // the tree groups; a narrower row tile buys bigger groups; past that one block per CU with the biggest
  // groups wins.  In order of preference:
  //   256 rows x 4 tree threads, two blocks per CU, while >= 16 KB remain for a group   (up to ~60 features)
  //   128 x 8, two blocks, while >= 20 KB remain                                        (up to ~118)
  //    64 x 16, two blocks, while >= 40 KB remain                                       (up to ~155)
  //   128 x 8, one block, while >= 56 KB remain                                         (up to ~195)
  //    64 x 16, one block                                                               (as long as the tile fits)
  const int32_t halfLds = limits.ldsBytesPerBlock / 2;
  bool words = false;
  auto treeThreadsFor = [&](int32_t r) {
    int32_t tt = std::max(1, 1024 / r);
    if (ov && ov->numTreeThreads > 0) tt = std::max(1, std::min(ov->numTreeThreads, 1024 / r));
    return tt;
  };
  // LDS left for a tree group beside the row tile (and the classifiers' meeting area)
  auto roomFor = [&](int32_t r, int32_t ldsBytes) -> int64_t {
    const int64_t tile = (int64_t)(forest.numFeatures + 1) * r * 4;
    const int64_t meetBytes = forest.numClasses > 0 ? (int64_t)r * treeThreadsFor(r) * 8 : 0;
    return (int64_t)ldsBytes - tile - meetBytes - 512;
  };
  int32_t rb = 64;
  int32_t budget = limits.ldsBytesPerBlock;
  if (ov && ov->numRowsPerTB > 0) { // the caller's block shape: two blocks per CU if 16 KB remain, else one
    rb = std::max(64, FloorPow2(ov->numRowsPerTB));
    while (rb > 64 && roomFor(rb, limits.ldsBytesPerBlock) < 16384) rb /= 2;
    if (roomFor(rb, halfLds) >= 16384) budget = halfLds;
  } else if (roomFor(256, halfLds) >= 16384) {
    rb = 256, budget = halfLds;
  } else if (roomFor(128, halfLds) >= 20480) {
    rb = 128, budget = halfLds;
  } else if (roomFor(64, halfLds) >= 40960) {
    rb = 64, budget = halfLds;
  } else if (roomFor(128, limits.ldsBytesPerBlock) >= 57344) {
    rb = 128;
  }
  if (!RowTileFits(forest.numFeatures, rb, budget, &words))
    throw Error("row tile of " + std::to_string(forest.numFeatures) + " features does not fit LDS");
  plan.rowsPerBlock = rb;
  plan.featureOffsetInWords = words;
  plan.treeThreads = treeThreadsFor(rb);

  plan.interleave = 4;
  if (ov && ov->treeWalkInterleaveFactor > 0)
    plan.interleave = std::min(kMaxInterleave, FloorPow2(ov->treeWalkInterleaveFactor));

  const int64_t rowTile = (int64_t)(forest.numFeatures + 1) * rb * 4;
  const int64_t need = (BiggestTreeNodes(forest) + 2) * kNodeBytes;
  if (need > 65536) throw Error("a tree does not fit one LDS tree group");
  const int64_t meet = forest.numClasses > 0 ? (int64_t)rb * plan.treeThreads * 8 : 0; // cross-wave pass
  // (LDS is handed out in coarse pieces: leave slack or the second block will not fit)
  int64_t group = std::min<int64_t>(65536, budget - rowTile - meet - 512);
  if (group < need) group = std::min<int64_t>(65536, limits.ldsBytesPerBlock - rowTile - meet - 512);
  group = std::min<int64_t>(group, 256LL * rb * plan.treeThreads); // 16 prefetch registers of 16 bytes per lane
  if (group < need) throw Error("the biggest tree does not fit LDS next to the row tile");
  plan.groupBytes = (int32_t)(group & ~15);

  // Tree slices: when the batch alone cannot fill the chip, blocks share a row
  // tile and split the tree groups between them.
  const int64_t rowBlocks = std::max<int64_t>(1, (batchSize + rb - 1) / rb);
  const int64_t totalBytes = (int64_t)forest.NumNodes() * kNodeBytes;
  int64_t groups = std::max<int64_t>(1, (totalBytes + plan.groupBytes - 1) / plan.groupBytes);
  int64_t slices = 1;
  const int64_t wantBlocks = 2LL * limits.computeUnits;
  if (rowBlocks < wantBlocks) slices = (wantBlocks + rowBlocks - 1) / rowBlocks;
  slices = std::min<int64_t>(slices, std::max<int64_t>(1, totalBytes / 16384)); // >= 16 KB of trees per slice
  if (slices > groups) { // more, smaller groups so that every slice has one
    int64_t perSlice = std::max<int64_t>((totalBytes + slices - 1) / slices + 4096, need);
    if (perSlice < plan.groupBytes) plan.groupBytes = (int32_t)((perSlice + 15) & ~15);
  }
  plan.treeSlices = (int32_t)std::max<int64_t>(1, slices);
  return plan;
}

} // namespace

std::vector<LaunchPlan> CandidatePlans(const Forest &forest, int64_t batchSize, const DeviceLimits &limits,
                                       const WalkOptions &walk) {
  std::vector<LaunchPlan> out;
  LaunchPlan base = ChoosePlan(forest, batchSize, nullptr, limits, walk);
  out.push_back(base);
  if (base.tileSize > 1) { // block shapes and interleave factors of the tiled walk
    for (int32_t rb : {64, 128, 256})
      for (int32_t k : {1, 2, 4}) {
        LaunchPlan p = base;
        p.rowsPerBlock = rb;
        p.treeThreads = 1024 / rb;
        p.interleave = k;
        const int64_t tile = (int64_t)(forest.numFeatures + 1) * rb * 4;
        if (tile > 0xFFFF) continue;
        const int64_t meet = forest.numClasses > 0 ? (int64_t)rb * p.treeThreads * 8 : 0;
        int64_t group = std::min<int64_t>(65536, limits.ldsBytesPerBlock / 2 - tile - meet - 2048);
        if (group < TiledGroupNeed(forest, base.tileSize)) continue;
        if (base.treeSlices > 1) group = std::min<int64_t>(group, base.groupBytes);
        p.groupBytes = (int32_t)(group & ~15);
        bool dup = false;
        for (auto &q : out)
          dup = dup || (q.rowsPerBlock == p.rowsPerBlock && q.interleave == p.interleave && q.groupBytes == p.groupBytes);
        if (!dup) out.push_back(p);
      }
    return out;
  }
  if (base.kernel == LaunchPlan::Kernel::kGlobalWalk) {
    for (int32_t k : {1, 2, 8}) {
      LaunchPlan p = base;
      p.interleave = k;
      out.push_back(p);
    }
    return out;
  }
  if (base.kernel == LaunchPlan::Kernel::kTreeParallel) {
    for (int32_t lanes : {base.treeLanes / 2, base.treeLanes * 2})
      for (int32_t k : {1, 2}) {
        LaunchPlan p = base;
        p.treeLanes = lanes;
        p.interleave = k;
        if (lanes < 1 || p.ThreadsPerBlock() > 1024 || p.ThreadsPerBlock() % 64 != 0) continue;
        if (lanes < 64 && 64 % lanes != 0) continue;
        out.push_back(p);
      }
    return out;
  }
  const int64_t need = (BiggestTreeNodes(forest) + 2) * kNodeBytes;
  for (int32_t rb : {64, 128, 256, 512})
    for (int32_t tt : {1, 2, 4, 8, 16})
      for (int32_t k : {2, 4, 8})
        for (int blocksPerCu : {1, 2, 3, 4, 6, 8}) {
          if (rb * tt > 1024 || rb * tt * blocksPerCu > 2048) continue; // (a compute unit holds 32 waves)
          bool words = false;
          const int32_t budget = limits.ldsBytesPerBlock / blocksPerCu;
          if (!RowTileFits(forest.numFeatures, rb, budget + 8192, &words)) continue;
          LaunchPlan p = base;
          p.rowsPerBlock = rb;
          p.treeThreads = tt;
          p.featureOffsetInWords = words;
          p.interleave = k;
          const int64_t rowTile = (int64_t)(forest.numFeatures + 1) * rb * 4;
          int64_t group = std::min<int64_t>(65536, budget - rowTile - (forest.numClasses > 0 ? (int64_t)rb * tt * 8 : 0) - 2048);
          group = std::min<int64_t>(group, 256LL * rb * tt); // 16 prefetch registers of 16 bytes per lane
          if (group < need || group < 8192) continue;
          if (base.treeSlices > 1) group = std::min<int64_t>(group, base.groupBytes);
          p.groupBytes = (int32_t)(group & ~15);
          if (base.deferTails) {
            p.deferTails = false;
            if (!DeferTailsFit(forest, &p)) continue;
            p.deferTails = true;
          }
          bool dup = false;
          for (auto &q : out)
            dup = dup || (q.rowsPerBlock == p.rowsPerBlock && q.treeThreads == p.treeThreads &&
                          q.interleave == p.interleave && q.groupBytes == p.groupBytes);
          if (!dup) out.push_back(p);
        }
  // Two-byte rank rows (a ranking kernel in front of the walk, half the row tile): the timed search counts both
  // kernels, so the form is kept only where the walk gains more than the ranking costs.
  if (!base.quantizedRows && base.treeSlices == 1)
    for (int32_t rb : {256, 512}) {
      const int64_t rowTile = (int64_t)((forest.numFeatures + 2) / 2) * rb * 4;
      if (rowTile > 0xFFFF) continue;
      LaunchPlan p = base;
      p.rankRows16 = true;
      p.deferTails = false;
      p.featureOffsetInWords = false;
      p.rowsPerBlock = rb;
      p.treeThreads = 1024 / rb;
      p.interleave = 4;
      int64_t group = std::min<int64_t>(65536, limits.ldsBytesPerBlock / 2 - rowTile - (forest.numClasses > 0 ? 1024 * 8 : 0) - 2048);
      if (group < need || group < 8192) continue;
      p.groupBytes = (int32_t)(group & ~15);
      out.push_back(p);
    }
  return out;
}

} // namespace tbamd
