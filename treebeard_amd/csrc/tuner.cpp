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

void FitGroupBytes(LaunchPlan &plan, const Forest &forest, const DeviceLimits &limits, int blocksPerCu) {
  const int64_t rowTile = (int64_t)(forest.numFeatures + 1) * plan.rowsPerBlock * 4;
  int64_t perBlock = limits.ldsBytesPerBlock / blocksPerCu;
  int64_t group = std::min<int64_t>(65536, perBlock - rowTile);
  // the biggest tree has to fit a group (+ null leaf + alignment pad)
  int64_t biggest = 0;
  for (auto &t : forest.trees) biggest = std::max<int64_t>(biggest, (int64_t)t.NumNodes());
  const int64_t need = (biggest + 2) * kNodeBytes;
  if (group < need) group = std::min<int64_t>(65536, std::min<int64_t>(limits.ldsBytesPerBlock - rowTile, std::max<int64_t>(need, 16384)));
  plan.groupBytes = (int32_t)(group & ~15);
}

} // namespace

namespace {

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

LaunchPlan ChoosePlan(const Forest &forest, int64_t batchSize, const GPUAutoScheduleOptions *ov,
                      const DeviceLimits &limits) {
  bool fitsTransposed = false;
  {
    bool words = false;
    fitsTransposed = RowTileFits(forest.numFeatures, 64, limits.ldsBytesPerBlock, &words);
  }
  if (!fitsTransposed || (batchSize > 0 && batchSize <= 128))
    return ChooseTreeParallelPlan(forest, batchSize, ov, limits);

  LaunchPlan plan;
  plan.kernel = LaunchPlan::Kernel::kRowParallelLds;

  int32_t rb = 256;
  if (ov && ov->numRowsPerTB > 0) rb = std::max(64, FloorPow2(ov->numRowsPerTB));
  if (batchSize > 0 && batchSize < rb) rb = std::max<int32_t>(64, FloorPow2(std::max<int64_t>(batchSize, 1) * 2 - 1));
  bool words = false;
  while (rb > 64 && !RowTileFits(forest.numFeatures, rb, limits.ldsBytesPerBlock, &words)) rb /= 2;
  if (!RowTileFits(forest.numFeatures, rb, limits.ldsBytesPerBlock, &words))
    throw Error("row tile of " + std::to_string(forest.numFeatures) + " features does not fit LDS");
  plan.rowsPerBlock = rb;
  plan.featureOffsetInWords = words;

  plan.interleave = 4;
  if (ov && ov->treeWalkInterleaveFactor > 0)
    plan.interleave = std::min(kMaxInterleave, FloorPow2(ov->treeWalkInterleaveFactor));

  FitGroupBytes(plan, forest, limits, /*blocksPerCu=*/2);

  // Tree slices: when the batch alone cannot fill the chip, blocks share a row
  // tile and split the tree groups between them.
  const int64_t rowBlocks = std::max<int64_t>(1, (batchSize + rb - 1) / rb);
  int64_t totalNodes = (int64_t)forest.NumNodes();
  int64_t groups = std::max<int64_t>(1, (totalNodes * kNodeBytes + plan.groupBytes - 1) / plan.groupBytes);
  int64_t slices = 1;
  const int64_t wantBlocks = 2LL * limits.computeUnits;
  if (rowBlocks < wantBlocks) slices = std::min<int64_t>(groups, (wantBlocks + rowBlocks - 1) / rowBlocks);
  if (ov && ov->numTreeThreads > 0) slices = std::min<int64_t>(groups, ov->numTreeThreads);
  if (slices > 1) {
    // more, smaller groups so that every slice has at least one
    int64_t perSlice = (totalNodes * kNodeBytes + slices - 1) / slices + 4096;
    int64_t biggest = 0;
    for (auto &t : forest.trees) biggest = std::max<int64_t>(biggest, (int64_t)t.NumNodes());
    perSlice = std::max<int64_t>(perSlice, (biggest + 2) * kNodeBytes);
    if (perSlice < plan.groupBytes) plan.groupBytes = (int32_t)((perSlice + 15) & ~15);
  }
  plan.treeSlices = (int32_t)std::max<int64_t>(1, slices);
  return plan;
}

std::vector<LaunchPlan> CandidatePlans(const Forest &forest, int64_t batchSize, const DeviceLimits &limits) {
  std::vector<LaunchPlan> out;
  LaunchPlan base = ChoosePlan(forest, batchSize, nullptr, limits);
  out.push_back(base);
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
  for (int32_t rb : {64, 128, 256, 512})
    for (int32_t k : {2, 4, 8})
      for (int blocksPerCu : {1, 2, 3}) {
        bool words = false;
        if (!RowTileFits(forest.numFeatures, rb, limits.ldsBytesPerBlock / blocksPerCu, &words)) continue;
        LaunchPlan p = base;
        p.rowsPerBlock = rb;
        p.featureOffsetInWords = words;
        p.interleave = k;
        FitGroupBytes(p, forest, limits, blocksPerCu);
        if ((int64_t)(forest.numFeatures + 1) * rb * 4 + p.groupBytes > limits.ldsBytesPerBlock) continue;
        const int64_t rowBlocks = std::max<int64_t>(1, (batchSize + rb - 1) / rb);
        if (base.treeSlices > 1) {
          int64_t groups = std::max<int64_t>(1, ((int64_t)forest.NumNodes() * kNodeBytes + p.groupBytes - 1) / p.groupBytes);
          p.treeSlices = (int32_t)std::min<int64_t>(groups, std::max<int64_t>(1, 2LL * limits.computeUnits / rowBlocks));
        }
        bool dup = false;
        for (auto &q : out)
          dup = dup || (q.rowsPerBlock == p.rowsPerBlock && q.interleave == p.interleave &&
                        q.groupBytes == p.groupBytes && q.treeSlices == p.treeSlices);
        if (!dup) out.push_back(p);
      }
  return out;
}

} // namespace tbamd
