#include "packer.h"

#include <algorithm>
#include <cmath>
#include <functional>
#include <limits>
#include <cstring>
#include <numeric>

namespace tbamd {

Forest NormalizeToLessThan(const Forest &forest) {
  if (forest.predicate == Predicate::kLT) return forest;
  Forest out = forest;
  out.predicate = Predicate::kLT;
  const bool swapChildren = forest.predicate == Predicate::kGE || forest.predicate == Predicate::kGT;
  // x <= t  <=>  x < nextafter(t, +inf)   and   x > t  <=>  !(x <= t)
  const bool bumpThreshold = forest.predicate == Predicate::kLE || forest.predicate == Predicate::kGT;
  for (auto &tree : out.trees)
    for (size_t i = 0; i < tree.NumNodes(); ++i) {
      if (tree.IsLeaf((int32_t)i)) continue;
      if (bumpThreshold) tree.value[i] = std::nextafter(tree.value[i], std::numeric_limits<float>::infinity());
      if (swapChildren) std::swap(tree.left[i], tree.right[i]);
    }
  return out;
}

uint32_t PackedModel::PadFeatureOffset() const { return plan.FeatureOffset((uint32_t)numFeatures); }

size_t PackedModel::RowTileBytes() const {
  if (plan.rankRows16) return (size_t)((numFeatures + 2) / 2) * plan.rowsPerBlock * 4; // pairs of two-byte ranks, pad feature included
  return (size_t)(numFeatures + 1) * plan.rowsPerBlock * (plan.quantizedRows ? 1 : 4); // (+ the pad feature's column)
}

size_t PackedModel::LdsBytes() const {
  if (plan.kernel == LaunchPlan::Kernel::kGlobalWalk) return 0;
  size_t bytes = RowTileBytes() + (size_t)GroupRegionBytes();
  if (plan.kernel == LaunchPlan::Kernel::kTreeParallel) {
    // cross-wave reduction scratch + per-row, per-class accumulators (doubles)
    const size_t waves = (size_t)(plan.ThreadsPerBlock() + 63) / 64;
    bytes = (bytes + 7) & ~(size_t)7;
    bytes += waves * 8 + (size_t)plan.rowsPerBlock * (numClasses > 0 ? numClasses : 1) * 8;
  } else if (plan.treeThreads > 1 && numClasses > 0) {
    bytes = (bytes + 7) & ~(size_t)7;
    bytes += (size_t)plan.ThreadsPerBlock() * 8; // classifiers: cross-wave pass behind the row tile
  }
  if (plan.deferTails) {
    bytes = (bytes + 15) & ~(size_t)15;
    bytes += (size_t)(plan.ThreadsPerBlock() / 64) * kDeferBytesPerWave; // every wave's queue of deferred walks
  }
  return bytes;
}

namespace {

// Sorted distinct thresholds per feature of a forest already normalised to "x < t".
std::vector<std::vector<float>> ThresholdsPerFeature(const Forest &forest) {
  std::vector<std::vector<float>> out((size_t)forest.numFeatures);
  for (auto &tree : forest.trees)
    for (size_t i = 0; i < tree.NumNodes(); ++i)
      if (!tree.IsLeaf((int32_t)i)) out[(size_t)tree.feature[i]].push_back(tree.value[i]);
  for (auto &v : out) {
    std::sort(v.begin(), v.end());
    v.erase(std::unique(v.begin(), v.end()), v.end());
  }
  return out;
}

} // namespace

int32_t MaxThresholdsPerFeature(const Forest &forest) {
  size_t most = 0;
  for (auto &v : ThresholdsPerFeature(NormalizeToLessThan(forest))) most = std::max(most, v.size());
  return (int32_t)most;
}

namespace {

// Level-order node list of one tree with siblings adjacent.
struct LevelOrder {
  std::vector<int32_t> order;    // packed position -> original node
  std::vector<int32_t> position; // original node -> packed position
};

LevelOrder MakeLevelOrder(const Tree &tree) {
  LevelOrder lo;
  lo.position.assign(tree.NumNodes(), -1);
  lo.order.push_back(0);
  for (size_t head = 0; head < lo.order.size(); ++head) {
    int32_t n = lo.order[head];
    lo.position[n] = (int32_t)head;
    if (tree.IsLeaf(n)) continue;
    lo.order.push_back(tree.left[n]);
    lo.order.push_back(tree.right[n]);
  }
  return lo;
}

} // namespace


namespace {

// ---------------------------------------------------------------------------
// Tiling of one tree (LaunchPlan::tileSize > 1).
// ---------------------------------------------------------------------------
struct TileInfo {
  int32_t count = 0;                       // internal nodes in the tile; 0: a leaf tile
  int32_t members[kMaxTileSize] = {};      // original node ids, level order inside the tile
  int32_t numExits = 0;
  int32_t exits[kMaxTileSize + 1] = {};    // original node ids the tile's children start at, left to right
  int32_t leafNode = -1;                   // leaf tiles: the original leaf
  uint32_t firstChild = 0;                 // tile index (inside the tree) of child 0; own index on a leaf tile
  uint64_t select = 0;                     // child number per outcome word, TileSelectBits() each (tiles of up to 4 nodes)
  uint64_t links = kLeafTileLinks;         // a 4-bit link per slot and outcome (tiles of 5 to 8 nodes, device_model.h)
  int32_t hops = 1;                        // links a walk follows inside the tile at most (its levels of nodes)
  int32_t depth = 0;                       // tile steps from this tile down to its deepest leaf
  int32_t level = 0;                       // tile steps from the root tile
};

struct TiledTree {
  std::vector<TileInfo> tiles; // children of a tile are consecutive
  int32_t depth = 0;           // tile steps that bring every row to a leaf tile
  int32_t hops = 1;            // the most levels of nodes any tile holds
  bool byProfile = false;
};

// Members of the tile rooted at `root`, breadth first over internal nodes, left before right
// (src/mlir/UniformTilingTransformation.cpp:148-168).
int GatherUniform(const Tree &tree, int32_t root, int T, int32_t *members) {
  int32_t queue[2 * kMaxTileSize + 2];
  int head = 0, tail = 0, n = 0;
  queue[tail++] = root;
  while (head < tail && n < T) {
    const int32_t node = queue[head++];
    members[n++] = node;
    if (!tree.IsLeaf(tree.left[node])) queue[tail++] = tree.left[node];
    if (!tree.IsLeaf(tree.right[node])) queue[tail++] = tree.right[node];
  }
  return n;
}

// Members chosen by visit counts: the tile grows by the most-visited internal child of any member
// (src/mlir/ProbabilityBasedTilingTransform.cpp:152-190: members are scanned in node order, left child before
// right, and a candidate wins only with strictly more hits).
int GatherByHits(const Tree &tree, const std::vector<int64_t> &hits, int32_t root, int T, int32_t *members) {
  int n = 0;
  members[n++] = root;
  while (n < T) {
    int32_t sorted[kMaxTileSize];
    std::copy(members, members + n, sorted);
    std::sort(sorted, sorted + n);
    int64_t bestHits = -1;
    int32_t best = -1;
    for (int i = 0; i < n; ++i)
      for (int32_t child : {tree.left[sorted[i]], tree.right[sorted[i]]}) {
        if (tree.IsLeaf(child) || hits[child] <= bestHits) continue;
        if (std::find(members, members + n, child) != members + n) continue;
        bestHits = hits[child];
        best = child;
      }
    if (best < 0) break;
    members[n++] = best;
  }
  return n;
}

// src/mlir/ProbabilityBasedTilingTransform.cpp:208-225: the most-visited tenth of the leaves takes more
// than 90 % of the rows.
bool IsSkewed(const Tree &tree, const std::vector<int64_t> &hits) {
  std::vector<int64_t> leafHits;
  for (size_t i = 0; i < tree.NumNodes(); ++i)
    if (tree.IsLeaf((int32_t)i)) leafHits.push_back(hits[i]);
  std::sort(leafHits.begin(), leafHits.end(), std::greater<int64_t>());
  const size_t consider = (size_t)((double)leafHits.size() * 0.10);
  int64_t covered = 0;
  for (size_t i = 0; i < consider; ++i) covered += leafHits[i];
  return hits[0] > 0 && (double)covered / (double)hits[0] > 0.9;
}

TiledTree TileTree(const Tree &tree, int T, int tiling, const std::vector<int64_t> *hits) {
  TiledTree out;
  out.byProfile = tiling != 0 && hits != nullptr && IsSkewed(tree, *hits);
  // depth of every original node, for the level order inside a tile
  std::vector<int32_t> nodeDepth(tree.NumNodes(), -1);
  {
    std::vector<int32_t> stack{0};
    nodeDepth[0] = 0;
    while (!stack.empty()) {
      const int32_t n = stack.back();
      stack.pop_back();
      if (tree.IsLeaf(n)) continue;
      nodeDepth[tree.left[n]] = nodeDepth[tree.right[n]] = nodeDepth[n] + 1;
      stack.push_back(tree.left[n]);
      stack.push_back(tree.right[n]);
    }
  }
  std::vector<int32_t> roots{0}; // node each tile starts at, in tile order
  for (size_t ti = 0; ti < roots.size(); ++ti) {
    TileInfo tile;
    const int32_t root = roots[ti];
    if (tree.IsLeaf(root)) {
      tile.leafNode = root;
      tile.firstChild = (uint32_t)ti;
      out.tiles.push_back(tile);
      continue;
    }
    bool byHits = out.byProfile;
    if (byHits && tiling == 2 && (double)(*hits)[root] / (double)(*hits)[0] < 0.20) byHits = false; // hybrid
    int32_t members[kMaxTileSize];
    const int n = byHits ? GatherByHits(tree, *hits, root, T, members) : GatherUniform(tree, root, T, members);
    // level order inside the tile: by depth, then left to right (position in an in-order walk of the tile)
    std::vector<int32_t> inorder;
    {
      // in-order walk restricted to the members
      std::vector<std::pair<int32_t, int>> stack{{root, 0}};
      while (!stack.empty()) {
        auto [node, state] = stack.back();
        stack.pop_back();
        const bool member = std::find(members, members + n, node) != members + n;
        if (!member) continue;
        if (state == 0) {
          stack.push_back({node, 1});
          stack.push_back({tree.left[node], 0});
        } else {
          inorder.push_back(node);
          stack.push_back({tree.right[node], 0});
        }
      }
    }
    std::vector<int32_t> ordered(members, members + n);
    std::stable_sort(ordered.begin(), ordered.end(), [&](int32_t a, int32_t b) {
      if (nodeDepth[a] != nodeDepth[b]) return nodeDepth[a] < nodeDepth[b];
      return std::find(inorder.begin(), inorder.end(), a) < std::find(inorder.begin(), inorder.end(), b);
    });
    tile.count = n;
    std::copy(ordered.begin(), ordered.end(), tile.members);
    // tile-local children (slot or -(exit number) - 1), exits numbered left to right
    int32_t leftSlot[kMaxTileSize], rightSlot[kMaxTileSize];
    auto slotOf = [&](int32_t node) {
      for (int i = 0; i < n; ++i)
        if (tile.members[i] == node) return i;
      return -1;
    };
    {
      std::vector<std::pair<int, int>> stack{{0, 0}};
      while (!stack.empty()) {
        auto [slot, state] = stack.back();
        stack.pop_back();
        const int32_t node = tile.members[slot];
        if (state == 0) {
          stack.push_back({slot, 1});
          const int child = slotOf(tree.left[node]);
          if (child >= 0) {
            leftSlot[slot] = child;
            stack.push_back({child, 0});
          } else {
            leftSlot[slot] = -(tile.numExits) - 1;
            tile.exits[tile.numExits++] = tree.left[node];
          }
        } else {
          const int child = slotOf(tree.right[node]);
          if (child >= 0) {
            rightSlot[slot] = child;
            stack.push_back({child, 0});
          } else {
            rightSlot[slot] = -(tile.numExits) - 1;
            tile.exits[tile.numExits++] = tree.right[node];
          }
        }
      }
    }
    if (T <= kMaxSelectTile) {
      // the tile's row of the child look-up table: outcome bit i set = node i sends the row left
      const uint32_t width = TileSelectBits(T);
      for (uint32_t outcome = 0; outcome < (1u << T); ++outcome) {
        int slot = 0;
        for (;;) {
          const int32_t next = ((outcome >> slot) & 1u) ? leftSlot[slot] : rightSlot[slot];
          if (next < 0) {
            tile.select |= (uint64_t)(-next - 1) << (outcome * width);
            break;
          }
          slot = next;
        }
      }
    } else {
      // the tile's shape itself: per slot where a row goes when the slot's predicate holds (left) and when not
      auto link = [](int32_t next) -> uint64_t { return next < 0 ? kTileLinkExit + (uint64_t)(-next - 1) : (uint64_t)(next - 1); };
      tile.links = 0;
      for (int slot = 0; slot < kMaxTileSize; ++slot) {
        const uint64_t left = slot < n ? link(leftSlot[slot]) : kTileLinkExit, right = slot < n ? link(rightSlot[slot]) : kTileLinkExit;
        tile.links |= (right << (4 * slot)) | (left << (32 + 4 * slot));
      }
      for (int i = 0; i < n; ++i) tile.hops = std::max(tile.hops, nodeDepth[tile.members[i]] - nodeDepth[tile.members[0]] + 1);
      out.hops = std::max(out.hops, tile.hops);
    }
    tile.firstChild = (uint32_t)roots.size();
    for (int e = 0; e < tile.numExits; ++e) roots.push_back(tile.exits[e]);
    out.tiles.push_back(tile);
  }
  // levels top down (children follow their parent in tile order), depths bottom up
  for (size_t ti = 0; ti < out.tiles.size(); ++ti)
    for (int e = 0; e < out.tiles[ti].numExits; ++e)
      out.tiles[out.tiles[ti].firstChild + e].level = out.tiles[ti].level + 1;
  for (size_t ti = out.tiles.size(); ti-- > 0;) {
    TileInfo &tile = out.tiles[ti];
    for (int e = 0; e < tile.numExits; ++e) tile.depth = std::max(tile.depth, 1 + out.tiles[tile.firstChild + e].depth);
  }
  out.depth = out.tiles[0].depth;
  return out;
}

// Bytes of one tile (see device_model.h) for a tree whose tile 0 sits at byte address `treeBase` of its group.
void EmitTile(const Tree &tree, const TileInfo &tile, int T, uint32_t treeBase, size_t tileIndex, uint32_t featureStride,
              uint32_t padOffset, unsigned char *dst) {
  const uint32_t bytes = TileBytes(T);
  float thr[kMaxTileSize] = {};
  uint16_t off[kMaxTileSize];
  for (int i = 0; i < kMaxTileSize; ++i) off[i] = (uint16_t)padOffset;
  if (tile.count == 0) {
    thr[0] = tree.value[tile.leafNode];
  } else {
    for (int i = 0; i < tile.count; ++i) {
      thr[i] = tree.value[tile.members[i]];
      off[i] = (uint16_t)((uint32_t)tree.feature[tile.members[i]] * featureStride);
    }
  }
  const uint32_t childAddress = treeBase + tile.firstChild * bytes;
  if (childAddress + (uint32_t)std::max(tile.numExits, 1) * bytes > 0x10000u) throw Error("internal error: tile address beyond the group");
  const uint16_t childBase = (uint16_t)childAddress;
  std::memset(dst, 0, bytes);
  if (T > kMaxSelectTile) { // eight slots whatever the tile size: { thr[8]; off[8]; links; childBase }
    std::memcpy(dst, thr, 32);
    std::memcpy(dst + 32, off, 16);
    std::memcpy(dst + 48, &tile.links, 8);
    std::memcpy(dst + 56, &childBase, 2);
    return;
  }
  std::memcpy(dst, thr, (size_t)T * 4);
  std::memcpy(dst + T * 4, off, (size_t)T * 2);
  std::memcpy(dst + T * 6, &childBase, 2);
  if (T == 4) {
    const uint16_t low = (uint16_t)(tile.select & 0xFFFFu);
    const uint32_t high = (uint32_t)(tile.select >> 16);
    std::memcpy(dst + 26, &low, 2);
    std::memcpy(dst + 28, &high, 4);
  } else {
    const uint16_t select = (uint16_t)tile.select;
    std::memcpy(dst + T * 6 + 2, &select, 2);
  }
  (void)tileIndex;
}

// Steps after which 90 % of the profiled rows of a tree have reached their leaf
// (src/utils/TreeTilingUtils.cpp:1722-1743); `leafLevel[i]` is the step count of leaf i, -1 for other nodes.
int32_t PeelDepth(const std::vector<int64_t> &hits, const std::vector<int32_t> &leafLevel, int32_t depth) {
  if (hits.empty() || hits[0] <= 0) return depth;
  for (int32_t d = 0; d <= depth; ++d) {
    int64_t covered = 0;
    for (size_t i = 0; i < leafLevel.size(); ++i)
      if (leafLevel[i] >= 0 && leafLevel[i] <= d) covered += hits[i];
    if ((double)covered / (double)hits[0] >= 0.9) return d;
  }
  return depth;
}

} // namespace

int64_t BiggestTiledTreeBytes(const Forest &forest, int tileSize) {
  if (tileSize < 2 || tileSize > kMaxTileSize) throw Error("internal error: tile size out of range");
  size_t most = 0;
  for (const Tree &tree : forest.trees) most = std::max(most, TileTree(tree, tileSize, 0, nullptr).tiles.size());
  return (int64_t)most * TileBytes(tileSize);
}

namespace {

// Global-memory layout: every tree breadth first (siblings adjacent), absolute node indices.
PackedModel PackForGlobalWalk(const Forest &forest, const LaunchPlan &plan) {
  if (plan.rowsPerBlock < 64 || plan.rowsPerBlock > 1024 || plan.rowsPerBlock % 64 != 0)
    throw Error("the global-memory walk needs a block of 64..1024 lanes");
  PackedModel pm;
  pm.plan = plan;
  pm.numFeatures = forest.numFeatures;
  pm.numClasses = forest.numClasses;
  pm.numTrees = (int32_t)forest.trees.size();
  std::vector<int32_t> depth(forest.trees.size());
  for (size_t t = 0; t < forest.trees.size(); ++t) depth[t] = forest.trees[t].Depth();
  std::vector<int32_t> order(forest.trees.size());
  std::iota(order.begin(), order.end(), 0);
  std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) {
    const int32_t ca = forest.numClasses > 0 ? forest.trees[a].classId : 0;
    const int32_t cb = forest.numClasses > 0 ? forest.trees[b].classId : 0;
    if (ca != cb) return ca < cb;
    return depth[a] < depth[b];
  });
  if (forest.NumNodes() > 0x7FFFFFF0u) throw Error("forest has too many nodes");
  for (int32_t t : order) {
    const Tree &tree = forest.trees[t];
    const LevelOrder lo = MakeLevelOrder(tree);
    const uint32_t base = (uint32_t)pm.globalNodes.size();
    pm.globalTrees.push_back(DeviceGlobalTree{base, (uint32_t)depth[t],
                                              (uint32_t)(forest.numClasses > 0 ? tree.classId : 0), t});
    for (size_t i = 0; i < lo.order.size(); ++i) {
      const int32_t n = lo.order[i];
      DeviceGlobalNode dn;
      dn.value = tree.value[n];
      dn.origin = n;
      if (tree.IsLeaf(n)) {
        dn.feature = kGlobalLeaf;
        dn.left = base + (uint32_t)i;
      } else {
        dn.feature = (uint32_t)tree.feature[n];
        dn.left = base + (uint32_t)lo.position[tree.left[n]];
      }
      pm.globalNodes.push_back(dn);
    }
  }
  return pm;
}

} // namespace

PackedModel PackForest(const Forest &input, const LaunchPlan &plan, const HitCountProfile *profile) {
  // Plans also come out of files: every field is brought into its range before anything is computed from it.
  if (plan.kernel != LaunchPlan::Kernel::kRowParallelLds && plan.kernel != LaunchPlan::Kernel::kTreeParallel &&
      plan.kernel != LaunchPlan::Kernel::kGlobalWalk)
    throw Error("launch plan names no kernel");
  if (plan.rowsPerBlock < 1 || plan.rowsPerBlock > 1024 || plan.treeThreads < 1 || plan.treeThreads > 1024 || plan.treeLanes < 1 ||
      plan.treeLanes > 1024)
    throw Error("launch plan: rows per block, tree threads and tree lanes must be in [1, 1024]");
  if (plan.treeSlices < 1 || plan.treeSlices > 65535) throw Error("launch plan: tree slices must be in [1, 65535]");
  if (plan.tiling < 0 || plan.tiling > 2) throw Error("launch plan: tiling type must be 0, 1 or 2");
  const Forest forest = NormalizeToLessThan(input);
  if (profile && profile->hits.size() != forest.trees.size()) throw Error("hit-count profile does not match the forest");
  if (plan.kernel == LaunchPlan::Kernel::kGlobalWalk) {
    if (plan.tileSize > 1) throw Error("tile sizes above 1 need the row-parallel LDS kernel; this forest has a tree too big for LDS");
    return PackForGlobalWalk(forest, plan);
  }
  const int K = plan.interleave;
  if (K < 1 || K > kMaxInterleave || (K & (K - 1))) throw Error("interleave must be 1, 2, 4 or 8");
  if (plan.kernel == LaunchPlan::Kernel::kRowParallelLds) {
    if (plan.rowsPerBlock < 64 || (plan.rowsPerBlock & (plan.rowsPerBlock - 1)) || plan.rowsPerBlock > 1024)
      throw Error("rowsPerBlock must be a power of two in [64, 1024]");
    if (plan.treeThreads < 1 || plan.ThreadsPerBlock() > 1024)
      throw Error("rowsPerBlock * treeThreads must not exceed 1024 lanes");
  } else {
    if (plan.treeLanes < 1 || (plan.treeLanes & (plan.treeLanes - 1)) || plan.rowsPerBlock < 1 ||
        plan.ThreadsPerBlock() > 1024 || plan.ThreadsPerBlock() % 64 != 0)
      throw Error("tree-parallel plan needs a power-of-two treeLanes and a block of 64..1024 lanes");
    if (plan.treeLanes < 64 && 64 % plan.treeLanes != 0) throw Error("treeLanes must divide 64");
  }
  if (plan.groupBytes > 256 * plan.ThreadsPerBlock())
    throw Error("groupBytes must not exceed 256 bytes per lane of the block (group prefetch registers)");
  if (plan.groupBytes < 1024 || plan.groupBytes > 65536) throw Error("groupBytes must be in [1024, 65536]");

  if (plan.quantizedRows && (plan.kernel != LaunchPlan::Kernel::kRowParallelLds || plan.rowsPerBlock != 64))
    throw Error("rank-quantised rows need the row-parallel kernel with 64 rows per block");
  if (plan.rankRows16 && (plan.kernel != LaunchPlan::Kernel::kRowParallelLds || plan.quantizedRows || plan.featureOffsetInWords))
    throw Error("two-byte rank rows need the row-parallel kernel (and exclude one-byte ranks and word offsets)");
  const int T = plan.tileSize;
  if (T < 1 || T > kMaxTileSize)
    throw Error("tile size " + std::to_string(T) + " is not supported: the device kernels walk tiles of 1 to " +
                std::to_string(kMaxTileSize) + " nodes");
  if (plan.deferTails && (plan.kernel != LaunchPlan::Kernel::kRowParallelLds || T != 1 || plan.quantizedRows || plan.rankRows16 ||
                          plan.featureOffsetInWords || forest.numClasses > 0 || !profile))
    throw Error("deferred tails need a profile and the scalar row-parallel kernel on float32 rows of a model without classes");
  if (T > 1 && (plan.kernel != LaunchPlan::Kernel::kRowParallelLds || plan.quantizedRows || plan.rankRows16))
    throw Error("tile sizes above 1 need the row-parallel kernel on float32 rows");
  if (T > 1 && (plan.featureOffsetInWords || (int64_t)(forest.numFeatures + 1) * plan.rowsPerBlock * 4 > 0x10000))
    throw Error("tile sizes above 1 need a row tile below 64 KB (tiles hold byte offsets): fewer rows per block");

  PackedModel pm;
  pm.plan = plan;
  pm.numFeatures = forest.numFeatures;
  pm.numClasses = forest.numClasses;
  pm.numTrees = (int32_t)forest.trees.size();
  if (plan.deferTails) { // tail node 0: a leaf of value 0, what a lane without a queue entry walks
    pm.tailNodes.push_back(DeviceNode{0.0f, (0u << kTailFeatureBits) | (uint32_t)forest.numFeatures});
    pm.tailOrigin.push_back(-1);
  }
  const uint64_t padOffset = pm.PadFeatureOffset();
  if (padOffset > 0xFFFFu)
    throw Error("feature offsets do not fit 16 bits for this rowsPerBlock / feature count");
  const uint32_t featureStride = plan.FeatureStride();
  if (plan.rankRows16 && pm.RowTileBytes() > 0x10000u) throw Error("two-byte rank rows: the row tile must stay below 64 KB (byte offsets)");
  const uint32_t groupCapacity = (uint32_t)plan.groupBytes / kNodeBytes; // in 8-byte units
  const uint32_t tileUnits = TileBytes(T) / kNodeBytes;                    // units per tile (1 for scalar nodes)

  // Rank quantisation: x < t_j  <=>  #{t : t <= x} <= j for the sorted distinct thresholds t_0 < t_1 < ...
  // of the feature, so an internal node stores j and the kernel compares the row's one-byte rank with it.
  std::vector<std::vector<float>> ranks;
  if (plan.quantizedRows) {
    ranks = ThresholdsPerFeature(forest);
    size_t most = 0;
    for (auto &v : ranks) most = std::max(most, v.size());
    if (most > 254) throw Error("a feature has more than 254 distinct thresholds: rows cannot be rank-quantised to bytes");
    int32_t depth = 1;
    while ((size_t)depth < most) depth = depth * 2 + 1; // 2^n - 1 >= most
    pm.binTableDepth = depth;
    // features per block of the binning kernel: one per lane of a wave
    const int32_t chunk = 64;
    pm.binChunkFeatures = chunk;
    const int32_t chunks = (forest.numFeatures + chunk - 1) / chunk;
    pm.binThresholds.assign((size_t)chunks * depth * chunk, std::numeric_limits<float>::infinity());
    for (int32_t f = 0; f < forest.numFeatures; ++f)
      for (size_t k = 0; k < ranks[f].size(); ++k)
        pm.binThresholds[((size_t)(f / chunk) * depth + k) * chunk + (f % chunk)] = ranks[f][k];
  }

  if (plan.rankRows16) {
    ranks = ThresholdsPerFeature(forest);
    // LDS of one block of the ranking kernel: the chunk's tables and a staging tile of 1025 floats per feature of
    // the chunk (two blocks per compute unit)
    constexpr size_t kChunkBytes = 76 * 1024, kStageBytesPerFeature = 1025 * 4;
    pm.rankFeatures.resize((size_t)((forest.numFeatures + 2) / 2) * 2); // every slot of the tile, the pad feature's included
    auto tableEntries = [&](size_t f) -> size_t {
      if (f >= ranks.size() || ranks[f].empty()) return 0;
      size_t entries = 1;
      while (entries < ranks[f].size()) entries = entries * 2 + 1; // 2^n - 1 >= thresholds
      return entries;
    };
    for (size_t f = 0; f < ranks.size(); ++f)
      if (ranks[f].size() > 65534) throw Error("a feature has more than 65534 distinct thresholds: rows cannot be ranked in two bytes");
    size_t f = 0;
    while (f < pm.rankFeatures.size()) {
      RankChunkDesc chunk{(uint32_t)f, 0, (uint32_t)pm.rankTables.size(), 0};
      size_t entries = 0;
      while (f < pm.rankFeatures.size()) {
        const size_t pairEntries = tableEntries(f) + tableEntries(f + 1);
        if (pairEntries * 4 + 2 * kStageBytesPerFeature > 150 * 1024) throw Error("the thresholds of one feature pair do not fit the ranking kernel's LDS");
        if (chunk.numFeatures > 0 && (entries + pairEntries) * 4 + (chunk.numFeatures + 2) * kStageBytesPerFeature > kChunkBytes) break;
        for (size_t g = f; g < f + 2; ++g) {
          const size_t n = tableEntries(g);
          uint32_t levels = 0;
          while (((size_t)1 << levels) - 1 < n) ++levels;
          pm.rankFeatures[g] = RankFeatureDesc{(uint32_t)entries, levels};
          // breadth-first order of the complete search tree over the sorted thresholds (+inf beyond the last)
          std::vector<float> bfs(n, std::numeric_limits<float>::infinity());
          std::function<void(size_t, size_t, size_t)> fill = [&](size_t node, size_t lo, size_t hi) { // keys [lo, hi)
            if (node >= n) return;
            const size_t mid = lo + (hi - lo) / 2;
            if (mid < ranks[g].size()) bfs[node] = ranks[g][mid];
            fill(2 * node + 1, lo, mid);
            fill(2 * node + 2, mid + 1, hi);
          };
          fill(0, 0, n);
          pm.rankTables.insert(pm.rankTables.end(), bfs.begin(), bfs.end());
          entries += n;
        }
        chunk.numFeatures += 2;
        f += 2;
      }
      chunk.tableEntries = (uint32_t)entries;
      pm.rankChunks.push_back(chunk);
    }
    pm.rankThresholds = ranks;
  }

  // Per tree: its size in the packed layout, the steps of a lock-step walk, and the steps after which the walk
  // starts looking whether any lane still moves (walk peeling; equal to the depth when there is no tail).
  const size_t numTrees = forest.trees.size();
  std::vector<TiledTree> tiled(T > 1 ? numTrees : 0);
  std::vector<int32_t> depth(numTrees), peel(numTrees);
  std::vector<int32_t> fullDepth(numTrees, 0); // deferred tails: the tree's own depth (depth[] is then where its walk stops)
  int64_t tailBudget = plan.deferTails && forest.numFeatures + 1 < (1 << kTailFeatureBits) ? (int64_t)kMaxTailNodes - 1 : 0;
  std::vector<uint32_t> units(numTrees);
  for (size_t t = 0; t < numTrees; ++t) {
    const Tree &tree = forest.trees[t];
    const std::vector<int64_t> *hits = profile ? &profile->hits[t] : nullptr;
    std::vector<int32_t> leafLevel(tree.NumNodes(), -1);
    std::vector<int32_t> nodeLevel; // scalar nodes: the level of every node
    if (T > 1) {
      tiled[t] = TileTree(tree, T, plan.tiling, hits);
      depth[t] = tiled[t].depth;
      units[t] = (uint32_t)tiled[t].tiles.size() * tileUnits;
      pm.treesTiledByProfile += tiled[t].byProfile ? 1 : 0;
      pm.maxTileHops = std::max(pm.maxTileHops, tiled[t].hops);
      for (const TileInfo &tile : tiled[t].tiles)
        if (tile.count == 0) leafLevel[tile.leafNode] = tile.level;
    } else {
      depth[t] = tree.Depth();
      units[t] = (uint32_t)tree.NumNodes();
      std::vector<int32_t> stack{0};
      leafLevel[0] = 0;
      while (!stack.empty()) { // (the level of every node; only the leaves' entries are used)
        const int32_t n = stack.back();
        stack.pop_back();
        if (tree.IsLeaf(n)) continue;
        leafLevel[tree.left[n]] = leafLevel[tree.right[n]] = leafLevel[n] + 1;
        stack.push_back(tree.left[n]);
        stack.push_back(tree.right[n]);
      }
      nodeLevel = leafLevel;
      for (size_t i = 0; i < tree.NumNodes(); ++i)
        if (!tree.IsLeaf((int32_t)i)) leafLevel[i] = -1;
    }
    peel[t] = plan.peelWalks && hits ? PeelDepth(*hits, leafLevel, depth[t]) : depth[t];
    fullDepth[t] = depth[t];
    if (plan.deferTails) {
      // Where the lock-step walk of this tree stops.  Costs in cycles of a compute unit per 64 rows: a lock-step
      // level is a node read (2.5 cycles while the level has at most 32 nodes, 4.3 for 64, 6.0 beyond) and a
      // feature read (2.4), as measured on MI355X; a deferred walk costs 20 to queue, fetch and hand back plus 20
      // per step down to the deepest leaf below the stub (a wave of 64 queue entries runs to the deepest of them),
      // and the stub test costs every row of the tree 2: the values that, of those tried (6 to 150 per step), gave
      // the shortest kernel times on two models of 1000 and 800 trees.
      std::vector<double> alive((size_t)depth[t] + 1, 0.0);
      {
        std::vector<std::pair<int32_t, int32_t>> stack{{0, 0}};
        while (!stack.empty()) {
          auto [n, level] = stack.back();
          stack.pop_back();
          if (tree.IsLeaf(n)) continue;
          alive[(size_t)level] += (*hits)[0] > 0 ? (double)(*hits)[n] / (double)(*hits)[0] : 1.0;
          stack.push_back({tree.left[n], level + 1});
          stack.push_back({tree.right[n], level + 1});
        }
      }
      auto levelCost = [](int32_t d) { return (d <= 5 ? 2.5 : d == 6 ? 4.3 : 6.0) + 2.4; };
      double whole = 0.0;
      for (int32_t d = 0; d < depth[t]; ++d) whole += levelCost(d);
      double best = whole, head = 0.0;
      int32_t cut = depth[t];
      for (int32_t d = 1; d < depth[t]; ++d) {
        head += levelCost(d - 1);
        const double cost = head + 2.0 + alive[(size_t)d] * ((depth[t] - d) * 20.0 + 20.0);
        if (cost < best && cost < 0.92 * whole) best = cost, cut = d;
      }
      bool nanLeaf = false; // (a NaN is what marks a stub)
      for (size_t i = 0; i < tree.NumNodes(); ++i) nanLeaf = nanLeaf || (tree.IsLeaf((int32_t)i) && tree.value[i] != tree.value[i]);
      if (cut < depth[t] && tailBudget > 0 && !nanLeaf) {
        uint32_t above = 0;
        for (size_t i = 0; i < tree.NumNodes(); ++i)
          if (nodeLevel[i] <= cut) ++above; // the top of the tree, the cut level's internal nodes as stubs
        tailBudget -= (int64_t)(tree.NumNodes() - above) + 64;
        units[t] = above;
        depth[t] = cut;
        peel[t] = cut;
        pm.treesDeferred += 1;
        pm.deferredEntriesPerRow += alive[(size_t)cut];
      }
    }
    pm.lockStepSteps += depth[t];
    if (hits && (*hits)[0] > 0) {
      double steps = 0.0;
      for (size_t i = 0; i < tree.NumNodes(); ++i)
        if (leafLevel[i] >= 0) steps += (double)(*hits)[i] * leafLevel[i];
      pm.profiledSteps += steps / (double)(*hits)[0];
    }
  }

  // Order: class, then depth (the reference sorts by depth for its GPU schedules,
  // src/mlir/GPUAutoSchedule.cpp:115-122); stable so equal keys keep model order.
  std::vector<int32_t> order(numTrees);
  std::iota(order.begin(), order.end(), 0);
  std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) {
    int32_t ca = forest.numClasses > 0 ? forest.trees[a].classId : 0;
    int32_t cb = forest.numClasses > 0 ? forest.trees[b].classId : 0;
    if (ca != cb) return ca < cb;
    if (depth[a] != depth[b]) return depth[a] < depth[b];
    return peel[a] < peel[b];
  });

  // The null leaf that padding trees of a bundle point at: a leaf of value 0 at address 0 of every group.
  auto pushNullLeaf = [&]() {
    if (T > 1) {
      Tree nullTree;
      nullTree.value = {0.0f};
      nullTree.feature = {0};
      nullTree.left = nullTree.right = {-1};
      TileInfo leaf;
      leaf.leafNode = 0;
      std::vector<unsigned char> bytes(TileBytes(T));
      EmitTile(nullTree, leaf, T, 0, 0, featureStride, (uint32_t)padOffset, bytes.data());
      for (uint32_t u = 0; u < tileUnits; ++u) {
        DeviceNode unit;
        std::memcpy(&unit, bytes.data() + u * kNodeBytes, kNodeBytes);
        pm.nodes.push_back(unit);
        pm.nodeOrigin.push_back(-1);
      }
    } else {
      pm.nodes.push_back(DeviceNode{0.0f, (0u << 16) | (uint32_t)padOffset});
      pm.nodeOrigin.push_back(-1);
    }
  };
  auto openGroup = [&]() {
    DeviceGroup g{};
    g.nodeBegin = (uint32_t)pm.nodes.size();
    g.bundleBegin = (uint32_t)pm.bundles.size();
    pm.groups.push_back(g);
    pushNullLeaf();
  };
  auto closeGroup = [&]() {
    DeviceGroup &g = pm.groups.back();
    if ((pm.nodes.size() - g.nodeBegin) & 1) { // whole 16-byte pieces
      pm.nodes.push_back(DeviceNode{0.0f, (0u << 16) | (uint32_t)padOffset});
      pm.nodeOrigin.push_back(-1);
    }
    g.nodeCount = (uint32_t)pm.nodes.size() - g.nodeBegin;
    g.bundleCount = (uint32_t)pm.bundles.size() - g.bundleBegin;
    g.uniformClass = 0;
    if (g.bundleCount > 0) {
      const uint32_t first = pm.bundles[g.bundleBegin].classId;
      bool uniform = true;
      for (uint32_t b = 1; b < g.bundleCount; ++b) uniform = uniform && pm.bundles[g.bundleBegin + b].classId == first;
      if (uniform) g.uniformClass = first + 1;
    }
    pm.maxGroupNodes = std::max(pm.maxGroupNodes, g.nodeCount);
  };
  // Writes tree t with its first unit at unit `base` of the current group.
  auto emitTree = [&](int32_t t, uint32_t base) {
    const Tree &tree = forest.trees[t];
    if (T > 1) {
      std::vector<unsigned char> bytes(TileBytes(T));
      for (size_t ti = 0; ti < tiled[t].tiles.size(); ++ti) {
        const TileInfo &tile = tiled[t].tiles[ti];
        EmitTile(tree, tile, T, base * kNodeBytes, ti, featureStride, (uint32_t)padOffset, bytes.data());
        for (uint32_t u = 0; u < tileUnits; ++u) {
          DeviceNode unit;
          std::memcpy(&unit, bytes.data() + u * kNodeBytes, kNodeBytes);
          pm.nodes.push_back(unit);
          pm.nodeOrigin.push_back(u == 0 ? (tile.count == 0 ? tile.leafNode : tile.members[0]) : -1);
        }
      }
      return;
    }
    if (plan.deferTails && depth[t] < fullDepth[t]) {
      // The walk of this tree stops at level depth[t]: the internal nodes of that level are represented by stubs
      // (a NaN whose payload is the index of the node itself in the tail array); their subtrees go to the tail
      // array in global memory, each in level order with siblings adjacent.
      const int32_t cut = depth[t];
      std::vector<int32_t> top, cutNodes, where(tree.NumNodes(), -1);
      {
        std::vector<std::pair<int32_t, int32_t>> queue{{0, 0}};
        for (size_t head = 0; head < queue.size(); ++head) {
          auto [n, level] = queue[head];
          where[n] = (int32_t)top.size();
          top.push_back(n);
          if (tree.IsLeaf(n)) continue;
          if (level == cut) { cutNodes.push_back(n); continue; }
          queue.push_back({tree.left[n], level + 1});
          queue.push_back({tree.right[n], level + 1});
        }
      }
      if (top.size() != units[t]) throw Error("internal error: deferred tree size out of step");
      std::vector<uint32_t> tailIndex(tree.NumNodes(), 0);
      for (int32_t first : cutNodes) {
        std::vector<int32_t> queue{first};
        for (size_t head = 0; head < queue.size(); ++head) {
          const int32_t n = queue[head];
          if (!tree.IsLeaf(n)) { queue.push_back(tree.left[n]); queue.push_back(tree.right[n]); }
        }
        const uint32_t begin = (uint32_t)pm.tailNodes.size();
        if ((size_t)begin + queue.size() > kMaxTailNodes) throw Error("internal error: tail array overflow");
        for (size_t i = 0; i < queue.size(); ++i) tailIndex[queue[i]] = begin + (uint32_t)i;
        for (int32_t n : queue) {
          DeviceNode dn;
          dn.value = tree.value[n];
          if (tree.IsLeaf(n)) {
            dn.meta = (tailIndex[n] << kTailFeatureBits) | (uint32_t)forest.numFeatures; // stays put: the pad feature holds -inf
          } else {
            if (tailIndex[tree.right[n]] != tailIndex[tree.left[n]] + 1) throw Error("internal error: siblings not adjacent");
            dn.meta = (tailIndex[tree.left[n]] << kTailFeatureBits) | (uint32_t)tree.feature[n];
          }
          pm.tailNodes.push_back(dn);
          pm.tailOrigin.push_back(n);
        }
      }
      for (size_t i = 0; i < top.size(); ++i) {
        const int32_t n = top[i];
        const uint32_t self = (base + (uint32_t)i) * kNodeBytes;
        DeviceNode dn;
        if (tree.IsLeaf(n)) {
          dn.value = tree.value[n];
          dn.meta = (self << 16) | (uint32_t)padOffset;
        } else if (tailIndex[n] != 0) { // a stub: NaN compares false, so the walk takes the "right" child: the stub itself
          const uint32_t bits = kStubValueBits | tailIndex[n];
          std::memcpy(&dn.value, &bits, sizeof(bits));
          dn.meta = ((self - kNodeBytes) << 16) | (uint32_t)padOffset;
        } else {
          dn.value = tree.value[n];
          if (where[tree.right[n]] != where[tree.left[n]] + 1) throw Error("internal error: siblings not adjacent");
          dn.meta = (((base + (uint32_t)where[tree.left[n]]) * kNodeBytes) << 16) | plan.FeatureOffset((uint32_t)tree.feature[n]);
        }
        pm.nodes.push_back(dn);
        pm.nodeOrigin.push_back(n);
      }
      pm.maxTailDepth = std::max<uint32_t>(pm.maxTailDepth, (uint32_t)(fullDepth[t] - cut));
      return;
    }
    const LevelOrder lo = MakeLevelOrder(tree);
    for (size_t i = 0; i < lo.order.size(); ++i) {
      const int32_t n = lo.order[i];
      DeviceNode dn;
      dn.value = tree.value[n];
      if ((plan.quantizedRows || plan.rankRows16) && !tree.IsLeaf(n)) {
        const auto &sorted = ranks[(size_t)tree.feature[n]];
        const uint32_t j = (uint32_t)(std::lower_bound(sorted.begin(), sorted.end(), tree.value[n]) - sorted.begin());
        static_assert(sizeof(float) == sizeof(uint32_t), "node value holds the rank bit pattern");
        std::memcpy(&dn.value, &j, sizeof(j));
      }
      if (tree.IsLeaf(n)) {
        dn.meta = (((base + (uint32_t)i) * kNodeBytes) << 16) | (uint32_t)padOffset;
      } else {
        const uint32_t child = base + (uint32_t)lo.position[tree.left[n]];
        if (lo.position[tree.right[n]] != lo.position[tree.left[n]] + 1)
          throw Error("internal error: siblings not adjacent");
        dn.meta = ((child * kNodeBytes) << 16) | plan.FeatureOffset((uint32_t)tree.feature[n]);
      }
      pm.nodes.push_back(dn);
      pm.nodeOrigin.push_back(n);
    }
  };

  size_t next = 0;
  while (next < order.size()) {
    openGroup();
    DeviceGroup &g = pm.groups.back();
    // one spare unit keeps room for the alignment pad
    auto freeNodes = [&]() { return groupCapacity - 1 - ((uint32_t)pm.nodes.size() - g.nodeBegin); };
    bool any = false;
    struct Mark { size_t nodes, slots, next, tail; };
    std::vector<Mark> marks; // state before each bundle of this group
    const size_t multiple = plan.kernel == LaunchPlan::Kernel::kRowParallelLds ? (size_t)plan.treeThreads : 1;
    while (next < order.size()) {
      // gather up to K consecutive trees of one class that still fit
      DeviceBundle b{};
      const int32_t cls = forest.numClasses > 0 ? forest.trees[order[next]].classId : 0;
      uint32_t need = 0;
      int count = 0;
      while (count < K && next + count < order.size()) {
        const int32_t t = order[next + count];
        const int32_t c = forest.numClasses > 0 ? forest.trees[t].classId : 0;
        if (c != cls) break;
        if (units[t] + 2 * tileUnits > groupCapacity)
          throw Error("a tree of " + std::to_string(forest.trees[t].NumNodes()) + " nodes does not fit one LDS tree group");
        if (need + units[t] > freeNodes()) break;
        need += units[t];
        ++count;
      }
      if (count == 0) break; // group full
      marks.push_back(Mark{pm.nodes.size(), pm.slotTree.size(), next, pm.tailNodes.size()});
      b.classId = (uint16_t)cls;
      b.firstSlot = (uint32_t)pm.slotTree.size();
      for (int k = 0; k < K; ++k) {
        if (k >= count) {
          b.root[k] = 0; // null leaf
          pm.slotTree.push_back(-1);
          continue;
        }
        const int32_t t = order[next + k];
        const uint32_t base = (uint32_t)pm.nodes.size() - g.nodeBegin; // unit index inside the group
        b.root[k] = (uint16_t)(base * kNodeBytes);
        b.depth = std::max<uint32_t>(b.depth, (uint32_t)depth[t]);
        b.peelDepth = std::max<uint32_t>(b.peelDepth, (uint32_t)peel[t]);
        if (plan.deferTails && depth[t] < fullDepth[t]) b.hasStubs = 1;
        pm.slotTree.push_back(t);
        emitTree(t, base);
      }
      for (int k = 0; k < K; ++k) pm.bundleRoots.push_back(pm.nodes[g.nodeBegin + b.root[k] / kNodeBytes]);
      pm.bundles.push_back(b);
      next += count;
      any = true;
    }
    // Tree threads take bundles round-robin: when more trees follow, end the group on a
    // multiple of treeThreads bundles so that no thread idles through a last partial round.
    if (next < order.size() && multiple > 1 && marks.size() > multiple && marks.size() % multiple != 0) {
      const size_t keep = marks.size() - marks.size() % multiple;
      pm.nodes.resize(marks[keep].nodes);
      pm.nodeOrigin.resize(marks[keep].nodes);
      pm.slotTree.resize(marks[keep].slots);
      pm.tailNodes.resize(marks[keep].tail);
      pm.tailOrigin.resize(marks[keep].tail);
      pm.bundles.resize(g.bundleBegin + keep);
      pm.bundleRoots.resize((size_t)(g.bundleBegin + keep) * K);
      next = marks[keep].next;
    }
    closeGroup();
    if (!any) throw Error("internal error: empty tree group");
  }
  if (pm.groups.empty()) { // a forest without trees still needs one (empty) group
    openGroup();
    closeGroup();
  }
  if (pm.bundleRoots.size() != pm.bundles.size() * (size_t)K) throw Error("internal error: bundle root table out of step");
  return pm;
}

Tree UnpackTree(const PackedModel &pm, int32_t treeIndex) {
  if (pm.plan.tileSize > 1) throw Error("tiled models are checked through their walks, not unpacked");
  if (pm.plan.kernel == LaunchPlan::Kernel::kGlobalWalk) {
    for (const DeviceGlobalTree &gt : pm.globalTrees) {
      if (gt.origin != treeIndex) continue;
      Tree tree;
      tree.classId = (int32_t)gt.classId;
      std::vector<uint32_t> queue{gt.root};
      size_t total = 0;
      for (size_t head = 0; head < queue.size(); ++head) {
        const DeviceGlobalNode &dn = pm.globalNodes[queue[head]];
        total = std::max<size_t>(total, (size_t)dn.origin + 1);
        if (dn.feature != kGlobalLeaf) { queue.push_back(dn.left); queue.push_back(dn.left + 1); }
      }
      tree.value.assign(total, 0.f);
      tree.feature.assign(total, 0);
      tree.left.assign(total, -1);
      tree.right.assign(total, -1);
      for (uint32_t q : queue) {
        const DeviceGlobalNode &dn = pm.globalNodes[q];
        tree.value[dn.origin] = dn.value;
        if (dn.feature != kGlobalLeaf) {
          tree.feature[dn.origin] = (int32_t)dn.feature;
          tree.left[dn.origin] = pm.globalNodes[dn.left].origin;
          tree.right[dn.origin] = pm.globalNodes[dn.left + 1].origin;
        }
      }
      return tree;
    }
    throw Error("tree not found in packed model");
  }
  const int K = pm.plan.interleave;
  for (const DeviceGroup &g : pm.groups)
    for (uint32_t bi = g.bundleBegin; bi < g.bundleBegin + g.bundleCount; ++bi)
      for (int k = 0; k < K; ++k) {
        if (pm.slotTree[pm.bundles[bi].firstSlot + k] != treeIndex) continue;
        // walk the packed tree breadth first, restoring original node ids (a stub stands for the node its value
        // field points at)
        // (units of the group's image; a stub stands for a node of the tail array, noted as kTailBit | index)
        constexpr uint32_t kTailBit = 0x80000000u;
        auto resolve = [&](uint32_t unit) {
          const DeviceNode &dn = pm.nodes[g.nodeBegin + unit];
          uint32_t bits;
          std::memcpy(&bits, &dn.value, sizeof(bits));
          const bool stub = pm.plan.deferTails && (dn.meta >> 16) / kNodeBytes + 1 == unit && (bits & ~kStubIndexMask) == kStubValueBits;
          if (!stub) return unit;
          return kTailBit | (bits & kStubIndexMask);
        };
        auto nodeAt = [&](uint32_t q) -> const DeviceNode & { return q & kTailBit ? pm.tailNodes[q & ~kTailBit] : pm.nodes[g.nodeBegin + q]; };
        auto originAt = [&](uint32_t q) { return q & kTailBit ? pm.tailOrigin[q & ~kTailBit] : pm.nodeOrigin[g.nodeBegin + q]; };
        auto leftOf = [&](uint32_t q) -> uint32_t { // the left child (same notation), or q itself on a leaf
          const DeviceNode &dn = nodeAt(q);
          if (q & kTailBit) return kTailBit | (dn.meta >> kTailFeatureBits);
          return resolve((dn.meta >> 16) / kNodeBytes);
        };
        auto rightOf = [&](uint32_t q) -> uint32_t {
          const DeviceNode &dn = nodeAt(q);
          if (q & kTailBit) return kTailBit | ((dn.meta >> kTailFeatureBits) + 1);
          return resolve((dn.meta >> 16) / kNodeBytes + 1);
        };
        auto isLeaf = [&](uint32_t q) {
          const DeviceNode &dn = nodeAt(q);
          return q & kTailBit ? (dn.meta >> kTailFeatureBits) == (q & ~kTailBit) : (dn.meta >> 16) / kNodeBytes == q;
        };
        auto featureOf = [&](uint32_t q) -> int32_t {
          const DeviceNode &dn = nodeAt(q);
          return q & kTailBit ? (int32_t)(dn.meta & ((1u << kTailFeatureBits) - 1u)) : (int32_t)pm.plan.FeatureOfOffset(dn.meta & 0xFFFFu);
        };
        Tree tree;
        tree.classId = pm.bundles[bi].classId;
        std::vector<uint32_t> queue{resolve(pm.bundles[bi].root[k] / kNodeBytes)};
        size_t total = 0;
        for (size_t head = 0; head < queue.size(); ++head) {
          total = std::max<size_t>(total, (size_t)originAt(queue[head]) + 1);
          if (!isLeaf(queue[head])) { queue.push_back(leftOf(queue[head])); queue.push_back(rightOf(queue[head])); }
        }
        tree.value.assign(total, 0.f);
        tree.feature.assign(total, 0);
        tree.left.assign(total, -1);
        tree.right.assign(total, -1);
        for (uint32_t q : queue) {
          const DeviceNode &dn = nodeAt(q);
          const int32_t me = originAt(q);
          tree.value[me] = dn.value;
          const bool leaf = isLeaf(q);
          if (!leaf && pm.plan.quantizedRows) { // rank -> threshold through the binning table
            uint32_t j;
            std::memcpy(&j, &dn.value, sizeof(j));
            const int32_t f = featureOf(q);
            const int32_t chunk = pm.binChunkFeatures;
            tree.value[me] = pm.binThresholds[((size_t)(f / chunk) * pm.binTableDepth + j) * chunk + (f % chunk)];
          }
          if (!leaf && pm.plan.rankRows16) {
            uint32_t j;
            std::memcpy(&j, &dn.value, sizeof(j));
            tree.value[me] = pm.rankThresholds.at((size_t)featureOf(q)).at(j);
          }
          if (!leaf) {
            tree.feature[me] = featureOf(q);
            tree.left[me] = originAt(leftOf(q));
            tree.right[me] = originAt(rightOf(q));
          }
        }
        return tree;
      }
  throw Error("tree not found in packed model");
}

} // namespace tbamd
