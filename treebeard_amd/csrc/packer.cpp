#include "packer.h"

#include <algorithm>
#include <cmath>
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

uint32_t PackedModel::PadFeatureOffset() const { return (uint32_t)numFeatures * plan.FeatureStride(); }

size_t PackedModel::RowTileBytes() const {
  return (size_t)(numFeatures + 1) * plan.rowsPerBlock * (plan.quantizedRows ? 1 : 4);
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

PackedModel PackForest(const Forest &input, const LaunchPlan &plan) {
  const Forest forest = NormalizeToLessThan(input);
  if (plan.kernel == LaunchPlan::Kernel::kGlobalWalk) return PackForGlobalWalk(forest, plan);
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

  PackedModel pm;
  pm.plan = plan;
  pm.numFeatures = forest.numFeatures;
  pm.numClasses = forest.numClasses;
  pm.numTrees = (int32_t)forest.trees.size();
  const uint64_t padOffset = pm.PadFeatureOffset();
  if (padOffset > 0xFFFFu)
    throw Error("feature offsets do not fit 16 bits for this rowsPerBlock / feature count");
  const uint32_t featureStride = plan.FeatureStride();
  const uint32_t groupCapacity = (uint32_t)plan.groupBytes / kNodeBytes;

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

  // Order: class, then depth (the reference sorts by depth for its GPU schedules,
  // src/mlir/GPUAutoSchedule.cpp:115-122); stable so equal keys keep model order.
  std::vector<int32_t> depth(forest.trees.size());
  for (size_t t = 0; t < forest.trees.size(); ++t) depth[t] = forest.trees[t].Depth();
  std::vector<int32_t> order(forest.trees.size());
  std::iota(order.begin(), order.end(), 0);
  std::stable_sort(order.begin(), order.end(), [&](int32_t a, int32_t b) {
    int32_t ca = forest.numClasses > 0 ? forest.trees[a].classId : 0;
    int32_t cb = forest.numClasses > 0 ? forest.trees[b].classId : 0;
    if (ca != cb) return ca < cb;
    return depth[a] < depth[b];
  });

  auto openGroup = [&]() {
    DeviceGroup g{};
    g.nodeBegin = (uint32_t)pm.nodes.size();
    g.bundleBegin = (uint32_t)pm.bundles.size();
    pm.groups.push_back(g);
    // node 0 of every group: the null leaf padding trees point at
    pm.nodes.push_back(DeviceNode{0.0f, (0u << 16) | (uint32_t)padOffset});
    pm.nodeOrigin.push_back(-1);
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

  size_t next = 0;
  while (next < order.size()) {
    openGroup();
    DeviceGroup &g = pm.groups.back();
    // one spare node keeps room for the alignment pad
    auto freeNodes = [&]() { return groupCapacity - 1 - ((uint32_t)pm.nodes.size() - g.nodeBegin); };
    bool any = false;
    struct Mark { size_t nodes, slots, next; };
    std::vector<Mark> marks; // state before each bundle of this group
    const size_t multiple = plan.kernel == LaunchPlan::Kernel::kRowParallelLds ? (size_t)plan.treeThreads : 1;
    while (next < order.size()) {
      // gather up to K consecutive trees of one class that still fit
      DeviceBundle b{};
      const int32_t cls = forest.numClasses > 0 ? forest.trees[order[next]].classId : 0;
      uint32_t need = 0;
      int count = 0;
      while (count < K && next + count < order.size()) {
        const Tree &tree = forest.trees[order[next + count]];
        const int32_t c = forest.numClasses > 0 ? tree.classId : 0;
        if (c != cls) break;
        if ((uint32_t)tree.NumNodes() + 2 > groupCapacity)
          throw Error("a tree of " + std::to_string(tree.NumNodes()) + " nodes does not fit one LDS tree group");
        if (need + tree.NumNodes() > freeNodes()) break;
        need += (uint32_t)tree.NumNodes();
        ++count;
      }
      if (count == 0) break; // group full
      marks.push_back(Mark{pm.nodes.size(), pm.slotTree.size(), next});
      b.classId = (uint32_t)cls;
      b.firstSlot = (uint32_t)pm.slotTree.size();
      for (int k = 0; k < K; ++k) {
        if (k >= count) {
          b.root[k] = 0; // null leaf
          pm.slotTree.push_back(-1);
          continue;
        }
        const int32_t t = order[next + k];
        const Tree &tree = forest.trees[t];
        const LevelOrder lo = MakeLevelOrder(tree);
        const uint32_t base = (uint32_t)pm.nodes.size() - g.nodeBegin; // node index inside the group
        b.root[k] = (uint16_t)(base * kNodeBytes);
        b.depth = std::max<uint32_t>(b.depth, (uint32_t)depth[t]);
        pm.slotTree.push_back(t);
        for (size_t i = 0; i < lo.order.size(); ++i) {
          const int32_t n = lo.order[i];
          DeviceNode dn;
          dn.value = tree.value[n];
          if (plan.quantizedRows && !tree.IsLeaf(n)) {
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
            dn.meta = ((child * kNodeBytes) << 16) | ((uint32_t)tree.feature[n] * featureStride);
          }
          pm.nodes.push_back(dn);
          pm.nodeOrigin.push_back(n);
        }
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
  const uint32_t featureStride = pm.plan.FeatureStride();
  for (const DeviceGroup &g : pm.groups)
    for (uint32_t bi = g.bundleBegin; bi < g.bundleBegin + g.bundleCount; ++bi)
      for (int k = 0; k < K; ++k) {
        if (pm.slotTree[pm.bundles[bi].firstSlot + k] != treeIndex) continue;
        // walk the packed tree breadth first, restoring original node ids
        Tree tree;
        tree.classId = pm.bundles[bi].classId;
        std::vector<uint32_t> queue{pm.bundles[bi].root[k] / kNodeBytes};
        size_t total = 0;
        for (size_t head = 0; head < queue.size(); ++head) {
          const DeviceNode &dn = pm.nodes[g.nodeBegin + queue[head]];
          total = std::max<size_t>(total, (size_t)pm.nodeOrigin[g.nodeBegin + queue[head]] + 1);
          const uint32_t child = (dn.meta >> 16) / kNodeBytes;
          if (child != queue[head]) { queue.push_back(child); queue.push_back(child + 1); }
        }
        tree.value.assign(total, 0.f);
        tree.feature.assign(total, 0);
        tree.left.assign(total, -1);
        tree.right.assign(total, -1);
        for (uint32_t q : queue) {
          const DeviceNode &dn = pm.nodes[g.nodeBegin + q];
          const int32_t me = pm.nodeOrigin[g.nodeBegin + q];
          const uint32_t child = (dn.meta >> 16) / kNodeBytes;
          tree.value[me] = dn.value;
          if (child != q && pm.plan.quantizedRows) { // rank -> threshold through the binning table
            uint32_t j;
            std::memcpy(&j, &dn.value, sizeof(j));
            const int32_t f = (int32_t)((dn.meta & 0xFFFFu) / featureStride);
            const int32_t chunk = pm.binChunkFeatures;
            tree.value[me] = pm.binThresholds[((size_t)(f / chunk) * pm.binTableDepth + j) * chunk + (f % chunk)];
          }
          if (child != q) {
            tree.feature[me] = (int32_t)((dn.meta & 0xFFFFu) / featureStride);
            tree.left[me] = pm.nodeOrigin[g.nodeBegin + child];
            tree.right[me] = pm.nodeOrigin[g.nodeBegin + child + 1];
          }
        }
        return tree;
      }
  throw Error("tree not found in packed model");
}

} // namespace tbamd
