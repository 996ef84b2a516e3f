#include "forest.h"

#include <cmath>

namespace tbamd {

int32_t Tree::Depth() const {
  if (value.empty()) return 0;
  int32_t best = 0;
  std::vector<std::pair<int32_t, int32_t>> stack{{0, 0}};
  while (!stack.empty()) {
    auto [n, d] = stack.back();
    stack.pop_back();
    if (IsLeaf(n)) {
      if (d > best) best = d;
      continue;
    }
    stack.push_back({left[n], d + 1});
    stack.push_back({right[n], d + 1});
  }
  return best;
}

void Tree::Validate(int32_t numFeatures, size_t treeIndex) const {
  const int32_t n = (int32_t)NumNodes();
  auto fail = [&](const std::string &what) {
    throw Error("tree " + std::to_string(treeIndex) + ": " + what);
  };
  if (n == 0) fail("has no nodes");
  if ((int32_t)feature.size() != n || (int32_t)left.size() != n || (int32_t)right.size() != n)
    fail("node arrays differ in length");
  std::vector<uint8_t> seen(n, 0);
  std::vector<int32_t> stack{0};
  int32_t visited = 0;
  while (!stack.empty()) {
    int32_t i = stack.back();
    stack.pop_back();
    if (i < 0 || i >= n) fail("child index out of range");
    if (seen[i]) fail("node reachable twice (not a tree)");
    seen[i] = 1;
    ++visited;
    if (IsLeaf(i)) {
      if (!std::isfinite(value[i])) fail("non-finite leaf value");
      continue;
    }
    if (left[i] == -1 || right[i] == -1) fail("internal node with a single child");
    if (feature[i] < 0 || feature[i] >= numFeatures) fail("feature index out of range");
    if (std::isnan(value[i])) fail("NaN threshold");
    stack.push_back(left[i]);
    stack.push_back(right[i]);
  }
  (void)visited;
}

void Forest::Validate() const {
  if (numFeatures <= 0) throw Error("model has no features");
  if (numClasses < 0 || numClasses > 127) throw Error("unsupported number of classes");
  for (size_t t = 0; t < trees.size(); ++t) {
    trees[t].Validate(numFeatures, t);
    if (numClasses > 0 && (trees[t].classId < 0 || trees[t].classId >= numClasses))
      throw Error("tree " + std::to_string(t) + ": class id out of range");
  }
}

} // namespace tbamd
