// In-memory decision forest shared by the loaders, the packer and the runner.
//
// Mirrors the role of the reference's DecisionForest / DecisionTree
// (src/include/DecisionForest.h:30-263) with f32 thresholds, which is what the
// reference's default CompilerOptions instantiate
// (src/include/TreebeardContext.h:73-80).
#pragma once

#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

namespace tbamd {

enum class Transform : int32_t { kIdentity = 0, kSigmoid = 1, kSoftMax = 2 };
// Which comparison sends a row to the LEFT (true) child.
enum class Predicate : int32_t { kLT = 0, kGE = 1, kGT = 2, kLE = 3 };

struct Error : std::runtime_error {
  using std::runtime_error::runtime_error;
};

struct Tree {
  // value[i] is the split threshold of an internal node or the prediction of a
  // leaf (the reference keeps leaf values in the threshold field too,
  // src/json/xgboostparser.h:205).
  std::vector<float> value;
  std::vector<int32_t> feature;
  std::vector<int32_t> left, right; // local node index, -1 when absent
  int32_t classId = 0;

  size_t NumNodes() const { return value.size(); }
  bool IsLeaf(int32_t n) const { return left[n] == -1 && right[n] == -1; }
  // Number of internal nodes on the longest root-to-leaf path.
  int32_t Depth() const;
  void Validate(int32_t numFeatures, size_t treeIndex) const;
};

struct Forest {
  int32_t numFeatures = 0;
  double initialValue = 0.0;
  Transform transform = Transform::kIdentity;
  int32_t numClasses = 0; // 0: regression / binary
  Predicate predicate = Predicate::kLT;
  std::vector<Tree> trees;

  size_t NumNodes() const {
    size_t n = 0;
    for (auto &t : trees) n += t.NumNodes();
    return n;
  }
  void Validate() const;
};

// Leaf hit counts of a profiling run (the reference's probability profile, src/utils/StatsUtils.cpp:10-52),
// with the counts of the internal nodes filled in from their subtrees.
struct HitCountProfile {
  int64_t numRows = 0;
  std::vector<std::vector<int64_t>> hits; // per tree, per node
};

// src/json/xgboostparser.h:117-219
Forest LoadXGBoostJSON(const std::string &path);
// src/json/onnxmodelparser.h:50-374; numFeatures comes from CompilerOptions.
Forest LoadONNX(const std::string &path, int32_t numFeatures);

} // namespace tbamd
