// C driver around the reference's own header-only forest model
// (src/include/DecisionForest.h) so that its scalar walker can be called from
// the tests.  TEST INFRASTRUCTURE ONLY.  Compiled by oracle/Makefile straight
// from the reference checkout where it lies (-I<reference>/src/include); no
// reference source is copied here and the output goes to oracle/_ref/ only.
#include "DecisionForest.h"

#include <cstdint>
#include <vector>

using mlir::decisionforest::DecisionForest;
using mlir::decisionforest::PredictionTransformation;

namespace {
struct Handle {
  DecisionForest forest;
};
} // namespace

extern "C" {

void *tbref_create(double initialValue, int32_t transform, int32_t numClasses) {
  auto *h = new Handle{DecisionForest(initialValue)};
  h->forest.SetPredictionTransformation(
      transform == 0   ? PredictionTransformation::kIdentity
      : transform == 1 ? PredictionTransformation::kSigmoid
                       : PredictionTransformation::kSoftMax);
  h->forest.SetNumClasses(numClasses);
  return h;
}

void tbref_destroy(void *hv) { delete static_cast<Handle *>(hv); }

// Same call sequence as XGBoostJSONParser::ConstructSingleTree
// (src/json/xgboostparser.h:199-218): NewNode for every node, then links.
void tbref_add_tree(void *hv, int32_t n, const double *thr, const int32_t *feat,
                    const int32_t *left, const int32_t *right, int32_t classId) {
  auto &forest = static_cast<Handle *>(hv)->forest;
  auto &tree = forest.NewTree();
  std::vector<int64_t> ids;
  for (int32_t i = 0; i < n; ++i)
    ids.push_back(tree.NewNode(thr[i], feat[i]));
  tree.SetNodeParent(ids[0], -1);
  for (int32_t i = 0; i < n; ++i) {
    if (left[i] != -1) {
      tree.SetNodeLeftChild(ids[i], ids[left[i]]);
      tree.SetNodeParent(ids[left[i]], ids[i]);
    }
    if (right[i] != -1) {
      tree.SetNodeRightChild(ids[i], ids[right[i]]);
      tree.SetNodeParent(ids[right[i]], ids[i]);
    }
  }
  tree.SetClassId(classId);
  forest.EndTree();
}

void tbref_predict_float(void *hv, const float *x, int64_t rows, int32_t F, float *out) {
  auto &forest = static_cast<Handle *>(hv)->forest;
  std::vector<float> row(F);
  for (int64_t r = 0; r < rows; ++r) {
    row.assign(x + r * F, x + (r + 1) * F);
    out[r] = forest.Predict_Float(row);
  }
}

void tbref_predict_double(void *hv, const double *x, int64_t rows, int32_t F, double *out) {
  auto &forest = static_cast<Handle *>(hv)->forest;
  std::vector<double> row(F);
  for (int64_t r = 0; r < rows; ++r) {
    row.assign(x + r * F, x + (r + 1) * F);
    out[r] = forest.Predict(row);
  }
}

void tbref_tree_values_float(void *hv, const float *x, int64_t rows, int32_t F, float *out) {
  auto &forest = static_cast<Handle *>(hv)->forest;
  const int64_t T = forest.NumTrees();
  std::vector<float> row(F);
  for (int64_t r = 0; r < rows; ++r) {
    row.assign(x + r * F, x + (r + 1) * F);
    for (int64_t t = 0; t < T; ++t)
      out[r * T + t] = forest.GetTree(t).PredictTree_Float(row);
  }
}

int32_t tbref_tree_depth(void *hv, int32_t t) {
  return static_cast<Handle *>(hv)->forest.GetTree(t).GetTreeDepth();
}

int32_t tbref_dense_size(void *hv, int32_t t) {
  return (int32_t)static_cast<Handle *>(hv)->forest.GetTree(t).GetThresholdArray().size();
}

void tbref_dense_arrays(void *hv, int32_t t, double *thr, int32_t *idx) {
  auto &tree = static_cast<Handle *>(hv)->forest.GetTree(t);
  auto a = tree.GetThresholdArray();
  auto b = tree.GetFeatureIndexArray();
  for (size_t i = 0; i < a.size(); ++i) { thr[i] = a[i]; idx[i] = b[i]; }
}

int32_t tbref_sparse_size(void *hv, int32_t t) {
  return (int32_t)static_cast<Handle *>(hv)->forest.GetTree(t).GetSparseThresholdArray().size();
}

void tbref_sparse_arrays(void *hv, int32_t t, double *thr, int32_t *idx, int32_t *child) {
  auto &tree = static_cast<Handle *>(hv)->forest.GetTree(t);
  auto a = tree.GetSparseThresholdArray();
  auto b = tree.GetSparseFeatureIndexArray();
  auto c = tree.GetChildIndexArray();
  for (size_t i = 0; i < a.size(); ++i) { thr[i] = a[i]; idx[i] = b[i]; child[i] = c[i]; }
}
}
