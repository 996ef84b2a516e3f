// XGBoost-JSON front end.  Same reading rules as the reference's
// XGBoostJSONParser (src/json/xgboostparser.h):
//   :94-114   base_score / objective -> initial value and output transform
//   :117-145  features counted from learner.feature_types
//   :156-174  one class id per tree from gradient_booster.model.tree_info
//   :177-219  node i = (split_conditions[i] narrowed to f32, split_indices[i]);
//             a node is a leaf iff both children are -1 and its prediction is
//             split_conditions[leaf]; default_left is ignored.
#include "forest.h"
#include "json_reader.h"

#include <cmath>

namespace tbamd {

Forest LoadXGBoostJSON(const std::string &path) {
  JsonValue doc = ParseJsonFile(path);
  const JsonValue &learner = doc["learner"];
  const JsonValue &params = learner["learner_model_param"];

  Forest forest;
  const double baseScore = std::stod(params["base_score"].AsString());
  const std::string &objective = learner["objective"]["name"].AsString();
  if (objective == "binary:logistic") {
    forest.initialValue = -std::log(1.0 / baseScore - 1.0);
    forest.transform = Transform::kSigmoid;
  } else if (objective == "reg:squarederror") {
    forest.initialValue = baseScore;
    forest.transform = Transform::kIdentity;
  } else if (objective == "multi:softmax") {
    forest.initialValue = baseScore;
    forest.transform = Transform::kSoftMax;
  } else {
    throw Error("Unknown objective type " + objective);
  }
  forest.numClasses = std::stoi(params["num_class"].AsString());
  forest.numFeatures = (int32_t)learner["feature_types"].Size();
  if (forest.numFeatures == 0 && params.Has("num_feature"))
    forest.numFeatures = std::stoi(params["num_feature"].AsString());

  const JsonValue &model = learner["gradient_booster"]["model"];
  const size_t numTrees = (size_t)std::stoi(model["gbtree_model_param"]["num_trees"].AsString());
  const JsonValue &trees = model["trees"];
  std::vector<double> treeInfo = model["tree_info"].AsNumbers();
  if (trees.Size() != numTrees || treeInfo.size() != numTrees)
    throw Error("num_trees does not match the trees / tree_info arrays");

  forest.trees.reserve(numTrees);
  for (size_t t = 0; t < numTrees; ++t) {
    const JsonValue &tj = trees.array[t];
    const size_t n = (size_t)std::stoi(tj["tree_param"]["num_nodes"].AsString());
    std::vector<double> left = tj["left_children"].AsNumbers();
    std::vector<double> right = tj["right_children"].AsNumbers();
    std::vector<double> cond = tj["split_conditions"].AsNumbers();
    std::vector<double> index = tj["split_indices"].AsNumbers();
    if (left.size() != n || right.size() != n || cond.size() != n || index.size() != n)
      throw Error("tree " + std::to_string(t) + ": node arrays do not match num_nodes");
    Tree tree;
    tree.value.resize(n);
    tree.feature.resize(n);
    tree.left.resize(n);
    tree.right.resize(n);
    for (size_t i = 0; i < n; ++i) {
      tree.value[i] = (float)cond[i];
      tree.feature[i] = (int32_t)index[i];
      tree.left[i] = (int32_t)left[i];
      tree.right[i] = (int32_t)right[i];
    }
    tree.classId = (int32_t)treeInfo[t];
    forest.trees.push_back(std::move(tree));
  }
  forest.Validate();
  return forest;
}

} // namespace tbamd
