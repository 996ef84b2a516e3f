// ONNX TreeEnsembleRegressor / TreeEnsembleClassifier front end with a
// hand-written protobuf wire-format reader (no libprotobuf).
//
// Reading rules follow the reference's ONNXFileParser
// (src/json/onnxmodelparser.h):
//   :71-83    exactly one graph node of type TreeEnsemble{Regressor,Classifier}
//   :94-177   attributes; one comparison mode per model, scanned from index 1
//   :227-261  true branch = left child; a child link is kept only when its id is
//             > 0 and < the total node count, otherwise that side is absent
//   :274-281  a new tree starts whenever nodes_treeids changes
//   :289-304  leaf prediction = target_weights; class ids gathered per tree
//   :315-334  nodes renumbered in pre-order (node, left subtree, right subtree)
//   :355-374  classifier: exactly one class id per tree
// Field numbers: src/json/onnx.proto:138-174 (AttributeProto), :196-213
// (NodeProto), :380 (ModelProto.graph = 7), :441 (GraphProto.node = 1).
#include "forest.h"
#include "json_reader.h"

#include <cstring>
#include <map>
#include <set>

namespace tbamd {

namespace {

struct Reader {
  const uint8_t *p, *end;
  bool Done() const { return p >= end; }
  uint64_t Varint() {
    uint64_t v = 0;
    int shift = 0;
    while (true) {
      if (p >= end || shift > 63) throw Error("ONNX: truncated varint");
      uint8_t b = *p++;
      v |= (uint64_t)(b & 0x7F) << shift;
      if (!(b & 0x80)) return v;
      shift += 7;
    }
  }
  Reader Bytes() {
    uint64_t n = Varint();
    if (n > (uint64_t)(end - p)) throw Error("ONNX: truncated field");
    Reader r{p, p + n};
    p += n;
    return r;
  }
  float Fixed32() {
    if (end - p < 4) throw Error("ONNX: truncated fixed32");
    float f;
    std::memcpy(&f, p, 4);
    p += 4;
    return f;
  }
  void Skip(uint32_t wireType) {
    switch (wireType) {
    case 0: Varint(); break;
    case 1: if (end - p < 8) throw Error("ONNX: truncated fixed64"); p += 8; break;
    case 2: Bytes(); break;
    case 5: if (end - p < 4) throw Error("ONNX: truncated fixed32"); p += 4; break;
    default: throw Error("ONNX: unsupported wire type");
    }
  }
};

struct Attribute {
  std::string name, s;
  int64_t i = 0;
  std::vector<float> floats;
  std::vector<int64_t> ints;
  std::vector<std::string> strings;
};

Attribute ParseAttribute(Reader r) {
  Attribute a;
  while (!r.Done()) {
    uint64_t key = r.Varint();
    uint32_t field = (uint32_t)(key >> 3), wt = (uint32_t)(key & 7);
    if (field == 1 && wt == 2) { Reader b = r.Bytes(); a.name.assign((const char *)b.p, b.end - b.p); }
    else if (field == 3 && wt == 0) a.i = (int64_t)r.Varint();
    else if (field == 4 && wt == 2) { Reader b = r.Bytes(); a.s.assign((const char *)b.p, b.end - b.p); }
    else if (field == 7 && wt == 5) a.floats.push_back(r.Fixed32());
    else if (field == 7 && wt == 2) { Reader b = r.Bytes(); while (!b.Done()) a.floats.push_back(b.Fixed32()); }
    else if (field == 8 && wt == 0) a.ints.push_back((int64_t)r.Varint());
    else if (field == 8 && wt == 2) { Reader b = r.Bytes(); while (!b.Done()) a.ints.push_back((int64_t)b.Varint()); }
    else if (field == 9 && wt == 2) { Reader b = r.Bytes(); a.strings.emplace_back((const char *)b.p, b.end - b.p); }
    else r.Skip(wt);
  }
  return a;
}

struct RawNode {
  int64_t feature;
  float value;
  int64_t leftKey = -1, rightKey = -1; // index into the raw node list, -1 absent
};

} // namespace

Forest LoadONNX(const std::string &path, int32_t numFeatures) {
  if (numFeatures <= 0) throw Error("Number of features must be greater than 0");
  std::string file = ReadFile(path);
  Reader model{(const uint8_t *)file.data(), (const uint8_t *)file.data() + file.size()};
  Reader graph{nullptr, nullptr};
  while (!model.Done()) {
    uint64_t key = model.Varint();
    if ((key >> 3) == 7 && (key & 7) == 2) graph = model.Bytes();
    else model.Skip((uint32_t)(key & 7));
  }
  if (!graph.p) throw Error("ONNX: model has no graph");
  std::vector<Reader> nodes;
  while (!graph.Done()) {
    uint64_t key = graph.Varint();
    if ((key >> 3) == 1 && (key & 7) == 2) nodes.push_back(graph.Bytes());
    else graph.Skip((uint32_t)(key & 7));
  }
  if (nodes.size() != 1) throw Error("Only one node is supported");
  std::string opType;
  std::map<std::string, Attribute> attrs;
  Reader node = nodes[0];
  while (!node.Done()) {
    uint64_t key = node.Varint();
    uint32_t field = (uint32_t)(key >> 3), wt = (uint32_t)(key & 7);
    if (field == 4 && wt == 2) { Reader b = node.Bytes(); opType.assign((const char *)b.p, b.end - b.p); }
    else if (field == 5 && wt == 2) { Attribute a = ParseAttribute(node.Bytes()); attrs[a.name] = std::move(a); }
    else node.Skip(wt);
  }
  if (opType != "TreeEnsembleRegressor" && opType != "TreeEnsembleClassifier")
    throw Error("Only TreeEnsembleRegressor and TreeEnsembleClassifier are supported");
  const bool isClassifier = opType == "TreeEnsembleClassifier";
  auto need = [&](const char *name) -> Attribute & {
    auto it = attrs.find(name);
    if (it == attrs.end()) throw Error(std::string("ONNX: missing attribute ") + name);
    return it->second;
  };

  Forest forest;
  forest.numFeatures = numFeatures;
  if (attrs.count("base_values")) {
    if (attrs["base_values"].floats.size() != 1) throw Error("Only one base value is supported");
    forest.initialValue = attrs["base_values"].floats[0];
  }
  std::string post = attrs.count("post_transform") ? attrs["post_transform"].s : "NONE";
  if (post == "NONE") forest.transform = Transform::kIdentity;
  else if (post == "SOFTMAX") forest.transform = Transform::kSoftMax;
  else if (post == "LOGISTIC") forest.transform = Transform::kSigmoid;
  else throw Error("Unknown post_transform");
  if (attrs.count("nodes_missing_value_tracks_true"))
    for (int64_t v : attrs["nodes_missing_value_tracks_true"].ints)
      if (v != 0) throw Error("Missing tracks are not supported");

  std::set<std::string> modes;
  const auto &modeStrings = need("nodes_modes").strings;
  for (size_t i = 1; i < modeStrings.size(); ++i)
    if (modeStrings[i] != "LEAF") modes.insert(modeStrings[i]);
  if (modes.size() != 1) throw Error("Only one node mode is supported");
  const std::string mode = *modes.begin();
  if (mode == "BRANCH_LT") forest.predicate = Predicate::kLT;
  else if (mode == "BRANCH_GEQ") forest.predicate = Predicate::kGE;
  else if (mode == "BRANCH_GT") forest.predicate = Predicate::kGT;
  else if (mode == "BRANCH_LEQ") forest.predicate = Predicate::kLE;
  else throw Error("Only BRANCH_{LT, GEQ, GT, LEQ} is supported");

  const auto &treeIds = need("nodes_treeids").ints;
  const auto &nodeIds = need("nodes_nodeids").ints;
  const auto &featureIds = need("nodes_featureids").ints;
  const auto &values = need("nodes_values").floats;
  const auto &trueIds = need("nodes_truenodeids").ints;
  const auto &falseIds = need("nodes_falsenodeids").ints;
  const int64_t numNodes = (int64_t)nodeIds.size();
  if ((int64_t)treeIds.size() != numNodes || (int64_t)featureIds.size() != numNodes ||
      (int64_t)values.size() != numNodes || (int64_t)trueIds.size() != numNodes ||
      (int64_t)falseIds.size() != numNodes)
    throw Error("ONNX: node attribute arrays differ in length");
  forest.numClasses = isClassifier && attrs.count("n_targets") ? (int32_t)attrs["n_targets"].i : 0;

  std::map<std::pair<int64_t, int64_t>, int64_t> keyToRaw;
  std::vector<RawNode> raw(numNodes);
  for (int64_t i = 0; i < numNodes; ++i) {
    raw[i].feature = featureIds[i];
    raw[i].value = values[i];
    keyToRaw[{treeIds[i], nodeIds[i]}] = i;
  }
  for (int64_t i = 0; i < numNodes; ++i) {
    auto l = keyToRaw.find({treeIds[i], trueIds[i]});
    auto r = keyToRaw.find({treeIds[i], falseIds[i]});
    if (l == keyToRaw.end()) throw Error("Left child not found");
    if (r == keyToRaw.end()) throw Error("Right child not found");
    if (trueIds[i] > 0 && trueIds[i] < numNodes) raw[i].leftKey = l->second;
    if (falseIds[i] > 0 && falseIds[i] < numNodes) raw[i].rightKey = r->second;
  }
  std::vector<int64_t> roots;
  for (int64_t i = 0; i < numNodes; ++i)
    if (i == 0 || treeIds[i] != treeIds[i - 1]) roots.push_back(i);

  std::map<int64_t, std::set<int64_t>> treeClasses;
  const auto &tTree = need("target_treeids").ints;
  const auto &tNode = need("target_nodeids").ints;
  const auto &tIds = need("target_ids").ints;
  const auto &tWeights = need("target_weights").floats;
  if (tTree.size() != tWeights.size() || tNode.size() != tWeights.size() || tIds.size() != tWeights.size())
    throw Error("ONNX: target attribute arrays differ in length");
  for (size_t i = 0; i < tWeights.size(); ++i) {
    auto it = keyToRaw.find({tTree[i], tNode[i]});
    if (it == keyToRaw.end()) throw Error("Key not found");
    treeClasses[tTree[i]].insert(tIds[i]);
    raw[it->second].value = tWeights[i];
  }

  forest.trees.reserve(roots.size());
  for (size_t idx = 0; idx < roots.size(); ++idx) {
    Tree tree;
    struct Item { int64_t raw; int32_t parent; int side; };
    std::vector<Item> stack{{roots[idx], -1, 0}};
    while (!stack.empty()) {
      Item it = stack.back();
      stack.pop_back();
      const int32_t me = (int32_t)tree.value.size();
      tree.value.push_back(raw[it.raw].value);
      tree.feature.push_back((int32_t)raw[it.raw].feature);
      tree.left.push_back(-1);
      tree.right.push_back(-1);
      if (it.parent >= 0) (it.side == 0 ? tree.left : tree.right)[it.parent] = me;
      if (raw[it.raw].rightKey >= 0) stack.push_back({raw[it.raw].rightKey, me, 1});
      if (raw[it.raw].leftKey >= 0) stack.push_back({raw[it.raw].leftKey, me, 0});
    }
    if (isClassifier && forest.numClasses > 0) {
      auto &cls = treeClasses[(int64_t)idx];
      if (cls.size() != 1)
        throw Error("ONNX classifier with multiple class IDs per tree is not supported");
      tree.classId = (int32_t)*cls.begin();
    }
    forest.trees.push_back(std::move(tree));
  }
  forest.Validate();
  return forest;
}

} // namespace tbamd
