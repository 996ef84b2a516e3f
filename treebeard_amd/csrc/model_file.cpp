// "Compile once, reload": a compiled model (forest + launch plan) saved to one binary file and
// reopened without the source model, and the reader of the reference's leaf hit-count profiles.
//
// Stands where the reference persists its model buffers in `<model>.treebeard-globals.json`
// (src/utils/TreeTilingUtils.cpp:145-170) and reopens a compiled model with
// InitializeInferenceRunner (src/runtime/runtime.cpp:35-54).  The file keeps the forest in model
// numbering (so leaf ids survive) and the plan; packing for the device takes milliseconds at load.
//
// Profile format (src/utils/StatsUtils.cpp:10-52 writer, :86-118 reader): first line
// `numTrees, numRows`; then one line per tree with `hitCount, depth` for every leaf in node order.
#include "model_file.h"

#include "json_reader.h"

#include <cstring>
#include <fstream>
#include <sstream>

namespace tbamd {

namespace {

constexpr char kMagic[8] = {'T', 'B', 'A', 'M', 'D', 'M', 'D', 'L'};
constexpr uint32_t kVersion = 5;

struct Writer {
  std::string bytes;
  template <typename T> void Put(const T &v) { bytes.append(reinterpret_cast<const char *>(&v), sizeof(T)); }
  template <typename T> void PutVector(const std::vector<T> &v) {
    Put<uint64_t>(v.size());
    bytes.append(reinterpret_cast<const char *>(v.data()), v.size() * sizeof(T));
  }
};

struct Reader {
  const std::string &bytes;
  size_t pos = 0;
  template <typename T> T Get() {
    if (pos + sizeof(T) > bytes.size()) throw Error("model file is truncated");
    T v;
    std::memcpy(&v, bytes.data() + pos, sizeof(T));
    pos += sizeof(T);
    return v;
  }
  template <typename T> std::vector<T> GetVector() {
    const uint64_t n = Get<uint64_t>();
    if (n > (bytes.size() - pos) / sizeof(T)) throw Error("model file is truncated");
    std::vector<T> v(n);
    if (n) std::memcpy(v.data(), bytes.data() + pos, n * sizeof(T));
    pos += n * sizeof(T);
    return v;
  }
};

} // namespace

void SaveCompiledModel(const std::string &path, const Forest &forest, const LaunchPlan &plan, int32_t batchSize,
                       int32_t returnTypeWidth, bool returnTypeFloatType, const HitCountProfile *profile) {
  Writer w;
  w.bytes.append(kMagic, sizeof(kMagic));
  w.Put<uint32_t>(kVersion);
  w.Put<int32_t>(batchSize);
  w.Put<int32_t>(returnTypeWidth);
  w.Put<int32_t>(returnTypeFloatType ? 1 : 0);
  w.Put<int32_t>(forest.numFeatures);
  w.Put<double>(forest.initialValue);
  w.Put<int32_t>((int32_t)forest.transform);
  w.Put<int32_t>(forest.numClasses);
  w.Put<int32_t>((int32_t)forest.predicate);
  w.Put<int32_t>((int32_t)plan.kernel);
  w.Put<int32_t>(plan.rowsPerBlock);
  w.Put<int32_t>(plan.treeThreads);
  w.Put<int32_t>(plan.treeLanes);
  w.Put<int32_t>(plan.interleave);
  w.Put<int32_t>(plan.groupBytes);
  w.Put<int32_t>(plan.treeSlices);
  w.Put<int32_t>(plan.featureOffsetInWords ? 1 : 0);
  w.Put<int32_t>(plan.quantizedRows ? 1 : 0);
  w.Put<int32_t>(plan.rankRows16 ? 1 : 0);
  w.Put<int32_t>(plan.tileSize);
  w.Put<int32_t>(plan.tiling);
  w.Put<int32_t>(plan.peelWalks ? 1 : 0);
  w.Put<int32_t>(plan.deferTails ? 1 : 0);
  w.Put<uint64_t>(forest.trees.size());
  for (const Tree &t : forest.trees) {
    w.Put<int32_t>(t.classId);
    w.PutVector(t.value);
    w.PutVector(t.feature);
    w.PutVector(t.left);
    w.PutVector(t.right);
  }
  w.Put<int64_t>(profile ? profile->numRows : -1);
  if (profile)
    for (const auto &hits : profile->hits) w.PutVector(hits);
  std::ofstream out(path, std::ios::binary | std::ios::trunc);
  if (!out) throw Error("cannot write " + path);
  out.write(w.bytes.data(), (std::streamsize)w.bytes.size());
  if (!out) throw Error("cannot write " + path);
}

CompiledModel LoadCompiledModel(const std::string &path) {
  const std::string bytes = ReadFile(path);
  if (bytes.size() < sizeof(kMagic) || std::memcmp(bytes.data(), kMagic, sizeof(kMagic)) != 0)
    throw Error(path + " is not a compiled model file");
  Reader r{bytes, sizeof(kMagic)};
  if (r.Get<uint32_t>() != kVersion) throw Error("unsupported compiled model version");
  CompiledModel m;
  m.batchSize = r.Get<int32_t>();
  m.returnTypeWidth = r.Get<int32_t>();
  m.returnTypeFloatType = r.Get<int32_t>() != 0;
  m.forest.numFeatures = r.Get<int32_t>();
  m.forest.initialValue = r.Get<double>();
  m.forest.transform = (Transform)r.Get<int32_t>();
  m.forest.numClasses = r.Get<int32_t>();
  m.forest.predicate = (Predicate)r.Get<int32_t>();
  m.plan.kernel = (LaunchPlan::Kernel)r.Get<int32_t>();
  m.plan.rowsPerBlock = r.Get<int32_t>();
  m.plan.treeThreads = r.Get<int32_t>();
  m.plan.treeLanes = r.Get<int32_t>();
  m.plan.interleave = r.Get<int32_t>();
  m.plan.groupBytes = r.Get<int32_t>();
  m.plan.treeSlices = r.Get<int32_t>();
  m.plan.featureOffsetInWords = r.Get<int32_t>() != 0;
  m.plan.quantizedRows = r.Get<int32_t>() != 0;
  m.plan.rankRows16 = r.Get<int32_t>() != 0;
  m.plan.tileSize = r.Get<int32_t>();
  m.plan.tiling = r.Get<int32_t>();
  m.plan.peelWalks = r.Get<int32_t>() != 0;
  m.plan.deferTails = r.Get<int32_t>() != 0;
  const uint64_t trees = r.Get<uint64_t>();
  if (trees > (bytes.size() - r.pos) / 36) throw Error("model file is truncated"); // (a tree takes 36 bytes at least)
  m.forest.trees.resize(trees);
  for (Tree &t : m.forest.trees) {
    t.classId = r.Get<int32_t>();
    t.value = r.GetVector<float>();
    t.feature = r.GetVector<int32_t>();
    t.left = r.GetVector<int32_t>();
    t.right = r.GetVector<int32_t>();
  }
  m.forest.Validate();
  const int64_t profileRows = r.Get<int64_t>();
  if (profileRows >= 0) {
    m.profile = std::make_unique<HitCountProfile>();
    m.profile->numRows = profileRows;
    m.profile->hits.resize(trees);
    for (size_t t = 0; t < trees; ++t) {
      m.profile->hits[t] = r.GetVector<int64_t>();
      if (m.profile->hits[t].size() != m.forest.trees[t].NumNodes()) throw Error("model file: profile does not match the forest");
    }
  }
  return m;
}

HitCountProfile LoadHitCountProfile(const Forest &forest, const std::string &path) {
  std::ifstream in(path);
  if (!in) throw Error("cannot open " + path);
  auto numbers = [](const std::string &line) {
    std::vector<int64_t> out;
    std::stringstream ss(line);
    std::string cell;
    while (std::getline(ss, cell, ',')) {
      if (cell.find_first_not_of(" \t\r") == std::string::npos) continue;
      out.push_back((int64_t)std::strtod(cell.c_str(), nullptr));
    }
    return out;
  };
  std::string line;
  if (!std::getline(in, line)) throw Error("hit-count profile is empty");
  const std::vector<int64_t> header = numbers(line);
  if (header.size() != 2) throw Error("hit-count profile: the first line must be `numTrees, numRows`");
  if ((size_t)header[0] != forest.trees.size()) throw Error("hit-count profile: tree count differs from the model");
  HitCountProfile profile;
  profile.numRows = header[1];
  profile.hits.resize(forest.trees.size());
  for (size_t t = 0; t < forest.trees.size(); ++t) {
    if (!std::getline(in, line)) throw Error("hit-count profile: missing line for tree " + std::to_string(t));
    const std::vector<int64_t> row = numbers(line);
    const Tree &tree = forest.trees[t];
    std::vector<int32_t> leaves;
    for (int32_t n = 0; n < (int32_t)tree.NumNodes(); ++n)
      if (tree.IsLeaf(n)) leaves.push_back(n);
    if (row.size() != 2 * leaves.size())
      throw Error("hit-count profile: tree " + std::to_string(t) + " has " + std::to_string(leaves.size()) +
                  " leaves but the profile lists " + std::to_string(row.size() / 2));
    profile.hits[t].assign(tree.NumNodes(), 0);
    for (size_t j = 0; j < leaves.size(); ++j) profile.hits[t][leaves[j]] = row[2 * j];
    // internal nodes: rows that pass through (src/include/DecisionForest.h:428-435)
    std::vector<int32_t> order;
    order.push_back(0);
    for (size_t head = 0; head < order.size(); ++head) {
      const int32_t n = order[head];
      if (!tree.IsLeaf(n)) { order.push_back(tree.left[n]); order.push_back(tree.right[n]); }
    }
    for (size_t k = order.size(); k-- > 0;) {
      const int32_t n = order[k];
      if (!tree.IsLeaf(n)) profile.hits[t][n] = profile.hits[t][tree.left[n]] + profile.hits[t][tree.right[n]];
    }
  }
  return profile;
}

double ExpectedWalkSteps(const Forest &forest, const HitCountProfile &profile) {
  // rows that pass through an internal node take one step there
  double steps = 0.0;
  for (size_t t = 0; t < forest.trees.size(); ++t) {
    const Tree &tree = forest.trees[t];
    for (int32_t n = 0; n < (int32_t)tree.NumNodes(); ++n)
      if (!tree.IsLeaf(n)) steps += (double)profile.hits[t][n];
  }
  return profile.numRows > 0 ? steps / (double)profile.numRows : 0.0;
}

} // namespace tbamd
