// Drives the C ABI (runtime.cpp + runner.cpp + the host sources) over the host-only HIP stand-in
// (hip_host_shim.cpp) so that AddressSanitizer / UBSan / ThreadSanitizer see every buffer the runner
// sizes and every copy it makes: host entry points with pageable and "pinned" inputs of many sizes (one
// copy, staged pieces, windows), device entry points, plan changes, the plan search, the compiled-model
// file, the entry points on a caller's stream.  Predictions are compared with a plain walk of the forest.
#include "../../include/tbruntime_amd.h"

#include <hip/hip_runtime_api.h>

#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstdint>
#include <cstring>
#include <fstream>
#include <iterator>
#include <random>
#include <string>
#include <vector>

namespace {

struct HostTree {
  std::vector<float> value;
  std::vector<int32_t> feature, left, right;
  int32_t classId = 0;
};

struct HostForest {
  std::vector<HostTree> trees;
  int64_t numFeatures = 0, numClasses = 0, transform = 0;
  double initial = 0.0;
};

int gFailures = 0;
#define EXPECT(cond, ...)                                                                                              \
  do {                                                                                                                 \
    if (!(cond)) {                                                                                                     \
      std::printf("FAILED %s:%d: ", __FILE__, __LINE__);                                                               \
      std::printf(__VA_ARGS__);                                                                                        \
      std::printf(" [%s]\n", tbmi_last_error());                                                                       \
      ++gFailures;                                                                                                     \
    }                                                                                                                  \
  } while (0)

HostForest LoadForest(const char *path) {
  HostForest f;
  const intptr_t h = tbmi_load_forest(path, "xgboost_json", 0);
  if (!h) {
    std::printf("cannot load %s: %s\n", path, tbmi_last_error());
    std::exit(2);
  }
  int64_t info[6];
  tbmi_forest_info(h, info, &f.initial);
  f.numFeatures = info[1];
  f.numClasses = info[2];
  f.transform = info[3];
  f.trees.resize((size_t)info[0]);
  for (size_t t = 0; t < f.trees.size(); ++t) {
    const int32_t n = tbmi_forest_tree_size(h, (int32_t)t);
    HostTree &tree = f.trees[t];
    tree.value.resize(n);
    tree.feature.resize(n);
    tree.left.resize(n);
    tree.right.resize(n);
    tbmi_forest_tree(h, (int32_t)t, tree.value.data(), tree.feature.data(), tree.left.data(), tree.right.data(), &tree.classId);
  }
  tbmi_delete_forest(h);
  return f;
}

// Prediction of one row as RunInference returns it (class id for classifiers).
float Predict(const HostForest &f, const float *row, int32_t *leafIds) {
  std::vector<double> sums((size_t)std::max<int64_t>(1, f.numClasses), 0.0);
  for (size_t t = 0; t < f.trees.size(); ++t) {
    const HostTree &tree = f.trees[t];
    int32_t n = 0;
    while (tree.left[n] != -1) n = row[tree.feature[n]] < tree.value[n] ? tree.left[n] : tree.right[n];
    if (leafIds) leafIds[t] = n;
    sums[f.numClasses > 0 ? tree.classId : 0] += (double)tree.value[n];
  }
  if (f.numClasses == 0) {
    const double margin = f.initial + sums[0];
    return (float)(f.transform == 1 ? 1.0 / (1.0 + std::exp(-margin)) : margin);
  }
  float best = -INFINITY;
  int bestClass = 0;
  for (int c = 0; c < (int)f.numClasses; ++c) {
    const float m = (float)(f.initial + sums[c]);
    if (!(best > m)) best = m, bestClass = c;
  }
  return (float)bestClass;
}

bool Close(float a, float b) { return std::fabs((double)a - (double)b) <= 1e-6 + 1e-5 * std::fabs((double)b); }

struct Case {
  HostForest forest;
  std::string path;
  std::vector<float> x;        // rows x F
  std::vector<float> expected; // rows
  int64_t rows = 0;
};

void Compare(const Case &c, const float *got, int64_t first, int64_t rows, const char *what) {
  int64_t bad = 0;
  for (int64_t r = 0; r < rows; ++r) bad += !Close(got[r], c.expected[first + r]);
  EXPECT(bad == 0, "%s: %lld of %lld rows differ (%s)", what, (long long)bad, (long long)rows, c.path.c_str());
}

// Leaf hit counts of the case's own rows in the reference's profile format (first line `numTrees, numRows`,
// then per tree `hitCount, depth` for every leaf in node order).
std::string WriteProfile(const Case &c, const std::string &path) {
  const int64_t F = c.forest.numFeatures;
  const size_t T = c.forest.trees.size();
  std::vector<std::vector<int64_t>> hits(T);
  for (size_t t = 0; t < T; ++t) hits[t].assign(c.forest.trees[t].value.size(), 0);
  std::vector<int32_t> ids(T);
  for (int64_t r = 0; r < c.rows; ++r) {
    Predict(c.forest, c.x.data() + r * F, ids.data());
    for (size_t t = 0; t < T; ++t) ++hits[t][ids[t]];
  }
  FILE *out = std::fopen(path.c_str(), "w");
  std::fprintf(out, "%zu, %lld\n", T, (long long)c.rows);
  for (size_t t = 0; t < T; ++t) {
    const HostTree &tree = c.forest.trees[t];
    bool first = true;
    for (size_t n = 0; n < tree.value.size(); ++n) {
      if (tree.left[n] != -1) continue;
      std::fprintf(out, "%s%lld, 0", first ? "" : ", ", (long long)hits[t][n]);
      first = false;
    }
    std::fprintf(out, "\n");
  }
  std::fclose(out);
  return path;
}

intptr_t MakeRunner(const Case &c, int32_t batch, bool int8Classes, int32_t tileSize = 1, int32_t tilingType = 0,
                    const char *profile = "") {
  const intptr_t options = CreateCompilerOptions();
  Set_batchSize(options, batch);
  Set_tileSize(options, tileSize);
  Set_tilingType(options, tilingType);
  Set_statsProfileCSVPath(options, profile);
  if (int8Classes) {
    Set_returnTypeWidth(options, 8);
    Set_returnTypeFloatType(options, 0);
  }
  const intptr_t runner = CreateInferenceRunner(c.path.c_str(), "", options);
  DeleteCompilerOptions(options);
  EXPECT(runner != 0 || tileSize > 1, "CreateInferenceRunner");
  return runner;
}

// SANITIZE_QUICK=1: only the largest batch through the host entry points and the default plan through the
// device entry points (the thread sanitizer's slower build looks at the copier threads, not at plan shapes).
bool Quick() { return std::getenv("SANITIZE_QUICK") != nullptr; }

void HostEntryPoints(const Case &c) {
  const int64_t F = c.forest.numFeatures;
  // exact-size result buffers (heap, so that an overrun is seen), several batch sizes incl. the staged path
  for (int64_t rows : {(int64_t)1, (int64_t)63, (int64_t)1000, (int64_t)8192, c.rows}) {
    if (rows > c.rows || (Quick() && rows != c.rows)) continue;
    const intptr_t runner = MakeRunner(c, (int32_t)rows, false);
    if (!runner) continue;
    std::vector<float> in(c.x.begin(), c.x.begin() + rows * F), out((size_t)rows, -1.f);
    RunInference(runner, in.data(), out.data());
    Compare(c, out.data(), 0, rows, "RunInference");
    RunInference(runner, in.data(), out.data()); // buffers reused
    Compare(c, out.data(), 0, rows, "RunInference again");
    // "pinned" input: memory the runtime knows as host memory is read where it lies
    void *pinned = nullptr;
    if (hipHostMalloc(&pinned, (size_t)rows * F * sizeof(float), 0) == hipSuccess) {
      std::memcpy(pinned, in.data(), (size_t)rows * F * sizeof(float));
      std::fill(out.begin(), out.end(), -1.f);
      RunInference(runner, pinned, out.data());
      Compare(c, out.data(), 0, rows, "RunInference pinned");
      (void)hipHostFree(pinned);
    }
    // any number of rows through a runner compiled for `rows`
    for (int64_t n : {(int64_t)0, rows / 3, rows, std::min(c.rows, rows * 2 + 5), c.rows}) {
      if (Quick() && n != c.rows) continue;
      std::vector<float> in2(c.x.begin(), c.x.begin() + n * F), out2((size_t)n, -1.f);
      EXPECT(tbmi_run_host(runner, in2.data(), out2.data(), n) == 0, "tbmi_run_host %lld", (long long)n);
      Compare(c, out2.data(), 0, n, "tbmi_run_host");
    }
    const int64_t whole = c.rows / rows * rows;
    if (whole > 0 && whole <= (int64_t)1 << 30 && !Quick()) {
      std::vector<float> in3(c.x.begin(), c.x.begin() + whole * F), out3((size_t)whole, -1.f);
      RunInferenceOnMultipleBatches(runner, in3.data(), out3.data(), (int32_t)whole);
      Compare(c, out3.data(), 0, whole, "RunInferenceOnMultipleBatches");
    }
    DeleteInferenceRunner(runner);
  }
}

void DeviceEntryPoints(const Case &c, int64_t rows, int32_t tileSize = 1, int32_t tilingType = 0, const char *profile = "",
                       bool peel = false) {
  const int64_t F = c.forest.numFeatures;
  const int32_t T = (int32_t)c.forest.trees.size();
  const bool multiclass = c.forest.numClasses > 0;
  SetPeeledCodeGenForProbabilityBasedTiling(peel ? 1 : 0);
  const intptr_t runner = MakeRunner(c, (int32_t)rows, multiclass, tileSize, tilingType, profile);
  SetPeeledCodeGenForProbabilityBasedTiling(0);
  if (!runner) {
    // tiled walks are refused where the row tile cannot hold byte offsets (very wide rows), never silently dropped
    EXPECT(tileSize > 1 && std::strstr(tbmi_last_error(), "tile size"), "runner with tile size %d", tileSize);
    return;
  }
  {
    char plan[1024];
    tbmi_describe_plan(runner, plan, sizeof(plan));
    char want[64];
    std::snprintf(want, sizeof(want), " tileSize=%d ", tileSize);
    EXPECT(std::strstr(plan, want) != nullptr, "plan does not carry the tile size: %s", plan);
  }
  float *dx = nullptr;
  void *dout = nullptr;
  int32_t *dids = nullptr;
  EXPECT(hipMalloc((void **)&dx, (size_t)rows * F * sizeof(float)) == hipSuccess, "hipMalloc");
  EXPECT(hipMalloc(&dout, (size_t)rows * tbmi_result_bytes(runner)) == hipSuccess, "hipMalloc");
  EXPECT(hipMalloc((void **)&dids, (size_t)rows * T * sizeof(int32_t)) == hipSuccess, "hipMalloc");
  std::memcpy(dx, c.x.data(), (size_t)rows * F * sizeof(float));
  std::vector<int32_t> wantIds((size_t)rows * T);
  for (int64_t r = 0; r < rows; ++r) Predict(c.forest, c.x.data() + r * F, wantIds.data() + r * T);

  auto check = [&](const char *what) {
    std::vector<float> got((size_t)rows);
    for (int64_t r = 0; r < rows; ++r)
      got[r] = multiclass ? (float)static_cast<int8_t *>(dout)[r] : static_cast<float *>(dout)[r];
    Compare(c, got.data(), 0, rows, what);
    std::memset(dout, 0x5A, (size_t)rows * tbmi_result_bytes(runner));
  };
  auto runAll = [&](const char *what) {
    EXPECT(tbmi_run_device(runner, dx, dout, rows) == 0, "tbmi_run_device (%s)", what);
    check(what);
    EXPECT(tbmi_run_device_async(runner, dx, dout, rows, nullptr) == 0, "tbmi_run_device_async (%s)", what);
    check(what);
    if (tbmi_run_device_noalloc(runner, dx, dout, rows, nullptr) == 0) check(what);
    else EXPECT(std::strstr(tbmi_last_error(), "scratch memory") != nullptr, "tbmi_run_device_noalloc (%s)", what);
    EXPECT(tbmi_run_device_noalloc(runner, dx, dout, rows / 2, nullptr) == 0 || std::strstr(tbmi_last_error(), "scratch memory"),
           "tbmi_run_device_noalloc half (%s)", what);
    std::memset(dids, 0xFF, (size_t)rows * T * sizeof(int32_t));
    EXPECT(tbmi_dump_leaf_ids(runner, dx, dids, rows) == 0, "tbmi_dump_leaf_ids (%s)", what);
    EXPECT(std::memcmp(dids, wantIds.data(), wantIds.size() * sizeof(int32_t)) == 0, "leaf ids differ (%s)", what);
    double w = 0, f = 0, b = 0;
    EXPECT(tbmi_time_kernels(runner, dx, dout, rows, 2, &w, &f, &b) == 0, "tbmi_time_kernels (%s)", what);
    char small[16], big[1024];
    EXPECT(tbmi_describe_plan(runner, small, sizeof(small)) > 0 && std::strlen(small) == sizeof(small) - 1, "describe (small)");
    EXPECT(tbmi_describe_plan(runner, big, sizeof(big)) > 0, "describe");
  };
  runAll("default plan");
  if (tileSize > 1) { // block shapes of the tiled walk, the plan search, save and reload
    const int tiledPlans[][5] = {{64, 1, 1, 16384, 1}, {128, 8, 2, 32768, 3}, {256, 4, 4, 40960, 2}, {64, 16, 2, 24576, 5}, {128, 4, 1, 65536, 2}};
    for (auto &p : tiledPlans)
      if (tbmi_set_plan(runner, p[0], p[1], p[2], p[3], p[4]) == 0) runAll("tiled plan");
    EXPECT(tbmi_set_tree_parallel_plan(runner, 4, 64, 1, 0, 1) == -1, "tree-parallel plan must refuse tiles");
    double best = 0;
    EXPECT(tbmi_autotune(runner, dx, rows < 96 ? rows : 96, &best) == 0, "tbmi_autotune (tiled)"); // (a few rows: the search re-packs and launches hundreds of times)
    runAll("tiled, after the plan search");
    const std::string file = std::string(std::getenv("TMPDIR") ? std::getenv("TMPDIR") : "/tmp") + "/sanitize_tiled.tbamd";
    EXPECT(tbmi_save_compiled_model(runner, file.c_str()) == 0, "tbmi_save_compiled_model (tiled)");
    const intptr_t again = tbmi_load_compiled_model(file.c_str(), 0);
    EXPECT(again != 0, "tbmi_load_compiled_model (tiled)");
    if (again) {
      char a[1024], b[1024];
      tbmi_describe_plan(runner, a, sizeof(a));
      tbmi_describe_plan(again, b, sizeof(b));
      EXPECT(std::strcmp(a, b) == 0, "reloaded tiled plan differs: %s / %s", a, b);
      EXPECT(tbmi_run_device(again, dx, dout, rows) == 0, "reloaded tiled runner");
      check("reloaded tiled runner");
      DeleteInferenceRunner(again);
    }
  }
  if (Quick() || tileSize > 1) {
    DeleteInferenceRunner(runner);
    (void)hipFree(dx);
    (void)hipFree(dout);
    (void)hipFree(dids);
    return;
  }
  // the plan shapes the GPU tests pin, one after the other on one runner (re-pack, upload, free)
  const int rowsLds[][5] = {{64, 1, 1, 16384, 1}, {128, 1, 2, 32768, 3}, {256, 1, 8, 65536, 1}, {512, 1, 4, 49152, 5}, {256, 1, 4, 8192, 40},
                            {256, 4, 4, 65536, 1}, {128, 8, 2, 40960, 2}, {64, 3, 1, 16384, 1}, {512, 2, 8, 32768, 1}};
  for (auto &p : rowsLds)
    if (tbmi_set_plan(runner, p[0], p[1], p[2], p[3], p[4]) == 0) {
      runAll("rows_lds plan");
      for (int mode : {1, 2, 0}) { // tree groups through registers, copied directly, by rule
        EXPECT(tbmi_set_group_staging(runner, mode) == 0, "tbmi_set_group_staging");
        runAll("rows_lds plan, group staging pinned");
      }
    }
  EXPECT(tbmi_set_group_staging(runner, 7) != 0, "tbmi_set_group_staging refuses an unknown mode");
  const int treeParallel[][5] = {{1, 256, 1, 0, 0}, {4, 64, 1, 32768, 7}, {16, 16, 2, 0, 1}, {2, 128, 1, 16384, 0}, {8, 8, 4, 0, 3}, {64, 1, 1, 0, 2}, {1, 1024, 1, 65536, 1}};
  for (auto &p : treeParallel)
    if (tbmi_set_tree_parallel_plan(runner, p[0], p[1], p[2], p[3], p[4]) == 0) runAll("tree_parallel plan");
  const int quantized[][4] = {{8, 4, 0, 1}, {16, 1, 16384, 1}, {4, 2, 32768, 3}, {1, 8, 16384, 1}};
  for (auto &p : quantized)
    if (tbmi_set_quantized_plan(runner, p[0], p[1], p[2], p[3]) == 0) runAll("rank-quantised plan");
  const int rank16[][5] = {{256, 4, 4, 0, 1}, {512, 2, 4, 32768, 1}, {128, 8, 2, 16384, 3}, {64, 1, 1, 16384, 2}};
  for (auto &p : rank16)
    if (tbmi_set_rank16_plan(runner, p[0], p[1], p[2], p[3], p[4]) == 0) runAll("two-byte rank plan");
  if (tbmi_set_global_walk_plan(runner, 256, 4, 3) == 0) runAll("global walk plan");
  double best = 0;
  EXPECT(tbmi_autotune(runner, dx, rows < 96 ? rows : 96, &best) == 0, "tbmi_autotune");
  runAll("after the plan search");
  if (multiclass) {
    int8_t *cls = nullptr;
    float *margins = nullptr, *probs = nullptr;
    EXPECT(hipMalloc((void **)&cls, (size_t)rows) == hipSuccess, "hipMalloc");
    EXPECT(hipMalloc((void **)&margins, (size_t)rows * c.forest.numClasses * sizeof(float)) == hipSuccess, "hipMalloc");
    EXPECT(hipMalloc((void **)&probs, (size_t)rows * c.forest.numClasses * sizeof(float)) == hipSuccess, "hipMalloc");
    EXPECT(tbmi_run_device_multiclass(runner, dx, rows, cls, margins, probs) == 0, "tbmi_run_device_multiclass");
    EXPECT(tbmi_run_device_multiclass(runner, dx, rows, nullptr, margins, nullptr) == 0, "tbmi_run_device_multiclass");
    for (int64_t r = 0; r < rows; ++r) EXPECT((float)cls[r] == c.expected[r], "class id of row %lld", (long long)r);
    (void)hipFree(cls);
    (void)hipFree(margins);
    (void)hipFree(probs);
  }
  const std::string file = std::string(std::getenv("TMPDIR") ? std::getenv("TMPDIR") : "/tmp") + "/sanitize_runner.tbamd";
  EXPECT(tbmi_save_compiled_model(runner, file.c_str()) == 0, "tbmi_save_compiled_model");
  const intptr_t again = tbmi_load_compiled_model(file.c_str(), 0);
  EXPECT(again != 0, "tbmi_load_compiled_model");
  if (again) {
    EXPECT(tbmi_run_device(again, dx, dout, rows) == 0, "reloaded runner");
    check("reloaded runner");
    DeleteInferenceRunner(again);
  }
  DeleteInferenceRunner(runner);
  (void)hipFree(dx);
  (void)hipFree(dout);
  (void)hipFree(dids);
}

} // namespace

// Compiled-model files with mutated bytes through tbmi_load_compiled_model and, where one loads, through a host call
// of a few rows: the header's plan, batch size and return type are what a runner is built from.
static int MutatedCompiledModels(const char *path, int iterations) {
  std::ifstream in(path, std::ios::binary);
  const std::vector<char> good((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
  EXPECT(!good.empty(), "cannot read %s", path);
  const std::string scratch = std::string(std::getenv("TMPDIR") ? std::getenv("TMPDIR") : "/tmp") + "/mutated.tbamd";
  std::mt19937 rng(13);
  long loaded = 0;
  for (int i = 0; i < iterations; ++i) {
    std::vector<char> bytes = good;
    if (i > 0) {
      const int edits = 1 + (int)(rng() % 3);
      for (int e = 0; e < edits; ++e) {
        const int32_t words[] = {0, 1, -1, 2, 3, 7, 8, 9, 63, 64, 65, 255, 1000, 1024, 65536, 1 << 20, 1 << 30, INT32_MIN};
        const int32_t w = words[rng() % 18];
        const size_t limit = rng() % 4 ? std::min<size_t>(bytes.size(), 140) : bytes.size(); // mostly the header
        const size_t p = (rng() % limit) & ~(size_t)3;
        std::memcpy(bytes.data() + p, &w, std::min<size_t>(4, bytes.size() - p));
      }
    }
    {
      std::ofstream out(scratch, std::ios::binary | std::ios::trunc);
      out.write(bytes.data(), (std::streamsize)bytes.size());
    }
    const intptr_t runner = tbmi_load_compiled_model(scratch.c_str(), 0);
    if (!runner) {
      EXPECT(i > 0, "the intact compiled model was refused: %s", tbmi_last_error());
      continue;
    }
    ++loaded;
    const int32_t F = GetRowSize(runner);
    EXPECT(F > 0 && F < (1 << 20), "row size %d of a loaded model", F);
    const int64_t rows = 70;
    std::vector<float> x((size_t)rows * F, 0.25f);
    std::vector<unsigned char> out((size_t)rows * (size_t)tbmi_result_bytes(runner), 0xEE); // exactly what the call may write
    (void)tbmi_run_host(runner, x.data(), out.data(), rows); // may be refused; must not overrun
    DeleteInferenceRunner(runner);
  }
  std::printf("mutated compiled models: %ld of %d loaded\n", loaded, iterations);
  return gFailures;
}

int main(int argc, char **argv) {
  // argv: pairs of <model.json> <rows>, or --mutate <compiled model> <iterations>
  if (argc == 4 && std::strcmp(argv[1], "--mutate") == 0) {
    if (int rc = MutatedCompiledModels(argv[2], std::atoi(argv[3]))) return rc;
    std::printf("ok\n");
    return 0;
  }
  std::mt19937 rng(7);
  std::normal_distribution<float> normal(0.f, 1.f);
  for (int a = 1; a + 1 < argc; a += 2) {
    Case c;
    c.path = argv[a];
    c.rows = std::atoll(argv[a + 1]);
    c.forest = LoadForest(argv[a]);
    const int64_t F = c.forest.numFeatures;
    c.x.resize((size_t)c.rows * F);
    for (auto &v : c.x) v = normal(rng);
    c.expected.resize((size_t)c.rows);
    for (int64_t r = 0; r < c.rows; ++r) c.expected[r] = Predict(c.forest, c.x.data() + r * F, nullptr);
    HostEntryPoints(c);
    DeviceEntryPoints(c, std::min<int64_t>(c.rows, 203));
    if (!Quick()) {
      const std::string profile =
          WriteProfile(c, std::string(std::getenv("TMPDIR") ? std::getenv("TMPDIR") : "/tmp") + "/sanitize_profile.csv");
      // (every tile layout on every model; the profiled variants of the odd sizes on the first model only)
      for (int32_t tileSize : {2, 3, 4, 5, 8}) {
        DeviceEntryPoints(c, std::min<int64_t>(c.rows, 203), tileSize);
        if (a > 1 && (tileSize == 3 || tileSize == 5)) continue;
        DeviceEntryPoints(c, std::min<int64_t>(c.rows, 203), tileSize, 1, profile.c_str(), true);
        if (a > 1 && tileSize != 4) continue;
        DeviceEntryPoints(c, std::min<int64_t>(c.rows, 203), tileSize, 2, profile.c_str(), false);
      }
      DeviceEntryPoints(c, std::min<int64_t>(c.rows, 203), 1, 1, profile.c_str(), true); // scalar nodes, peeled walks
      const intptr_t options = CreateCompilerOptions();
      Set_batchSize(options, 64);
      Set_tileSize(options, 9);
      EXPECT(CreateInferenceRunner(c.path.c_str(), "", options) == 0 && std::strstr(tbmi_last_error(), "tile size 9"),
             "tile size 9 must be refused");
      DeleteCompilerOptions(options);
    }
    std::printf("%s: %lld rows done, %d failures so far\n", argv[a], (long long)c.rows, gFailures);
    std::fflush(stdout);
  }
  // error paths keep their hands off the caller's buffers
  EXPECT(tbmi_run_device(0, nullptr, nullptr, 4) == -1, "null runner");
  EXPECT(CreateInferenceRunner("/nonexistent/model.json", "", 0) == 0, "missing options");
  if (gFailures) return 1;
  std::printf("ok\n");
  return 0;
}
