// Host-only stress of loaders, packer, tuner, model file and the copier under AddressSanitizer.
#include "forest.h"
#include "host_copy.h"
#include "model_file.h"
#include "packer.h"
#include "tuner.h"
#include <array>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <random>
using namespace tbamd;
namespace tbamd { Forest LoadXGBoostJSON(const std::string &path); }
int main(int argc, char **argv) {
  std::mt19937 rng(1);
  DeviceLimits limits; limits.computeUnits = 256; limits.ldsBytesPerBlock = 160 * 1024;
  long packs = 0, refused = 0;
  for (int a = 1; a < argc; ++a) {
    Forest f = LoadXGBoostJSON(argv[a]);
    f.Validate();
    for (int64_t batch : {1, 7, 100, 203, 3001, 1 << 20}) {
      LaunchPlan base = ChoosePlan(f, batch, nullptr, limits);
      std::vector<LaunchPlan> plans = CandidatePlans(f, batch, limits);
      plans.push_back(base);
      // the plan shapes the GPU tests pin
      for (auto t : std::vector<std::array<int, 5>>{{1, 256, 1, 0, 0}, {4, 64, 1, 32768, 7}, {16, 16, 2, 0, 1}, {2, 128, 1, 16384, 0}, {8, 8, 4, 0, 3}, {64, 1, 1, 0, 2}, {1, 1024, 1, 65536, 1}}) {
        LaunchPlan p = base; p.kernel = LaunchPlan::Kernel::kTreeParallel; p.quantizedRows = false; p.treeThreads = 1;
        p.rowsPerBlock = t[0]; p.treeLanes = t[1]; p.interleave = t[2]; if (t[3]) p.groupBytes = t[3]; if (t[4]) p.treeSlices = t[4];
        p.featureOffsetInWords = (int64_t)(f.numFeatures + 1) * 4 > 0xFFFF;
        plans.push_back(p);
      }
      for (auto t : std::vector<std::array<int, 5>>{{64, 1, 1, 16384, 1}, {128, 1, 2, 32768, 3}, {256, 1, 8, 65536, 1}, {512, 1, 4, 49152, 5}, {256, 1, 4, 8192, 40}, {256, 4, 4, 65536, 1}, {128, 8, 2, 40960, 2}, {64, 3, 1, 16384, 1}, {512, 2, 8, 32768, 1}, {64, 2, 1, 4096, 24}}) {
        LaunchPlan p = base; p.kernel = LaunchPlan::Kernel::kRowParallelLds; p.quantizedRows = false; p.treeLanes = 1;
        p.rowsPerBlock = t[0]; p.treeThreads = t[1]; p.interleave = t[2]; p.groupBytes = t[3]; p.treeSlices = t[4];
        p.featureOffsetInWords = (int64_t)(f.numFeatures + 1) * p.rowsPerBlock * 4 > 0xFFFF;
        plans.push_back(p);
      }
      for (auto t : std::vector<std::array<int, 3>>{{8, 4, 0}, {16, 1, 16384}, {4, 2, 32768}, {1, 8, 16384}, {16, 2, 33728}}) {
        LaunchPlan p = base; p.kernel = LaunchPlan::Kernel::kRowParallelLds; p.quantizedRows = true; p.treeLanes = 1; p.rowsPerBlock = 64;
        p.treeThreads = t[0]; p.interleave = t[1]; if (t[2]) p.groupBytes = t[2]; p.featureOffsetInWords = true;
        plans.push_back(p);
      }
      { LaunchPlan p; p.kernel = LaunchPlan::Kernel::kGlobalWalk; p.rowsPerBlock = 256; p.interleave = 4; p.groupBytes = 0; p.treeSlices = 3; plans.push_back(p); }
      for (const LaunchPlan &p : plans) {
        try {
          PackedModel pm = PackForest(f, p);
          ++packs;
          const Forest norm = NormalizeToLessThan(f);
          for (size_t t = 0; t < norm.trees.size(); t += 37) {
            Tree u = UnpackTree(pm, (int32_t)t);
            if (u.left != norm.trees[t].left || u.right != norm.trees[t].right) { printf("MISMATCH tree %zu\n", t); return 1; }
          }
        } catch (const Error &e) { ++refused; }
      }
    }
    LaunchPlan plan = ChoosePlan(f, 4096, nullptr, limits);
    SaveCompiledModel((std::string(getenv("TMPDIR") ? getenv("TMPDIR") : "/tmp") + "/sanitize_model.tbamd"), f, plan, 4096, 32, true);
    CompiledModel m = LoadCompiledModel((std::string(getenv("TMPDIR") ? getenv("TMPDIR") : "/tmp") + "/sanitize_model.tbamd"));
    if (m.forest.trees.size() != f.trees.size()) return 2;
  }
  ParallelCopier copier(8);
  std::vector<char> src(37 << 20), dst(37 << 20);
  for (size_t i = 0; i < src.size(); ++i) src[i] = (char)(i * 131);
  for (size_t bytes : {(size_t)1, (size_t)4095, (size_t)1 << 20, ((size_t)1 << 20) + 1, (size_t)16 << 20, src.size()}) {
    std::memset(dst.data(), 0, dst.size());
    copier.Copy(dst.data(), src.data(), bytes);
    if (std::memcmp(dst.data(), src.data(), bytes) != 0 || (bytes < dst.size() && dst[bytes] != 0)) { printf("COPY MISMATCH %zu\n", bytes); return 3; }
  }
  printf("packs %ld refused %ld: ok\n", packs, refused);
  return 0;
}
