// Mutated model files through the loaders under AddressSanitizer + UndefinedBehaviorSanitizer: flipped bytes,
// overwritten words, cut and doubled pieces.  A loader may refuse a file (tbamd::Error) or load it; a loaded forest
// must pass Validate() or be refused there, and a validated forest must pack and unpack.  Anything else - a
// sanitizer report, another exception type, an allocation sized by a corrupt count - fails the run.
// usage: mutate_loaders <iterations> (<kind> <file> [<features> | <model.json>])...   kind: json | onnx <features> | compiled | profile <model.json>
#include "forest.h"
#include "model_file.h"
#include "packer.h"
#include "tuner.h"
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <iterator>
#include <random>
#include <string>
#include <vector>
using namespace tbamd;

static std::vector<char> Mutate(const std::vector<char> &good, std::mt19937 &rng) {
  std::vector<char> bytes = good;
  auto at = [&](size_t n) { return (size_t)(rng() % (n ? n : 1)); };
  const int edits = 1 + (int)at(3);
  for (int e = 0; e < edits && !bytes.empty(); ++e) {
    switch (at(7)) {
    case 6: { // a small, a negative or a huge number in one of the header's words
      const int32_t words[] = {0, 1, -1, 3, 7, 63, 65, 1000, 65536, 1 << 30, INT32_MIN};
      const int32_t w = words[at(11)];
      const size_t p = at(std::min<size_t>(bytes.size(), 160)) & ~(size_t)3;
      std::memcpy(bytes.data() + p, &w, std::min<size_t>(4, bytes.size() - p));
      break;
    }
    case 0: // flip a few bits
      for (int i = 0, n = 1 + (int)at(8); i < n; ++i) bytes[at(bytes.size())] ^= (char)(1u << at(8));
      break;
    case 1: { // a word of all ones, of zeros, or the largest positive value
      const uint32_t words[] = {0xFFFFFFFFu, 0u, 0x7FFFFFFFu, 0x80000000u, 0x00010000u};
      const uint32_t w = words[at(5)];
      const size_t p = at(bytes.size());
      std::memcpy(bytes.data() + p, &w, std::min<size_t>(4, bytes.size() - p));
      break;
    }
    case 2: // cut the tail
      bytes.resize(at(bytes.size()));
      break;
    case 3: { // cut a piece out of the middle
      const size_t p = at(bytes.size()), n = std::min(bytes.size() - p, 1 + at(64));
      bytes.erase(bytes.begin() + (long)p, bytes.begin() + (long)(p + n));
      break;
    }
    case 4: { // double a piece
      const size_t p = at(bytes.size()), n = std::min(bytes.size() - p, 1 + at(64));
      const std::vector<char> piece(bytes.begin() + (long)p, bytes.begin() + (long)(p + n));
      bytes.insert(bytes.begin() + (long)p, piece.begin(), piece.end());
      break;
    }
    default: // a digit, a sign, a bracket or a quote somewhere (text formats)
      bytes[at(bytes.size())] = "0123456789-+.eE[]{},:\"\\ n"[at(26)];
      break;
    }
  }
  return bytes;
}

int main(int argc, char **argv) {
  if (argc < 4) return 64;
  const int iterations = std::atoi(argv[1]);
  std::mt19937 rng(7);
  DeviceLimits limits;
  limits.computeUnits = 256;
  limits.ldsBytesPerBlock = 160 * 1024;
  const std::string scratch = std::string(std::getenv("TMPDIR") ? std::getenv("TMPDIR") : "/tmp") + "/mutated_model";
  long loaded = 0, refused = 0, packed = 0;
  for (int a = 2; a + 1 < argc;) {
    const std::string kind = argv[a], path = argv[a + 1];
    int features = 0;
    a += 2;
    if (kind == "onnx") features = std::atoi(argv[a++]);
    Forest profiled; // kind "profile": the forest the hit-count profile belongs to
    if (kind == "profile") profiled = LoadXGBoostJSON(argv[a++]);
    std::ifstream in(path, std::ios::binary);
    const std::vector<char> good((std::istreambuf_iterator<char>(in)), std::istreambuf_iterator<char>());
    if (good.empty()) { std::printf("cannot read %s\n", path.c_str()); return 65; }
    for (int i = 0; i < iterations; ++i) {
      const std::vector<char> bytes = i == 0 ? good : Mutate(good, rng); // (the intact file first: it must load)
      {
        std::ofstream out(scratch, std::ios::binary | std::ios::trunc);
        out.write(bytes.data(), (std::streamsize)bytes.size());
      }
      try {
        Forest forest;
        if (kind == "profile") {
          const HitCountProfile profile = LoadHitCountProfile(profiled, scratch);
          LaunchPlan plan = ChoosePlan(profiled, 4096, nullptr, limits);
          plan.tileSize = 4, plan.tiling = 1, plan.peelWalks = true, plan.interleave = 2, plan.featureOffsetInWords = false;
          (void)PackForest(profiled, plan, &profile); // tile membership and peel depths come out of the counts
          ++loaded, ++packed;
          continue;
        }
        if (kind == "json") forest = LoadXGBoostJSON(scratch);
        else if (kind == "onnx") forest = LoadONNX(scratch, features);
        else {
          CompiledModel model = LoadCompiledModel(scratch);
          forest = model.forest;
          try { // the plan the file names is what the runner packs with: refused or packed, never trusted blindly
            (void)PackForest(forest, model.plan);
          } catch (const Error &) {
          }
        }
        forest.Validate();
        ++loaded;
        const LaunchPlan plan = ChoosePlan(forest, 4096, nullptr, limits);
        const PackedModel pm = PackForest(forest, plan);
        if (plan.kernel != LaunchPlan::Kernel::kGlobalWalk && !forest.trees.empty()) (void)UnpackTree(pm, 0);
        ++packed;
      } catch (const Error &) {
        if (i == 0) { std::printf("the intact file %s was refused\n", path.c_str()); return 66; }
        ++refused;
      }
    }
  }
  std::printf("loaded %ld refused %ld packed %ld: ok\n", loaded, refused, packed);
  return 0;
}
