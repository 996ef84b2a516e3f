// Host-only stand-in for the HIP runtime and for the kernel launchers of kernels.h, so that the runner
// and the C ABI (runner.cpp, runtime.cpp) can run under AddressSanitizer / ThreadSanitizer without a GPU.
//
// "Device" memory is ordinary heap memory, so every buffer the library allocates gets the sanitizer's
// red zones; copies are memcpy; streams and events are tokens.  The launchers below interpret the packed
// model on the CPU with the kernels' addressing rules (group-relative node addresses, pre-multiplied
// feature offsets, rank tiles, per-class partial sums, tree slices, finalize), reading every input and
// writing every output element the kernels touch: a buffer sized or indexed wrongly by the host code is
// reported by the sanitizer, and a wrongly packed model gives wrong predictions.  Test infrastructure only.
#include "kernels.h"

#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <mutex>
#include <vector>

namespace {
std::mutex gMutex;
std::map<const void *, std::pair<size_t, bool>> gAllocations; // pointer -> (bytes, pinned host)
hipError_t gLastError = hipSuccess;

hipError_t Fail(hipError_t e) {
  gLastError = e;
  return e;
}
} // namespace

extern "C" {

hipError_t hipMalloc(void **ptr, size_t size) {
  if (!ptr) return Fail(hipErrorInvalidValue);
  *ptr = std::malloc(size ? size : 1);
  if (!*ptr) return Fail(hipErrorOutOfMemory);
  std::memset(*ptr, 0xA5, size); // device memory starts with garbage
  std::lock_guard<std::mutex> lock(gMutex);
  gAllocations[*ptr] = {size, false};
  return hipSuccess;
}

hipError_t hipFree(void *ptr) {
  if (!ptr) return hipSuccess;
  {
    std::lock_guard<std::mutex> lock(gMutex);
    if (!gAllocations.erase(ptr)) return Fail(hipErrorInvalidValue);
  }
  std::free(ptr);
  return hipSuccess;
}

hipError_t hipHostMalloc(void **ptr, size_t size, unsigned int) {
  if (!ptr) return Fail(hipErrorInvalidValue);
  *ptr = std::malloc(size ? size : 1);
  if (!*ptr) return Fail(hipErrorOutOfMemory);
  std::lock_guard<std::mutex> lock(gMutex);
  gAllocations[*ptr] = {size, true};
  return hipSuccess;
}

hipError_t hipHostFree(void *ptr) { return hipFree(ptr); }

hipError_t hipMemcpy(void *dst, const void *src, size_t bytes, hipMemcpyKind) {
  if (bytes) std::memcpy(dst, src, bytes);
  return hipSuccess;
}

hipError_t hipMemcpyAsync(void *dst, const void *src, size_t bytes, hipMemcpyKind, hipStream_t) {
  if (bytes) std::memcpy(dst, src, bytes);
  return hipSuccess;
}

hipError_t hipPointerGetAttributes(hipPointerAttribute_t *attr, const void *ptr) {
  std::lock_guard<std::mutex> lock(gMutex);
  auto it = gAllocations.upper_bound(ptr);
  if (it == gAllocations.begin()) return Fail(hipErrorInvalidValue);
  --it;
  const char *base = static_cast<const char *>(it->first);
  if (static_cast<const char *>(ptr) >= base + it->second.first) return Fail(hipErrorInvalidValue);
  std::memset(attr, 0, sizeof(*attr));
  attr->type = it->second.second ? hipMemoryTypeHost : hipMemoryTypeDevice;
  return hipSuccess;
}

hipError_t hipStreamCreateWithFlags(hipStream_t *stream, unsigned int) {
  *stream = reinterpret_cast<hipStream_t>(new int(0));
  return hipSuccess;
}
hipError_t hipStreamDestroy(hipStream_t stream) {
  delete reinterpret_cast<int *>(stream);
  return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t) { return hipSuccess; }
hipError_t hipStreamWaitEvent(hipStream_t, hipEvent_t, unsigned int) { return hipSuccess; }
hipError_t hipEventCreate(hipEvent_t *event) {
  *event = reinterpret_cast<hipEvent_t>(new int(0));
  return hipSuccess;
}
hipError_t hipEventCreateWithFlags(hipEvent_t *event, unsigned) { return hipEventCreate(event); }
hipError_t hipEventDestroy(hipEvent_t event) {
  delete reinterpret_cast<int *>(event);
  return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t, hipStream_t) { return hipSuccess; }
hipError_t hipEventSynchronize(hipEvent_t) { return hipSuccess; }
hipError_t hipEventElapsedTime(float *ms, hipEvent_t, hipEvent_t) {
  static float fake = 1.0f; // every measurement a little longer than the last: plan searches keep the first
  fake += 0.001f;
  *ms = fake;
  return hipSuccess;
}
hipError_t hipGetDeviceCount(int *count) {
  *count = 1;
  return hipSuccess;
}
hipError_t hipGetDevice(int *device) {
  *device = 0;
  return hipSuccess;
}
hipError_t hipGetDevicePropertiesR0600(hipDeviceProp_tR0600 *prop, int) {
  std::memset(prop, 0, sizeof(*prop));
  prop->multiProcessorCount = 256;
  prop->sharedMemPerBlock = 160 * 1024;
  return hipSuccess;
}
hipError_t hipGetSymbolAddress(void **devPtr, const void *symbol) {
  *devPtr = const_cast<void *>(symbol);
  return hipSuccess;
}
const char *hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "emulated HIP error"; }
hipError_t hipGetLastError(void) {
  const hipError_t e = gLastError;
  gLastError = hipSuccess;
  return e;
}

} // extern "C"

namespace tbamd {

namespace {

uint32_t Bits(float v) {
  uint32_t u;
  std::memcpy(&u, &v, sizeof(u));
  return u;
}

// One row through the slice's groups of an LDS-layout model.  `stride` is the node-offset distance between
// two features; rankRows: x points at the rank tile [row block][feature][64 rows].
// rankRows: 0 f32 rows, 1 one-byte ranks, 2 two-byte ranks ([row block][feature pair][row][2], `stride` = bytes of
// one feature pair's column = rows per block x 4)
void WalkRowLds(const WalkParams &p, int K, uint32_t stride, int rankRows, int64_t row, int slice, double *classSums,
                bool *classSeen) {
  const DeviceNode *nodes = reinterpret_cast<const DeviceNode *>(p.nodes16);
  const int F = p.s.numFeatures;
  const int gBegin = (int)(((int64_t)p.s.numGroups * slice) / p.s.treeSlices);
  const int gEnd = (int)(((int64_t)p.s.numGroups * (slice + 1)) / p.s.treeSlices);
  for (int g = gBegin; g < gEnd; ++g) {
    const DeviceGroup grp = p.groups[g];
    for (uint32_t b = 0; b < grp.bundleCount; ++b) {
      const DeviceBundle bd = p.bundles[grp.bundleBegin + b];
      for (int k = 0; k < K; ++k) {
        uint32_t addr = bd.root[k];
        for (uint32_t d = 0; d < bd.depth; ++d) {
          if (addr % kNodeBytes != 0 || addr / kNodeBytes >= grp.nodeCount) std::abort(); // pointer outside the group
          const DeviceNode node = nodes[grp.nodeBegin + addr / kNodeBytes];
          const uint32_t offset = node.meta & 0xFFFFu;
          const uint32_t f = rankRows == 2 ? offset / stride * 2u + ((offset >> 1) & 1u) : offset / stride;
          if ((rankRows == 2 ? (offset % stride) & ~2u : offset % stride) != 0 || (int)f > F) std::abort(); // offset outside the row tile
          bool left;
          if (rankRows == 2) {
            const uint16_t *ranks = reinterpret_cast<const uint16_t *>(p.x);
            const int64_t RB = stride / 4, pairs = (F + 2) / 2;
            const uint32_t rank = ranks[(((row / RB) * pairs + f / 2) * RB + row % RB) * 2 + (f & 1)]; // (the pad feature's slot holds 0)
            left = rank <= Bits(node.value);
          } else if (rankRows) {
            const uint8_t *ranks = reinterpret_cast<const uint8_t *>(p.x);
            const uint32_t rank = (int)f == F ? 0u : ranks[((row / 64) * F + f) * 64 + (row % 64)];
            left = rank <= Bits(node.value);
          } else {
            const float x = (int)f >= F ? -INFINITY : p.x[row * F + f]; // (the pad feature and the stub feature hold -inf)
            left = x < node.value;
          }
          addr = (node.meta >> 16) + (left ? 0u : kNodeBytes);
        }
        if (addr / kNodeBytes >= grp.nodeCount) std::abort();
        bool inTail = false;
        uint32_t at = 0;
        if (p.s.deferTails) {
          // a stub (NaN value, child pointer one node before itself) stands for the node of the tail array its
          // payload names: the walk goes on there for at most tailDepth steps
          const DeviceNode stop = nodes[grp.nodeBegin + addr / kNodeBytes];
          if (rankRows != 0 || stride == 0) std::abort();
          if (stop.value != stop.value) { // a NaN marks a stub; its payload is the tail index
            if (!bd.hasStubs || (stop.meta >> 16) + kNodeBytes != addr || (Bits(stop.value) & ~kStubIndexMask) != kStubValueBits ||
                !p.tailNodes || !p.tailOrigin)
              std::abort();
            inTail = true;
            at = Bits(stop.value) & kStubIndexMask;
            if (at == 0) std::abort();
            for (int d = 0; d < p.s.tailDepth; ++d) {
              const DeviceNode node = p.tailNodes[at];
              const uint32_t f = node.meta & ((1u << kTailFeatureBits) - 1u);
              if ((int)f > F) std::abort();
              const float x = (int)f == F ? -INFINITY : p.x[row * F + f];
              at = (node.meta >> kTailFeatureBits) + (x < node.value ? 0u : 1u);
            }
            const DeviceNode leaf = p.tailNodes[at];
            if ((leaf.meta >> kTailFeatureBits) != at || (leaf.meta & ((1u << kTailFeatureBits) - 1u)) != (uint32_t)F) std::abort(); // tailDepth must reach a leaf
          }
        }
        if (inTail) {
          classSums[0] += (double)p.tailNodes[at].value;
          classSeen[0] = true;
          if (p.leafIds) {
            const int tree = p.slotTree[bd.firstSlot + k];
            if (tree >= 0) p.leafIds[row * p.s.numTrees + tree] = p.tailOrigin[at];
          }
          continue;
        }
        const int cls = p.s.numClasses > 0 ? (int)bd.classId : 0;
        classSums[cls] += (double)nodes[grp.nodeBegin + addr / kNodeBytes].value;
        classSeen[cls] = true;
        if (p.leafIds) {
          const int tree = p.slotTree[bd.firstSlot + k];
          if (tree >= 0) p.leafIds[row * p.s.numTrees + tree] = p.nodeOrigin[grp.nodeBegin + addr / kNodeBytes];
        }
      }
    }
  }
}

void StoreRow(const WalkParams &p, int64_t row, int slice, const double *classSums) {
  const int C = p.s.numClasses;
  if (p.s.fuseArgmax) { // the kernel's own running arg-max (ties go to the larger class id)
    if (C <= 0 || p.s.treeSlices != 1 || p.partial || (!p.out && !p.classOut)) std::abort();
    float best = -INFINITY;
    int bestClass = 0;
    for (int c = 0; c < C; ++c) {
      const float m = (float)(p.s.initialValue + classSums[c]);
      if (!(best > m)) best = m, bestClass = c;
    }
    if (p.classOut) p.classOut[row] = (int8_t)bestClass;
    else p.out[row] = (float)bestClass;
    return;
  }
  if (C > 0 || p.partial) {
    if (!p.partial) std::abort(); // classifiers always go through the finalize kernel
    double *dst = p.partial + ((int64_t)slice * p.s.rows + row) * (C > 0 ? C : 1);
    for (int c = 0; c < (C > 0 ? C : 1); ++c) dst[c] = classSums[c];
  } else {
    const double margin = p.s.initialValue + classSums[0];
    p.out[row] = (float)(p.s.transform == 1 ? 1.0 / (1.0 + std::exp(-margin)) : margin);
  }
}

hipError_t WalkLds(const WalkParams &p, int K, uint32_t stride, int rankRows) {
  if (K != 1 && K != 2 && K != 4 && K != 8) return hipErrorInvalidValue;
  if (p.s.treeSlices > 1 && !p.partial) std::abort(); // slices meet in the partial-sum buffer
  const int Cn = p.s.numClasses > 0 ? p.s.numClasses : 1;
  std::vector<double> sums((size_t)Cn);
  std::vector<char> seen((size_t)Cn);
  for (int slice = 0; slice < p.s.treeSlices; ++slice)
    for (int64_t row = 0; row < p.s.rows; ++row) {
      std::fill(sums.begin(), sums.end(), 0.0);
      WalkRowLds(p, K, stride, rankRows, row, slice, sums.data(), reinterpret_cast<bool *>(seen.data()));
      StoreRow(p, row, slice, sums.data());
    }
  return hipSuccess;
}

} // namespace

hipError_t LaunchWalkRowsLds(const WalkParams &p, int interleave, int tileMode, size_t ldsBytes, hipStream_t) {
  if (p.s.rows <= 0) return hipSuccess;
  const int RB = p.s.rowsPerBlock, TT = p.s.treeThreads;
  if (ldsBytes > 160 * 1024 || RB < 64 || (RB & (RB - 1)) || TT < 1 || RB * TT > 1024) return hipErrorInvalidValue;
  if (p.s.treeSlices < 1 || p.s.treeSlices > 65535) return hipErrorInvalidValue;
  const int prefetch = (int)((p.s.groupRegionBytes / 16 + RB * TT - 1) / (RB * TT));
  if (prefetch > 16) return hipErrorInvalidValue;
  if (tileMode == 2 && RB != 64) return hipErrorInvalidValue;
  if (tileMode < 0 || tileMode > 3) return hipErrorInvalidValue;
  if (tileMode == 3 && (int64_t)((p.s.numFeatures + 2) / 2) * RB * 4 > 0x10000) return hipErrorInvalidValue;
  const uint32_t stride = tileMode == 0 || tileMode == 3 ? (uint32_t)RB * 4u : tileMode == 1 ? (uint32_t)RB : (uint32_t)RB / 4u;
  return WalkLds(p, interleave, stride, tileMode == 3 ? 2 : tileMode == 2 ? 1 : 0);
}

namespace {

// One tile step of the tiled layout (device_model.h): returns the byte address of the child tile.
uint32_t TileStepHost(const unsigned char *group, uint32_t groupBytes, uint32_t addr, int T, const float *row, int F,
                      uint32_t stride, int hops) {
  const uint32_t bytes = TileBytes(T);
  if (addr % 8 != 0 || addr + bytes > groupBytes) std::abort(); // tile outside the group
  const unsigned char *tile = group + addr;
  if (T > kMaxSelectTile) { // the eight-slot tile: { thr[8]; off[8]; links; childBase }
    float thr8[8];
    uint16_t off8[8], base;
    uint64_t links;
    std::memcpy(thr8, tile, 32);
    std::memcpy(off8, tile + 32, 16);
    std::memcpy(&links, tile + 48, 8);
    std::memcpy(&base, tile + 56, 2);
    uint32_t slot = 0;
    for (int hop = 0; hop < hops; ++hop) { // (the kernel follows `hops` links: they must reach a child)
      if (off8[slot] % stride != 0 || (int)(off8[slot] / stride) > F) std::abort();
      const int f = (int)(off8[slot] / stride);
      const float x = f == F ? -INFINITY : row[f];
      const uint32_t link = (uint32_t)(links >> (4 * slot + (x < thr8[slot] ? 32 : 0))) & 15u;
      if (link >= kTileLinkExit) return base + (link - kTileLinkExit) * bytes;
      slot = link + 1;
    }
    std::abort(); // links that never reach a child
  }
  float thr[kMaxTileSize];
  uint16_t off[kMaxTileSize], childBase;
  std::memcpy(thr, tile, (size_t)T * 4);
  std::memcpy(off, tile + T * 4, (size_t)T * 2);
  std::memcpy(&childBase, tile + T * 6, 2);
  uint64_t select = 0;
  if (T == 4) {
    uint16_t low;
    uint32_t high;
    std::memcpy(&low, tile + 26, 2);
    std::memcpy(&high, tile + 28, 4);
    select = (uint64_t)low | ((uint64_t)high << 16);
  } else {
    uint16_t s16;
    std::memcpy(&s16, tile + T * 6 + 2, 2);
    select = s16;
  }
  uint32_t outcome = 0;
  for (int i = 0; i < T; ++i) {
    if (off[i] % stride != 0 || (int)(off[i] / stride) > F) std::abort();
    const int f = (int)(off[i] / stride);
    const float x = f == F ? -INFINITY : row[f];
    outcome |= (x < thr[i] ? 1u : 0u) << i;
  }
  const uint32_t width = TileSelectBits(T);
  const uint32_t child = (uint32_t)(select >> (outcome * width)) & ((1u << width) - 1u);
  return childBase + child * bytes;
}

} // namespace

hipError_t LaunchWalkRowsTiled(const WalkParams &p, int tileSize, int interleave, size_t ldsBytes, hipStream_t) {
  if (p.s.rows <= 0) return hipSuccess;
  const int RB = p.s.rowsPerBlock, TT = p.s.treeThreads, T = tileSize, K = interleave;
  if (ldsBytes > 160 * 1024 || RB < 64 || (RB & (RB - 1)) || TT < 1 || RB * TT > 1024) return hipErrorInvalidValue;
  if ((int64_t)(p.s.numFeatures + 1) * RB * 4 > 0x10000) return hipErrorInvalidValue;
  if (p.s.treeSlices < 1 || p.s.treeSlices > 65535) return hipErrorInvalidValue;
  if (T < 2 || T > kMaxTileSize || (K != 1 && K != 2 && K != 4)) return hipErrorInvalidValue;
  if (p.s.treeSlices > 1 && !p.partial) std::abort();
  const DeviceNode *nodes = reinterpret_cast<const DeviceNode *>(p.nodes16);
  const int F = p.s.numFeatures;
  const int Cn = p.s.numClasses > 0 ? p.s.numClasses : 1;
  std::vector<double> sums((size_t)Cn);
  for (int slice = 0; slice < p.s.treeSlices; ++slice) {
    const int gBegin = (int)(((int64_t)p.s.numGroups * slice) / p.s.treeSlices);
    const int gEnd = (int)(((int64_t)p.s.numGroups * (slice + 1)) / p.s.treeSlices);
    for (int64_t row = 0; row < p.s.rows; ++row) {
      std::fill(sums.begin(), sums.end(), 0.0);
      for (int g = gBegin; g < gEnd; ++g) {
        const DeviceGroup grp = p.groups[g];
        const unsigned char *group = reinterpret_cast<const unsigned char *>(nodes + grp.nodeBegin);
        for (uint32_t b = 0; b < grp.bundleCount; ++b) {
          const DeviceBundle bd = p.bundles[grp.bundleBegin + b];
          if (bd.peelDepth > bd.depth) std::abort();
          for (int k = 0; k < K; ++k) {
            uint32_t addr = bd.root[k];
            // the kernel stops early only when no lane moves any more, which leaves every lane where `depth`
            // steps would: the full walk is the specification
            for (uint32_t d = 0; d < bd.depth; ++d)
              addr = TileStepHost(group, grp.nodeCount * kNodeBytes, addr, T, p.x + row * F, F, (uint32_t)RB * 4u, p.s.tileHops);
            const uint32_t settled = TileStepHost(group, grp.nodeCount * kNodeBytes, addr, T, p.x + row * F, F, (uint32_t)RB * 4u, p.s.tileHops);
            if (settled != addr) std::abort(); // `depth` steps must end on a leaf tile
            float value;
            std::memcpy(&value, group + addr, 4);
            sums[p.s.numClasses > 0 ? bd.classId : 0] += (double)value;
            if (p.leafIds) {
              const int tree = p.slotTree[bd.firstSlot + k];
              if (tree >= 0) p.leafIds[row * p.s.numTrees + tree] = p.nodeOrigin[grp.nodeBegin + addr / kNodeBytes];
            }
          }
        }
      }
      StoreRow(p, row, slice, sums.data());
    }
  }
  return hipSuccess;
}

hipError_t LaunchWalkTreeParallel(const WalkParams &p, int interleave, size_t ldsBytes, hipStream_t) {
  if (p.s.rows <= 0) return hipSuccess;
  if (ldsBytes > 160 * 1024 || p.s.rowsPerBlock < 1 || p.s.treeLanes < 1) return hipErrorInvalidValue;
  const int threads = p.s.rowsPerBlock * p.s.treeLanes;
  if (threads > 1024 || threads % 64 != 0) return hipErrorInvalidValue;
  if (p.s.treeSlices < 1 || p.s.treeSlices > 65535) return hipErrorInvalidValue;
  if ((int)((p.s.groupRegionBytes / 16 + threads - 1) / threads) > 16) return hipErrorInvalidValue;
  return WalkLds(p, interleave, 4u, 0);
}

hipError_t LaunchWalkGlobal(const WalkParams &p, int interleave, hipStream_t) {
  if (p.s.rows <= 0) return hipSuccess;
  const int threads = p.s.rowsPerBlock;
  if (threads < 64 || threads > 1024 || threads % 64 != 0) return hipErrorInvalidValue;
  if (interleave != 1 && interleave != 2 && interleave != 4 && interleave != 8) return hipErrorInvalidValue;
  const int Cn = p.s.numClasses > 0 ? p.s.numClasses : 1;
  std::vector<double> sums((size_t)Cn);
  for (int slice = 0; slice < p.s.treeSlices; ++slice) {
    const int tBegin = (int)(((int64_t)p.s.numTrees * slice) / p.s.treeSlices);
    const int tEnd = (int)(((int64_t)p.s.numTrees * (slice + 1)) / p.s.treeSlices);
    for (int64_t row = 0; row < p.s.rows; ++row) {
      std::fill(sums.begin(), sums.end(), 0.0);
      for (int t = tBegin; t < tEnd; ++t) {
        const DeviceGlobalTree tree = p.globalTrees[t];
        uint32_t n = tree.root;
        for (uint32_t d = 0; d < tree.depth; ++d) {
          const DeviceGlobalNode node = p.globalNodes[n];
          if (node.feature != kGlobalLeaf) n = node.left + (p.x[row * p.s.numFeatures + node.feature] < node.value ? 0u : 1u);
        }
        sums[p.s.numClasses > 0 ? tree.classId : 0] += (double)p.globalNodes[n].value;
        if (p.leafIds) p.leafIds[row * p.s.numTrees + tree.origin] = p.globalNodes[n].origin;
      }
      StoreRow(p, row, slice, sums.data());
    }
  }
  return hipSuccess;
}

hipError_t LaunchBinRows(const float *x, const float *table, uint8_t *ranks, int64_t rows, int numFeatures, int tableDepth,
                         int chunkFeatures, hipStream_t) {
  if (rows <= 0) return hipSuccess;
  if (chunkFeatures != 64) return hipErrorInvalidValue;
  if (tableDepth < 1 || tableDepth > 255 || ((tableDepth + 1) & tableDepth)) return hipErrorInvalidValue;
  const int64_t rowBlocks = (rows + 63) / 64;
  for (int64_t rb = 0; rb < rowBlocks; ++rb)
    for (int f = 0; f < numFeatures; ++f)
      for (int r = 0; r < 64; ++r) {
        const int64_t row = std::min<int64_t>(rb * 64 + r, rows - 1);
        const float v = x[row * numFeatures + f];
        const float *column = table + ((int64_t)(f / 64) * tableDepth) * 64 + (f % 64);
        int rank = 0;
        for (int step = (tableDepth + 1) / 2; step >= 1; step /= 2)
          if (!(v < column[(int64_t)(rank + step - 1) * 64])) rank += step;
        ranks[(rb * numFeatures + f) * 64 + r] = (uint8_t)rank;
      }
  return hipSuccess;
}

hipError_t LaunchRankRows16(const float *x, const float *tables, const RankFeatureDesc *features, const RankChunkDesc *chunks,
                            int numChunks, uint32_t maxChunkEntries, uint32_t maxChunkFeatures, uint16_t *ranks, int64_t rows,
                            int numFeatures, int rowsPerBlock, hipStream_t) {
  if (rows <= 0) return hipSuccess;
  if (numChunks < 1 || (size_t)maxChunkEntries * 4 + (size_t)maxChunkFeatures * 1025 * 4 + 16 > 160 * 1024 || rowsPerBlock < 64 ||
      rowsPerBlock % 64 != 0)
    return hipErrorInvalidValue;
  const int64_t RB = rowsPerBlock, pairs = (numFeatures + 2) / 2;
  // the kernel ranks whole row blocks, rounded up to its own tiles of 1024 rows: the buffer has to hold them
  const int64_t rowBlocks = (((rows + RB - 1) / RB * RB + 1023) / 1024 * 1024 + RB - 1) / RB;
  std::vector<char> written((size_t)pairs * 2, 0);
  for (int c = 0; c < numChunks; ++c) {
    const RankChunkDesc ck = chunks[c];
    if (ck.firstFeature % 2 || ck.numFeatures % 2 || ck.firstFeature + ck.numFeatures > (uint32_t)pairs * 2 ||
        ck.tableEntries > maxChunkEntries || ck.numFeatures > maxChunkFeatures)
      std::abort();
    for (uint32_t f = ck.firstFeature; f < ck.firstFeature + ck.numFeatures; ++f) {
      written[f] = 1;
      const RankFeatureDesc fd = features[f];
      const uint32_t entries = (1u << fd.levels) - 1u;
      if (fd.tableOffset + entries > ck.tableEntries) std::abort(); // table outside its chunk
      if ((int)f >= numFeatures && fd.levels != 0) std::abort();     // the pad slots have no table
      const float *table = tables + ck.tableBegin + fd.tableOffset;
      for (int64_t slot = 0; slot < rowBlocks * RB; ++slot) {
        const int64_t row = std::min<int64_t>(slot, rows - 1);
        uint32_t node = 0;
        if (fd.levels) {
          const float v = x[row * numFeatures + f];
          for (uint32_t level = 0; level < fd.levels; ++level) node = 2 * node + (v < table[node] ? 1u : 2u);
        }
        ranks[(((slot / RB) * pairs + f / 2) * RB + slot % RB) * 2 + (f & 1)] = (uint16_t)(node - entries);
      }
    }
  }
  for (char w : written)
    if (!w) std::abort(); // a slot of the tile no chunk fills
  return hipSuccess;
}

hipError_t LaunchFinalize(const FinalizeParams &p, hipStream_t) {
  if (p.rows <= 0) return hipSuccess;
  const int C = p.numClasses;
  for (int64_t row = 0; row < p.rows; ++row) {
    if (C == 0) {
      double margin = p.initialValue;
      for (int s = 0; s < p.treeSlices; ++s) margin += p.partial[(int64_t)s * p.rows + row];
      p.out[row] = (float)(p.transform == 1 ? 1.0 / (1.0 + std::exp(-margin)) : margin);
      continue;
    }
    float best = -INFINITY;
    int bestClass = 0;
    double maxMargin = -INFINITY;
    std::vector<double> margins((size_t)C);
    for (int c = 0; c < C; ++c) {
      double margin = p.initialValue;
      for (int s = 0; s < p.treeSlices; ++s) margin += p.partial[((int64_t)s * p.rows + row) * C + c];
      margins[c] = margin;
      const float m = (float)margin;
      if (p.margins) p.margins[row * C + c] = m;
      if (!(best > m)) {
        best = m;
        bestClass = c;
      }
      maxMargin = std::max(maxMargin, margin);
    }
    if (p.classOut) p.classOut[row] = (int8_t)bestClass;
    if (p.out) p.out[row] = (float)bestClass;
    if (p.probabilities) {
      double z = 0.0;
      for (int c = 0; c < C; ++c) z += std::exp(margins[c] - maxMargin);
      for (int c = 0; c < C; ++c) p.probabilities[row * C + c] = (float)(std::exp(margins[c] - maxMargin) / z);
    }
  }
  return hipSuccess;
}

} // namespace tbamd
