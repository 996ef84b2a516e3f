// Host-callable launchers of the HIP kernels (kernels.hip).
#pragma once

#include "device_model.h"

#include <hip/hip_runtime.h>

namespace tbamd {

// Scalars of the row-parallel walk (passed by value, live in SGPRs).
struct WalkScalars {
  int64_t rows = 0;
  int32_t numFeatures = 0;
  int32_t numClasses = 0;
  int32_t numGroups = 0;
  int32_t treeSlices = 1;
  uint32_t groupRegionBytes = 0; // LDS bytes reserved for one tree group (multiple of 16)
  int32_t transform = 0;         // 0 identity, 1 sigmoid
  int32_t numTrees = 0;
  int32_t rowsPerBlock = 0;      // rows per block (both kernels)
  int32_t treeThreads = 1;       // row-parallel kernel: lanes (in different waves) that share a row
  int32_t treeLanes = 1;         // tree-parallel kernel: lanes per row (power of two)
  // Row-parallel kernels, classifiers with one tree slice: the kernel keeps the running arg-max of the class
  // sums (which arrive in ascending class order) and stores the class id itself; no partial sums, no finalize.
  int32_t fuseArgmax = 0;
  // Scalar row-parallel walk on an f32 tile with byte offsets: trees may end in stubs (device_model.h); the row
  // tile then has a column for the stub feature and every wave a queue of deferred walks behind it.
  int32_t deferTails = 0;
  int32_t tailDepth = 0;         // steps the deepest deferred walk takes below its stub
  int32_t tileHops = 1;          // eight-slot tiles: links a tile step follows at most (levels of nodes inside a tile)
  double initialValue = 0.0;
};

struct WalkParams {
  WalkScalars s;
  const float *x = nullptr;       // rows x numFeatures, row-major, device
  const uint4 *nodes16 = nullptr; // packed nodes viewed as 16-byte pieces
  const DeviceBundle *bundles = nullptr;
  const DeviceNode *bundleRoots = nullptr; // interleave root-node copies per bundle (row-parallel f32 walk)
  const DeviceGroup *groups = nullptr;
  const DeviceNode *tailNodes = nullptr;   // deferred tails: the subtrees below the stubs (PackedModel::tailNodes)
  const int32_t *tailOrigin = nullptr;     // ... and their original node ids (leaf-id dump)
  const DeviceGlobalNode *globalNodes = nullptr; // global-memory walk only
  const DeviceGlobalTree *globalTrees = nullptr;
  bool peelWalks = false;         // tiled walk: bundles carry peel depths below their depths
  // Row-parallel scalar walk: tree groups go straight from global memory into LDS (no staging registers); the
  // block waits for its copy, so this pays when a second block on the CU walks meanwhile.
  bool directStaging = false;
  float *out = nullptr;           // used when the epilogue is fused (1 slice; class ids as float32 with fuseArgmax)
  int8_t *classOut = nullptr;     // fuseArgmax: class ids as int8 (out is then null)
  double *partial = nullptr;      // [partials][rows][max(1, classes)] otherwise
  // leaf-id dump (parity checks only)
  int32_t *leafIds = nullptr;     // [rows][numTrees]
  const int32_t *nodeOrigin = nullptr;
  const int32_t *slotTree = nullptr;
};

// From this many tree slices on, small batches are finalized by a wave per (row, class); classifiers then need
// one spare slot of [rows][classes] doubles behind the last slice of the partial sums.
constexpr int kWideFinalizeSlices = 16;

struct FinalizeParams {
  double *partial = nullptr;   // [slices (+ 1 spare, see kWideFinalizeSlices)][rows][max(1, classes)]
  int64_t rows = 0;
  int32_t numClasses = 0;
  int32_t treeSlices = 1;      // number of partial sums per (row, class)
  double initialValue = 0.0;
  int32_t transform = 0;
  float *out = nullptr;        // regression / binary prediction, may be null for multiclass
  int8_t *classOut = nullptr;  // multiclass: arg-max class id
  float *margins = nullptr;    // optional [rows][classes] per-class sums
  float *probabilities = nullptr; // optional [rows][classes] softmax
};

// Row-parallel walk over LDS-staged tree groups: block = s.rowsPerBlock * s.treeThreads lanes.
// `interleave` in {1,2,4,8}; `tileMode`: 0 f32 tile with byte offsets, 1 f32 tile with offsets in units of
// 4 bytes, 2 one-byte rank tile (p.x then points at the output of LaunchBinRows; 64 rows per block), 3 two-byte
// rank tile (p.x points at the output of LaunchRankRows16 for the same rowsPerBlock).
hipError_t LaunchWalkRowsLds(const WalkParams &p, int interleave, int tileMode, size_t ldsBytes, hipStream_t stream);
// The same block shape over tiled trees (tiles of 2 to 8 nodes, f32 row tile with byte offsets below 64 KB);
// `interleave` in {1,2,4}.  Tree groups are staged by direct global-to-LDS copies.
hipError_t LaunchWalkRowsTiled(const WalkParams &p, int tileSize, int interleave, size_t ldsBytes, hipStream_t stream);
// Rank-quantises rows x[rows][numFeatures] into ranks[ceil(rows/64)][numFeatures][64] (bytes) with the
// packer's threshold table ([chunk][k][64], +inf padded, tableDepth = 2^n - 1).
hipError_t LaunchBinRows(const float *x, const float *table, uint8_t *ranks, int64_t rows, int numFeatures,
                         int tableDepth, int chunkFeatures, hipStream_t stream);
// Ranks rows x[rows][numFeatures] into two-byte ranks laid out as [ceil(rows / rowsPerBlock)][(numFeatures + 2) / 2]
// [rowsPerBlock][2] with the packer's tables (PackedModel::rankTables / rankFeatures / rankChunks on the device);
// maxChunkEntries / maxChunkFeatures = the largest chunk's table entries / slots (the kernel's LDS need).  The rank
// buffer must hold the rows rounded up to whole row blocks and then to a multiple of 1024 rows.
hipError_t LaunchRankRows16(const float *x, const float *tables, const RankFeatureDesc *features, const RankChunkDesc *chunks,
                            int numChunks, uint32_t maxChunkEntries, uint32_t maxChunkFeatures, uint16_t *ranks, int64_t rows,
                            int numFeatures, int rowsPerBlock, hipStream_t stream);
// Tree-parallel walk: s.rowsPerBlock rows per block (row-major in LDS),
// s.treeLanes lanes per row; block = rowsPerBlock * treeLanes lanes.
hipError_t LaunchWalkTreeParallel(const WalkParams &p, int interleave, size_t ldsBytes, hipStream_t stream);
// Global-memory walk (fallback for trees that do not fit an LDS group): block = s.rowsPerBlock lanes,
// one per row; p.globalNodes / p.globalTrees instead of groups and bundles.
hipError_t LaunchWalkGlobal(const WalkParams &p, int interleave, hipStream_t stream);
hipError_t LaunchFinalize(const FinalizeParams &p, hipStream_t stream);

} // namespace tbamd
