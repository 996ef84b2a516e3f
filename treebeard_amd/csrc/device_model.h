// Device-facing model layout shared by the packer (host) and the HIP kernels.
//
// This replaces the reference's tiled-tree model buffers
// (src/utils/TreeTilingUtils.cpp:363-413 tile byte layout, :434-495
// offsets/lengths/classIds, src/mlir/Representations.cpp:1038-1052/:1728-1744
// tile structs, src/gpu/GPURepresentations.cpp:90-256 device packing) with a
// layout made for staging whole tree groups in LDS:
//
//  * A forest is cut into GROUPS of trees; one group's nodes are a contiguous
//    run of 8-byte nodes that is copied verbatim into LDS, so every pointer a
//    node holds is a byte address relative to the start of its group.
//  * Node = { f32 value; u32 meta }.  value is the split threshold or, on a
//    leaf, the prediction.  meta = (left-child byte address << 16) | feature
//    offset.  The right child always follows the left one (+8 bytes).
//  * The feature offset is pre-multiplied for the transposed row tile the
//    kernel keeps in LDS (feature-major, one column per row of the block), so
//    the address of the feature value is `featureOffset + 4*rowSlot`.
//  * A leaf points at itself and tests the pad feature (index numFeatures),
//    whose column holds -inf: `x < value` is then always true, the walk takes
//    the "left" pointer and stays on the leaf.  A walk of `depth` steps thus
//    needs no leaf test: it ends on the leaf for every row.
//  * Deferred tails (LaunchPlan::deferTails; the reference's peeled walks for skewed trees,
//    src/mlir/ProbabilityBasedTilingTransform.cpp:66-73, src/mlir/WalkDecisionTreeLoweringPass.cpp:231-315): the
//    lock-step walk of a tree may stop at a level above its leaves.  The internal nodes of that level are then
//    represented by STUBS, which hold the walk in place like a leaf: the value field is a NaN (every compare
//    fails, the walk takes the "right" child) and the child pointer is the stub's own address minus one node, so
//    the right child is the stub itself.  The NaN's payload is the index of the node the stub stands for in the
//    TAIL ARRAY: the subtrees below the stubs stay in global memory, out of the tree groups, as nodes
//    { value; (left child index << kTailFeatureBits) | feature index } (PackedModel::tailNodes).  A model with a
//    NaN leaf value keeps its trees whole.
//  * Trees are walked K at a time (a BUNDLE) to give every lane K independent
//    dependency chains.  A bundle records the K root addresses, the trip count
//    (deepest tree of the bundle) and the class the trees add to.
//
// Tiled layout (LaunchPlan::tileSize T in 2..8; the reference's tile of T connected internal nodes,
// src/mlir/UniformTilingTransformation.cpp:148-195, src/mlir/ProbabilityBasedTilingTransform.cpp:124-198):
//  * A TILE holds its nodes in level order, struct-of-arrays: T thresholds, T feature offsets, the byte
//    address of its first child tile and a child-select table, in 16 / 24 / 32 bytes for T = 2 / 3 / 4:
//      T = 2: { f32 thr[2]; u16 off[2]; u16 childBase; u16 select }                      one 16-byte read
//      T = 3: { f32 thr[3]; u16 off[3]; u16 childBase; u16 select; u16 pad }             three 8-byte reads
//      T = 4: { f32 thr[4]; u16 off[4]; u16 childBase; u16 selectLow; u32 selectHigh }   two 16-byte reads
//  * The children of a tile (tiles or leaves, numbered left to right as in
//    docs/TileShapesAndLUT/TileShapesAndLUT.md:23-27) are consecutive tiles, child c at childBase + c * tile
//    bytes.  `select` is the tile's own row of the reference's LUT[shape][outcome]
//    (src/utils/TreeTilingUtils.cpp:1932-2018): field number `outcome` (2 bits wide for T <= 3, 3 bits for
//    T = 4) is the child reached when bit i of `outcome` says that node i's predicate held (node 0 in the
//    least significant bit, src/mlir/CodeGenStateMachine.cpp:284-506).  Keeping the row in the tile saves the
//    shape id and the table lookup.
//  * Unused node slots of a short tile test the pad feature; their outcome bits are don't-cares of `select`.
//  * A leaf is a tile of its own: thr[0] is the prediction, every slot tests the pad feature, childBase is
//    the tile's own address and select is 0, so a walk of `depth` tile steps needs no leaf test either.
//  * Tile sizes 5 to 8 share one 64-byte tile of eight slots (four 16-byte reads), the reference's default
//    tile size 8 among them (test/python/cpu_tests.py:14, src/test/GPUTests.cpp:995):
//      { f32 thr[8]; u16 off[8]; u64 links; u16 childBase; u16 pad[3] }
//    A table of 256 outcomes does not fit a tile, and one row of the reference's LUT per shape present in a
//    model (1430 shapes of 256 entries) fits no LDS, so the tile carries its own shape instead: `links` holds
//    a 4-bit link per slot and outcome, nibble s of the high word taken when slot s sends the row left (its
//    predicate holds) and nibble s of the low word when it sends it right.  A link below 7 names the next slot
//    (link + 1: slot 0 is nobody's child), a link of 7 or more the child reached (link - 7, children numbered
//    left to right, 0..8).  A tile step picks the eight links its comparisons select with one masked insert of
//    the high word into the low one and follows them from slot 0, as many as the tiles of the model have
//    levels of nodes; this is the reference's LUT[shape][outcome] evaluated instead of stored, so the outcome
//    bit order and the child numbering are the same.  A leaf tile's links
//    all say "child 0" and its childBase is its own address.
#pragma once

#include <cstdint>

namespace tbamd {

constexpr int kMaxInterleave = 8;
constexpr uint32_t kNodeBytes = 8;
constexpr uint32_t kDeferBytesPerWave = 512; // LDS of one wave's queue of deferred walks (LaunchPlan::deferTails)
// Deferred tails: a tail node's meta word holds the index of its left child above kTailFeatureBits bits of feature
// index; a queue entry holds a tail index below 6 bits of lane (bits 26 to 31).
constexpr uint32_t kTailFeatureBits = 12;
constexpr uint32_t kMaxTailNodes = 1u << 20;
// A stub's value field: a quiet NaN whose low bits are the tail index.
constexpr uint32_t kStubValueBits = 0x7FC00000u;
constexpr uint32_t kStubIndexMask = kMaxTailNodes - 1u;
constexpr int kMaxTileSize = 8;
// Tiles of more than kMaxSelectTile nodes carry links instead of a child-select table.
constexpr int kMaxSelectTile = 4;
// Bytes of one tile of T nodes (T = 1 is the scalar node).
constexpr uint32_t TileBytes(int tileSize) {
  return tileSize <= 1 ? kNodeBytes : tileSize == 2 ? 16u : tileSize == 3 ? 24u : tileSize == 4 ? 32u : 64u;
}
// Width of one field of a tile's child-select table (tiles of up to kMaxSelectTile nodes).
constexpr uint32_t TileSelectBits(int tileSize) { return tileSize == 4 ? 3u : 2u; }
// Links of the 64-byte tile: values below kTileLinkExit name a slot (value + 1), the others a child (value - kTileLinkExit).
constexpr uint32_t kTileLinkExit = 7;
constexpr uint64_t kLeafTileLinks = 0x7777777777777777ull; // every link: child 0

struct DeviceNode {
  float value;
  uint32_t meta;
};

struct alignas(32) DeviceBundle {
  uint16_t root[kMaxInterleave]; // byte address of each tree's root inside the group
  uint32_t depth;                // walk steps (tile steps in the tiled layout) that bring every row to a leaf (or to a stub)
  uint16_t classId;              // (the kernels fetch a bundle with scalar loads only)
  uint16_t hasStubs;             // deferred tails: some tree of the bundle ends in stubs
  uint32_t firstSlot;            // index of root[0] in the slot->tree table
  uint32_t peelDepth;            // steps taken without looking; the rest runs while any lane still moves (== depth: no tail)
};

// Node of the global-memory walk (trees too big for an LDS group): 16 bytes, absolute indices.
struct DeviceGlobalNode {
  float value;        // threshold, or the prediction on a leaf
  uint32_t feature;   // feature index; kGlobalLeaf on a leaf
  uint32_t left;      // index of the left child in the node array (right = left + 1)
  int32_t origin;     // node id in the model file's numbering
};
constexpr uint32_t kGlobalLeaf = 0xFFFFFFFFu;

// Per-tree record of the global-memory walk.
struct DeviceGlobalTree {
  uint32_t root;
  uint32_t depth;
  uint32_t classId;
  int32_t origin;     // tree index in the model file
};

// Ranking kernel of the two-byte rank rows: where a feature's threshold table (a complete search tree in
// breadth-first order, 2^levels - 1 entries) starts inside its chunk, and which whole feature pairs a chunk holds.
struct RankFeatureDesc {
  uint32_t tableOffset;
  uint32_t levels;
};
struct RankChunkDesc {
  uint32_t firstFeature, numFeatures;
  uint32_t tableBegin, tableEntries;
};

struct DeviceGroup {
  uint32_t nodeBegin;   // first node of the group in the packed node array
  uint32_t nodeCount;   // multiple of 2 so that the group is a whole number of 16-byte pieces
  uint32_t bundleBegin;
  uint32_t bundleCount;
  uint32_t uniformClass; // class id + 1 when every bundle of the group votes for one class, else 0
  uint32_t reserved[3];
};
static_assert(sizeof(DeviceGroup) == 32, "group descriptors are fetched with one 32-byte scalar load");

} // namespace tbamd
