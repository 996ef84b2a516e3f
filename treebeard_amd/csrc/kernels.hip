// Hand-written gfx950 kernels for decision-forest inference.
//
// They replace the kernels the reference generates from its schedules
// (src/gpu/GPUSchedules.cpp, src/mlir/CodeGenStateMachine.cpp:149-243 scalar
// tile step, src/mlir/WalkDecisionTreeLoweringPass.cpp:23-110 walk loops,
// src/gpu/GPURepresentations.cpp:279-399 row caching, src/mlir/LowerReduceOps.cpp
// :119-187 and :921-1003 reductions, src/mlir/LowerToMidLevelIR.cpp:554-648
// result initialisation and sigmoid).
#include "kernels.h"

#include <atomic>
#include <cmath>

namespace tbamd {

namespace {

__device__ __forceinline__ float AsFloat(uint32_t u) { return __uint_as_float(u); }

// LDS reads by absolute LDS address.  The kernels below use dynamic LDS only,
// which the compiler places at LDS address 0, so an offset into the dynamic
// array is the address itself and no base has to be added per access.
typedef uint32_t U32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t U32x4 __attribute__((ext_vector_type(4)));
typedef const __attribute__((address_space(3))) U32x2 *LdsNodePtr;
typedef const __attribute__((address_space(3))) float *LdsFloatPtr;
__device__ __forceinline__ U32x2 LdsLoadNode(uint32_t address) { return *(LdsNodePtr)(uintptr_t)address; }
__device__ __forceinline__ float LdsLoadFloat(uint32_t address) { return *(LdsFloatPtr)(uintptr_t)address; }
typedef const __attribute__((address_space(3))) uint8_t *LdsBytePtr;
__device__ __forceinline__ uint32_t LdsLoadByte(uint32_t address) { return *(LdsBytePtr)(uintptr_t)address; }
typedef const __attribute__((address_space(3))) uint16_t *LdsHalfPtr;
__device__ __forceinline__ uint32_t LdsLoadHalf(uint32_t address) { return *(LdsHalfPtr)(uintptr_t)address; }

// How a node's 16-bit feature offset addresses the row tile of the row-parallel kernel.
enum RowTileMode : int {
  kTileF32Bytes = 0, // f32 tile, offset in bytes
  kTileF32Words = 1, // f32 tile, offset in units of 4 bytes (tiles above 64 KB)
  kTileRankU8 = 2,   // one-byte rank tile (rank-quantised rows), offset in units of 4 bytes
  kTileRankU16 = 3   // two-byte rank tile [feature pair][row][2], offset in bytes
};
constexpr bool IsRankTile(int mode) { return mode == kTileRankU8 || mode == kTileRankU16; }

// A rank tile's comparison: the row's rank among the feature's thresholds against the node's threshold index.
template <int kMode>
__device__ __forceinline__ bool RankGoesLeft(uint32_t address, uint32_t thresholdIndex) {
  return (kMode == kTileRankU8 ? LdsLoadByte(address) : LdsLoadHalf(address)) <= thresholdIndex;
}


// Copies the block's rows (contiguous, row-major in global memory) into the LDS tile.
// kTransposed: tile[f * R + r] (row-parallel kernel), else tile[r * rowWords + f].
// Loads are 16-byte wide, issued kStageUnroll at a time per lane and unconditional (index
// clamped into the live part of the batch) so that they overlap; rows past the end of the
// batch read as 0 and nothing outside the batch is touched.
constexpr int kStageUnroll = 8;

template <bool kTransposed>
__device__ __forceinline__ void StageRows(const float *__restrict__ src, int valid, int R, int F, int rowWords,
                                          float *tile, int tid, int threads) {
  const int total = R * F;
  const int live = valid * F;
  const bool aligned = (reinterpret_cast<uintptr_t>(src) & 15u) == 0;
  const int vecs = aligned ? total >> 2 : 0;    // 16-byte pieces handled by the vector path
  const int liveVecs = aligned ? live >> 2 : 0; // pieces that lie entirely inside the batch
  const float invF = 1.0f / (float)F;
  typedef float F32x4 __attribute__((ext_vector_type(4)));
  const F32x4 *src4 = reinterpret_cast<const F32x4 *>(src);
  for (int base = 0; base < vecs; base += threads * kStageUnroll) {
    F32x4 v[kStageUnroll];
#pragma unroll
    for (int u = 0; u < kStageUnroll; ++u) {
      const int idx = base + u * threads + tid;
      const int clamped = idx < liveVecs ? idx : (liveVecs > 0 ? liveVecs - 1 : 0);
      v[u] = liveVecs > 0 ? src4[clamped] : F32x4{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int u = 0; u < kStageUnroll; ++u) {
      const int idx = base + u * threads + tid;
      if (idx >= vecs) continue;
      const int e0 = idx << 2;
      int r = (int)((float)e0 * invF);
      if (r * F > e0) --r;
      if ((r + 1) * F <= e0) ++r;
      int f = e0 - r * F;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int e = e0 + j;
        // elements of the one partially live piece are left to the scalar tail below
        if (idx < liveVecs || e >= live) {
          const float value = idx < liveVecs ? v[u][j] : 0.0f;
          if (kTransposed) tile[f * R + r] = value;
          else tile[r * rowWords + f] = value;
        }
        if (++f == F) { f = 0; ++r; }
      }
    }
  }
  // scalar: the live elements of the partially live piece, which the vector path skipped ...
  const int skippedEnd = live < (vecs << 2) ? live : (vecs << 2);
  for (int e = (liveVecs << 2) + tid; e < skippedEnd; e += threads) {
    const int r = e / F;
    const int f = e - r * F;
    if (kTransposed) tile[f * R + r] = src[e];
    else tile[r * rowWords + f] = src[e];
  }
  // ... and whatever lies behind the last whole 16-byte piece (everything, for unaligned input)
  for (int e = (vecs << 2) + tid; e < total; e += threads) {
    const int r = e / F;
    const int f = e - r * F;
    const float value = e < live ? src[e] : 0.0f;
    if (kTransposed) tile[f * R + r] = value;
    else tile[r * rowWords + f] = value;
  }
}

// ---------------------------------------------------------------------------
// Row-parallel walk.  The block owns `rowsPerBlock` rows, kept transposed in
// LDS (feature-major) so that lane i always reads bank i%64 no matter which
// feature its node tests.  Trees are streamed through LDS one group at a time:
// either the next group is fetched into registers while the current one is walked
// (PF > 0), or the group is copied by direct global-to-LDS loads between the two
// barriers of its round while the compute unit's other blocks walk (PF == 0).
// A lane walks K trees at a time in lock step: all lanes take `depth` steps and
// leaves hold the walk in place (see device_model.h), so the loop body has no
// leaf test and no divergence.  `treeThreads` lanes (in different waves) share
// one row and split each group's bundles between them, which buys occupancy
// without growing the row tile; their sums meet in an LDS cross-wave pass.
// Sums are kept in double; trees are added in packed order.
// ---------------------------------------------------------------------------
// kDefer (peeled walks, src/mlir/ProbabilityBasedTilingTransform.cpp:66-73, src/mlir/WalkDecisionTreeLoweringPass.cpp
// :231-315, the way this hardware wants them): the lock-step walk of a tree stops at the level a hit-count
// profile says it still pays (device_model.h: stubs).  A row that ends on a stub is queued by its wave as
// (row, tail node); whenever 64 entries have come together - whatever trees they belong to - the wave walks
// them on densely, one entry per lane, to their leaves, and hands the leaf values back to the rows' lanes
// through LDS.  The subtrees below the stubs are not part of the tree groups: the dense walk reads its nodes
// from global memory (they stay in L2), so the queue outlives the groups and is emptied once more at the end.
// Lock step spends its LDS reads on all 64 rows of a wave even when three of them still move; the queue spends
// 64 lanes on 64 rows that do, its node reads go through the vector memory path, which the walk leaves idle,
// and only its feature reads (at scattered addresses now) come out of LDS.
//
// kVariant picks what is compiled in beside the plain walk (each costs the plain walk about a percent when it
// is merely present): kWalkDump the leaf-id dump of the parity checks, kWalkDefer the deferred tails, kWalkFuse
// the classifiers' running arg-max (WalkScalars::fuseArgmax).
enum WalkVariant : int { kWalkPlain = 0, kWalkDump = 1, kWalkDefer = 2, kWalkFuse = 3 };

template <int K, int PF, int kMode, int kVariant>
__global__ void __launch_bounds__(1024)
WalkRowsLdsKernel(const float *__restrict__ x, const uint4 *__restrict__ nodes16,
                  const DeviceBundle *__restrict__ bundles, const DeviceNode *__restrict__ bundleRoots,
                  const DeviceGroup *__restrict__ groups,
                  const WalkScalars s, float *__restrict__ out, int8_t *__restrict__ classOut,
                  double *__restrict__ partial, int32_t *__restrict__ leafIds, const int32_t *__restrict__ nodeOrigin,
                  const int32_t *__restrict__ slotTree, const U32x2 *__restrict__ tailNodes, const int32_t *__restrict__ tailOrigin) {
  constexpr bool kDump = kVariant == kWalkDump, kDefer = kVariant == kWalkDefer, kFuse = kVariant == kWalkFuse;
  // LDS: [tree group nodes | transposed row tile].  The group sits at LDS
  // address 0 so that node pointers are LDS addresses as stored.
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x;
  const int threads = blockDim.x;
  const int RB = s.rowsPerBlock;
  const int TT = s.treeThreads;
  const int lane = tid & (RB - 1);
  // uniform inside a wave (RB is a multiple of 64); readfirstlane tells the compiler so
  const int tt = __builtin_amdgcn_readfirstlane(tid / RB);
  const int F = s.numFeatures;
  const int64_t row0 = (int64_t)blockIdx.x * RB;
  const int64_t remaining = s.rows - row0;
  const int valid = remaining < RB ? (int)remaining : RB;

  uint32_t column; // LDS address of this row's feature 0
  if (IsRankTile(kMode)) {
    // Ranks arrive already tiled: plain copy.  One byte each as [row block][feature][row] (the pad feature's
    // column is filled here), or two bytes each as [row block][feature pair][row][2], pad feature included.
    typedef uint32_t Piece __attribute__((ext_vector_type(4)));
    const int tileBytes = kMode == kTileRankU8 ? F * RB : ((F + 2) >> 1) * RB * 4;
    const Piece *src = reinterpret_cast<const Piece *>(reinterpret_cast<const uint8_t *>(x) + (int64_t)blockIdx.x * tileBytes);
    Piece *dst = reinterpret_cast<Piece *>(lds + s.groupRegionBytes);
    const int pieces = tileBytes >> 4;
    for (int base = 0; base < pieces; base += threads * kStageUnroll) {
      Piece v[kStageUnroll];
#pragma unroll
      for (int u = 0; u < kStageUnroll; ++u) {
        const int idx = base + u * threads + tid;
        v[u] = src[idx < pieces ? idx : pieces - 1];
      }
#pragma unroll
      for (int u = 0; u < kStageUnroll; ++u) {
        const int idx = base + u * threads + tid;
        if (idx < pieces) dst[idx] = v[u];
      }
    }
    if (kMode == kTileRankU8) {
      for (int i = tid; i < RB; i += threads) lds[s.groupRegionBytes + (uint32_t)F * RB + i] = 0; // pad feature: rank 0
      column = s.groupRegionBytes + (uint32_t)lane;
    } else {
      column = s.groupRegionBytes + (uint32_t)lane * 4u;
    }
  } else {
    float *rowTile = reinterpret_cast<float *>(lds + s.groupRegionBytes);
    // Stage the block's rows: coalesced reads of the contiguous row-major tile, transposed writes.
    StageRows<true>(x + row0 * F, valid, RB, F, 0, rowTile, tid, threads);
    for (int i = tid; i < RB; i += threads) rowTile[F * RB + i] = -INFINITY; // pad feature: keeps leaves in place
    column = s.groupRegionBytes + (uint32_t)lane * 4u;
  }
  // Deferred tails: the wave's queue of (row, node) entries, 128 of 4 bytes behind the row tile; while the wave
  // walks 64 of them on, the same 512 bytes take the leaf values on their way back (a double per lane).
  const uint32_t queueAddress = ((s.groupRegionBytes + (uint32_t)(F + 1) * RB * 4u + 15u) & ~15u) +
                                (uint32_t)__builtin_amdgcn_readfirstlane(tid >> 6) * kDeferBytesPerWave;
  uint32_t *queue = reinterpret_cast<uint32_t *>(lds + queueAddress);
  double *handBack = reinterpret_cast<double *>(lds + queueAddress);
  const uint32_t waveColumn = column - (uint32_t)(tid & 63) * 4u; // LDS address of feature 0 of the wave's first row
  const uint32_t laneTag = (uint32_t)(tid & 63) << 26;            // a queue entry: lane << 26 | tail index
  uint32_t queued = 0;                                            // entries in the queue (the same in every lane)

  const int slice = blockIdx.y;
  const int gBegin = (int)(((int64_t)s.numGroups * slice) / s.treeSlices);
  const int gEnd = (int)(((int64_t)s.numGroups * (slice + 1)) / s.treeSlices);
  const int C = s.numClasses;
  const int64_t row = row0 + lane;
  double *partialRow = partial ? partial + ((int64_t)slice * s.rows + row) * (C > 0 ? C : 1) : nullptr;
  // LDS cross-wave pass: the tree threads of a row leave their sums here and tree thread 0 adds
  // them in thread order.  Classifiers meet at class boundaries, while a tree group is live, so
  // their meeting area sits behind the row tile; otherwise the (then idle) group region is used.
  double *meet = reinterpret_cast<double *>(
      C > 0 ? lds + ((s.groupRegionBytes + (kMode == kTileRankU16 ? (uint32_t)((F + 2) >> 1) * RB * 4u
                                                                  : (uint32_t)(F + 1) * RB * (kMode == kTileRankU8 ? 1u : 4u)) + 7u) & ~7u)
            : lds);

  double acc = 0.0;
  int curClass = 0;
  float best = -INFINITY; // fuseArgmax: running maximum of the class sums and its class (tree thread 0)
  int bestClass = 0;

  // Register double buffer for the next tree group.  Loads are unconditional
  // (index clamped) so that they stay in flight across the walk.  PF == 0 is the other way of staging: no
  // registers, the group goes straight from global memory into LDS between the two barriers (below).
  U32x4 fetched[PF > 0 ? PF : 1];
#define TBAMD_PREFETCH_GROUP(NEXTGRP)                                                                                  \
  {                                                                                                                    \
    const DeviceGroup nextGrp = (NEXTGRP);                                                                             \
    const U32x4 *src = reinterpret_cast<const U32x4 *>(nodes16) + (nextGrp.nodeBegin >> 1);                            \
    const int last = (int)(nextGrp.nodeCount >> 1) - 1;                                                                \
    _Pragma("unroll") for (int i = 0; i < PF; ++i) {                                                                   \
      const int idx = tid + i * threads;                                                                               \
      fetched[i] = src[idx < last ? idx : last];                                                                       \
    }                                                                                                                  \
  }
  // Ends class `curClass`: the row's tree threads meet in LDS and thread 0 stores the class sum.
  // Uniform across the block (class boundaries are bundle positions), so the barriers are safe.
#define TBAMD_FLUSH_CLASS(UPTO)                                                                                        \
  {                                                                                                                    \
    if (TT > 1) {                                                                                                      \
      __syncthreads();                                                                                                 \
      meet[tid] = acc;                                                                                                 \
      __syncthreads();                                                                                                 \
      if (tt == 0) {                                                                                                   \
        acc = 0.0;                                                                                                     \
        for (int t = 0; t < TT; ++t) acc += meet[t * RB + lane];                                                       \
      }                                                                                                                \
    }                                                                                                                  \
    if (kFuse) {                                                                                                       \
      /* running arg-max with the generated code's tie rule (replace unless strictly greater); a class */              \
      /* without trees scores the initial value */                                                                     \
      const float m = (float)(s.initialValue + acc);                                                                   \
      if (!(best > m)) { best = m; bestClass = curClass; }                                                             \
      const float m0 = (float)s.initialValue;                                                                          \
      for (int c = curClass + 1; c < (UPTO); ++c)                                                                      \
        if (!(best > m0)) { best = m0; bestClass = c; }                                                                \
    } else if (tt == 0 && lane < valid) {                                                                              \
      partialRow[curClass] = acc;                                                                                      \
      for (int c = curClass + 1; c < (UPTO); ++c) partialRow[c] = 0.0;                                                 \
    }                                                                                                                  \
    acc = 0.0;                                                                                                         \
  }
  // Walks the first 64 (or fewer) entries of the wave's queue to their leaves, one entry per lane, and adds the
  // leaf values to the sums of the rows they belong to; what the queue holds beyond 64 moves to its front.  A
  // lane without an entry walks tail node 0, a leaf of value 0.  Only LDS accesses of this one wave touch the
  // queue, and a wave's LDS accesses complete in program order.
  const uint32_t tileShift = (uint32_t)__builtin_ctz((unsigned)RB) + 2u; // feature index -> byte offset in the row tile
#define TBAMD_WALK_QUEUE                                                                                               \
  {                                                                                                                    \
    const uint32_t me = (uint32_t)(tid & 63);                                                                          \
    const uint32_t take = queued < 64u ? queued : 64u;                                                                 \
    const uint32_t entry = me < take ? queue[me] : 0u;                                                                 \
    const uint32_t later = 64u + me < queued ? queue[64u + me] : 0u;                                                   \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                                             \
    __builtin_amdgcn_wave_barrier();                                                                                   \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");                                                             \
    handBack[me] = 0.0;                                                                                                \
    uint32_t at = entry & kStubIndexMask;                                                                              \
    const uint32_t owner = entry >> 26;                                                                                \
    const uint32_t ownerColumn = waveColumn + owner * 4u;                                                              \
    U32x2 node = tailNodes[at];                                                                                        \
    for (int d = 0; d < s.tailDepth; ++d) {                                                                            \
      const bool left = LdsLoadFloat(ownerColumn + ((node.y & ((1u << kTailFeatureBits) - 1u)) << tileShift)) < AsFloat(node.x); \
      const uint32_t next = (node.y >> kTailFeatureBits) + (left ? 0u : 1u);                                           \
      const bool moved = next != at;                                                                                   \
      at = next;                                                                                                       \
      if (!__any(moved)) break;                                                                                        \
      node = tailNodes[at];                                                                                            \
    }                                                                                                                  \
    const double leafValue = (double)AsFloat(node.x);                                                                  \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                                             \
    __builtin_amdgcn_wave_barrier();                                                                                   \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");                                                             \
    if (me < take) __hip_atomic_fetch_add(&handBack[owner], leafValue, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WAVEFRONT); \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                                             \
    __builtin_amdgcn_wave_barrier();                                                                                   \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");                                                             \
    acc += handBack[me];                                                                                               \
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");                                                             \
    __builtin_amdgcn_wave_barrier();                                                                                   \
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");                                                             \
    if (64u + me < queued) queue[me] = later;                                                                          \
    queued = queued > 64u ? queued - 64u : 0u;                                                                         \
  }
  if (PF > 0 && gBegin < gEnd) TBAMD_PREFETCH_GROUP(groups[gBegin])

  for (int g = gBegin; g < gEnd; ++g) {
    const DeviceGroup grp = groups[g];
    __syncthreads(); // rows staged / previous group no longer read
    if (PF > 0) {
      U32x4 *dst = reinterpret_cast<U32x4 *>(lds);
      const int pieces = (int)(grp.nodeCount >> 1);
#pragma unroll
      for (int i = 0; i < PF; ++i) {
        const int idx = tid + i * threads;
        if (idx < pieces) dst[idx] = fetched[i];
      }
    } else {
      // Direct staging: the group is copied by global -> LDS loads (lane i of a wave-wide load leaves its 16 bytes
      // at base + 16 i, lanes switched off write nothing): no staging registers, no LDS store instructions.  The
      // block waits for its own copy; the CU's other block walks meanwhile, which is why launch plans ask for
      // this form only when two blocks fit a CU.
      const U32x4 *src = reinterpret_cast<const U32x4 *>(nodes16) + (grp.nodeBegin >> 1);
      const int pieces = (int)(grp.nodeCount >> 1);
      const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
      for (int first = wave * 64; first < pieces; first += threads)
        if (first + (tid & 63) < pieces)
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src + first + (tid & 63)),
                                           (__attribute__((address_space(3))) void *)(lds + (uint32_t)first * 16u), 16, 0, 0);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();
    if (PF > 0 && g + 1 < gEnd) TBAMD_PREFETCH_GROUP(groups[g + 1]) // in flight while this group is walked

    // Walking waves go before waves that are staging (this block's or the other block's on the CU): the walk is
    // what keeps the LDS and the VALUs busy.
    __builtin_amdgcn_s_setprio(1);
    // Bundles are sorted by class; a segment is a run of bundles of one class.
    uint32_t b0 = 0;
    while (b0 < grp.bundleCount) {
      uint32_t b1 = grp.bundleCount;
      if (C > 0) {
        // most groups vote for one class: the descriptor says so and no bundle has to be looked at
        const int cls = grp.uniformClass ? (int)grp.uniformClass - 1 : (int)bundles[grp.bundleBegin + b0].classId;
        if (cls != curClass) { // classes arrive in ascending order
          TBAMD_FLUSH_CLASS(cls)
          curClass = cls;
        }
        if (!grp.uniformClass) {
          b1 = b0 + 1;
          while (b1 < grp.bundleCount && (int)bundles[grp.bundleBegin + b1].classId == cls) ++b1;
        }
      }
      for (uint32_t b = b0 + tt; b < b1; b += TT) {
        const DeviceBundle bd = bundles[grp.bundleBegin + b];
        uint32_t addr[K];
#pragma unroll
        for (int k = 0; k < K; ++k) addr[k] = bd.root[k];
        const int depth = (int)bd.depth;
        // Level 0 of the f32 tiles: copies of the root nodes sit next to the bundles and arrive in scalar
        // registers, only the feature is read from LDS.  A root that is a leaf holds the walk in place like any other leaf, so the step is safe
        // for depth 0.  (On rank tiles, whose rounds are latency-bound, the extra scalar load did not pay.)
        if (kMode != kTileRankU8) {
          const DeviceNode *roots = bundleRoots + (size_t)(grp.bundleBegin + b) * K;
#pragma unroll
          for (int k = 0; k < K; ++k) {
            const DeviceNode root = roots[k];
            const uint32_t off = kMode == kTileF32Words ? (root.meta & 0xFFFFu) << 2 : (root.meta & 0xFFFFu);
            bool left;
            if (kMode == kTileRankU16) left = RankGoesLeft<kMode>(column + off, __float_as_uint(root.value));
            else left = LdsLoadFloat(column + off) < root.value;
            addr[k] = (root.meta >> 16) + (left ? 0u : kNodeBytes);
          }
        }
#pragma unroll 2
        for (int d = kMode != kTileRankU8 ? 1 : 0; d < depth; ++d) {
#pragma unroll
          for (int k = 0; k < K; ++k) {
            const U32x2 node = LdsLoadNode(addr[k]);
            const uint32_t off = kMode == kTileF32Bytes || kMode == kTileRankU16 ? (node.y & 0xFFFFu) : (node.y & 0xFFFFu) << 2;
            bool left;
            if (IsRankTile(kMode)) left = RankGoesLeft<kMode>(column + off, node.x); // rank <= threshold index
            else left = LdsLoadFloat(column + off) < AsFloat(node.x);
            addr[k] = (node.y >> 16) + (left ? 0u : kNodeBytes);
          }
        }
        if (kDefer && bd.hasStubs) {
          // rows on a stub are queued, the others add their leaf; the queue is walked on as soon as it holds a wave's worth
          float value[K];
#pragma unroll
          for (int k = 0; k < K; ++k) value[k] = LdsLoadFloat(addr[k]);
#pragma unroll
          for (int k = 0; k < K; ++k) {
            const bool stub = __builtin_amdgcn_classf(value[k], 0x3); // a stub's value is a NaN (no leaf's is)
            acc += (double)(stub ? 0.0f : value[k]);
            const uint64_t who = __ballot(stub);
            if (who != 0) {
              const uint32_t before = __builtin_amdgcn_mbcnt_hi((uint32_t)(who >> 32), __builtin_amdgcn_mbcnt_lo((uint32_t)who, 0u));
              // entry: the NaN's payload (index of the node the stub stands for) below the lane's number
              if (stub) queue[queued + before] = (__float_as_uint(value[k]) & kStubIndexMask) | laneTag;
              queued += (uint32_t)__builtin_popcountll(who);
              if (queued >= 64u) TBAMD_WALK_QUEUE
            }
          }
        } else {
          if (kDump && s.deferTails && bd.hasStubs) {
            // the dump walks the rows that stand on a stub on at once, each lane for itself, through the tail array
#pragma unroll
            for (int k = 0; k < K; ++k) {
              const float stop = LdsLoadFloat(addr[k]);
              if (__builtin_amdgcn_classf(stop, 0x3)) {
                uint32_t at = __float_as_uint(stop) & kStubIndexMask;
                U32x2 node = tailNodes[at];
                for (int d = 0; d < s.tailDepth; ++d) {
                  const bool left = LdsLoadFloat(column + ((node.y & ((1u << kTailFeatureBits) - 1u)) << tileShift)) < AsFloat(node.x);
                  at = (node.y >> kTailFeatureBits) + (left ? 0u : 1u);
                  node = tailNodes[at];
                }
                acc += (double)AsFloat(node.x);
                const int tree = slotTree[bd.firstSlot + k];
                if (lane < valid && tree >= 0) leafIds[row * s.numTrees + tree] = tailOrigin[at];
                addr[k] = 0; // (the null leaf: adds 0 below and names no tree's node)
              }
            }
          }
#pragma unroll
          for (int k = 0; k < K; ++k) acc += (double)LdsLoadFloat(addr[k]);
        }
        if (kDump) {
          if (lane < valid) {
#pragma unroll
            for (int k = 0; k < K; ++k) {
              const int tree = slotTree[bd.firstSlot + k];
              if (tree >= 0 && !(s.deferTails && addr[k] == 0u))
                leafIds[row * s.numTrees + tree] = nodeOrigin[grp.nodeBegin + addr[k] / kNodeBytes];
            }
          }
        }
      }
      b0 = b1;
    }
    __builtin_amdgcn_s_setprio(0);
  }
  if (kDefer) // what is still queued is walked on now
    while (queued > 0u) TBAMD_WALK_QUEUE

  if (C > 0) {
    TBAMD_FLUSH_CLASS(C)
    if (kFuse && tt == 0 && lane < valid) {
      if (classOut) classOut[row] = (int8_t)bestClass;
      else out[row] = (float)bestClass;
    }
    return;
  }
  if (TT > 1) {
    __syncthreads();
    meet[tid] = acc;
    __syncthreads();
    if (tt != 0) return;
    acc = 0.0;
    for (int t = 0; t < TT; ++t) acc += meet[t * RB + lane];
  }
  if (lane >= valid) return;
  if (partial) {
    partialRow[0] = acc;
  } else {
    const double margin = s.initialValue + acc;
    out[row] = (float)(s.transform == 1 ? 1.0 / (1.0 + exp(-margin)) : margin);
  }
#undef TBAMD_FLUSH_CLASS
#undef TBAMD_PREFETCH_GROUP
#undef TBAMD_WALK_QUEUE
}

// ---------------------------------------------------------------------------
// Row-parallel walk over TILED trees (tiles of T = 2 to 8 nodes, layout in device_model.h): the
// reference's tile step (src/mlir/CodeGenStateMachine.cpp:284-506, cooperative GPU form
// src/gpu/GPUSimtPass.cpp:39-133) as branch-free per-lane code.  One step reads the tile (thresholds,
// feature offsets, child base and the tile's own child-select row) with one to four wide LDS reads, gathers
// the T feature values of the lane's row, turns the T comparisons into an outcome word (node i in bit i)
// and picks the child out of the select row with one shift (tiles of up to 4 nodes) or by following the
// tile's links (the eight-slot tile of tile sizes 5 to 8).  Leaves are tiles that select themselves, so a
// bundle walks `depth` tile steps without a leaf test.  Block shape, row tile, tree groups (staged by direct
// global-to-LDS copies), tree threads, class flush and epilogue are those of WalkRowsLdsKernel.
//
// Bundles carry a peel depth (taken from a hit-count profile: the steps that bring 90 % of the profiled
// rows to a leaf, src/mlir/ProbabilityBasedTilingTransform.cpp:66-73; equal to the depth without one): the
// walk takes that many steps blind and then goes on only while some lane of the wave still moves, at most to
// the full depth.
// ---------------------------------------------------------------------------
typedef const __attribute__((address_space(3))) U32x4 *LdsQuadPtr;
__device__ __forceinline__ U32x4 LdsLoadQuad(uint32_t address) { return *(LdsQuadPtr)(uintptr_t)address; }

template <int T> // 2, 3, 4, or kMaxTileSize for the eight-slot tile of tile sizes 5 to 8
__device__ __forceinline__ uint32_t TileStep(uint32_t addr, uint32_t column, int hops) {
  static_assert(T >= 2 && (T <= kMaxSelectTile || T == kMaxTileSize), "tile sizes 5 to 8 share the eight-slot tile");
  float thr[T];
  uint32_t off[T];
  uint32_t childBase;
  uint64_t select; // the child-select row, or the links of the eight-slot tile
  if constexpr (T == 2) {
    const U32x4 q = LdsLoadQuad(addr);
    thr[0] = AsFloat(q.x), thr[1] = AsFloat(q.y);
    off[0] = q.z & 0xFFFFu, off[1] = q.z >> 16;
    childBase = q.w & 0xFFFFu;
    select = q.w >> 16;
  } else if constexpr (T == 3) {
    const U32x2 a = LdsLoadNode(addr), b = LdsLoadNode(addr + 8), c = LdsLoadNode(addr + 16);
    thr[0] = AsFloat(a.x), thr[1] = AsFloat(a.y), thr[2] = AsFloat(b.x);
    off[0] = b.y & 0xFFFFu, off[1] = b.y >> 16, off[2] = c.x & 0xFFFFu;
    childBase = c.x >> 16;
    select = c.y & 0xFFFFu;
  } else if constexpr (T == 4) {
    const U32x4 q0 = LdsLoadQuad(addr), q1 = LdsLoadQuad(addr + 16);
    thr[0] = AsFloat(q0.x), thr[1] = AsFloat(q0.y), thr[2] = AsFloat(q0.z), thr[3] = AsFloat(q0.w);
    off[0] = q1.x & 0xFFFFu, off[1] = q1.x >> 16, off[2] = q1.y & 0xFFFFu, off[3] = q1.y >> 16;
    childBase = q1.z & 0xFFFFu;
    select = (uint64_t)(q1.z >> 16) | ((uint64_t)q1.w << 16);
  } else {
    const U32x4 q0 = LdsLoadQuad(addr), q1 = LdsLoadQuad(addr + 16), q2 = LdsLoadQuad(addr + 32), q3 = LdsLoadQuad(addr + 48);
    thr[0] = AsFloat(q0.x), thr[1] = AsFloat(q0.y), thr[2] = AsFloat(q0.z), thr[3] = AsFloat(q0.w);
    thr[4] = AsFloat(q1.x), thr[5] = AsFloat(q1.y), thr[6] = AsFloat(q1.z), thr[7] = AsFloat(q1.w);
    off[0] = q2.x & 0xFFFFu, off[1] = q2.x >> 16, off[2] = q2.y & 0xFFFFu, off[3] = q2.y >> 16;
    off[4] = q2.z & 0xFFFFu, off[5] = q2.z >> 16, off[6] = q2.w & 0xFFFFu, off[7] = q2.w >> 16;
    select = (uint64_t)q3.x | ((uint64_t)q3.y << 32);
    childBase = q3.z & 0xFFFFu;
  }
  if constexpr (T > kMaxSelectTile) {
    // The eight comparisons pick, slot by slot, the link the slot sends its row along: nibble s of the high word
    // of `select` when slot s sends the row left, nibble s of the low word otherwise (one bit-field insert under a
    // mask of eight nibbles).  Then the links are followed from slot 0: a link below kTileLinkExit names the next
    // slot (link + 1), the others the child; a tile holds `hops` levels of nodes, so `hops` links reach a child.
    uint32_t wentLeft = 0;
#pragma unroll
    for (int i = 0; i < T; ++i) {
      const float x = LdsLoadFloat(column + off[i]);
      wentLeft |= x < thr[i] ? 0xFu << (4 * i) : 0u;
    }
    const uint32_t taken = ((uint32_t)(select >> 32) & wentLeft) | ((uint32_t)select & ~wentLeft);
    uint32_t link = taken & 15u;
    for (int hop = 1; hop < hops; ++hop) {
      const uint32_t next = __builtin_amdgcn_ubfe(taken, (link + 1u) << 2, 4u); // (the field offset wraps at 32 for a link that names a child: ignored below)
      link = link < kTileLinkExit ? next : link;
    }
    return childBase + (link - kTileLinkExit) * TileBytes(T);
  } else {
    uint32_t outcome = 0;
#pragma unroll
    for (int i = 0; i < T; ++i) {
      const float x = LdsLoadFloat(column + off[i]);
      outcome |= (x < thr[i] ? 1u : 0u) << i;
    }
    const uint32_t child = (uint32_t)(select >> (outcome * TileSelectBits(T))) & ((1u << TileSelectBits(T)) - 1u);
    return childBase + child * TileBytes(T);
  }
}

template <int T, int K, int kVariant> // kVariant: kWalkPlain, kWalkDump or kWalkFuse (the peel tail is always there)
__global__ void __launch_bounds__(1024)
WalkRowsTiledKernel(const float *__restrict__ x, const uint4 *__restrict__ nodes16,
                    const DeviceBundle *__restrict__ bundles, const DeviceGroup *__restrict__ groups,
                    const WalkScalars s, float *__restrict__ out, int8_t *__restrict__ classOut,
                    double *__restrict__ partial, int32_t *__restrict__ leafIds, const int32_t *__restrict__ nodeOrigin,
                    const int32_t *__restrict__ slotTree) {
  constexpr bool kDump = kVariant == kWalkDump, kFuse = kVariant == kWalkFuse;
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x;
  const int threads = blockDim.x;
  const int RB = s.rowsPerBlock;
  const int TT = s.treeThreads;
  const int lane = tid & (RB - 1);
  const int tt = __builtin_amdgcn_readfirstlane(tid / RB);
  const int F = s.numFeatures;
  const int64_t row0 = (int64_t)blockIdx.x * RB;
  const int64_t remaining = s.rows - row0;
  const int valid = remaining < RB ? (int)remaining : RB;

  float *rowTile = reinterpret_cast<float *>(lds + s.groupRegionBytes);
  StageRows<true>(x + row0 * F, valid, RB, F, 0, rowTile, tid, threads);
  for (int i = tid; i < RB; i += threads) rowTile[F * RB + i] = -INFINITY; // pad feature: keeps leaves in place
  const uint32_t column = s.groupRegionBytes + (uint32_t)lane * 4u;

  const int slice = blockIdx.y;
  const int gBegin = (int)(((int64_t)s.numGroups * slice) / s.treeSlices);
  const int gEnd = (int)(((int64_t)s.numGroups * (slice + 1)) / s.treeSlices);
  const int C = s.numClasses;
  const int64_t row = row0 + lane;
  double *partialRow = partial ? partial + ((int64_t)slice * s.rows + row) * (C > 0 ? C : 1) : nullptr;
  double *meet = reinterpret_cast<double *>(C > 0 ? lds + ((s.groupRegionBytes + (uint32_t)(F + 1) * RB * 4u + 7u) & ~7u) : lds);

  double acc = 0.0;
  int curClass = 0;
  float best = -INFINITY; // fuseArgmax: running maximum of the class sums and its class (tree thread 0)
  int bestClass = 0;
#define TBAMD_FLUSH_CLASS(UPTO)                                                                                        \
  {                                                                                                                    \
    if (TT > 1) {                                                                                                      \
      __syncthreads();                                                                                                 \
      meet[tid] = acc;                                                                                                 \
      __syncthreads();                                                                                                 \
      if (tt == 0) {                                                                                                   \
        acc = 0.0;                                                                                                     \
        for (int t = 0; t < TT; ++t) acc += meet[t * RB + lane];                                                       \
      }                                                                                                                \
    }                                                                                                                  \
    if (kFuse) {                                                                                                \
      /* running arg-max with the generated code's tie rule (replace unless strictly greater); a class */              \
      /* without trees scores the initial value */                                                                     \
      const float m = (float)(s.initialValue + acc);                                                                   \
      if (!(best > m)) { best = m; bestClass = curClass; }                                                             \
      const float m0 = (float)s.initialValue;                                                                          \
      for (int c = curClass + 1; c < (UPTO); ++c)                                                                      \
        if (!(best > m0)) { best = m0; bestClass = c; }                                                                \
    } else if (tt == 0 && lane < valid) {                                                                              \
      partialRow[curClass] = acc;                                                                                      \
      for (int c = curClass + 1; c < (UPTO); ++c) partialRow[c] = 0.0;                                                 \
    }                                                                                                                  \
    acc = 0.0;                                                                                                         \
  }
  for (int g = gBegin; g < gEnd; ++g) {
    const DeviceGroup grp = groups[g];
    __syncthreads();
    {
      // The group goes straight from global memory into LDS (lane i of a wave-wide load leaves its 16 bytes at
      // base + 16 i, lanes switched off write nothing), as in the scalar kernel's direct form.
      const U32x4 *src = reinterpret_cast<const U32x4 *>(nodes16) + (grp.nodeBegin >> 1);
      const int pieces = (int)(grp.nodeCount >> 1);
      const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
      for (int first = wave * 64; first < pieces; first += threads)
        if (first + (tid & 63) < pieces)
          __builtin_amdgcn_global_load_lds((const __attribute__((address_space(1))) void *)(src + first + (tid & 63)),
                                           (__attribute__((address_space(3))) void *)(lds + (uint32_t)first * 16u), 16, 0, 0);
      asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    __syncthreads();

    uint32_t b0 = 0;
    while (b0 < grp.bundleCount) {
      uint32_t b1 = grp.bundleCount;
      if (C > 0) {
        const int cls = grp.uniformClass ? (int)grp.uniformClass - 1 : (int)bundles[grp.bundleBegin + b0].classId;
        if (cls != curClass) {
          TBAMD_FLUSH_CLASS(cls)
          curClass = cls;
        }
        if (!grp.uniformClass) {
          b1 = b0 + 1;
          while (b1 < grp.bundleCount && (int)bundles[grp.bundleBegin + b1].classId == cls) ++b1;
        }
      }
      for (uint32_t b = b0 + tt; b < b1; b += TT) {
        const DeviceBundle bd = bundles[grp.bundleBegin + b];
        uint32_t addr[K];
#pragma unroll
        for (int k = 0; k < K; ++k) addr[k] = bd.root[k];
        const int depth = (int)bd.depth;
        const int blind = (int)bd.peelDepth;
        for (int d = 0; d < blind; ++d) {
#pragma unroll
          for (int k = 0; k < K; ++k) addr[k] = TileStep<T>(addr[k], column, s.tileHops);
        }
        for (int d = blind; d < depth; ++d) {
          bool moved = false;
#pragma unroll
          for (int k = 0; k < K; ++k) {
            const uint32_t next = TileStep<T>(addr[k], column, s.tileHops);
            moved = moved || next != addr[k];
            addr[k] = next;
          }
          if (!__any(moved)) break; // every lane of the wave sits on a leaf tile (leaves select themselves)
        }
#pragma unroll
        for (int k = 0; k < K; ++k) acc += (double)LdsLoadFloat(addr[k]);
        if (kDump) {
          if (lane < valid) {
#pragma unroll
            for (int k = 0; k < K; ++k) {
              const int tree = slotTree[bd.firstSlot + k];
              if (tree >= 0) leafIds[row * s.numTrees + tree] = nodeOrigin[grp.nodeBegin + addr[k] / kNodeBytes];
            }
          }
        }
      }
      b0 = b1;
    }
  }

  if (C > 0) {
    TBAMD_FLUSH_CLASS(C)
    if (kFuse && tt == 0 && lane < valid) {
      if (classOut) classOut[row] = (int8_t)bestClass;
      else out[row] = (float)bestClass;
    }
    return;
  }
  if (TT > 1) {
    __syncthreads();
    meet[tid] = acc;
    __syncthreads();
    if (tt != 0) return;
    acc = 0.0;
    for (int t = 0; t < TT; ++t) acc += meet[t * RB + lane];
  }
  if (lane >= valid) return;
  if (partial) {
    partialRow[0] = acc;
  } else {
    const double margin = s.initialValue + acc;
    out[row] = (float)(s.transform == 1 ? 1.0 / (1.0 + exp(-margin)) : margin);
  }
#undef TBAMD_FLUSH_CLASS
}

// ---------------------------------------------------------------------------
// Tree-parallel walk.  The block keeps `rowsPerBlock` rows row-major in LDS and
// gives each row `treeLanes` lanes; lane j of a row walks bundles j, j+treeLanes,
// ... of the staged tree group, so a row's trees are shared between its lanes.
// The lanes' partial sums are combined with a wave-level butterfly (lanes of a
// row are contiguous), then across waves through LDS when a row spans several
// waves.  One lane per row owns the row's per-class accumulators in LDS, which
// keeps the summation order fixed.  Used when a row is too wide to transpose
// 64 of them into LDS, and when the batch has too few rows to fill the chip
// with one lane per row.
// ---------------------------------------------------------------------------
// One butterfly step on doubles.  Partners 1, 2, 4 and 8 lanes away are reached with DPP operand swizzles
// inside the VALU (quad permutes, the mirror of half a row and of a row: after the steps before them every
// lane of the mirrored group already holds the same partial sum, so the mirror partner is as good as the
// xor partner); only the steps across rows of 16 lanes go through the LDS crossbar (ds_bpermute).
template <int kDppCtrl>
__device__ __forceinline__ double DppMove(double v) {
  int lo = __double2loint(v), hi = __double2hiint(v);
  lo = __builtin_amdgcn_update_dpp(0, lo, kDppCtrl, 0xF, 0xF, false);
  hi = __builtin_amdgcn_update_dpp(0, hi, kDppCtrl, 0xF, 0xF, false);
  return __hiloint2double(hi, lo);
}

__device__ __forceinline__ double ShuffleXor(double v, int mask) {
  switch (mask) {
  case 1: return DppMove<0xB1>(v);  // quad_perm [1,0,3,2]
  case 2: return DppMove<0x4E>(v);  // quad_perm [2,3,0,1]
  case 4: return DppMove<0x141>(v); // row_half_mirror
  case 8: return DppMove<0x140>(v); // row_mirror
  default: break;
  }
  int lo = __double2loint(v), hi = __double2hiint(v);
  lo = __shfl_xor(lo, mask, 64);
  hi = __shfl_xor(hi, mask, 64);
  return __hiloint2double(hi, lo);
}

template <int K, int PF, bool kDump>
__global__ void __launch_bounds__(1024)
WalkTreeParallelKernel(const float *__restrict__ x, const uint4 *__restrict__ nodes16,
                       const DeviceBundle *__restrict__ bundles, const DeviceGroup *__restrict__ groups,
                       const WalkScalars s, float *__restrict__ out, double *__restrict__ partial,
                       int32_t *__restrict__ leafIds, const int32_t *__restrict__ nodeOrigin,
                       const int32_t *__restrict__ slotTree) {
  // LDS: [tree group nodes | rows, (F+1) floats each | cross-wave scratch | per-row class sums]
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x;
  const int threads = blockDim.x;
  const int F = s.numFeatures;
  const int R = s.rowsPerBlock;
  const int TL = s.treeLanes;
  const int r = tid / TL;
  const int j = tid - r * TL;
  const int C = s.numClasses;
  const int Cn = C > 0 ? C : 1;
  const int64_t row0 = (int64_t)blockIdx.x * R;
  const int64_t remaining = s.rows - row0;
  const int valid = remaining < R ? (int)remaining : R;
  const int rowWords = F + 1;

  float *rowsLds = reinterpret_cast<float *>(lds + s.groupRegionBytes);
  const uint32_t scratchOffset = (s.groupRegionBytes + (uint32_t)R * rowWords * 4u + 7u) & ~7u;
  double *waveScratch = reinterpret_cast<double *>(lds + scratchOffset);
  double *classSums = waveScratch + (threads + 63) / 64;

  StageRows<false>(x + row0 * F, valid, R, F, rowWords, rowsLds, tid, threads);
  for (int rr = tid; rr < R; rr += threads) rowsLds[rr * rowWords + F] = -INFINITY;
  for (int i = tid; i < R * Cn; i += threads) classSums[i] = 0.0;
  const uint32_t rowBase = s.groupRegionBytes + (uint32_t)r * rowWords * 4u;

  const int slice = blockIdx.y;
  const int gBegin = (int)(((int64_t)s.numGroups * slice) / s.treeSlices);
  const int gEnd = (int)(((int64_t)s.numGroups * (slice + 1)) / s.treeSlices);
  const int64_t row = row0 + r;

  // Register double buffer for the next tree group (loads stay in flight across the walk).
  U32x4 fetched[PF];
#define TBAMD_PREFETCH_GROUP(NEXTGRP)                                                                                  \
  {                                                                                                                    \
    const DeviceGroup nextGrp = (NEXTGRP);                                                                             \
    const U32x4 *src = reinterpret_cast<const U32x4 *>(nodes16) + (nextGrp.nodeBegin >> 1);                            \
    const int last = (int)(nextGrp.nodeCount >> 1) - 1;                                                                \
    _Pragma("unroll") for (int i = 0; i < PF; ++i) {                                                                   \
      const int idx = tid + i * threads;                                                                               \
      fetched[i] = src[idx < last ? idx : last];                                                                       \
    }                                                                                                                  \
  }
  if (gBegin < gEnd) TBAMD_PREFETCH_GROUP(groups[gBegin])

  for (int g = gBegin; g < gEnd; ++g) {
    const DeviceGroup grp = groups[g];
    __syncthreads();
    {
      U32x4 *dst = reinterpret_cast<U32x4 *>(lds);
      const int pieces = (int)(grp.nodeCount >> 1);
#pragma unroll
      for (int i = 0; i < PF; ++i) {
        const int idx = tid + i * threads;
        if (idx < pieces) dst[idx] = fetched[i];
      }
    }
    __syncthreads();
    if (g + 1 < gEnd) TBAMD_PREFETCH_GROUP(groups[g + 1])

    // bundles are sorted by class: handle one class segment at a time
    uint32_t b0 = 0;
    while (b0 < grp.bundleCount) {
      const int cls = bundles[grp.bundleBegin + b0].classId;
      uint32_t b1 = b0 + 1;
      while (b1 < grp.bundleCount && bundles[grp.bundleBegin + b1].classId == cls) ++b1;

      double acc = 0.0;
      for (uint32_t b = b0 + j; b < b1; b += TL) {
        const DeviceBundle bd = bundles[grp.bundleBegin + b];
        uint32_t addr[K];
#pragma unroll
        for (int k = 0; k < K; ++k) addr[k] = bd.root[k];
        const int depth = bd.depth;
        for (int d = 0; d < depth; ++d) {
#pragma unroll
          for (int k = 0; k < K; ++k) {
            const U32x2 node = LdsLoadNode(addr[k]);
            const float xv = LdsLoadFloat(rowBase + (node.y & 0xFFFFu));
            addr[k] = (node.y >> 16) + (xv < AsFloat(node.x) ? 0u : kNodeBytes);
          }
        }
#pragma unroll
        for (int k = 0; k < K; ++k) acc += (double)LdsLoadFloat(addr[k]);
        if (kDump) {
          if (r < valid) {
#pragma unroll
            for (int k = 0; k < K; ++k) {
              const int tree = slotTree[bd.firstSlot + k];
              if (tree >= 0) leafIds[row * s.numTrees + tree] = nodeOrigin[grp.nodeBegin + addr[k] / kNodeBytes];
            }
          }
        }
      }

      // combine the lanes of each row: butterfly inside the wave ...
      const int inWave = TL < 64 ? TL : 64;
      for (int m = 1; m < inWave; m <<= 1) acc += ShuffleXor(acc, m); // (ascending: see ShuffleXor)
      if (TL > 64) { // ... then across the row's waves through LDS
        __syncthreads();
        if ((tid & 63) == 0) waveScratch[tid >> 6] = acc;
        __syncthreads();
        if (j == 0) {
          acc = 0.0;
          for (int w = 0; w < TL / 64; ++w) acc += waveScratch[(tid >> 6) + w];
        }
      }
      if (j == 0) classSums[r * Cn + cls] += acc;
      b0 = b1;
    }
  }

  if (j != 0 || r >= valid) return;
  if (C > 0 || partial) {
    double *dst = partial + ((int64_t)slice * s.rows + row) * Cn;
    for (int c = 0; c < Cn; ++c) dst[c] = classSums[r * Cn + c];
  } else {
    const double margin = s.initialValue + classSums[r];
    out[row] = (float)(s.transform == 1 ? 1.0 / (1.0 + exp(-margin)) : margin);
  }
#undef TBAMD_PREFETCH_GROUP
}

// ---------------------------------------------------------------------------
// Global-memory walk: the fallback for forests with a tree that does not fit one LDS group.  One
// lane per row; nodes (16 bytes, absolute child indices) and row values are read from global memory
// through L1/L2, K trees at a time in lock step with an explicit leaf test.  Same accumulation,
// class flush and tree-slice scheme as the LDS kernels.
// ---------------------------------------------------------------------------
template <int K, bool kDump>
__global__ void __launch_bounds__(1024)
WalkGlobalKernel(const float *__restrict__ x, const DeviceGlobalNode *__restrict__ nodes,
                 const DeviceGlobalTree *__restrict__ trees, const WalkScalars s, float *__restrict__ out,
                 double *__restrict__ partial, int32_t *__restrict__ leafIds) {
  const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const bool valid = row < s.rows;
  const float *xr = x + (valid ? row : s.rows - 1) * s.numFeatures;
  const int slice = blockIdx.y;
  const int tBegin = (int)(((int64_t)s.numTrees * slice) / s.treeSlices);
  const int tEnd = (int)(((int64_t)s.numTrees * (slice + 1)) / s.treeSlices);
  const int C = s.numClasses;
  double *partialRow = partial ? partial + ((int64_t)slice * s.rows + (valid ? row : 0)) * (C > 0 ? C : 1) : nullptr;
  typedef uint32_t Quad __attribute__((ext_vector_type(4)));
  const Quad *nodeQuads = reinterpret_cast<const Quad *>(nodes);

  double acc = 0.0;
  int curClass = 0;
  for (int t0 = tBegin; t0 < tEnd; t0 += K) {
    uint32_t n[K];
    uint32_t depth = 0;
#pragma unroll
    for (int k = 0; k < K; ++k) {
      const int t = t0 + k < tEnd ? t0 + k : tEnd - 1; // the tail repeats the last tree; its result is dropped
      n[k] = trees[t].root;
      depth = trees[t].depth > depth ? trees[t].depth : depth;
    }
    for (uint32_t d = 0; d < depth; ++d) {
#pragma unroll
      for (int k = 0; k < K; ++k) {
        const Quad node = nodeQuads[n[k]];
        if (node.y != kGlobalLeaf) n[k] = node.z + (xr[node.y] < AsFloat(node.x) ? 0u : 1u);
      }
    }
#pragma unroll
    for (int k = 0; k < K; ++k) {
      if (t0 + k >= tEnd) break;
      const DeviceGlobalTree tree = trees[t0 + k];
      const Quad leaf = nodeQuads[n[k]];
      if (C > 0 && (int)tree.classId != curClass) { // classes arrive in ascending order
        if (valid) {
          partialRow[curClass] = acc;
          for (int c = curClass + 1; c < (int)tree.classId; ++c) partialRow[c] = 0.0;
        }
        acc = 0.0;
        curClass = (int)tree.classId;
      }
      acc += (double)AsFloat(leaf.x);
      if (kDump && valid) leafIds[row * s.numTrees + tree.origin] = (int32_t)leaf.w;
    }
  }
  if (!valid) return;
  if (C > 0) {
    partialRow[curClass] = acc;
    for (int c = curClass + 1; c < C; ++c) partialRow[c] = 0.0;
  } else if (partial) {
    partialRow[0] = acc;
  } else {
    const double margin = s.initialValue + acc;
    out[row] = (float)(s.transform == 1 ? 1.0 / (1.0 + exp(-margin)) : margin);
  }
}

// ---------------------------------------------------------------------------
// Rank quantisation of the rows.  For every (row, feature) the kernel counts how many of the
// feature's sorted distinct split thresholds are <= the value and writes the count as one byte into
// the tile layout the row-parallel kernel copies verbatim: [block of 64 rows][feature][row].  The
// table is padded with +inf up to 2^n - 1 entries; NaN and +inf count all of them (the largest rank,
// above every node's threshold index, so they go right at every node like the f32 compare sends
// them).  Rows past the end of the batch in the last block get the ranks of the last row; the walk
// never stores their results.
//
// A block owns a chunk of 64 features, whose threshold table sits in LDS as [k][feature]; its waves
// take 64-row blocks in turn.  A lane owns ONE feature of the chunk: whatever level of the search a
// lane is at, lane i reads bank i, so the table reads never conflict, and a wave's row load is 256
// contiguous bytes.  The lane's 64 result bytes pass through a per-wave LDS area (80-byte lane
// stride: conflict-free 16-byte writes) so that the wave stores its 4 KB of tile in four contiguous
// 1 KB pieces.
// ---------------------------------------------------------------------------
constexpr int kBinRows = 64;        // rows per tile = rows per block of the quantised walk
constexpr int kBinFeatures = 64;    // features per block = lanes per wave
constexpr int kBinRowsPerPass = 16; // rows a lane searches side by side
constexpr int kBinWaves = 8;
constexpr int kBinLaneStride = 80;  // bytes of staging per lane (64 used)

// Sixteen rows of one feature, all loads in flight; rows past the batch re-read the last row.
__device__ __forceinline__ void BinLoadRows(const float *__restrict__ x, int64_t rows, int F, int feature, int64_t rowBase,
                                            float (&v)[kBinRowsPerPass]) {
#pragma unroll
  for (int u = 0; u < kBinRowsPerPass; ++u) {
    const int64_t row = rowBase + u;
    v[u] = x[(row < rows ? row : rows - 1) * F + feature];
  }
}

// Ranks of sixteen values of the lane's feature, left as one 16-byte piece at LDS address `piece`.
// Branch-free binary search on byte offsets into the [k][feature] table (lane offset included); every
// level first issues the reads of all rows, then consumes them, so a wave keeps 16 LDS reads in flight.
template <int kLevels>
__device__ __forceinline__ void BinSearchRows(const float (&v)[kBinRowsPerPass], uint32_t laneBytes, unsigned char *piece) {
  typedef uint32_t Piece __attribute__((ext_vector_type(4)));
  constexpr uint32_t strideBytes = kBinFeatures * 4u; // one table level
  uint32_t pos[kBinRowsPerPass];
#pragma unroll
  for (int u = 0; u < kBinRowsPerPass; ++u) pos[u] = laneBytes;
#pragma unroll
  for (int level = kLevels - 1; level >= 0; --level) {
    const uint32_t step = strideBytes << level;
    float probe[kBinRowsPerPass];
#pragma unroll
    for (int u = 0; u < kBinRowsPerPass; ++u) probe[u] = LdsLoadFloat(pos[u] + (step - strideBytes));
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < kBinRowsPerPass; ++u) pos[u] += !(v[u] < probe[u]) ? step : 0u; // NaN: every step taken
    __builtin_amdgcn_sched_barrier(0);
  }
  // byte 1 of every offset is the rank (offset = rank * 256 + lane * 4): gather four of them per word
  uint32_t packed[kBinRowsPerPass / 4];
#pragma unroll
  for (int i = 0; i < kBinRowsPerPass / 4; ++i) {
    const uint32_t lo = __builtin_amdgcn_perm(pos[4 * i + 1], pos[4 * i], 0x0c0c0501u);
    const uint32_t hi = __builtin_amdgcn_perm(pos[4 * i + 3], pos[4 * i + 2], 0x0c0c0501u);
    packed[i] = __builtin_amdgcn_perm(hi, lo, 0x05040100u);
  }
  *reinterpret_cast<Piece *>(piece) = Piece{packed[0], packed[1], packed[2], packed[3]};
}

template <int kLevels> // search depth: the table holds 2^kLevels - 1 thresholds per feature
__global__ void __launch_bounds__(kBinWaves * 64)
BinRowsKernel(const float *__restrict__ x, const float *__restrict__ table, uint8_t *__restrict__ ranks,
              int64_t rows, int F, int rowBlocksPerBlock, int chunks) {
  extern __shared__ __align__(16) unsigned char lds[];
  typedef uint32_t Piece __attribute__((ext_vector_type(4)));
  static_assert(kBinRows == 4 * kBinRowsPerPass, "four passes per row block");
  // Workgroups go to the 8 XCDs in turn, each with its own L2.  A row is not aligned to cache lines
  // (F * 4 bytes is no multiple of 128 in general), so neighbouring feature chunks of the same rows
  // share lines: blocks 8 apart in launch order (same XCD, back to back) take neighbouring chunks of
  // one group of row blocks, and the shared lines are fetched from HBM once.
  const uint32_t linear = blockIdx.x;
  const int chunk = (int)((linear >> 3) % (uint32_t)chunks);
  const int64_t rowGroup = (int64_t)(linear & 7u) + 8 * (int64_t)(linear / (8u * (uint32_t)chunks));
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int f0 = chunk * kBinFeatures;
  const int f = f0 + lane;
  constexpr int depth = (1 << kLevels) - 1;
  constexpr uint32_t tableBytes = (uint32_t)depth * kBinFeatures * 4u;
  {
    float *tab = reinterpret_cast<float *>(lds);
    const float *src = table + (int64_t)chunk * depth * kBinFeatures;
    for (int i = tid; i < depth * kBinFeatures; i += kBinWaves * 64) tab[i] = src[i];
  }
  __syncthreads(); // the only block-wide barrier: from here on the waves run on their own
  unsigned char *stage = lds + tableBytes + (uint32_t)wave * (64u * kBinLaneStride);
  unsigned char *mine = stage + lane * kBinLaneStride;
  const int64_t numRowBlocks = (rows + kBinRows - 1) / kBinRows;
  const int64_t rbBegin = rowGroup * rowBlocksPerBlock; // (past the end for the padding blocks of the last 8 groups)
  const int64_t rbEnd = rbBegin + rowBlocksPerBlock < numRowBlocks ? rbBegin + rowBlocksPerBlock : numRowBlocks;
  const int fClamped = f < F ? f : F - 1;
  const uint32_t laneBytes = (uint32_t)lane * 4u;
  // The rows of the next pass are requested before the current pass is searched (two register
  // buffers), so that the wave always has loads in flight.
  float va[kBinRowsPerPass], vb[kBinRowsPerPass];
  int64_t rb = rbBegin + wave;
  if (rb < rbEnd) BinLoadRows(x, rows, F, fClamped, rb * kBinRows, va);
  for (; rb < rbEnd; rb += kBinWaves) {
    const int64_t rowBase = rb * kBinRows;
    BinLoadRows(x, rows, F, fClamped, rowBase + kBinRowsPerPass, vb);
    BinSearchRows<kLevels>(va, laneBytes, mine);
    BinLoadRows(x, rows, F, fClamped, rowBase + 2 * kBinRowsPerPass, va);
    BinSearchRows<kLevels>(vb, laneBytes, mine + 16);
    BinLoadRows(x, rows, F, fClamped, rowBase + 3 * kBinRowsPerPass, vb);
    BinSearchRows<kLevels>(va, laneBytes, mine + 32);
    const int64_t rbNext = rb + kBinWaves < rbEnd ? rb + kBinWaves : rb; // (the last block re-reads its own rows)
    BinLoadRows(x, rows, F, fClamped, rbNext * kBinRows, va);
    BinSearchRows<kLevels>(vb, laneBytes, mine + 48);
    // the wave's 64 features x 64 rows leave as contiguous 16-byte pieces (piece = feature * 4 + pass)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    uint8_t *dst = ranks + (rb * F + f0) * kBinRows;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int piece = j * 64 + lane;
      const Piece value = *reinterpret_cast<const Piece *>(stage + (piece >> 2) * kBinLaneStride + (piece & 3) * 16);
      if (f0 + (piece >> 2) < F) *reinterpret_cast<Piece *>(dst + piece * 16) = value;
    }
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier(); // the staging area is rewritten by the next row block
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
  }
}

// ---------------------------------------------------------------------------
// Two-byte ranks for narrow models.  For every (row, feature) the kernel counts how many of the feature's
// sorted distinct split thresholds are <= the value and writes the count as 16 bits into the tile layout the
// row-parallel kernel copies verbatim: [block of RB rows][feature pair][row][2] (the two ranks of a pair share
// a dword, so a row's LDS column keeps one bank of its own).  NaN and +inf count every entry of the table (a
// rank above every node's threshold index: they go right at every node, as the f32 compare sends them).  The
// slots of the pad feature (and of the unused half of an odd last pair) get rank 0.
//
// A block owns one chunk of feature pairs, whose threshold tables sit in LDS, and a range of rows, which it
// takes 1024 at a time: the chunk's columns of those rows are read with row-contiguous loads and left
// transposed in LDS (a lane that walked its row's columns in global memory would touch a cache line per load
// and evict it before the next: measured 1.2 to 2 times slower), then a lane is a row: it picks its values out
// of its own LDS bank and searches one feature after the other.  Every table is a complete search tree in
// breadth-first order (entry 0 the root, then its children, ...) and the feature is the same for the whole
// wave, so at search step l the lanes read among 2^l neighbouring entries (one bank each up to 64, broadcast
// where they meet).  Blocks 8 apart in launch order (same XCD, back to back) take the chunks of one row range,
// so that the cache lines of a row, which the chunks share, are fetched from HBM once.
// ---------------------------------------------------------------------------
// (measured on configurations 2, 3 and 5 at 2^20 rows: 16 waves x 1 group 0.105 / 0.169 / 0.290 ms, 8 x 2 0.120 / 0.189 /
// 0.310, 4 x 4 0.152 / 0.252 / 0.365: the two phases of a tile are latency-bound, and waves hide latency better
// than chains do)
constexpr int kRankWaves = 16;
constexpr int kRankChains = 1;                              // 64-row groups a lane searches side by side
constexpr int kRankTileRows = kRankWaves * kRankChains * 64; // rows a block ranks between two barriers
constexpr int kRankStride = kRankTileRows + 1;              // floats per feature column of the staging tile
constexpr int kRankLoads = 8;                               // loads a lane keeps in flight while staging

__global__ void __launch_bounds__(kRankWaves * 64)
RankRows16Kernel(const float *__restrict__ x, const float *__restrict__ tables, const RankFeatureDesc *__restrict__ features,
                 const RankChunkDesc *__restrict__ chunks, uint32_t *__restrict__ ranks, int64_t rows, int F, int RB,
                 int numChunks, int tilesPerBlock, int64_t rowTiles, uint32_t tableRegionBytes) {
  extern __shared__ __align__(16) unsigned char lds[];
  const uint32_t linear = blockIdx.x;
  const int chunk = (int)((linear >> 3) % (uint32_t)numChunks);
  const int64_t range = (int64_t)(linear & 7u) + 8 * (int64_t)(linear / (8u * (uint32_t)numChunks));
  const RankChunkDesc ck = chunks[chunk];
  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  constexpr int threads = kRankWaves * 64;
  {
    float *tab = reinterpret_cast<float *>(lds);
    const float *src = tables + ck.tableBegin;
    for (uint32_t i = tid; i < ck.tableEntries; i += threads) tab[i] = src[i];
  }
  float *stage = reinterpret_cast<float *>(lds + tableRegionBytes); // [feature of the chunk][kRankStride]
  const uint32_t stageAddress = tableRegionBytes;
  const int pairsTotal = (F + 2) >> 1;
  const int Fc = (int)ck.numFeatures;                                // slots of the chunk (whole pairs)
  const int live = (int)ck.firstFeature + Fc <= F ? Fc : F - (int)ck.firstFeature; // of which real features (may be <= 0)
  const float invLive = live > 0 ? 1.0f / (float)live : 0.0f;
  const int64_t tBegin = range * tilesPerBlock; // (past the end for the padding blocks of the last 8 ranges)
  const int64_t tEnd = tBegin + tilesPerBlock < rowTiles ? tBegin + tilesPerBlock : rowTiles;
  for (int64_t tile = tBegin; tile < tEnd; ++tile) {
    const int64_t row0 = tile * kRankTileRows;
    __syncthreads(); // tables loaded / the staging tile is no longer read
    // The chunk's columns of the tile's rows: element e = (row, column) in row-major order, so that a wave's load
    // covers whole row segments; rows past the batch (padding of the last row block) take the last row's values.
    const int total = kRankTileRows * live;
    for (int e0 = tid; e0 < total; e0 += threads * kRankLoads) {
      float value[kRankLoads];
      int where[kRankLoads];
#pragma unroll
      for (int u = 0; u < kRankLoads; ++u) {
        const int e = e0 + u * threads < total ? e0 + u * threads : total - 1;
        int r = (int)((float)e * invLive);
        if (r * live > e) --r;
        if ((r + 1) * live <= e) ++r;
        const int j = e - r * live;
        const int64_t row = row0 + r < rows ? row0 + r : rows - 1;
        value[u] = x[row * F + ck.firstFeature + j];
        where[u] = j * kRankStride + r;
      }
#pragma unroll
      for (int u = 0; u < kRankLoads; ++u)
        if (e0 + u * threads < total) stage[where[u]] = value[u];
    }
    __syncthreads();
    // a lane is a row in each of its wave's kRankChains groups of 64 rows
    const int r0 = wave * (kRankChains * 64) + lane;
    int64_t slot[kRankChains];
#pragma unroll
    for (int c = 0; c < kRankChains; ++c) {
      const int64_t row = row0 + r0 + c * 64;
      slot[c] = (row / RB) * (int64_t)pairsTotal * RB + (row % RB) + (int64_t)(ck.firstFeature >> 1) * RB;
    }
    for (int j0 = 0; j0 < Fc; j0 += 2) {
      uint32_t rank[2][kRankChains];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int j = j0 + h;
        if (j >= live) { // the pad feature's slot and the unused half of an odd last pair
#pragma unroll
          for (int c = 0; c < kRankChains; ++c) rank[h][c] = 0;
          continue;
        }
        const RankFeatureDesc fd = features[ck.firstFeature + j]; // (the same for the whole wave)
        const uint32_t base = fd.tableOffset * 4u;                 // LDS byte address of the table's root
        const uint32_t goLeft = 4u - base, goRight = 8u - base;
        float v[kRankChains];
        uint32_t pos[kRankChains];
#pragma unroll
        for (int c = 0; c < kRankChains; ++c) {
          v[c] = LdsLoadFloat(stageAddress + (uint32_t)(j * kRankStride + r0 + c * 64) * 4u);
          pos[c] = base;
        }
        for (uint32_t level = 0; level < fd.levels; ++level) {
          float probe[kRankChains];
#pragma unroll
          for (int c = 0; c < kRankChains; ++c) probe[c] = LdsLoadFloat(pos[c]);
#pragma unroll
          for (int c = 0; c < kRankChains; ++c) pos[c] = (pos[c] << 1) + (v[c] < probe[c] ? goLeft : goRight); // NaN: right at every step
        }
        // entry index reached below the last table level, minus the 2^levels - 1 entries of the table = thresholds <= value
        const uint32_t entries = (1u << fd.levels) - 1u;
#pragma unroll
        for (int c = 0; c < kRankChains; ++c) rank[h][c] = ((pos[c] - base) >> 2) - entries;
      }
#pragma unroll
      for (int c = 0; c < kRankChains; ++c) ranks[slot[c] + (int64_t)(j0 >> 1) * RB] = rank[0][c] | (rank[1][c] << 16);
    }
  }
}

// ---------------------------------------------------------------------------
// Sums the tree-slice partials of each row (in slice order, starting from the
// initial value), then applies the output transform.  Multiclass rows get the
// arg-max of the f32 per-class sums with the generated-code tie rule (running
// maximum replaced unless strictly greater, so ties go to the larger class id;
// src/mlir/LowerReduceOps.cpp:148-187) and, on request, the sums and their
// softmax.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256) FinalizeKernel(const FinalizeParams p) {
  const int64_t row = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (row >= p.rows) return;
  const int C = p.numClasses;
  if (C == 0) {
    double margin = p.initialValue;
    for (int s = 0; s < p.treeSlices; ++s) margin += p.partial[(int64_t)s * p.rows + row];
    p.out[row] = (float)(p.transform == 1 ? 1.0 / (1.0 + exp(-margin)) : margin);
    return;
  }
  float best = -INFINITY;
  int bestClass = 0;
  double maxMargin = -INFINITY;
  for (int c = 0; c < C; ++c) {
    double margin = p.initialValue;
    for (int s = 0; s < p.treeSlices; ++s) margin += p.partial[((int64_t)s * p.rows + row) * C + c];
    const float m = (float)margin;
    if (p.margins) p.margins[row * C + c] = m;
    if (!(best > m)) { best = m; bestClass = c; }
    maxMargin = margin > maxMargin ? margin : maxMargin;
  }
  if (p.classOut) p.classOut[row] = (int8_t)bestClass;
  if (p.out) p.out[row] = (float)bestClass;
  if (p.probabilities) {
    double z = 0.0;
    for (int c = 0; c < C; ++c) {
      double margin = p.initialValue;
      for (int s = 0; s < p.treeSlices; ++s) margin += p.partial[((int64_t)s * p.rows + row) * C + c];
      z += exp(margin - maxMargin);
    }
    for (int c = 0; c < C; ++c) {
      double margin = p.initialValue;
      for (int s = 0; s < p.treeSlices; ++s) margin += p.partial[((int64_t)s * p.rows + row) * C + c];
      p.probabilities[row * C + c] = (float)(exp(margin - maxMargin) / z);
    }
  }
}

// Small batches split over many tree slices (kWideFinalizeSlices or more): one wave per (row, class).  The lanes fetch the slice
// partials side by side (one memory latency instead of one per slice), each adds its slices in slice
// order, and a fixed butterfly combines the lanes - the order of additions depends only on the number
// of slices.
__global__ void __launch_bounds__(256) FinalizeWideKernel(const FinalizeParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t item = (int64_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int Cn = p.numClasses > 0 ? p.numClasses : 1;
  if (item >= p.rows * Cn) return; // (whole waves leave together)
  const int64_t row = item / Cn;
  const int c = (int)(item - row * Cn);
  double sum = 0.0;
  for (int s = lane; s < p.treeSlices; s += 64) sum += p.partial[((int64_t)s * p.rows + row) * Cn + c];
  for (int m = 1; m <= 32; m <<= 1) sum += ShuffleXor(sum, m); // (ascending: see ShuffleXor)
  const double margin = p.initialValue + sum;
  if (p.numClasses == 0) {
    if (lane == 0) p.out[row] = (float)(p.transform == 1 ? 1.0 / (1.0 + exp(-margin)) : margin);
    return;
  }
  // classifiers: the class sum goes into the spare slot behind the last slice; FinalizeKernel (1 slice, reading
  // that slot) does the rest.  The slices themselves stay as they are, so the launch can be repeated.
  if (lane == 0) p.partial[((int64_t)p.treeSlices * p.rows + row) * Cn + c] = margin - p.initialValue;
}

// The ceiling on dynamic LDS is an attribute of each kernel on each device: it is raised once per kernel and
// device, to the whole 160 KB, instead of on every launch (a runtime call that small batches would pay for each
// time).  Two threads that meet here for the first time both make the call, which is harmless.
template <auto Kernel> hipError_t AllowFullLds() {
  constexpr int kMaxDevices = 64;
  static std::atomic<bool> raised[kMaxDevices];
  int device = 0;
  hipError_t e = hipGetDevice(&device);
  if (e != hipSuccess) return e;
  if (device >= 0 && device < kMaxDevices && raised[device].load(std::memory_order_acquire)) return hipSuccess;
  e = hipFuncSetAttribute(reinterpret_cast<const void *>(Kernel), hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
  if (e == hipSuccess && device >= 0 && device < kMaxDevices) raised[device].store(true, std::memory_order_release);
  return e;
}

template <int K, int PF, int W, int V>
hipError_t LaunchWalkVariant(const WalkParams &p, dim3 grid, dim3 block, size_t ldsBytes, hipStream_t stream) {
  hipError_t e = AllowFullLds<&WalkRowsLdsKernel<K, PF, W, V>>();
  if (e != hipSuccess) return e;
  WalkRowsLdsKernel<K, PF, W, V><<<grid, block, ldsBytes, stream>>>(p.x, p.nodes16, p.bundles, p.bundleRoots, p.groups, p.s, p.out, p.classOut,
                                                                    p.partial, p.leafIds, p.nodeOrigin, p.slotTree,
                                                                    reinterpret_cast<const U32x2 *>(p.tailNodes), p.tailOrigin);
  return hipGetLastError();
}

template <int K, int PF, int W>
hipError_t LaunchWalkKP(const WalkParams &p, dim3 grid, dim3 block, size_t ldsBytes, hipStream_t stream) {
  if (p.leafIds) { // (the dump kernel walks every bundle to its full depth and leaves the arg-max to the finalize kernel)
    if (p.s.fuseArgmax || (p.s.deferTails && W != kTileF32Bytes)) return hipErrorInvalidValue;
    return LaunchWalkVariant<K, PF, W, kWalkDump>(p, grid, block, ldsBytes, stream);
  }
  if (p.s.fuseArgmax) return LaunchWalkVariant<K, PF, W, kWalkFuse>(p, grid, block, ldsBytes, stream);
  // deferred tails are built for the f32 tile with byte offsets only (the packer makes stubs for no other plan)
  if (p.s.deferTails) {
    if (W != kTileF32Bytes || p.s.numClasses > 0) return hipErrorInvalidValue;
    return LaunchWalkVariant<K, PF, kTileF32Bytes, kWalkDefer>(p, grid, block, ldsBytes, stream);
  }
  return LaunchWalkVariant<K, PF, W, kWalkPlain>(p, grid, block, ldsBytes, stream);
}

template <int K, int W>
hipError_t LaunchWalkK(const WalkParams &p, int prefetch, dim3 grid, dim3 block, size_t ldsBytes, hipStream_t stream) {
  if (p.directStaging) return LaunchWalkKP<K, 0, W>(p, grid, block, ldsBytes, stream);
  if (prefetch <= 4) return LaunchWalkKP<K, 4, W>(p, grid, block, ldsBytes, stream);
  if (prefetch <= 8) return LaunchWalkKP<K, 8, W>(p, grid, block, ldsBytes, stream);
  if (prefetch <= 16) return LaunchWalkKP<K, 16, W>(p, grid, block, ldsBytes, stream);
  return hipErrorInvalidValue;
}

template <int W>
hipError_t LaunchWalkW(const WalkParams &p, int interleave, int prefetch, dim3 grid, dim3 block, size_t ldsBytes,
                       hipStream_t stream) {
  switch (interleave) {
  case 1: return LaunchWalkK<1, W>(p, prefetch, grid, block, ldsBytes, stream);
  case 2: return LaunchWalkK<2, W>(p, prefetch, grid, block, ldsBytes, stream);
  case 4: return LaunchWalkK<4, W>(p, prefetch, grid, block, ldsBytes, stream);
  case 8: return LaunchWalkK<8, W>(p, prefetch, grid, block, ldsBytes, stream);
  default: return hipErrorInvalidValue;
  }
}

} // namespace

namespace {
// Outputs the walk kernels dereference must be there: a fused epilogue writes p.out (or p.classOut), everything
// else goes through p.partial.
bool OutputsConsistent(const WalkParams &p) {
  if (p.s.fuseArgmax) return p.s.numClasses > 0 && p.s.treeSlices == 1 && (p.out || p.classOut);
  if (p.s.numClasses > 0 || p.s.treeSlices > 1) return p.partial != nullptr;
  return p.out != nullptr || p.partial != nullptr;
}
} // namespace

hipError_t LaunchWalkRowsLds(const WalkParams &p, int interleave, int tileMode, size_t ldsBytes, hipStream_t stream) {
  if (p.s.rows <= 0) return hipSuccess;
  if (!OutputsConsistent(p)) return hipErrorInvalidValue;
  const int RB = p.s.rowsPerBlock, TT = p.s.treeThreads;
  if (ldsBytes > 160 * 1024 || RB < 64 || (RB & (RB - 1)) || TT < 1 || RB * TT > 1024) return hipErrorInvalidValue;
  const int64_t blocks = (p.s.rows + RB - 1) / RB;
  if (blocks > 0x7FFFFFFF || p.s.treeSlices < 1 || p.s.treeSlices > 65535) return hipErrorInvalidValue;
  // registers that hold the next tree group while the current one is walked
  const int prefetch = (int)((p.s.groupRegionBytes / 16 + RB * TT - 1) / (RB * TT));
  dim3 grid((unsigned)blocks, (unsigned)p.s.treeSlices), block((unsigned)(RB * TT));
  switch (tileMode) {
  case kTileF32Bytes: return LaunchWalkW<kTileF32Bytes>(p, interleave, prefetch, grid, block, ldsBytes, stream);
  case kTileF32Words: return LaunchWalkW<kTileF32Words>(p, interleave, prefetch, grid, block, ldsBytes, stream);
  case kTileRankU8:
    if (RB != 64) return hipErrorInvalidValue;
    return LaunchWalkW<kTileRankU8>(p, interleave, prefetch, grid, block, ldsBytes, stream);
  case kTileRankU16: // (tree groups always go straight from global memory into LDS)
    if ((int64_t)((p.s.numFeatures + 2) / 2) * RB * 4 > 0x10000) return hipErrorInvalidValue; // byte offsets
    switch (interleave) {
    case 1: return LaunchWalkKP<1, 0, kTileRankU16>(p, grid, block, ldsBytes, stream);
    case 2: return LaunchWalkKP<2, 0, kTileRankU16>(p, grid, block, ldsBytes, stream);
    case 4: return LaunchWalkKP<4, 0, kTileRankU16>(p, grid, block, ldsBytes, stream);
    case 8: return LaunchWalkKP<8, 0, kTileRankU16>(p, grid, block, ldsBytes, stream);
    default: return hipErrorInvalidValue;
    }
  default: return hipErrorInvalidValue;
  }
}

namespace {
template <int T, int K, int V>
hipError_t LaunchTiledVariant(const WalkParams &p, dim3 grid, dim3 block, size_t ldsBytes, hipStream_t stream) {
  hipError_t e = AllowFullLds<&WalkRowsTiledKernel<T, K, V>>();
  if (e != hipSuccess) return e;
  WalkRowsTiledKernel<T, K, V><<<grid, block, ldsBytes, stream>>>(p.x, p.nodes16, p.bundles, p.groups, p.s, p.out, p.classOut, p.partial,
                                                                  p.leafIds, p.nodeOrigin, p.slotTree);
  return hipGetLastError();
}

template <int T, int K>
hipError_t LaunchTiledTK(const WalkParams &p, dim3 grid, dim3 block, size_t ldsBytes, hipStream_t stream) {
  if (p.leafIds) {
    if (p.s.fuseArgmax) return hipErrorInvalidValue;
    return LaunchTiledVariant<T, K, kWalkDump>(p, grid, block, ldsBytes, stream);
  }
  if (p.s.fuseArgmax) return LaunchTiledVariant<T, K, kWalkFuse>(p, grid, block, ldsBytes, stream);
  return LaunchTiledVariant<T, K, kWalkPlain>(p, grid, block, ldsBytes, stream);
}

template <int T>
hipError_t LaunchTiledT(const WalkParams &p, int interleave, dim3 grid, dim3 block, size_t ldsBytes, hipStream_t stream) {
  switch (interleave) {
  case 1: return LaunchTiledTK<T, 1>(p, grid, block, ldsBytes, stream);
  case 2: return LaunchTiledTK<T, 2>(p, grid, block, ldsBytes, stream);
  case 4: return LaunchTiledTK<T, 4>(p, grid, block, ldsBytes, stream);
  default: return hipErrorInvalidValue;
  }
}
} // namespace

hipError_t LaunchWalkRowsTiled(const WalkParams &p, int tileSize, int interleave, size_t ldsBytes, hipStream_t stream) {
  if (p.s.rows <= 0) return hipSuccess;
  if (!OutputsConsistent(p)) return hipErrorInvalidValue;
  const int RB = p.s.rowsPerBlock, TT = p.s.treeThreads;
  if (ldsBytes > 160 * 1024 || RB < 64 || (RB & (RB - 1)) || TT < 1 || RB * TT > 1024) return hipErrorInvalidValue;
  // feature offsets are byte offsets into the f32 row tile: the tile has to end below 64 KB
  if ((int64_t)(p.s.numFeatures + 1) * RB * 4 > 0x10000) return hipErrorInvalidValue;
  const int64_t blocks = (p.s.rows + RB - 1) / RB;
  if (blocks > 0x7FFFFFFF || p.s.treeSlices < 1 || p.s.treeSlices > 65535) return hipErrorInvalidValue;
  dim3 grid((unsigned)blocks, (unsigned)p.s.treeSlices), block((unsigned)(RB * TT));
  switch (tileSize) {
  case 2: return LaunchTiledT<2>(p, interleave, grid, block, ldsBytes, stream);
  case 3: return LaunchTiledT<3>(p, interleave, grid, block, ldsBytes, stream);
  case 4: return LaunchTiledT<4>(p, interleave, grid, block, ldsBytes, stream);
  case 5: case 6: case 7: case 8: // one eight-slot tile for all four; the packer fills as many slots as the tile size says
    return LaunchTiledT<kMaxTileSize>(p, interleave, grid, block, ldsBytes, stream);
  default: return hipErrorInvalidValue;
  }
}

namespace {
template <int K, int PF>
hipError_t LaunchTreeParallelKP(const WalkParams &p, dim3 grid, dim3 block, size_t ldsBytes, hipStream_t stream) {
  if (p.leafIds) {
    hipError_t e = AllowFullLds<&WalkTreeParallelKernel<K, PF, true>>();
    if (e != hipSuccess) return e;
    WalkTreeParallelKernel<K, PF, true><<<grid, block, ldsBytes, stream>>>(p.x, p.nodes16, p.bundles, p.groups, p.s, p.out,
                                                                          p.partial, p.leafIds, p.nodeOrigin, p.slotTree);
  } else {
    hipError_t e = AllowFullLds<&WalkTreeParallelKernel<K, PF, false>>();
    if (e != hipSuccess) return e;
    WalkTreeParallelKernel<K, PF, false><<<grid, block, ldsBytes, stream>>>(p.x, p.nodes16, p.bundles, p.groups, p.s, p.out,
                                                                           p.partial, nullptr, nullptr, nullptr);
  }
  return hipGetLastError();
}

template <int K>
hipError_t LaunchTreeParallelK(const WalkParams &p, int prefetch, dim3 grid, dim3 block, size_t ldsBytes,
                               hipStream_t stream) {
  if (prefetch <= 4) return LaunchTreeParallelKP<K, 4>(p, grid, block, ldsBytes, stream);
  if (prefetch <= 8) return LaunchTreeParallelKP<K, 8>(p, grid, block, ldsBytes, stream);
  if (prefetch <= 16) return LaunchTreeParallelKP<K, 16>(p, grid, block, ldsBytes, stream);
  return hipErrorInvalidValue;
}
} // namespace

hipError_t LaunchWalkTreeParallel(const WalkParams &p, int interleave, size_t ldsBytes, hipStream_t stream) {
  if (p.s.rows <= 0) return hipSuccess;
  if (ldsBytes > 160 * 1024 || p.s.rowsPerBlock < 1 || p.s.treeLanes < 1) return hipErrorInvalidValue;
  const int threads = p.s.rowsPerBlock * p.s.treeLanes;
  if (threads > 1024 || threads % 64 != 0) return hipErrorInvalidValue;
  const int64_t blocks = (p.s.rows + p.s.rowsPerBlock - 1) / p.s.rowsPerBlock;
  if (blocks > 0x7FFFFFFF || p.s.treeSlices < 1 || p.s.treeSlices > 65535) return hipErrorInvalidValue;
  const int prefetch = (int)((p.s.groupRegionBytes / 16 + threads - 1) / threads);
  dim3 grid((unsigned)blocks, (unsigned)p.s.treeSlices), block((unsigned)threads);
  switch (interleave) {
  case 1: return LaunchTreeParallelK<1>(p, prefetch, grid, block, ldsBytes, stream);
  case 2: return LaunchTreeParallelK<2>(p, prefetch, grid, block, ldsBytes, stream);
  case 4: return LaunchTreeParallelK<4>(p, prefetch, grid, block, ldsBytes, stream);
  case 8: return LaunchTreeParallelK<8>(p, prefetch, grid, block, ldsBytes, stream);
  default: return hipErrorInvalidValue;
  }
}

namespace {
template <int K>
hipError_t LaunchGlobalK(const WalkParams &p, dim3 grid, dim3 block, hipStream_t stream) {
  if (p.leafIds)
    WalkGlobalKernel<K, true><<<grid, block, 0, stream>>>(p.x, p.globalNodes, p.globalTrees, p.s, p.out, p.partial, p.leafIds);
  else
    WalkGlobalKernel<K, false><<<grid, block, 0, stream>>>(p.x, p.globalNodes, p.globalTrees, p.s, p.out, p.partial, nullptr);
  return hipGetLastError();
}
} // namespace

hipError_t LaunchWalkGlobal(const WalkParams &p, int interleave, hipStream_t stream) {
  if (p.s.rows <= 0) return hipSuccess;
  const int threads = p.s.rowsPerBlock;
  if (threads < 64 || threads > 1024 || threads % 64 != 0) return hipErrorInvalidValue;
  const int64_t blocks = (p.s.rows + threads - 1) / threads;
  if (blocks > 0x7FFFFFFF || p.s.treeSlices < 1 || p.s.treeSlices > 65535) return hipErrorInvalidValue;
  dim3 grid((unsigned)blocks, (unsigned)p.s.treeSlices), block((unsigned)threads);
  switch (interleave) {
  case 1: return LaunchGlobalK<1>(p, grid, block, stream);
  case 2: return LaunchGlobalK<2>(p, grid, block, stream);
  case 4: return LaunchGlobalK<4>(p, grid, block, stream);
  case 8: return LaunchGlobalK<8>(p, grid, block, stream);
  default: return hipErrorInvalidValue;
  }
}

hipError_t LaunchBinRows(const float *x, const float *table, uint8_t *ranks, int64_t rows, int numFeatures,
                         int tableDepth, int chunkFeatures, hipStream_t stream) {
  if (rows <= 0) return hipSuccess;
  if (chunkFeatures != kBinFeatures) return hipErrorInvalidValue;
  const size_t ldsBytes = (size_t)tableDepth * kBinFeatures * sizeof(float) + (size_t)kBinWaves * 64 * kBinLaneStride;
  if (ldsBytes > 160 * 1024) return hipErrorInvalidValue;
  const int64_t rowBlocks = (rows + kBinRows - 1) / kBinRows;
  const int chunks = (numFeatures + kBinFeatures - 1) / kBinFeatures;
  // enough blocks to fill the chip, each amortising its table load over several row blocks per wave
  int64_t perBlock = (rowBlocks * chunks + 2047) / 2048;
  if (perBlock < kBinWaves) perBlock = kBinWaves;
  if (perBlock > 64 * kBinWaves) perBlock = 64 * kBinWaves;
  const int64_t rowGroups = (rowBlocks + perBlock - 1) / perBlock;
  const int64_t blocks = (rowGroups + 7) / 8 * 8 * chunks; // row groups padded to the 8 XCDs
  if (blocks > 0x7FFFFFFF) return hipErrorInvalidValue;
  const dim3 grid((unsigned)blocks), block(kBinWaves * 64);
#define TBAMD_BIN_CASE(LEVELS)                                                                                         \
  case (1 << LEVELS) - 1: {                                                                                            \
    hipError_t e = AllowFullLds<&BinRowsKernel<LEVELS>>();                                                             \
    if (e != hipSuccess) return e;                                                                                     \
    BinRowsKernel<LEVELS><<<grid, block, ldsBytes, stream>>>(x, table, ranks, rows, numFeatures, (int)perBlock,       \
                                                             chunks);                                                  \
    return hipGetLastError();                                                                                          \
  }
  switch (tableDepth) {
    TBAMD_BIN_CASE(1)
    TBAMD_BIN_CASE(2)
    TBAMD_BIN_CASE(3)
    TBAMD_BIN_CASE(4)
    TBAMD_BIN_CASE(5)
    TBAMD_BIN_CASE(6)
    TBAMD_BIN_CASE(7)
    TBAMD_BIN_CASE(8)
  default: return hipErrorInvalidValue;
  }
#undef TBAMD_BIN_CASE
}

hipError_t LaunchRankRows16(const float *x, const float *tables, const RankFeatureDesc *features, const RankChunkDesc *chunks,
                            int numChunks, uint32_t maxChunkEntries, uint32_t maxChunkFeatures, uint16_t *ranks, int64_t rows,
                            int numFeatures, int rowsPerBlock, hipStream_t stream) {
  if (rows <= 0) return hipSuccess;
  const uint32_t tableRegionBytes = (maxChunkEntries * (uint32_t)sizeof(float) + 15u) & ~15u;
  const size_t ldsBytes = (size_t)tableRegionBytes + (size_t)maxChunkFeatures * kRankStride * sizeof(float);
  if (numChunks < 1 || ldsBytes > 160 * 1024 || rowsPerBlock < 64 || rowsPerBlock % 64 != 0) return hipErrorInvalidValue;
  const int64_t rowBlocks = (rows + rowsPerBlock - 1) / rowsPerBlock;
  // whole row blocks (the walk copies whole tiles), in tiles of 1024 rows: smaller row blocks are ranked up to the
  // next multiple of 1024 rows, which the rank buffer has to hold
  const int64_t rowTiles = (rowBlocks * rowsPerBlock + kRankTileRows - 1) / kRankTileRows;
  // enough blocks to fill the chip, each amortising its table load over a few thousand rows
  int64_t perBlock = (rowTiles * numChunks + 4095) / 4096;
  if (perBlock < 2) perBlock = 2;
  if (perBlock > 16) perBlock = 16;
  const int64_t ranges = (rowTiles + perBlock - 1) / perBlock;
  const int64_t blocks = (ranges + 7) / 8 * 8 * numChunks; // row ranges padded to the 8 XCDs
  if (blocks > 0x7FFFFFFF) return hipErrorInvalidValue;
  hipError_t e = AllowFullLds<&RankRows16Kernel>();
  if (e != hipSuccess) return e;
  RankRows16Kernel<<<dim3((unsigned)blocks), dim3(kRankWaves * 64), ldsBytes, stream>>>(
      x, tables, features, chunks, reinterpret_cast<uint32_t *>(ranks), rows, numFeatures, rowsPerBlock, numChunks, (int)perBlock,
      rowTiles, tableRegionBytes);
  return hipGetLastError();
}

hipError_t LaunchFinalize(const FinalizeParams &p, hipStream_t stream) {
  if (p.rows <= 0) return hipSuccess;
  const int Cn = p.numClasses > 0 ? p.numClasses : 1;
  FinalizeParams q = p;
  if (p.treeSlices >= kWideFinalizeSlices && p.rows * Cn <= 65536) { // few rows, many slices: a wave per (row, class)
    const int64_t waves = p.rows * Cn;
    FinalizeWideKernel<<<dim3((unsigned)((waves + 3) / 4)), dim3(256), 0, stream>>>(p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess || p.numClasses == 0) return e;
    q.partial = p.partial + (int64_t)p.treeSlices * p.rows * Cn; // the class sums now sit in the spare slot
    q.treeSlices = 1;
  }
  const int64_t blocks = (q.rows + 255) / 256;
  FinalizeKernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(q);
  return hipGetLastError();
}

} // namespace tbamd
