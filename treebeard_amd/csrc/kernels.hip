// Hand-written gfx950 kernels for decision-forest inference.
//
// They replace the kernels the reference generates from its schedules
// (src/gpu/GPUSchedules.cpp, src/mlir/CodeGenStateMachine.cpp:149-243 scalar
// tile step, src/mlir/WalkDecisionTreeLoweringPass.cpp:23-110 walk loops,
// src/gpu/GPURepresentations.cpp:279-399 row caching, src/mlir/LowerReduceOps.cpp
// :119-187 and :921-1003 reductions, src/mlir/LowerToMidLevelIR.cpp:554-648
// result initialisation and sigmoid).
#include "kernels.h"

#include <cmath>

namespace tbamd {

namespace {

__device__ __forceinline__ float AsFloat(uint32_t u) { return __uint_as_float(u); }

// LDS reads by absolute LDS address.  The kernels below use dynamic LDS only,
// which the compiler places at LDS address 0, so an offset into the dynamic
// array is the address itself and no base has to be added per access.
typedef uint32_t U32x2 __attribute__((ext_vector_type(2)));
typedef const __attribute__((address_space(3))) U32x2 *LdsNodePtr;
typedef const __attribute__((address_space(3))) float *LdsFloatPtr;
__device__ __forceinline__ U32x2 LdsLoadNode(uint32_t address) { return *(LdsNodePtr)(uintptr_t)address; }
__device__ __forceinline__ float LdsLoadFloat(uint32_t address) { return *(LdsFloatPtr)(uintptr_t)address; }

// ---------------------------------------------------------------------------
// Row-parallel walk.  One lane owns one row of the block; the block's rows sit
// transposed in LDS (feature-major) so that lane i always reads bank i%32 no
// matter which feature its node tests.  Trees are streamed through LDS one
// group at a time and walked K at a time in lock step: all lanes take `depth`
// steps, leaves hold the walk in place (see device_model.h), so the loop body
// has no leaf test and no divergence.  The per-row sum is kept in double and
// trees are added in packed order.
// ---------------------------------------------------------------------------
template <int K, bool kOffsetsInWords, bool kDump>
__global__ void __launch_bounds__(1024)
WalkRowsLdsKernel(const float *__restrict__ x, const uint4 *__restrict__ nodes16,
                  const DeviceBundle *__restrict__ bundles, const DeviceGroup *__restrict__ groups,
                  const WalkScalars s, float *__restrict__ out, double *__restrict__ partial,
                  int32_t *__restrict__ leafIds, const int32_t *__restrict__ nodeOrigin,
                  const int32_t *__restrict__ slotTree) {
  // LDS: [tree group nodes | transposed row tile].  The group sits at LDS
  // address 0 so that node pointers are LDS addresses as stored.
  extern __shared__ __align__(16) unsigned char lds[];
  const int tid = threadIdx.x;
  const int RB = blockDim.x;
  const int F = s.numFeatures;
  const int64_t row0 = (int64_t)blockIdx.x * RB;
  const int64_t remaining = s.rows - row0;
  const int valid = remaining < RB ? (int)remaining : RB;

  unsigned char *group = lds;
  float *rowTile = reinterpret_cast<float *>(lds + s.groupRegionBytes);

  // Stage the block's rows: coalesced reads of the contiguous row-major tile,
  // transposed writes.  Rows past the end of the batch read as 0.
  {
    const float *src = x + row0 * F;
    const int total = RB * F;
    const int live = valid * F;
    for (int e = tid; e < total; e += RB) {
      const int r = e / F;
      const int f = e - r * F;
      rowTile[f * RB + r] = e < live ? src[e] : 0.0f;
    }
    rowTile[F * RB + tid] = -INFINITY; // pad feature: keeps leaves in place
  }
  const uint32_t column = s.groupRegionBytes + (uint32_t)tid * 4u; // LDS address of this row's feature 0

  const int slice = blockIdx.y;
  const int gBegin = (int)(((int64_t)s.numGroups * slice) / s.treeSlices);
  const int gEnd = (int)(((int64_t)s.numGroups * (slice + 1)) / s.treeSlices);
  const int C = s.numClasses;
  const int64_t row = row0 + tid;
  double *partialRow = partial ? partial + ((int64_t)slice * s.rows + row) * (C > 0 ? C : 1) : nullptr;

  double acc = 0.0;
  int curClass = 0;

  for (int g = gBegin; g < gEnd; ++g) {
    const DeviceGroup grp = groups[g];
    __syncthreads(); // rows staged / previous group no longer read
    {
      const uint4 *src = nodes16 + (grp.nodeBegin >> 1);
      uint4 *dst = reinterpret_cast<uint4 *>(group);
      const int pieces = (int)(grp.nodeCount >> 1);
      for (int i = tid; i < pieces; i += RB) dst[i] = src[i];
    }
    __syncthreads();

    for (uint32_t b = 0; b < grp.bundleCount; ++b) {
      const DeviceBundle bd = bundles[grp.bundleBegin + b];
      if (C > 0) {
        const int cls = bd.classId;
        if (cls != curClass) { // classes arrive in ascending order
          if (tid < valid) {
            partialRow[curClass] = acc;
            for (int c = curClass + 1; c < cls; ++c) partialRow[c] = 0.0;
          }
          acc = 0.0;
          curClass = cls;
        }
      }
      uint32_t addr[K];
#pragma unroll
      for (int k = 0; k < K; ++k) addr[k] = bd.root[k];
      const int depth = bd.depth;
      for (int d = 0; d < depth; ++d) {
#pragma unroll
        for (int k = 0; k < K; ++k) {
          const U32x2 node = LdsLoadNode(addr[k]);
          const uint32_t off = kOffsetsInWords ? (node.y & 0xFFFFu) << 2 : (node.y & 0xFFFFu);
          const float xv = LdsLoadFloat(column + off);
          addr[k] = (node.y >> 16) + (xv < AsFloat(node.x) ? 0u : kNodeBytes);
        }
      }
#pragma unroll
      for (int k = 0; k < K; ++k) acc += (double)LdsLoadFloat(addr[k]);
      if (kDump) {
        if (tid < valid) {
#pragma unroll
          for (int k = 0; k < K; ++k) {
            const int tree = slotTree[bd.firstSlot + k];
            if (tree >= 0) leafIds[row * s.numTrees + tree] = nodeOrigin[grp.nodeBegin + addr[k] / kNodeBytes];
          }
        }
      }
    }
  }

  if (tid >= valid) return;
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
__device__ __forceinline__ double ShuffleXor(double v, int mask) {
  int lo = __double2loint(v), hi = __double2hiint(v);
  lo = __shfl_xor(lo, mask, 64);
  hi = __shfl_xor(hi, mask, 64);
  return __hiloint2double(hi, lo);
}

template <int K, bool kDump>
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

  {
    const float *src = x + row0 * F;
    const int total = R * F;
    const int live = valid * F;
    for (int e = tid; e < total; e += threads) {
      const int rr = e / F;
      const int f = e - rr * F;
      rowsLds[rr * rowWords + f] = e < live ? src[e] : 0.0f;
    }
    for (int rr = tid; rr < R; rr += threads) rowsLds[rr * rowWords + F] = -INFINITY;
    for (int i = tid; i < R * Cn; i += threads) classSums[i] = 0.0;
  }
  const uint32_t rowBase = s.groupRegionBytes + (uint32_t)r * rowWords * 4u;

  const int slice = blockIdx.y;
  const int gBegin = (int)(((int64_t)s.numGroups * slice) / s.treeSlices);
  const int gEnd = (int)(((int64_t)s.numGroups * (slice + 1)) / s.treeSlices);
  const int64_t row = row0 + r;

  for (int g = gBegin; g < gEnd; ++g) {
    const DeviceGroup grp = groups[g];
    __syncthreads();
    {
      const uint4 *src = nodes16 + (grp.nodeBegin >> 1);
      uint4 *dst = reinterpret_cast<uint4 *>(lds);
      const int pieces = (int)(grp.nodeCount >> 1);
      for (int i = tid; i < pieces; i += threads) dst[i] = src[i];
    }
    __syncthreads();

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
      for (int m = inWave >> 1; m >= 1; m >>= 1) acc += ShuffleXor(acc, m);
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

template <int K, bool W>
hipError_t LaunchWalkK(const WalkParams &p, dim3 grid, dim3 block, size_t ldsBytes, hipStream_t stream) {
  if (p.leafIds) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&WalkRowsLdsKernel<K, W, true>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
    if (e != hipSuccess) return e;
    WalkRowsLdsKernel<K, W, true><<<grid, block, ldsBytes, stream>>>(p.x, p.nodes16, p.bundles, p.groups, p.s, p.out, p.partial,
                                                                     p.leafIds, p.nodeOrigin, p.slotTree);
  } else {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&WalkRowsLdsKernel<K, W, false>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
    if (e != hipSuccess) return e;
    WalkRowsLdsKernel<K, W, false><<<grid, block, ldsBytes, stream>>>(p.x, p.nodes16, p.bundles, p.groups, p.s, p.out,
                                                                      p.partial, nullptr, nullptr, nullptr);
  }
  return hipGetLastError();
}

template <bool W>
hipError_t LaunchWalkW(const WalkParams &p, int interleave, dim3 grid, dim3 block, size_t ldsBytes,
                       hipStream_t stream) {
  switch (interleave) {
  case 1: return LaunchWalkK<1, W>(p, grid, block, ldsBytes, stream);
  case 2: return LaunchWalkK<2, W>(p, grid, block, ldsBytes, stream);
  case 4: return LaunchWalkK<4, W>(p, grid, block, ldsBytes, stream);
  case 8: return LaunchWalkK<8, W>(p, grid, block, ldsBytes, stream);
  default: return hipErrorInvalidValue;
  }
}

} // namespace

hipError_t LaunchWalkRowsLds(const WalkParams &p, int rowsPerBlock, int interleave, bool featureOffsetInWords,
                             size_t ldsBytes, hipStream_t stream) {
  if (p.s.rows <= 0) return hipSuccess;
  if (ldsBytes > 160 * 1024) return hipErrorInvalidValue;
  const int64_t blocks = (p.s.rows + rowsPerBlock - 1) / rowsPerBlock;
  if (blocks > 0x7FFFFFFF || p.s.treeSlices < 1 || p.s.treeSlices > 65535) return hipErrorInvalidValue;
  dim3 grid((unsigned)blocks, (unsigned)p.s.treeSlices), block((unsigned)rowsPerBlock);
  return featureOffsetInWords ? LaunchWalkW<true>(p, interleave, grid, block, ldsBytes, stream)
                              : LaunchWalkW<false>(p, interleave, grid, block, ldsBytes, stream);
}

namespace {
template <int K>
hipError_t LaunchTreeParallelK(const WalkParams &p, dim3 grid, dim3 block, size_t ldsBytes, hipStream_t stream) {
  if (p.leafIds) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&WalkTreeParallelKernel<K, true>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
    if (e != hipSuccess) return e;
    WalkTreeParallelKernel<K, true><<<grid, block, ldsBytes, stream>>>(p.x, p.nodes16, p.bundles, p.groups, p.s, p.out,
                                                                      p.partial, p.leafIds, p.nodeOrigin, p.slotTree);
  } else {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&WalkTreeParallelKernel<K, false>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)ldsBytes);
    if (e != hipSuccess) return e;
    WalkTreeParallelKernel<K, false><<<grid, block, ldsBytes, stream>>>(p.x, p.nodes16, p.bundles, p.groups, p.s, p.out,
                                                                       p.partial, nullptr, nullptr, nullptr);
  }
  return hipGetLastError();
}
} // namespace

hipError_t LaunchWalkTreeParallel(const WalkParams &p, int interleave, size_t ldsBytes, hipStream_t stream) {
  if (p.s.rows <= 0) return hipSuccess;
  if (ldsBytes > 160 * 1024 || p.s.rowsPerBlock < 1 || p.s.treeLanes < 1) return hipErrorInvalidValue;
  const int threads = p.s.rowsPerBlock * p.s.treeLanes;
  if (threads > 1024 || threads % 64 != 0) return hipErrorInvalidValue;
  const int64_t blocks = (p.s.rows + p.s.rowsPerBlock - 1) / p.s.rowsPerBlock;
  if (blocks > 0x7FFFFFFF || p.s.treeSlices < 1 || p.s.treeSlices > 65535) return hipErrorInvalidValue;
  dim3 grid((unsigned)blocks, (unsigned)p.s.treeSlices), block((unsigned)threads);
  switch (interleave) {
  case 1: return LaunchTreeParallelK<1>(p, grid, block, ldsBytes, stream);
  case 2: return LaunchTreeParallelK<2>(p, grid, block, ldsBytes, stream);
  case 4: return LaunchTreeParallelK<4>(p, grid, block, ldsBytes, stream);
  case 8: return LaunchTreeParallelK<8>(p, grid, block, ldsBytes, stream);
  default: return hipErrorInvalidValue;
  }
}

hipError_t LaunchFinalize(const FinalizeParams &p, hipStream_t stream) {
  if (p.rows <= 0) return hipSuccess;
  const int64_t blocks = (p.rows + 255) / 256;
  FinalizeKernel<<<dim3((unsigned)blocks), dim3(256), 0, stream>>>(p);
  return hipGetLastError();
}

} // namespace tbamd
