// Bench-only library (libtbamd_bench.so): an LDS read micro-benchmark.  Not part of the runtime library
// and not needed for inference; bench.py and one GPU test load it to quote the walk kernels' LDS traffic
// against what the LDS of the device at hand delivers rather than against a datasheet figure.
#include <hip/hip_runtime.h>

#include <cstdint>
#include <random>
#include <vector>

namespace {

// What the LDS pipes of this device deliver for conflict-free reads of 4, 8 and 16 bytes per lane (lane i
// reads bank-aligned element i of a row; eight independent rows per iteration).
template <int kWidth>
__global__ void __launch_bounds__(1024) LdsReadBenchKernel(int iterations, uint32_t *sink) {
  extern __shared__ __align__(16) unsigned char lds[];
  for (int i = threadIdx.x; i < 16384; i += blockDim.x) reinterpret_cast<uint32_t *>(lds)[i] = (uint32_t)i;
  __syncthreads();
  const uint32_t lane = threadIdx.x & 63u;
  uint32_t address[8];
#pragma unroll
  for (int i = 0; i < 8; ++i) address[i] = (lane * kWidth + (uint32_t)i * 64u * kWidth) & 0xFFFFu;
  uint32_t issued = 0;
  for (int it = 0; it < iterations; ++it) {
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      if (kWidth == 4) {
        uint32_t v;
        asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(7)" : "=v"(v) : "v"(address[i]));
      } else if (kWidth == 8) {
        uint64_t v;
        asm volatile("ds_read_b64 %0, %1\n\ts_waitcnt lgkmcnt(7)" : "=v"(v) : "v"(address[i]));
      } else {
        __uint128_t v;
        asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(7)" : "=v"(v) : "v"(address[i]));
      }
      ++issued;
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)");
  if (issued == 0x7FFFFFFFu) sink[0] = issued; // (never true: keeps the loop alive)
}
hipError_t MeasureLdsReadBandwidth(int widthBytes, int computeUnits, hipStream_t stream, double *bytesPerSecond) {
  if (!bytesPerSecond || computeUnits < 1 || (widthBytes != 4 && widthBytes != 8 && widthBytes != 16)) return hipErrorInvalidValue;
  const int blocks = computeUnits * 2, threads = 1024, iterations = 2000;
  uint32_t *sink = nullptr;
  hipError_t e = hipMalloc(reinterpret_cast<void **>(&sink), sizeof(uint32_t));
  if (e != hipSuccess) return e;
  hipEvent_t start = nullptr, stop = nullptr;
  auto launch = [&](int it) {
    if (widthBytes == 4) LdsReadBenchKernel<4><<<blocks, threads, 65536, stream>>>(it, sink);
    else if (widthBytes == 8) LdsReadBenchKernel<8><<<blocks, threads, 65536, stream>>>(it, sink);
    else LdsReadBenchKernel<16><<<blocks, threads, 65536, stream>>>(it, sink);
  };
  float ms = 0.f;
  e = hipEventCreate(&start);
  if (e == hipSuccess) e = hipEventCreate(&stop);
  if (e == hipSuccess) {
    launch(10); // warm-up
    e = hipEventRecord(start, stream);
    launch(iterations);
    if (e == hipSuccess) e = hipEventRecord(stop, stream);
    if (e == hipSuccess) e = hipEventSynchronize(stop);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, start, stop);
    if (e == hipSuccess) e = hipGetLastError();
  }
  if (start) (void)hipEventDestroy(start);
  if (stop) (void)hipEventDestroy(stop);
  (void)hipFree(sink);
  if (e != hipSuccess) return e;
  const double bytes = (double)blocks * threads * iterations * 8.0 * widthBytes;
  *bytesPerSecond = bytes / (ms * 1e-3);
  return hipSuccess;
}


// What one wave-level LDS read costs, by instruction, address pattern and exec mask: every lane holds eight
// addresses prepared on the host and issues the eight reads back to back (independent, so the pipe and not the
// latency is measured); lanes switched off by `active` skip the loop.
enum ReadOp { kReadB32 = 0, kReadB64, kReadB128, kRead2B32, kReadU16, kReadU8, kReadB96, kReadOps };

template <int kOp>
__global__ void __launch_bounds__(512) LdsReadCostKernel(const uint32_t *__restrict__ addresses, const uint32_t *__restrict__ active,
                                                         int iterations, uint32_t *sink) {
  extern __shared__ __align__(16) unsigned char lds[];
  for (int i = threadIdx.x; i < 16384; i += blockDim.x) reinterpret_cast<uint32_t *>(lds)[i] = (uint32_t)i;
  __syncthreads();
  const int lane = blockIdx.x * blockDim.x + threadIdx.x;
  uint32_t address[8];
  for (int i = 0; i < 8; ++i) address[i] = addresses[(size_t)lane * 8 + i];
  uint32_t issued = 0;
  if (active[lane]) {
    for (int it = 0; it < iterations; ++it) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        if (kOp == kReadB32) { uint32_t v; asm volatile("ds_read_b32 %0, %1\n\ts_waitcnt lgkmcnt(7)" : "=v"(v) : "v"(address[i])); }
        if (kOp == kReadB64) { uint64_t v; asm volatile("ds_read_b64 %0, %1\n\ts_waitcnt lgkmcnt(7)" : "=v"(v) : "v"(address[i])); }
        if (kOp == kReadB128) { __uint128_t v; asm volatile("ds_read_b128 %0, %1\n\ts_waitcnt lgkmcnt(7)" : "=v"(v) : "v"(address[i])); }
        if (kOp == kRead2B32) { uint64_t v; asm volatile("ds_read2_b32 %0, %1 offset1:64\n\ts_waitcnt lgkmcnt(7)" : "=v"(v) : "v"(address[i])); }
        if (kOp == kReadU16) { uint32_t v; asm volatile("ds_read_u16 %0, %1\n\ts_waitcnt lgkmcnt(7)" : "=v"(v) : "v"(address[i])); }
        if (kOp == kReadU8) { uint32_t v; asm volatile("ds_read_u8 %0, %1\n\ts_waitcnt lgkmcnt(7)" : "=v"(v) : "v"(address[i])); }
        if (kOp == kReadB96) {
          typedef uint32_t U32x3 __attribute__((ext_vector_type(3)));
          U32x3 v;
          asm volatile("ds_read_b96 %0, %1\n\ts_waitcnt lgkmcnt(7)" : "=v"(v) : "v"(address[i]));
        }
        ++issued;
      }
    }
  }
  asm volatile("s_waitcnt lgkmcnt(0)");
  if (issued == 0x7FFFFFFFu) sink[0] = issued; // (never true: keeps the loop alive)
}

// pattern: 0 = lane i reads element i (conflict-free), 1 = random over 48 KB, 2 = random over 1 KB,
// 5..7 = random among 2^pattern consecutive elements (the nodes of one level of a level-order tree; elements are
// 8 bytes for ds_read_b64 and 4 bytes otherwise).  mask: 0 = all lanes, 1 = lanes 0-31, 2 = even lanes,
// 3 = a random half, 4 = a random quarter.
hipError_t MeasureLdsReadCost(int op, int pattern, int mask, int computeUnits, double clockHz, double *cyclesPerRead) {
  static const int kBytes[kReadOps] = {4, 8, 16, 4, 2, 1, 16};
  const bool patternOk = pattern == 0 || pattern == 1 || pattern == 2 || (pattern >= 5 && pattern <= 7);
  if (!cyclesPerRead || op < 0 || op >= kReadOps || !patternOk || mask < 0 || mask > 4 || computeUnits < 1) return hipErrorInvalidValue;
  const int blocks = computeUnits * 2, threads = 512, iterations = 1000;
  const size_t lanes = (size_t)blocks * threads;
  std::vector<uint32_t> addresses(lanes * 8), active(lanes);
  std::mt19937 rng(1);
  const uint32_t unit = (uint32_t)kBytes[op];
  for (size_t t = 0; t < lanes; ++t) {
    const uint32_t lane = (uint32_t)(t % 64);
    active[t] = mask == 0 ? 1u : mask == 1 ? (lane < 32) : mask == 2 ? ((lane & 1u) == 0) : mask == 3 ? (rng() % 2 == 0) : (rng() % 4 == 0);
    for (uint32_t i = 0; i < 8; ++i) {
      uint32_t a;
      if (pattern == 0) a = (lane * unit + i * 64u * unit) % 32768u;
      else if (pattern == 1) a = (rng() % (49152u / unit)) * unit;
      else if (pattern == 2) a = (rng() % (1024u / unit)) * unit;
      else a = 4096u + (rng() % (1u << pattern)) * (op == kReadB64 ? 8u : 4u);
      addresses[t * 8 + i] = a;
    }
  }
  uint32_t *dAddresses = nullptr, *dActive = nullptr, *sink = nullptr;
  hipEvent_t start = nullptr, stop = nullptr;
  float ms = 0.f;
  hipError_t e = hipMalloc(reinterpret_cast<void **>(&dAddresses), addresses.size() * 4);
  if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&dActive), active.size() * 4);
  if (e == hipSuccess) e = hipMalloc(reinterpret_cast<void **>(&sink), 4);
  if (e == hipSuccess) e = hipMemcpy(dAddresses, addresses.data(), addresses.size() * 4, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipMemcpy(dActive, active.data(), active.size() * 4, hipMemcpyHostToDevice);
  if (e == hipSuccess) e = hipEventCreate(&start);
  if (e == hipSuccess) e = hipEventCreate(&stop);
  if (e == hipSuccess) {
    auto launch = [&](int it) {
      switch (op) {
      case kReadB32: LdsReadCostKernel<kReadB32><<<blocks, threads, 65536, nullptr>>>(dAddresses, dActive, it, sink); break;
      case kReadB64: LdsReadCostKernel<kReadB64><<<blocks, threads, 65536, nullptr>>>(dAddresses, dActive, it, sink); break;
      case kReadB128: LdsReadCostKernel<kReadB128><<<blocks, threads, 65536, nullptr>>>(dAddresses, dActive, it, sink); break;
      case kRead2B32: LdsReadCostKernel<kRead2B32><<<blocks, threads, 65536, nullptr>>>(dAddresses, dActive, it, sink); break;
      case kReadU16: LdsReadCostKernel<kReadU16><<<blocks, threads, 65536, nullptr>>>(dAddresses, dActive, it, sink); break;
      case kReadU8: LdsReadCostKernel<kReadU8><<<blocks, threads, 65536, nullptr>>>(dAddresses, dActive, it, sink); break;
      default: LdsReadCostKernel<kReadB96><<<blocks, threads, 65536, nullptr>>>(dAddresses, dActive, it, sink); break;
      }
    };
    launch(10); // warm-up
    e = hipEventRecord(start, nullptr);
    launch(iterations);
    if (e == hipSuccess) e = hipEventRecord(stop, nullptr);
    if (e == hipSuccess) e = hipEventSynchronize(stop);
    if (e == hipSuccess) e = hipEventElapsedTime(&ms, start, stop);
    if (e == hipSuccess) e = hipGetLastError();
  }
  if (start) (void)hipEventDestroy(start);
  if (stop) (void)hipEventDestroy(stop);
  if (dAddresses) (void)hipFree(dAddresses);
  if (dActive) (void)hipFree(dActive);
  if (sink) (void)hipFree(sink);
  if (e != hipSuccess) return e;
  const double readsPerCu = (double)blocks * (threads / 64) * iterations * 8.0 / computeUnits;
  *cyclesPerRead = ms * 1e-3 * clockHz / readsPerCu;
  return hipSuccess;
}

} // namespace

// Bytes per second of conflict-free LDS reads of `widthBytes` (4, 8 or 16) per lane with every CU busy.
// Returns 0 on success, a HIP error code otherwise.
extern "C" __attribute__((visibility("default"))) int32_t tbbench_lds_read_bandwidth(int32_t widthBytes, double *bytesPerSecond) {
  int devices = 0;
  hipDeviceProp_t prop;
  if (hipGetDeviceCount(&devices) != hipSuccess || devices == 0) return (int32_t)hipErrorNoDevice;
  if (hipGetDeviceProperties(&prop, 0) != hipSuccess) return (int32_t)hipErrorInvalidDevice;
  return (int32_t)MeasureLdsReadBandwidth(widthBytes, prop.multiProcessorCount, nullptr, bytesPerSecond);
}

// Cycles (at the device's nominal shader clock) one compute unit spends per wave-level LDS read.
// op: 0 ds_read_b32, 1 ds_read_b64, 2 ds_read_b128, 3 ds_read2_b32, 4 ds_read_u16, 5 ds_read_u8, 6 ds_read_b96.
// pattern: 0 lane i reads element i, 1 random over 48 KB, 2 random over 1 KB, 5..7 random among 2^pattern
// consecutive elements.  mask: 0 all lanes, 1 lanes 0-31, 2 even lanes, 3 a random half, 4 a random quarter.
// Returns 0 on success, a HIP error code otherwise.
extern "C" __attribute__((visibility("default"))) int32_t tbbench_lds_read_cost(int32_t op, int32_t pattern, int32_t mask, double *cyclesPerRead) {
  int devices = 0;
  hipDeviceProp_t prop;
  if (hipGetDeviceCount(&devices) != hipSuccess || devices == 0) return (int32_t)hipErrorNoDevice;
  if (hipGetDeviceProperties(&prop, 0) != hipSuccess) return (int32_t)hipErrorInvalidDevice;
  return (int32_t)MeasureLdsReadCost(op, pattern, mask, prop.multiProcessorCount, prop.clockRate * 1e3, cyclesPerRead);
}
