// Bench-only library (libtbamd_bench.so): an LDS read micro-benchmark.  Not part of the runtime library
// and not needed for inference; bench.py and one GPU test load it to quote the walk kernels' LDS traffic
// against what the LDS of the device at hand delivers rather than against a datasheet figure.
#include <hip/hip_runtime.h>

#include <cstdint>

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
