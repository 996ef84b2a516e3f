// Copies between pageable host memory and a pinned staging buffer with several threads: one core
// moves about 10 GB/s, less than the PCIe link, so the host-buffer entry point splits each piece of
// a batch over a small pool that lives as long as the runner.
#pragma once
#include <condition_variable>
#include <cstddef>
#include <cstdint>
#include <mutex>
#include <thread>
#include <vector>

namespace tbamd {

class ParallelCopier {
public:
  explicit ParallelCopier(int threads); // the calling thread counts as one of them
  ~ParallelCopier();
  ParallelCopier(const ParallelCopier &) = delete;
  ParallelCopier &operator=(const ParallelCopier &) = delete;
  // memcpy(dst, src, bytes), striped over the pool; returns when every stripe is done.
  void Copy(void *dst, const void *src, size_t bytes);
  int Threads() const { return (int)m_workers.size() + 1; }

private:
  void Worker(int index);
  void CopyStripe(int index) const;
  std::vector<std::thread> m_workers;
  std::mutex m_mutex;
  std::condition_variable m_wake, m_done;
  uint64_t m_generation = 0;
  int m_pending = 0;
  bool m_stop = false;
  char *m_dst = nullptr;
  const char *m_src = nullptr;
  size_t m_bytes = 0;
};

} // namespace tbamd
