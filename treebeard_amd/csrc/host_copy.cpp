#include "host_copy.h"

#include <algorithm>
#include <cstring>

namespace tbamd {

ParallelCopier::ParallelCopier(int threads) {
  for (int i = 1; i < std::max(1, threads); ++i) m_workers.emplace_back([this, i] { Worker(i); });
}

ParallelCopier::~ParallelCopier() {
  {
    std::lock_guard<std::mutex> lock(m_mutex);
    m_stop = true;
  }
  m_wake.notify_all();
  for (auto &t : m_workers) t.join();
}

void ParallelCopier::CopyStripe(int index) const {
  const size_t parts = m_workers.size() + 1;
  const size_t stripe = ((m_bytes + parts - 1) / parts + 4095) & ~(size_t)4095; // whole pages per thread
  const size_t begin = std::min(m_bytes, stripe * (size_t)index);
  const size_t end = std::min(m_bytes, begin + stripe);
  if (end > begin) std::memcpy(m_dst + begin, m_src + begin, end - begin);
}

void ParallelCopier::Worker(int index) {
  uint64_t seen = 0;
  for (;;) {
    {
      std::unique_lock<std::mutex> lock(m_mutex);
      m_wake.wait(lock, [&] { return m_stop || m_generation != seen; });
      if (m_stop) return;
      seen = m_generation;
    }
    CopyStripe(index);
    {
      std::lock_guard<std::mutex> lock(m_mutex);
      if (--m_pending == 0) m_done.notify_one();
    }
  }
}

void ParallelCopier::Copy(void *dst, const void *src, size_t bytes) {
  if (bytes == 0) return;
  if (m_workers.empty() || bytes < ((size_t)1 << 20)) {
    std::memcpy(dst, src, bytes);
    return;
  }
  {
    std::lock_guard<std::mutex> lock(m_mutex);
    m_dst = static_cast<char *>(dst);
    m_src = static_cast<const char *>(src);
    m_bytes = bytes;
    m_pending = (int)m_workers.size();
    ++m_generation;
  }
  m_wake.notify_all();
  CopyStripe(0);
  std::unique_lock<std::mutex> lock(m_mutex);
  m_done.wait(lock, [&] { return m_pending == 0; });
}

} // namespace tbamd
