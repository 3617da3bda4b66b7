// Splits [0, n) over a few host threads (the host-side row gathers).
#pragma once
#include <stdint.h>

#include <algorithm>
#include <thread>
#include <vector>

namespace lrqk {

template <typename F>
inline void parallel_ranges(int64_t n, int threads, int64_t min_chunk, F&& fn) {
  if (threads < 1) threads = 1;
  int64_t parts = std::min<int64_t>(threads, (n + min_chunk - 1) / std::max<int64_t>(min_chunk, 1));
  if (parts <= 1) {
    fn(0, n);
    return;
  }
  std::vector<std::thread> pool;
  int64_t step = (n + parts - 1) / parts;
  for (int64_t p = 0; p < parts; ++p) {
    int64_t lo = p * step, hi = std::min(n, lo + step);
    if (lo >= hi) break;
    pool.emplace_back([=, &fn] { fn(lo, hi); });
  }
  for (auto& t : pool) t.join();
}

}  // namespace lrqk
