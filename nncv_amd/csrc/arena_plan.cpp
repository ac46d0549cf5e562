#include "arena_plan.hpp"

#include <algorithm>
#include <atomic>
#include <cstdlib>
#include <limits>
#include <numeric>

namespace nncv_hip {

namespace {
std::atomic<int>& overlap_state() {
  static std::atomic<int> v{[] {
    const char* e = getenv("NNCV_HIP_OVERLAP");
    const int n = e ? atoi(e) : 1;
    return n < 1 ? 1 : n;
  }()};
  return v;
}
}  // namespace

namespace {
thread_local int tl_overlap = 0;  // the value of the handle whose call this thread is serving; 0 = none
}

int overlap_hint() { return tl_overlap > 0 ? tl_overlap : overlap_state().load(std::memory_order_relaxed); }
int overlap_default() { return overlap_state().load(std::memory_order_relaxed); }
void set_overlap_hint(int passes) { overlap_state().store(passes < 1 ? 1 : passes, std::memory_order_relaxed); }
OverlapScope::OverlapScope(int passes) : prev_(tl_overlap) {
  if (passes > 0) tl_overlap = passes;
}
OverlapScope::~OverlapScope() { tl_overlap = prev_; }

namespace {
int linger_env() {
  static const int forced = [] {
    const char* e = getenv("NNCV_HIP_ARENA_LINGER");
    return e ? std::max(0, atoi(e)) : -1;
  }();
  return forced;
}
}  // namespace

int arena_linger() { return linger_env() >= 0 ? linger_env() : 3; }
bool arena_linger_forced() { return linger_env() >= 0; }

size_t plan_offsets(std::vector<TensorLife>& t, size_t align) {
  const size_t mask = align > 1 ? align - 1 : 0;
  auto up = [&](size_t v) { return (v + mask) & ~mask; };
  std::vector<int> order(t.size());
  std::iota(order.begin(), order.end(), 0);
  // non-increasing size; ties keep registration order, so the plan is deterministic
  std::stable_sort(order.begin(), order.end(), [&](int a, int b) { return up(t[a].bytes) > up(t[b].bytes); });
  std::vector<int> placed;  // indices, sorted by offset
  size_t total = 0;
  for (int id : order) {
    const size_t need = up(t[id].bytes);
    size_t prev_end = 0, best = std::numeric_limits<size_t>::max(), smallest_gap = std::numeric_limits<size_t>::max();
    for (int x : placed) {
      const int lo = std::max(t[id].first_op, t[x].first_op), hi = std::min(t[id].last_op, t[x].last_op);
      if (lo > hi) continue;  // never live together: may share memory
      if (t[x].offset > prev_end) {
        const size_t gap = t[x].offset - prev_end;
        if (gap >= need && gap < smallest_gap) {
          smallest_gap = gap;
          best = prev_end;
        }
      }
      prev_end = std::max(prev_end, t[x].offset + up(t[x].bytes));
    }
    if (best == std::numeric_limits<size_t>::max()) best = prev_end;
    t[id].offset = best;
    total = std::max(total, best + need);
    placed.insert(std::upper_bound(placed.begin(), placed.end(), id, [&](int a, int b) { return t[a].offset < t[b].offset; }), id);
  }
  return total;
}

}  // namespace nncv_hip
