// arena_plan.hpp -- places buffers with known lifetimes into one arena.
//
// A buffer is alive from the first to the last dispatch that binds one of its tensors; the dispatches of an instance run
// in order on one stream, so two buffers may share memory exactly when those closed intervals are disjoint.  The
// reference records first / last use per buffer (compiler/src/denox/compiler/placement/placement.cpp:276-300) and gives
// every buffer an allocation of its own (runtime/src/instance.cpp); this planner is the step it leaves out.
#pragma once
#include <algorithm>
#include <cstddef>
#include <cstdint>
#include <utility>
#include <vector>

namespace denox::runtime {

struct ArenaItem {
  uint64_t bytes = 0;      // what the buffer occupies, padding included
  int first = 0, last = 0; // closed interval of dispatch indices
};

// Offsets for every item, and the arena's size through `arenaBytes`.  Largest first, each at the lowest offset free of
// the items alive at the same time.
inline std::vector<uint64_t> plan_arena(const std::vector<ArenaItem> &items, uint64_t &arenaBytes) {
  std::vector<size_t> order(items.size());
  for (size_t i = 0; i < order.size(); ++i) order[i] = i;
  std::sort(order.begin(), order.end(), [&](size_t a, size_t b) { return items[a].bytes != items[b].bytes ? items[a].bytes > items[b].bytes : a < b; });
  std::vector<uint64_t> at(items.size(), 0);
  arenaBytes = 0;
  for (size_t k = 0; k < order.size(); ++k) {
    const ArenaItem &it = items[order[k]];
    std::vector<std::pair<uint64_t, uint64_t>> taken; // [begin, end) of placed items alive at the same time
    for (size_t j = 0; j < k; ++j) {
      const ArenaItem &o = items[order[j]];
      if (o.first <= it.last && it.first <= o.last) taken.emplace_back(at[order[j]], at[order[j]] + o.bytes);
    }
    std::sort(taken.begin(), taken.end());
    uint64_t pos = 0;
    for (const auto &iv : taken) {
      if (pos + it.bytes <= iv.first) break;
      pos = std::max(pos, iv.second);
    }
    at[order[k]] = pos;
    arenaBytes = std::max(arenaBytes, pos + it.bytes);
  }
  return at;
}

} // namespace denox::runtime
