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

// Offsets for every item, and the arena's size through `arenaBytes`.  Largest first (of equal sizes the one used later
// first).  An item goes where it does not grow the arena if such a place exists, and among those places to the one that
// shares the most bytes with items whose life ends right before its own begins, or begins right after its own ends --
// counted cyclically over the `period` dispatches of an inference, since the first dispatch of the next inference
// follows the last one of this: the successor then overwrites lines of its dead predecessor that still sit, modified, in
// the memory-side cache, and they are never written back.  Ties go to the lowest offset.
inline std::vector<uint64_t> plan_arena(const std::vector<ArenaItem> &items, uint64_t &arenaBytes, int period = 0) {
  std::vector<size_t> order(items.size());
  for (size_t i = 0; i < order.size(); ++i) order[i] = i;
  std::sort(order.begin(), order.end(), [&](size_t a, size_t b) {
    if (items[a].bytes != items[b].bytes) return items[a].bytes > items[b].bytes;
    if (items[a].first != items[b].first) return items[a].first > items[b].first;
    return a < b;
  });
  if (period >= 0) // (a negative period switches the preference off)
    for (const ArenaItem &it : items) period = std::max(period, it.last + 1);
  auto follows = [&](const ArenaItem &a, const ArenaItem &b) { // b begins right after a ends
    return period > 0 && (b.first - a.last + period) % period == 1;
  };
  std::vector<uint64_t> at(items.size(), 0);
  arenaBytes = 0;
  for (size_t k = 0; k < order.size(); ++k) {
    const ArenaItem &it = items[order[k]];
    std::vector<std::pair<uint64_t, uint64_t>> taken, liked; // [begin, end) of placed items alive at the same time / neighbours in time
    std::vector<uint64_t> cand{0};
    for (size_t j = 0; j < k; ++j) {
      const ArenaItem &o = items[order[j]];
      const uint64_t b = at[order[j]], e = b + o.bytes;
      if (o.first <= it.last && it.first <= o.last) {
        taken.emplace_back(b, e);
        cand.push_back(e);
      } else if (follows(o, it) || follows(it, o)) {
        liked.emplace_back(b, e);
        cand.push_back(b);
        if (e >= it.bytes) cand.push_back(e - it.bytes);
      }
    }
    std::sort(cand.begin(), cand.end());
    bool have = false, bestFits = false;
    uint64_t best = 0, bestShared = 0;
    for (uint64_t pos : cand) {
      const uint64_t end = pos + it.bytes;
      bool free = true;
      for (const auto &iv : taken)
        if (pos < iv.second && iv.first < end) { free = false; break; }
      if (!free) continue;
      const bool fits = end <= arenaBytes;
      uint64_t shared = 0;
      for (const auto &iv : liked)
        if (pos < iv.second && iv.first < end) shared += std::min(end, iv.second) - std::max(pos, iv.first);
      const bool better = !have || (fits && !bestFits) || (fits == bestFits && fits && shared > bestShared);
      if (better) { have = true; best = pos; bestFits = fits; bestShared = shared; }
    }
    at[order[k]] = best;
    arenaBytes = std::max(arenaBytes, best + it.bytes);
  }
  return at;
}

} // namespace denox::runtime
