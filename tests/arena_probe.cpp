// Test helper: exposes the arena planner of the runtime (a header-only routine) to ctypes.
#include "../denox_amd/csrc/runtime/arena_plan.hpp"

extern "C" int arena_probe_plan(int n, const unsigned long long *bytes, const int *first, const int *last, int period,
                                unsigned long long *offsets, unsigned long long *arena) {
  std::vector<denox::runtime::ArenaItem> items(static_cast<size_t>(n));
  for (int i = 0; i < n; ++i) items[static_cast<size_t>(i)] = denox::runtime::ArenaItem{bytes[i], first[i], last[i]};
  uint64_t total = 0;
  const std::vector<uint64_t> at = denox::runtime::plan_arena(items, total, period);
  for (int i = 0; i < n; ++i) offsets[i] = at[static_cast<size_t>(i)];
  *arena = total;
  return 0;
}
