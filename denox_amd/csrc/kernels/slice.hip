// slice.hip -- spatial crop, HWC binary16.
// Replaces compiler/src/denox/compiler/implement/shaders/slice/memory_slice.comp:29-112:
//   out[h, w, c] = in[h + IN_TOP, w + IN_LEFT, c].
// Definitions: CH, VEC; FLAT: rows moved as runs of halves (common.h).  grid.y = output rows.
#include "common.h"
#ifndef KERNEL_NAME
#define KERNEL_NAME memory_slice
#endif
struct PushConstants { unsigned int IN_TOP, IN_LEFT, IN_W, IN_H, OUT_W, OUT_H; };
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = DNX_CHUNKS(CH);
  const unsigned h = DNX_BID_Y;
  const unsigned i = DNX_ROW_INDEX();
#ifdef FLAT
  flat_row(IN + ((size_t)(h + pc.IN_TOP) * pc.IN_W + pc.IN_LEFT) * CH, OUT + (size_t)h * pc.OUT_W * CH, pc.OUT_W * CH, i, [](vec_t v) { return v; });
  return;
#endif
  if (i >= pc.OUT_W * CV) return;
  const unsigned w = i / CV, cv = i - w * CV;
  st_chunk<CH>(OUT + ((size_t)h * pc.OUT_W + w) * OPITCH, cv,
               ld_chunk<CH>(IN + ((size_t)(h + pc.IN_TOP) * pc.IN_W + (w + pc.IN_LEFT)) * CH, cv));
}
