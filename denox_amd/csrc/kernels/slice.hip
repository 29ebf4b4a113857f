// slice.hip -- spatial crop, HWC binary16.
// Replaces compiler/src/denox/compiler/implement/shaders/slice/memory_slice.comp:29-112:
//   out[h, w, c] = in[h + IN_TOP, w + IN_LEFT, c].
// Definitions: CH, VEC.
#include "common.h"
// The entry point is named per variant (KERNEL_NAME) so that profilers tell variants apart.
#ifndef KERNEL_NAME
#define KERNEL_NAME memory_slice
#endif
struct PushConstants { unsigned int IN_TOP, IN_LEFT, IN_W, IN_H, OUT_W, OUT_H; };
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = CH / VEC;
  const unsigned long long idx = (unsigned long long)DNX_BID_X * WG + DNX_TID;
  const unsigned long long total = (unsigned long long)pc.OUT_W * pc.OUT_H * CV;
  if (idx >= total) return;
  const unsigned cv = (unsigned)(idx % CV);
  const unsigned long long pix = idx / CV;
  const unsigned w = (unsigned)(pix % pc.OUT_W), h = (unsigned)(pix / pc.OUT_W);
  stv(OUT + (size_t)pix * CH + cv * VEC,
      ldv(IN + ((size_t)(h + pc.IN_TOP) * pc.IN_W + (w + pc.IN_LEFT)) * CH + cv * VEC));
}
