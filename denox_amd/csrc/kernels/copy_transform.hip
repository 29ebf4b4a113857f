// copy_transform.hip -- strided channel copy, the explicit-concat building block.
// Replaces compiler/src/denox/compiler/implement/shaders/copy/copy_transform.comp:27-149:
//   dst[h, w, OUT_CH_OFFSET + c] = src[h, w, IN_CH_OFFSET + c],  c < COUNT.
// Definitions: IN_CH, IN_CH_OFFSET, OUT_CH, OUT_CH_OFFSET, COUNT, VEC.
#include "common.h"
// The entry point is named per variant (KERNEL_NAME) so that profilers tell variants apart.
#ifndef KERNEL_NAME
#define KERNEL_NAME copy_transform
#endif
struct PushConstants { unsigned int W, H; };
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = COUNT / VEC;
  const unsigned long long idx = (unsigned long long)DNX_BID_X * WG + DNX_TID;
  const unsigned long long total = (unsigned long long)pc.W * pc.H * CV;
  if (idx >= total) return;
  const unsigned cv = (unsigned)(idx % CV);
  const unsigned long long pix = idx / CV;
  stv(OUT + (size_t)pix * OUT_CH + OUT_CH_OFFSET + cv * VEC,
      ldv(IN + (size_t)pix * IN_CH + IN_CH_OFFSET + cv * VEC));
}
