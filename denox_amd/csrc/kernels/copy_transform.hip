// copy_transform.hip -- strided channel copy, the explicit-concat building block.
// Replaces compiler/src/denox/compiler/implement/shaders/copy/copy_transform.comp:27-149:
//   dst[h, w, OUT_CH_OFFSET + c] = src[h, w, IN_CH_OFFSET + c],  c < COUNT.
// Definitions: IN_CH, IN_CH_OFFSET, OUT_CH, OUT_CH_OFFSET, COUNT, VEC.  grid.y = rows.
#include "common.h"
#ifndef KERNEL_NAME
#define KERNEL_NAME copy_transform
#endif
struct PushConstants { unsigned int W, H; };
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = COUNT / VEC;
  const unsigned h = DNX_BID_Y;
  const unsigned i = DNX_ROW_INDEX();
  if (i >= pc.W * CV) return;
  const unsigned w = i / CV, cv = i - w * CV;
  const size_t pix = (size_t)h * pc.W + w;
  stv(OUT + pix * OUT_CH + OUT_CH_OFFSET + cv * VEC, ldv(IN + pix * IN_CH + IN_CH_OFFSET + cv * VEC));
}
