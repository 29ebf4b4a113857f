// upsample.hip -- nearest-neighbour upsample by SCALE, HWC binary16.
// Replaces compiler/src/denox/compiler/implement/shaders/upsample/basic_upsample.comp:27-166:
//   out[h2, w2, c] = in[h2 / SCALE, w2 / SCALE, c].
// Definitions: CH, SCALE, VEC.  One thread per *input* vector (grid.y = input rows); it writes
// the SCALE x SCALE replicas, so every input byte is fetched once.
#include "common.h"
#ifndef KERNEL_NAME
#define KERNEL_NAME upsample_nearest
#endif
struct PushConstants { unsigned int W, H; }; // input extent
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = CH / VEC;
  const unsigned h = DNX_BID_Y;
  const unsigned i = DNX_ROW_INDEX();
  if (i >= pc.W * CV) return;
  const unsigned w = i / CV, cv = i - w * CV;
  const vec_t v = ldv(IN + ((size_t)h * pc.W + w) * CH + cv * VEC);
  const size_t W2 = (size_t)pc.W * SCALE;
#pragma unroll
  for (int r = 0; r < SCALE; ++r)
#pragma unroll
    for (int s = 0; s < SCALE; ++s)
      stv(OUT + (((size_t)h * SCALE + r) * W2 + (size_t)w * SCALE + s) * OPITCH + cv * VEC, v);
}
