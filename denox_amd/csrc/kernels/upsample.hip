// upsample.hip -- nearest-neighbour upsample by SCALE, HWC binary16.
// Replaces compiler/src/denox/compiler/implement/shaders/upsample/basic_upsample.comp:27-166:
//   out[h2, w2, c] = in[h2 / SCALE, w2 / SCALE, c].
// Definitions: CH, SCALE, VEC.  One thread per *input* vector; it writes the
// SCALE x SCALE replicas, so every input byte is fetched once.
#include "common.h"
// The entry point is named per variant (KERNEL_NAME) so that profilers tell variants apart.
#ifndef KERNEL_NAME
#define KERNEL_NAME upsample_nearest
#endif
struct PushConstants { unsigned int W, H; }; // input extent
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = CH / VEC;
  const unsigned long long idx = (unsigned long long)DNX_BID_X * WG + DNX_TID;
  const unsigned long long total = (unsigned long long)pc.W * pc.H * CV;
  if (idx >= total) return;
  const unsigned cv = (unsigned)(idx % CV);
  const unsigned long long pix = idx / CV;
  const unsigned w = (unsigned)(pix % pc.W), h = (unsigned)(pix / pc.W);
  const vec_t v = ldv(IN + (size_t)pix * CH + cv * VEC);
  const size_t W2 = (size_t)pc.W * SCALE;
#pragma unroll
  for (int r = 0; r < SCALE; ++r)
#pragma unroll
    for (int s = 0; s < SCALE; ++s)
      stv(OUT + (((size_t)h * SCALE + r) * W2 + (size_t)w * SCALE + s) * CH + cv * VEC, v);
}
