// pool.hip -- max pool with kernel == stride (KX x KY), no padding, HWC binary16.
// Replaces compiler/src/denox/compiler/implement/shaders/pool/basic_pool.comp:27-230:
//   out[oh, ow, c] = max_{r<KY, s<KX} in[oh*KY + r, ow*KX + s, c],
//   output extent floor(H/KY) x floor(W/KX).
// Definitions: CH, KX, KY, VEC.  One thread per output vector; grid.y = output rows.
#include "common.h"
#ifndef KERNEL_NAME
#define KERNEL_NAME pool_max
#endif
struct PushConstants { unsigned int W, H; };
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = CH / VEC;
  const unsigned W2 = pc.W / KX;
  const unsigned oh = DNX_BID_Y;
  const unsigned i = DNX_ROW_INDEX();
  if (i >= W2 * CV) return;
  const unsigned ow = i / CV, cv = i - ow * CV;
  const ushort_t *src = IN + ((size_t)(oh * KY) * pc.W + (size_t)ow * KX) * CH + cv * VEC;
  vec_t acc = ldv(src);
#pragma unroll
  for (int r = 0; r < KY; ++r)
#pragma unroll
    for (int s = 0; s < KX; ++s) {
      if (r == 0 && s == 0) continue;
      const vec_t v = ldv(src + ((size_t)r * pc.W + s) * CH);
#if VEC == 8
      half8 a = __builtin_bit_cast(half8, acc), b = __builtin_bit_cast(half8, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) a[e] = b[e] > a[e] ? b[e] : a[e];
      acc = __builtin_bit_cast(uint4v, a);
#else
      acc = max_keep_first(acc, v);
#endif
    }
  stv(OUT + ((size_t)oh * W2 + ow) * OPITCH + cv * VEC, acc);
}
