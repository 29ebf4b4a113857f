// activation.hip -- stand-alone elementwise activation in binary16.
// Replaces compiler/src/denox/compiler/implement/shaders/activation/basic_activation.comp:26-184:
//   ReLU: max(v, 0);  LeakyReLU: max(v, alpha * v) with alpha and the product in binary16.
// Definitions: CH, ACT (1 ReLU, 2 LeakyReLU), ALPHA, VEC; FLAT: rows moved as runs of halves (common.h).  grid.y = rows.
#include "common.h"
#ifndef ALPHA
#define ALPHA 0.0f
#endif
#ifndef KERNEL_NAME
#define KERNEL_NAME activation
#endif
struct PushConstants { unsigned int W, H; };
__device__ DNX_INLINE _Float16 act1(_Float16 v) {
#if ACT == 1
  return v > (_Float16)0.0f ? v : (_Float16)0.0f;
#else
  const _Float16 av = (_Float16)(ALPHA) * v;
  return v > av ? v : av;
#endif
}
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = DNX_CHUNKS(CH);
#ifdef PLANAR
  IN += (size_t)DNX_BID_Z * pc.W * pc.H * 8;
  OUT += (size_t)DNX_BID_Z * pc.W * pc.H * 8;
#endif
  const unsigned i = DNX_ROW_INDEX();
#ifdef FLAT
  {
    const size_t row = (size_t)DNX_BID_Y * pc.W * CH;
    flat_row(IN + row, OUT + row, pc.W * CH, i, [](vec_t v) {
      half8 a = __builtin_bit_cast(half8, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) a[e] = act1(a[e]);
      return __builtin_bit_cast(vec_t, a);
    });
    return;
  }
#endif
  if (i >= pc.W * CV) return;
  const unsigned w = i / CV, cv = i - w * CV;
  const size_t pix = (size_t)DNX_BID_Y * pc.W + w;
  const chunk_t v = ld_chunk<CH>(IN + pix * CH, cv);
  half8 a = __builtin_bit_cast(half8, v.a), b = __builtin_bit_cast(half8, v.b);
#pragma unroll
  for (int e = 0; e < 8; ++e) a[e] = act1(a[e]), b[e] = act1(b[e]);
  st_chunk<CH>(OUT + pix * OPITCH, cv, chunk_t{__builtin_bit_cast(uint4v, a), __builtin_bit_cast(uint4v, b)});
}
