// pool.hip -- pool with kernel == stride (KX x KY), no padding, HWC binary16.
// Replaces compiler/src/denox/compiler/implement/shaders/pool/basic_pool.comp:27-230:
//   out[oh, ow, c] = max_{r<KY, s<KX} in[oh*KY + r, ow*KX + s, c],
//   output extent floor(H/KY) x floor(W/KX).
// With AVG defined the window is averaged instead (PoolFunction::Avg, which the reference's model carries,
// common/src/denox/common/PoolFunction.hpp:7-10, but its shader refuses): the KX*KY values are summed in binary32 in
// row-major window order, the sum is multiplied by the binary32 constant 1/(KX*KY) and rounded once to binary16.
// Definitions: CH, KX, KY, VEC, [AVG].  One thread per output vector; grid.y = output rows.
#include "common.h"
#ifndef KERNEL_NAME
#define KERNEL_NAME pool_max
#endif
struct PushConstants { unsigned int W, H; };
#ifdef AVG
// The mean is defined with two roundings: the product to binary32, then that to binary16.  Left to itself the compiler
// merges the multiply and the conversion into one mixed-precision instruction that rounds the exact product once, which
// differs in the last place wherever the binary32 product lands on a binary16 tie (sums divisible by 3 under a 2x3 window
// do, often).  Passing the product through an empty asm keeps the two steps apart.
__device__ DNX_INLINE float rounded_f32(float x) {
  asm volatile("" : "+v"(x));
  return x;
}
#endif
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = CH / VEC;
  const unsigned W2 = pc.W / KX;
  const unsigned oh = DNX_BID_Y;
  const unsigned i = DNX_ROW_INDEX();
  if (i >= W2 * CV) return;
  const unsigned ow = i / CV, cv = i - ow * CV;
  const ushort_t *src = IN + ((size_t)(oh * KY) * pc.W + (size_t)ow * KX) * CH + cv * VEC;
#ifdef AVG
  float sum[VEC];
#pragma unroll
  for (int r = 0; r < KY; ++r)
#pragma unroll
    for (int s = 0; s < KX; ++s) {
      const vec_t v = ldv(src + ((size_t)r * pc.W + s) * CH);
#if VEC == 8
      const half8 h = __builtin_bit_cast(half8, v);
#pragma unroll
      for (int e = 0; e < 8; ++e) sum[e] = (r == 0 && s == 0) ? (float)h[e] : sum[e] + (float)h[e];
#else
      const float f = (float)__builtin_bit_cast(_Float16, v);
      sum[0] = (r == 0 && s == 0) ? f : sum[0] + f;
#endif
    }
  constexpr float inv = 1.0f / (float)(KX * KY);
#if VEC == 8
  half8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (_Float16)rounded_f32(sum[e] * inv);
  const vec_t acc = __builtin_bit_cast(uint4v, o);
#else
  const vec_t acc = __builtin_bit_cast(ushort_t, (_Float16)rounded_f32(sum[0] * inv));
#endif
#else
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
#endif
  stv(OUT + ((size_t)oh * W2 + ow) * OPITCH + cv * VEC, acc);
}
