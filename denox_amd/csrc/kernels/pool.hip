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
  constexpr unsigned CV = DNX_CHUNKS(CH);
  const unsigned W2 = pc.W / KX;
#ifdef PLANAR
  IN += (size_t)DNX_BID_Z * pc.W * pc.H * 8;
  OUT += (size_t)DNX_BID_Z * W2 * (pc.H / KY) * 8;
#endif
  const unsigned oh = DNX_BID_Y;
  const unsigned i = DNX_ROW_INDEX();
  if (i >= W2 * CV) return;
  const unsigned ow = i / CV, cv = i - ow * CV;
  const ushort_t *src = IN + ((size_t)(oh * KY) * pc.W + (size_t)ow * KX) * CH;
#ifdef AVG
  float sumA[8], sumB[8];
#pragma unroll
  for (int r = 0; r < KY; ++r)
#pragma unroll
    for (int s = 0; s < KX; ++s) {
      const chunk_t c = ld_chunk<CH>(src + ((size_t)r * pc.W + s) * CH, cv);
      const half8 ha = __builtin_bit_cast(half8, c.a), hb = __builtin_bit_cast(half8, c.b);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        sumA[e] = (r == 0 && s == 0) ? (float)ha[e] : sumA[e] + (float)ha[e];
        sumB[e] = (r == 0 && s == 0) ? (float)hb[e] : sumB[e] + (float)hb[e];
      }
    }
  constexpr float inv = 1.0f / (float)(KX * KY);
  half8 oa, ob;
#pragma unroll
  for (int e = 0; e < 8; ++e) oa[e] = (_Float16)rounded_f32(sumA[e] * inv), ob[e] = (_Float16)rounded_f32(sumB[e] * inv);
  const chunk_t acc = {__builtin_bit_cast(uint4v, oa), __builtin_bit_cast(uint4v, ob)};
#else
  chunk_t acc = ld_chunk<CH>(src, cv);
#pragma unroll
  for (int r = 0; r < KY; ++r)
#pragma unroll
    for (int s = 0; s < KX; ++s) {
      if (r == 0 && s == 0) continue;
      const chunk_t c = ld_chunk<CH>(src + ((size_t)r * pc.W + s) * CH, cv);
      acc.a = max_keep_first(acc.a, c.a);
      acc.b = max_keep_first(acc.b, c.b);
    }
#endif
  st_chunk<CH>(OUT + ((size_t)oh * W2 + ow) * OPITCH, cv, acc);
}
