// Shared helpers for the bandwidth kernels.  Every kernel processes VEC
// channels per thread: VEC = 8 (one 16-byte access) when all channel counts and
// offsets involved are multiples of 8, else VEC = 1 (2-byte accesses).
//
// Launch geometry (all of them): grid.y = rows of the iteration space, grid.x * WG threads
// cover one row of width * (channels / VEC) vectors.  Indices inside a row are 32-bit and
// only divided by compile-time constants; nothing divides by a run-time extent.
#include "prelude.h"
typedef unsigned short ushort_t;
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

#ifndef WG
#define WG 256
#endif
// Channels between consecutive OUTPUT pixels of the single-source kernels (pool, upsample, activation, pad, slice):
// their own channel count CH, or the channel count of a wider tensor when the result is stored straight into its
// channel range of a concat's output (OUT then points at the range's first channel).
#ifndef OPITCH
#define OPITCH CH
#endif

#if VEC == 8
typedef uint4v vec_t;
#elif VEC == 1
typedef ushort_t vec_t;
#else
#error "VEC must be 1 or 8"
#endif

__device__ DNX_INLINE vec_t ldv(const ushort_t *p) {
  return *reinterpret_cast<const vec_t *>(p);
}
__device__ DNX_INLINE void stv(ushort_t *p, vec_t v) {
  *reinterpret_cast<vec_t *>(p) = v;
}

// binary16 "replace only when strictly greater", the order-dependent max the
// pool uses; +0 and -0 compare equal so the earlier value is kept.
__device__ DNX_INLINE ushort_t max_keep_first(ushort_t acc, ushort_t v) {
  const _Float16 a = __builtin_bit_cast(_Float16, acc);
  const _Float16 b = __builtin_bit_cast(_Float16, v);
  return b > a ? v : acc;
}

// position of this thread inside its row: vector index `i` in [0, rowVectors)
#define DNX_ROW_INDEX() (DNX_BID_X * WG + (unsigned)DNX_TID)
