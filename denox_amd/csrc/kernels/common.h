// Shared helpers for the bandwidth kernels.  Every kernel moves one chunk of up to 8 channels (16 bytes) per thread.
//   VEC = 8: all channel counts, pitches and offsets involved are multiples of 8, every chunk is a full, 16-byte
//            aligned vector.
//   VEC = 1: any channel count.  A pixel of N channels has ceil(N / 8) chunks; the full ones are moved with 16-byte
//            accesses at 2-byte alignment (the memory system of this GPU serves such accesses, and the compiler emits a
//            single instruction for them), the last one, of N % 8 channels, with an 8-, a 4- and a 2-byte access as the
//            count's bits ask -- never a byte outside the pixel's own channel range, which may lie inside a wider tensor.
//
// Launch geometry (all of them): grid.y = rows of the iteration space, grid.x * WG threads
// cover one row of width * (chunks per pixel) vectors.  Indices inside a row are 32-bit and
// only divided by compile-time constants; nothing divides by a run-time extent.
#include "prelude.h"
typedef unsigned short ushort_t;
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

// PLANAR (pool, upsample, activation): the tensors are channel-block-major (CHWC8, [C/8][H][W][8]): every 8-channel plane is
// an HWC image of 8 channels, so the kernel is compiled with CH = 8, VEC = 8 and grid.z = C / 8 selects the plane.
#ifndef WG
#define WG 256
#endif
// Channels between consecutive OUTPUT pixels of the single-source kernels (pool, upsample, activation, pad, slice):
// their own channel count CH, or the channel count of a wider tensor when the result is stored straight into its
// channel range of a concat's output (OUT then points at the range's first channel).
#ifndef OPITCH
#define OPITCH CH
#endif

#if VEC != 8 && VEC != 1
#error "VEC must be 1 or 8"
#endif
typedef uint4v vec_t;
typedef unsigned int uint2v __attribute__((ext_vector_type(2)));
typedef uint4v uint4u __attribute__((aligned(2)));
typedef uint2v uint2u __attribute__((aligned(2)));
typedef unsigned int uint1u __attribute__((aligned(2)));

// What one thread moves: a chunk of 8 channels and, when VEC = 1 and it is the pixel's last full chunk, the partial chunk
// behind it too (so a 9-channel pixel is one thread's 16 + 2 bytes, not a full thread and a nearly idle one).
struct chunk_t { vec_t a, b; };

// threads per pixel of n channels
#define DNX_CHUNKS(n) (VEC == 8 ? (n) / 8 : ((n) < 8 ? 1 : (n) / 8))
// whether thread cv of a pixel of N channels also carries the partial chunk
template <unsigned N> __device__ DNX_INLINE bool has_tail(unsigned cv) {
  return VEC == 1 && N > 8 && N % 8 != 0 && cv == N / 8 - 1;
}

// R < 8 channels at p, as an 8-, a 4- and a 2-byte access where R's bits ask; the other lanes read as zero
template <unsigned R> __device__ DNX_INLINE vec_t ld_part(const ushort_t *p) {
  vec_t v = {};
  if (R & 4) {
    const uint2v a = *reinterpret_cast<const uint2u *>(p);
    v[0] = a[0];
    v[1] = a[1];
  }
  if (R & 2) v[(R & 4) / 2] = *reinterpret_cast<const uint1u *>(p + (R & 4));
  if (R & 1) v[(R & 6) / 2] = p[R & 6];
  return v;
}
template <unsigned R> __device__ DNX_INLINE void st_part(ushort_t *p, vec_t v) {
  if (R & 4) {
    uint2v a;
    a[0] = v[0];
    a[1] = v[1];
    *reinterpret_cast<uint2u *>(p) = a;
  }
  if (R & 2) *reinterpret_cast<uint1u *>(p + (R & 4)) = v[(R & 4) / 2];
  if (R & 1) p[R & 6] = (ushort_t)v[(R & 6) / 2];
}

// Thread cv's share of the pixel of N channels that starts at p.
template <unsigned N> __device__ DNX_INLINE chunk_t ld_chunk(const ushort_t *p, unsigned cv) {
  chunk_t c = {};
#if VEC == 8
  c.a = *reinterpret_cast<const uint4v *>(p + cv * 8);
#else
  if (N < 8) {
    c.a = ld_part<N % 8>(p);
  } else {
    c.a = *reinterpret_cast<const uint4u *>(p + cv * 8);
    if (has_tail<N>(cv)) c.b = ld_part<N % 8>(p + (N / 8) * 8);
  }
#endif
  return c;
}
template <unsigned N> __device__ DNX_INLINE void st_chunk(ushort_t *p, unsigned cv, chunk_t c) {
#if VEC == 8
  *reinterpret_cast<uint4v *>(p + cv * 8) = c.a;
#else
  if (N < 8) {
    st_part<N % 8>(p, c.a);
  } else {
    *reinterpret_cast<uint4u *>(p + cv * 8) = c.a;
    if (has_tail<N>(cv)) st_part<N % 8>(p + (N / 8) * 8, c.b);
  }
#endif
}

// binary16 "replace only when strictly greater", the order-dependent max the
// pool uses; +0 and -0 compare equal so the earlier value is kept.
__device__ DNX_INLINE vec_t max_keep_first(vec_t acc, vec_t v) {
  half8 a = __builtin_bit_cast(half8, acc);
  const half8 b = __builtin_bit_cast(half8, v);
#pragma unroll
  for (int e = 0; e < 8; ++e) a[e] = b[e] > a[e] ? b[e] : a[e];
  return __builtin_bit_cast(uint4v, a);
}

// FLAT (activation, pad, slice with VEC = 1 and a result that is a tensor of its own): a row of W pixels of any channel
// count is one run of W * CH consecutive halves in both tensors, so the row is moved as such a run instead of pixel by
// pixel.  Thread i stores the i-th 16-byte ALIGNED vector of the destination run -- whole cache lines from consecutive
// lanes, no 2-, 4- or 8-byte pieces -- and loads the 8 halves that belong there with one 16-byte load at whatever 2-byte
// alignment the source has.  The first and the last vector of a run may reach into the neighbouring rows: those two are
// moved element by element, inside the run only.  The grid covers W * CH / 8 + 1 vectors per row.
// F maps a vector of 8 halves (identity for the copies).
template <typename F>
__device__ DNX_INLINE void flat_row(const ushort_t *__restrict__ src, ushort_t *__restrict__ dst, unsigned n, unsigned i, F f) {
  const unsigned a = (unsigned)(((size_t)dst >> 1) & 7u); // halves between the previous 16-byte boundary and the run's start
  const int e0 = (int)(i * 8u) - (int)a;                   // first half of this thread's vector, relative to the run
  if (e0 >= (int)n)
    return;
  if (e0 >= 0 && e0 + 8 <= (int)n) {
    const vec_t v = *reinterpret_cast<const uint4u *>(src + e0);
    *reinterpret_cast<uint4v *>(dst + e0) = f(v);
  } else {
    const int lo = e0 < 0 ? 0 : e0, hi = e0 + 8 < (int)n ? e0 + 8 : (int)n;
    for (int e = lo; e < hi; ++e) {
      vec_t v = {};
      v[0] = src[e];
      dst[e] = (ushort_t)f(v)[0];
    }
  }
}
#define DNX_FLAT_VECTORS(w) (((w) * CH + 7u) / 8u + 1u) // vectors a row's grid must cover

// position of this thread inside its row: vector index `i` in [0, rowVectors)
#define DNX_ROW_INDEX() (DNX_BID_X * WG + (unsigned)DNX_TID)
