// upsample.hip -- nearest-neighbour upsample by SCALE, HWC binary16.
// Replaces compiler/src/denox/compiler/implement/shaders/upsample/basic_upsample.comp:27-166:
//   out[h2, w2, c] = in[h2 / SCALE, w2 / SCALE, c].
// Definitions: CH, SCALE, VEC; FLAT: rows moved as runs of aligned vectors (below).  One thread per chunk of an *output* row segment, grid.y = input rows: it loads the
// source chunk (the SCALE threads that share one are neighbours in a wave, so the load is one fetch) and stores it into
// the SCALE output rows that replicate the input row.  Every store instruction of a wave then covers a contiguous run of
// an output row; with threads mapped over the input the replicas along x were separate instructions that each wrote
// every other pixel, which left narrow pixels' cache lines half written.
#include "common.h"
#ifndef KERNEL_NAME
#define KERNEL_NAME upsample_nearest
#endif
struct PushConstants { unsigned int W, H; }; // input extent
#ifdef FLAT
// Pixels of CH >= 8 channels whose byte size is not a multiple of 16 (VEC = 1), a result that is a tensor of its own.  An
// output row is one run of W * SCALE * CH consecutive halves; thread i stores the i-th 16-byte ALIGNED vector of each of the
// SCALE runs that replicate input row h (whole cache lines from consecutive lanes, no 2- to 8-byte pieces).  The 8 halves of
// such a vector belong to at most two output pixels.  When those replicate two different source pixels they are consecutive
// in the source as well, and one 16-byte load (at whatever 2-byte alignment) fetches them; when both replicate the same
// source pixel the vector is the end of that pixel followed by its start, two loads and a select.  The first and the last
// vector of a run, which may reach into the neighbouring rows, and vectors whose loads would leave the tensor are moved
// element by element.  A thread per 8-channel chunk of a pixel reached 44 - 48 % of the memory bandwidth on 9 and 73 channels.
// grid.x covers W * SCALE * CH / 8 + 1 vectors, grid.y = input rows.
static_assert(CH >= 8, "at most one pixel boundary inside a vector");
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  const unsigned h = DNX_BID_Y;
  const unsigned i = DNX_ROW_INDEX();
  const unsigned nd = pc.W * SCALE * CH;           // halves of an output run
  const size_t srcRow = (size_t)h * pc.W * CH;     // first half of the source row
  const size_t srcEnd = (size_t)pc.W * pc.H * CH;  // halves in the source tensor
  auto source = [&](unsigned e) { // source half of half e of the run
    const unsigned op = e / CH, c = e - op * CH;
    return IN[srcRow + (size_t)(op / SCALE) * CH + c];
  };
  // When a run's length is a multiple of 8 halves, the SCALE runs start at the same offset from a 16-byte boundary and one
  // assembled vector serves them all (uniform branch).
  const unsigned copies = nd % 8u == 0u ? SCALE : 1u;
  for (unsigned r = 0; r < SCALE; r += copies) {
    ushort_t *dst = OUT + ((size_t)h * SCALE + r) * nd;
    const unsigned a = (unsigned)(((size_t)dst >> 1) & 7u); // halves between the previous 16-byte boundary and the run's start
    const int e0 = (int)(i * 8u) - (int)a;
    if (e0 >= (int)nd)
      continue;
    bool whole = e0 >= 0 && e0 + 8 <= (int)nd;
    if (whole) {
      const unsigned op = (unsigned)e0 / CH, c = (unsigned)e0 - op * CH;
      const unsigned t = CH - c;                                  // halves until the output pixel ends
      const size_t b1 = srcRow + (size_t)(op / SCALE) * CH + c;   // source of half 0 of the vector
      const size_t b2 = srcRow + (size_t)((op + 1) / SCALE) * CH; // source of half t (the next output pixel's first channel)
      whole = b1 + 8 <= srcEnd && b2 >= t && b2 - t + 8 <= srcEnd;
      if (whole) {
        const half8 v1 = __builtin_bit_cast(half8, *reinterpret_cast<const uint4u *>(IN + b1));
        half8 v = v1;
        if (t < 8 && b2 - t != b1) { // both output pixels replicate one source pixel: its end, then its start again
          const half8 v2 = __builtin_bit_cast(half8, *reinterpret_cast<const uint4u *>(IN + (b2 - t)));
#pragma unroll
          for (unsigned j = 0; j < 8; ++j) v[j] = j < t ? v1[j] : v2[j];
        }
        for (unsigned q = 0; q < copies; ++q)
          *reinterpret_cast<uint4v *>(dst + (size_t)q * nd + e0) = __builtin_bit_cast(uint4v, v);
      }
    }
    if (!whole) {
      const int lo = e0 < 0 ? 0 : e0, hi = e0 + 8 < (int)nd ? e0 + 8 : (int)nd;
      for (int e = lo; e < hi; ++e) {
        const ushort_t v = source((unsigned)e);
        for (unsigned q = 0; q < copies; ++q) dst[(size_t)q * nd + e] = v;
      }
    }
  }
}
#else
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = DNX_CHUNKS(CH);
#ifdef PLANAR
  IN += (size_t)DNX_BID_Z * pc.W * pc.H * 8;
  OUT += (size_t)DNX_BID_Z * pc.W * pc.H * (SCALE * SCALE * 8);
#endif
  const unsigned h = DNX_BID_Y;
  const unsigned i = DNX_ROW_INDEX();
  if (i >= pc.W * SCALE * CV) return;
  const unsigned w2 = i / CV, cv = i - w2 * CV;
  const unsigned w = w2 / SCALE;
  const chunk_t v = ld_chunk<CH>(IN + ((size_t)h * pc.W + w) * CH, cv);
  const size_t W2 = (size_t)pc.W * SCALE;
#pragma unroll
  for (int r = 0; r < SCALE; ++r) st_chunk<CH>(OUT + (((size_t)h * SCALE + r) * W2 + w2) * OPITCH, cv, v);
}
#endif
