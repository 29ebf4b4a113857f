// upsample.hip -- nearest-neighbour upsample by SCALE, HWC binary16.
// Replaces compiler/src/denox/compiler/implement/shaders/upsample/basic_upsample.comp:27-166:
//   out[h2, w2, c] = in[h2 / SCALE, w2 / SCALE, c].
// Definitions: CH, SCALE, VEC.  One thread per chunk of an *output* row segment, grid.y = input rows: it loads the
// source chunk (the SCALE threads that share one are neighbours in a wave, so the load is one fetch) and stores it into
// the SCALE output rows that replicate the input row.  Every store instruction of a wave then covers a contiguous run of
// an output row; with threads mapped over the input the replicas along x were separate instructions that each wrote
// every other pixel, which left narrow pixels' cache lines half written.
#include "common.h"
#ifndef KERNEL_NAME
#define KERNEL_NAME upsample_nearest
#endif
struct PushConstants { unsigned int W, H; }; // input extent
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
