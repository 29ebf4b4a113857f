// copy_transform.hip -- strided channel copy, the explicit-concat building block.
// Replaces compiler/src/denox/compiler/implement/shaders/copy/copy_transform.comp:27-149:
//   dst[h, w, OUT_CH_OFFSET + c] = src[h, w, IN_CH_OFFSET + c],  c < COUNT.
// Definitions: IN_CH, IN_CH_OFFSET, OUT_CH, OUT_CH_OFFSET, COUNT, VEC.  grid.y = rows.
// With COUNT1 defined the kernel has two sources of COUNT and COUNT1 channels and writes whole pixels of
// OUT_CH = COUNT + COUNT1 channels, dst[h, w, :] = src0[h, w, :] ++ src1[h, w, :]: both halves of a concat in one launch.
// Two launches that each fill half of every pixel leave each cache line half written for the time between them, and
// narrow pixels then cost the memory a read-modify-write per line (2.2 - 3 TB/s against 5 - 6 for whole lines).
#include "common.h"
#ifndef KERNEL_NAME
#define KERNEL_NAME copy_transform
#endif
struct PushConstants { unsigned int W, H; };
#ifdef COUNT1
// Rows per thread: with RPT > 1 a thread loads its chunk of RPT consecutive rows before it stores any of them
// (grid.y = ceil(rows / RPT); rows past the end are loaded from the last row and not stored).  Measured to help this
// kernel on narrow, unaligned pixels (9 + 9 channels: 53 % -> 57 % of the HBM peak, 3 + 3: 44 % -> 50 %) and none of
// the one-source kernels.
#ifndef RPT
#define RPT 1
#endif
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN0, const ushort_t *__restrict__ IN1, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV0 = DNX_CHUNKS(COUNT), CV = CV0 + DNX_CHUNKS(COUNT1);
  const unsigned h0 = DNX_BID_Y * RPT;
  const unsigned i = DNX_ROW_INDEX();
  if (i >= pc.W * CV) return;
  const unsigned w = i / CV, cv = i - w * CV;
  const bool second = cv >= CV0;
  chunk_t v[RPT];
#pragma unroll
  for (unsigned u = 0; u < RPT; ++u) {
    const size_t pix = (size_t)(h0 + u < pc.H ? h0 + u : pc.H - 1) * pc.W + w;
    v[u] = second ? ld_chunk<COUNT1>(IN1 + pix * COUNT1, cv - CV0) : ld_chunk<COUNT>(IN0 + pix * COUNT, cv);
  }
#pragma unroll
  for (unsigned u = 0; u < RPT; ++u) {
    if (h0 + u >= pc.H) break;
    ushort_t *dst = OUT + ((size_t)(h0 + u) * pc.W + w) * (COUNT + COUNT1);
    if (second) st_chunk<COUNT1>(dst + COUNT, cv - CV0, v[u]);
    else st_chunk<COUNT>(dst, cv, v[u]);
  }
}
#else
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = DNX_CHUNKS(COUNT);
  const unsigned h = DNX_BID_Y;
  const unsigned i = DNX_ROW_INDEX();
  if (i >= pc.W * CV) return;
  const unsigned w = i / CV, cv = i - w * CV;
  const size_t pix = (size_t)h * pc.W + w;
  st_chunk<COUNT>(OUT + pix * OUT_CH + OUT_CH_OFFSET, cv, ld_chunk<COUNT>(IN + pix * IN_CH + IN_CH_OFFSET, cv));
}
#endif
