// relayout.hip -- interface layout conversion between HWC, CHW and CHWC8
// (index formulas of common/src/denox/memory/tensor/ActivationLayout.hpp:37-66).
// The reference declares SSBO_CHW (dnx.fbs:86-95) but ships no shader that
// accepts it; this kernel is the missing conversion.  One thread per pixel
// moves all CH channels, so the pixel-major side is accessed contiguously per
// thread and the plane-major side is coalesced across threads.
// Definitions: CH, SRC_LAYOUT, DST_LAYOUT (0 HWC, 1 CHW, 2 CHWC8).
#include "prelude.h"
typedef unsigned short ushort_t;
#ifndef WG
#define WG 256
#endif
// The entry point is named per variant (KERNEL_NAME) so that profilers tell variants apart.
#ifndef KERNEL_NAME
#define KERNEL_NAME relayout
#endif
struct PushConstants { unsigned int W, H; };
__device__ DNX_INLINE size_t lidx(int layout, size_t HW, size_t pix, unsigned c) {
  if (layout == 0) return pix * CH + c;
  if (layout == 1) return (size_t)c * HW + pix;
  return (size_t)(c >> 3) * (HW * 8) + pix * 8 + (c & 7);
}
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  const size_t HW = (size_t)pc.W * pc.H;
  const size_t pix = (size_t)DNX_BID_X * WG + DNX_TID;
  if (pix >= HW) return;
#pragma unroll 8
  for (unsigned c = 0; c < CH; ++c)
    OUT[lidx(DST_LAYOUT, HW, pix, c)] = IN[lidx(SRC_LAYOUT, HW, pix, c)];
}
