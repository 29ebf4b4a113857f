// relayout.hip -- interface layout conversion between HWC, CHW and CHWC8
// (index formulas of common/src/denox/memory/tensor/ActivationLayout.hpp:37-66).
// The reference declares SSBO_CHW (dnx.fbs:86-95) but ships no shader that
// accepts it; this kernel is the missing conversion.
// Definitions: CH, SRC_LAYOUT, DST_LAYOUT (0 HWC, 1 CHW, 2 CHWC8).
//
// Three strategies, chosen at compile time:
//   * HWC <-> CHWC8 (CH % 8 == 0): both sides keep 8 channels contiguous, so one thread moves one
//     16-byte vector; 8 consecutive threads cover one pixel, a wave covers 128 contiguous bytes per plane.
//     Grid: ceil(H*W*CH/8 / WG) workgroups.
//   * HWC <-> CHW (CH <= 128): a workgroup transposes WG pixels through LDS, so that the plane-major
//     side is accessed one plane at a time (coalesced across pixels) and the pixel-major side as a flat
//     run of 16-byte vectors.  Grid: ceil(H*W / WG) workgroups.
//   * anything else: one thread per pixel, element by element.  Grid: ceil(H*W / WG).
#include "prelude.h"
typedef unsigned short ushort_t;
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
#ifndef WG
#define WG 256
#endif
#ifndef KERNEL_NAME
#define KERNEL_NAME relayout
#endif
struct PushConstants { unsigned int W, H; };

#define IS_BLOCKY(l) ((l) == 0 || (l) == 2)
#if IS_BLOCKY(SRC_LAYOUT) && IS_BLOCKY(DST_LAYOUT) && (CH % 8 == 0)
#define MODE_VEC8 1
#elif ((SRC_LAYOUT == 0 && DST_LAYOUT == 1) || (SRC_LAYOUT == 1 && DST_LAYOUT == 0)) && (CH <= 128)
#define MODE_LDS 1
#endif

__device__ DNX_INLINE size_t lidx(int layout, size_t HW, size_t pix, unsigned c) {
  if (layout == 0) return pix * CH + c;
  if (layout == 1) return (size_t)c * HW + pix;
  return (size_t)(c >> 3) * (HW * 8) + pix * 8 + (c & 7);
}

extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  const size_t HW = (size_t)pc.W * pc.H;
#if defined(MODE_VEC8)
  constexpr unsigned CV = CH / 8;
  const size_t i = (size_t)DNX_BID_X * WG + DNX_TID;
  if (i >= HW * CV) return;
  const size_t pix = i / CV;
  const unsigned c = (unsigned)(i - pix * CV) * 8;
  *reinterpret_cast<uint4v *>(OUT + lidx(DST_LAYOUT, HW, pix, c)) = *reinterpret_cast<const uint4v *>(IN + lidx(SRC_LAYOUT, HW, pix, c));
#elif defined(MODE_LDS)
  __shared__ __attribute__((aligned(16))) ushort_t tile[WG * CH];
  const size_t pix0 = (size_t)DNX_BID_X * WG;
  const unsigned t = DNX_TID;
  const size_t left = HW - pix0;
  const unsigned npix = left < WG ? (unsigned)left : WG; // pixels of this tile
  const unsigned nelem = npix * CH;
  // The pixel-major run of this tile starts at element pix0 * CH: a multiple of WG * CH * 2 bytes, so 16-byte aligned.
#if SRC_LAYOUT == 1 // CHW -> HWC
  if (t < npix)
#pragma unroll 8
    for (unsigned c = 0; c < CH; ++c) tile[t * CH + c] = IN[(size_t)c * HW + pix0 + t];
  DNX_SYNC();
  ushort_t *dst = OUT + pix0 * CH;
  for (unsigned e = t * 8; e < nelem; e += WG * 8) {
    if (e + 8 <= nelem) *reinterpret_cast<uint4v *>(dst + e) = *reinterpret_cast<const uint4v *>(tile + e);
    else for (unsigned k = e; k < nelem; ++k) dst[k] = tile[k];
  }
#else // HWC -> CHW
  const ushort_t *src = IN + pix0 * CH;
  for (unsigned e = t * 8; e < nelem; e += WG * 8) {
    if (e + 8 <= nelem) *reinterpret_cast<uint4v *>(tile + e) = *reinterpret_cast<const uint4v *>(src + e);
    else for (unsigned k = e; k < nelem; ++k) tile[k] = src[k];
  }
  DNX_SYNC();
  if (t < npix)
#pragma unroll 8
    for (unsigned c = 0; c < CH; ++c) OUT[(size_t)c * HW + pix0 + t] = tile[t * CH + c];
#endif
#else
  const size_t pix = (size_t)DNX_BID_X * WG + DNX_TID;
  if (pix >= HW) return;
#pragma unroll 8
  for (unsigned c = 0; c < CH; ++c)
    OUT[lidx(DST_LAYOUT, HW, pix, c)] = IN[lidx(SRC_LAYOUT, HW, pix, c)];
#endif
}
