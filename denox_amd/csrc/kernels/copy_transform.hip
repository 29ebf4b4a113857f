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
#if defined(COUNT1) && defined(FLAT)
// Two sources, pixels whose byte size is not a multiple of 16 (VEC = 1), assembled in LDS.  HWC rows are contiguous, so the
// concat is one-dimensional: output pixel q = src0 pixel q ++ src1 pixel q.  A workgroup takes PQ consecutive pixels (PQ
// a multiple of 8: the byte ranges of both sources and of the output then all start on 16-byte boundaries), loads the two
// source ranges with aligned 16-byte vectors into LDS, and writes the output range as aligned 4-byte words whose two
// halves it picks out of LDS.  Global memory sees nothing but aligned, coalesced accesses in both directions, whatever
// the channel counts; per-pixel accesses at 2-byte alignment reached 44 - 58 % of the memory bandwidth on such
// tensors.  grid.x = ceil(W * H / PQ).
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN0, const ushort_t *__restrict__ IN1, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned COUT = COUNT + COUNT1;
  static_assert(PQ % 8 == 0, "pixel groups of 8 keep every range 16-byte aligned");
  __shared__ __attribute__((aligned(16))) ushort_t s0[PQ * COUNT + 8]; // (+8: the word that ends a workgroup's range may look one pixel further;
  __shared__ __attribute__((aligned(16))) ushort_t s1[PQ * COUNT1];   //  with PQ * COUT even that half is never stored, only read)
  const unsigned total = pc.W * pc.H;
  const unsigned q0 = DNX_BID_X * PQ;
  const unsigned tid = (unsigned)DNX_TID;
  // whole vectors inside a source are loaded as such; the last, partial one element by element (never a byte outside the tensor)
  const unsigned elems0 = total * COUNT, elems1 = total * COUNT1;
  for (unsigned v = tid; v < PQ * COUNT / 8; v += WG) {
    const unsigned e0 = q0 * COUNT + v * 8;
    if (e0 + 8 <= elems0) *reinterpret_cast<uint4v *>(s0 + v * 8) = *reinterpret_cast<const uint4v *>(IN0 + e0);
    else
      for (unsigned e = 0; e < 8; ++e)
        if (e0 + e < elems0) s0[v * 8 + e] = IN0[e0 + e];
  }
  for (unsigned v = tid; v < PQ * COUNT1 / 8; v += WG) {
    const unsigned e0 = q0 * COUNT1 + v * 8;
    if (e0 + 8 <= elems1) *reinterpret_cast<uint4v *>(s1 + v * 8) = *reinterpret_cast<const uint4v *>(IN1 + e0);
    else
      for (unsigned e = 0; e < 8; ++e)
        if (e0 + e < elems1) s1[v * 8 + e] = IN1[e0 + e];
  }
  DNX_SYNC();
  // Output: one 4-byte word per lane and step, consecutive lanes on consecutive words.  The lanes of a wave then read
  // consecutive halves from LDS (no bank conflicts; a lane assembling a whole 16-byte vector reads at a 16-byte stride,
  // four lanes per bank) and a store instruction covers 256 contiguous bytes.
  const unsigned outElems = total * COUT;             // elements of the whole output
  const unsigned base = q0 * COUT;                    // first element of this workgroup's range (even: q0 is a multiple of 8)
  unsigned int *out32 = reinterpret_cast<unsigned int *>(OUT + base);
  // (pixel, channel) of a lane's word advance by a constant per step: no division inside the loop
  constexpr unsigned STEP = 2 * WG, STEP_PIX = STEP / COUT, STEP_CH = STEP % COUT;
  unsigned pix = (2 * tid) / COUT, ch = 2 * tid - pix * COUT;
  auto pick = [&](unsigned p, unsigned c) { return c < COUNT ? s0[p * COUNT + c] : s1[p * COUNT1 + (c - COUNT)]; };
  for (unsigned d = tid; d < PQ * COUT / 2; d += WG) {
    const unsigned e0 = 2 * d;
    if (base + e0 >= outElems) break;
    const ushort_t h0 = pick(pix, ch);
    const bool wrap = ch + 1 == COUT; // the word's second half is the next pixel's first channel
    const ushort_t h1 = pick(wrap ? pix + 1 : pix, wrap ? 0u : ch + 1);
    if (base + e0 + 2 <= outElems) out32[d] = (unsigned)h0 | ((unsigned)h1 << 16);
    else OUT[base + e0] = h0; // the tensor's last element when it has an odd number of them
    pix += STEP_PIX;
    ch += STEP_CH;
    if (ch >= COUT) {
      ch -= COUT;
      pix += 1;
    }
  }
}
#elif defined(COUNT1)
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
