// pad.hip -- replicate ("edge") or zero padding, HWC binary16.
// Replaces compiler/src/denox/compiler/implement/shaders/pad/memory_pad.comp:31-133:
//   out[ho, wo, c] = in[clamp(ho - PAD_T, 0, IN_H-1), clamp(wo - PAD_L, 0, IN_W-1), c];
// with ZERO = 1 the border is 0 instead (PaddingMode::Zero of the reference's model, which its shader does not implement).
// Definitions: CH, VEC, ZERO; FLAT: without left / right padding rows are moved as runs of halves (common.h).  grid.y = output rows.
#include "common.h"
#ifndef ZERO
#define ZERO 0
#endif
#ifndef KERNEL_NAME
#define KERNEL_NAME memory_pad
#endif
struct PushConstants { unsigned int OUT_W, OUT_H, PAD_L, PAD_R, PAD_T, PAD_B; };
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = DNX_CHUNKS(CH);
  const int ho = (int)DNX_BID_Y;
  const unsigned i = DNX_ROW_INDEX();
  const int IN_W = (int)(pc.OUT_W - pc.PAD_L - pc.PAD_R);
  const int IN_H = (int)(pc.OUT_H - pc.PAD_T - pc.PAD_B);
#ifdef FLAT
  if ((pc.PAD_L | pc.PAD_R) == 0u) { // rows are only added above and below: every output row is a whole source row (uniform branch)
    const int hr = ho - (int)pc.PAD_T;
    const int hc = hr < 0 ? 0 : (hr > IN_H - 1 ? IN_H - 1 : hr);
    const bool blank = ZERO && hr != hc;
    flat_row(IN + (size_t)hc * IN_W * CH, OUT + (size_t)ho * pc.OUT_W * CH, pc.OUT_W * CH, i, [blank](vec_t v) { const vec_t z = {}; return blank ? z : v; });
    return;
  }
#endif
  if (i >= pc.OUT_W * CV) return;
  const unsigned wo = i / CV, cv = i - wo * CV;
  int hi = ho - (int)pc.PAD_T, wi = (int)wo - (int)pc.PAD_L;
#if ZERO
  const bool inside = hi >= 0 && hi < IN_H && wi >= 0 && wi < IN_W;
#endif
  hi = hi < 0 ? 0 : (hi > IN_H - 1 ? IN_H - 1 : hi);
  wi = wi < 0 ? 0 : (wi > IN_W - 1 ? IN_W - 1 : wi);
  chunk_t v = ld_chunk<CH>(IN + ((size_t)hi * IN_W + wi) * CH, cv); // the clamped read is in range in both modes
#if ZERO
  const chunk_t zero = {};
  v = inside ? v : zero;
#endif
  st_chunk<CH>(OUT + ((size_t)ho * pc.OUT_W + wo) * OPITCH, cv, v);
}
