// pad.hip -- replicate ("edge") padding, HWC binary16.
// Replaces compiler/src/denox/compiler/implement/shaders/pad/memory_pad.comp:31-133:
//   out[ho, wo, c] = in[clamp(ho - PAD_T, 0, IN_H-1), clamp(wo - PAD_L, 0, IN_W-1), c].
// Definitions: CH, VEC.  grid.y = output rows.
#include "common.h"
#ifndef KERNEL_NAME
#define KERNEL_NAME memory_pad
#endif
struct PushConstants { unsigned int OUT_W, OUT_H, PAD_L, PAD_R, PAD_T, PAD_B; };
extern "C" __global__ DNX_LAUNCH_BOUNDS(WG) void KERNEL_NAME(
    const ushort_t *__restrict__ IN, ushort_t *__restrict__ OUT, PushConstants pc) {
  constexpr unsigned CV = CH / VEC;
  const int ho = (int)DNX_BID_Y;
  const unsigned i = DNX_ROW_INDEX();
  if (i >= pc.OUT_W * CV) return;
  const unsigned wo = i / CV, cv = i - wo * CV;
  const int IN_W = (int)(pc.OUT_W - pc.PAD_L - pc.PAD_R);
  const int IN_H = (int)(pc.OUT_H - pc.PAD_T - pc.PAD_B);
  int hi = ho - (int)pc.PAD_T; hi = hi < 0 ? 0 : (hi > IN_H - 1 ? IN_H - 1 : hi);
  int wi = (int)wo - (int)pc.PAD_L; wi = wi < 0 ? 0 : (wi > IN_W - 1 ? IN_W - 1 : wi);
  stv(OUT + ((size_t)ho * pc.OUT_W + wo) * OPITCH + cv * VEC, ldv(IN + ((size_t)hi * IN_W + wi) * CH + cv * VEC));
}
