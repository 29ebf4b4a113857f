// conv3x3_mfma.hip -- fused 3x3 convolution (stride 1, zero padding 1) as an fp16
// implicit GEMM on CDNA4 matrix cores, fp32 accumulation; weights streamed.
//
// Replaces the reference's three conv shaders
//   compiler/src/denox/compiler/implement/shaders/conv/direct_conv.comp:82-775
//   compiler/src/denox/compiler/implement/shaders/conv/direct_conv_cm.comp:119-1568
//   compiler/src/denox/compiler/implement/shaders/conv/concat_conv_cm.comp:1043-1128
// and, through compile-time switches (see conv_common.h), also absorbs a 2x nearest
// upsample, a channel concat, a replicate pad of a source, a 2x2 max pool or a crop
// of the result.
//
// One workgroup computes one (WAVES*RPW) x 32 pixel tile for KT output channels.
// Per step of CK input channels LDS holds the (TH+2) x 34 pixel halo and the
// 9 x KT x CK weight slice; rows are padded by 8 halves so that consecutive pixels /
// weight rows start in different 16-byte bank groups.  The loads of step i+1 are
// issued into registers before the matrix work of step i and written to LDS after it.
// Grid: x = ceil(W/32), y = ceil(H/TH), z = KOUTP/KT.
#include "conv_common.h"

#ifndef KERNEL_NAME
#define KERNEL_NAME conv3x3_mfma
#endif

#define NV_W ((NTAPS * KT * VPPK + NT - 1) / NT)

// weight slice of one step: global [tap][KT rows][L] -> registers -> LDS rows of CKP
template <int L>
__device__ DNX_INLINE void weights_fetch(const _Float16 *__restrict__ wchunk, uint4v (&st)[NV_W], int tid) {
  constexpr int VPP = L / 8;
#pragma unroll
  for (int it = 0; it < NV_W; ++it) {
    const int i = tid + it * NT;
    if (i < NTAPS * KT * VPP)
      st[it] = ld16(wchunk + (size_t)i * 8);
  }
}

template <int L>
__device__ DNX_INLINE void weights_commit(const uint4v (&st)[NV_W], _Float16 *sW, int tid) {
  constexpr int VPP = L / 8;
#pragma unroll
  for (int it = 0; it < NV_W; ++it) {
    const int i = tid + it * NT;
    if (i < NTAPS * KT * VPP) {
      const int row = i / VPP;
      const int v = i - row * VPP;
      *reinterpret_cast<uint4v *>(sW + row * CKP + v * 8) = st[it];
    }
  }
}

extern "C" __global__ DNX_LAUNCH_BOUNDS(NT) void KERNEL_NAME(
    const _Float16 *__restrict__ A,
#if CB > 0
    const _Float16 *__restrict__ B,
#endif
    _Float16 *__restrict__ OUT, const _Float16 *__restrict__ FILT,
#if HAS_BIAS
    const _Float16 *__restrict__ BIAS,
#endif
    PushConstants pc) {
  __shared__ __attribute__((aligned(16))) _Float16 sIn[HALO_ELEMS];
  __shared__ __attribute__((aligned(16))) _Float16 sW[NTAPS * KT * CKP];
  __shared__ __attribute__((aligned(16))) bias_t sBias[KT];
#if CB == 0
  const _Float16 *B = nullptr;
#endif
#if !HAS_BIAS
  const _Float16 *BIAS = nullptr;
#endif
  const int tid = DNX_TID;
  const OutBuf out = out_buffer(OUT, pc);
  const Sources srcs = make_sources(A, B, pc);
  const int wv = tid >> 6;
  const int lane = tid & 63;
  const bool rev = (pc.FLAGS & 1u) != 0;
  const int tilesX = (CONV_OUT_W(pc) + TW - 1) / TW, tilesY = (CONV_OUT_H(pc) + TH - 1) / TH;
  const int x0 = (rev ? tilesX - 1 - (int)DNX_BID_X : (int)DNX_BID_X) * TW;
  const int y0 = (rev ? tilesY - 1 - (int)DNX_BID_Y : (int)DNX_BID_Y) * TH;
  const int kt = DNX_BID_Z; // output-channel tile

  Acc acc;

  // packed filter: [kt][chunk][tap][KT][len(chunk)]
  const _Float16 *wbase = FILT + (size_t)kt * NTAPS * KT * CPAD;
  typedef Halo<NT> H;
  H::Map map;
  H::Src src;
  H::map_init(map, tid);
  H::src_init(src, map, y0, x0, pc);
  H::Regs stIn;
  uint4v stW[NV_W];
  H::fetch_step(srcs, stIn, map, src, 0);
  if (NCHUNK > 1 || TAIL == CK)
    weights_fetch<CK>(wbase, stW, tid);
  else
    weights_fetch<TAIL>(wbase, stW, tid);
  // The bias travels with the first step's loads and goes to LDS behind that step's halo and weights (loaded and staged in front
  // of them, it cost the kernel a memory round trip of its own).
#if HAS_BIAS
  constexpr int NBV = (KT + NT - 1) / NT;
  _Float16 biasv[NBV];
#pragma unroll
  for (int k = 0; k < NBV; ++k)
    biasv[k] = BIAS[kt * KT + (tid + k * NT < KT ? tid + k * NT : 0)];
#endif
  for (int chunk = 0; chunk < NCHUNK; ++chunk) {
    const bool fullNow = (TAIL == CK) || (chunk < NCHUNK - 1);
    H::commit_step(stIn, sIn, map, chunk);
    if (fullNow)
      weights_commit<CK>(stW, sW, tid);
    else
      weights_commit<TAIL>(stW, sW, tid);
#if HAS_BIAS
    if (chunk == 0) {
#pragma unroll
      for (int k = 0; k < NBV; ++k)
        if (tid + k * NT < KT)
          sBias[tid + k * NT] = (float)biasv[k];
    }
#endif
    DNX_SYNC();
    if (chunk == 0)
      init_acc(acc, sBias, lane); // the staged bias is visible from here on
    if (chunk + 1 < NCHUNK) { // loads for the next step fly during the MFMAs below
      const _Float16 *wnext = wbase + (size_t)NTAPS * KT * (chunk + 1) * CK;
      H::fetch_step(srcs, stIn, map, src, chunk + 1);
      if (TAIL == CK || chunk + 1 < NCHUNK - 1)
        weights_fetch<CK>(wnext, stW, tid);
      else
        weights_fetch<TAIL>(wnext, stW, tid);
    }
    mma_step<CKP>(sIn, sW, 0, acc, wv, lane, chunk);
    DNX_SYNC();
  }
  store_tile(acc, out, y0, x0, kt, wv, lane, pc);
}
