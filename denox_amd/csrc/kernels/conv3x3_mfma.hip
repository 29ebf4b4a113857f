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

#define NV_IN ((HALO_PIX * (CK / 8) + NT - 1) / NT)
#define NV_W ((9 * KT * (CK / 8) + NT - 1) / NT)

struct Staged {
  uint4v in[NV_IN];
  uint4v w[NV_W];
};

template <int L>
__device__ DNX_INLINE void
fetch_chunk(const _Float16 *__restrict__ A, const _Float16 *__restrict__ B, const _Float16 *__restrict__ wchunk,
            Staged &st, int c0, int y0, int x0, const PushConstants &pc, int tid) {
  constexpr int VPP = L / 8;
#pragma unroll
  for (int it = 0; it < NV_IN; ++it) {
    const int i = tid + it * NT;
    uint4v val = {0u, 0u, 0u, 0u};
    if (i < HALO_PIX * VPP)
      val = load_halo_vec<L>(A, B, i, c0, y0, x0, pc);
    st.in[it] = val;
  }
  // weight slice for these channels: global [tap][KT rows][L]
#pragma unroll
  for (int it = 0; it < NV_W; ++it) {
    const int i = tid + it * NT;
    if (i < 9 * KT * VPP)
      st.w[it] = ld16(wchunk + (size_t)i * 8);
  }
}

template <int L>
__device__ DNX_INLINE void commit_chunk(const Staged &st, _Float16 *sIn, _Float16 *sW, int tid) {
  constexpr int VPP = L / 8;
#pragma unroll
  for (int it = 0; it < NV_IN; ++it) {
    const int i = tid + it * NT;
    if (i < HALO_PIX * VPP) {
      const int pix = i / VPP;
      const int v = i - pix * VPP;
      *reinterpret_cast<uint4v *>(sIn + pix * CKP + v * 8) = st.in[it];
    }
  }
#pragma unroll
  for (int it = 0; it < NV_W; ++it) {
    const int i = tid + it * NT;
    if (i < 9 * KT * VPP) {
      const int row = i / VPP;
      const int v = i - row * VPP;
      *reinterpret_cast<uint4v *>(sW + row * CKP + v * 8) = st.w[it];
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
  __shared__ __attribute__((aligned(16))) _Float16 sIn[HALO_PIX * CKP];
  __shared__ __attribute__((aligned(16))) _Float16 sW[9 * KT * CKP];
#if CB == 0
  const _Float16 *B = nullptr;
#endif
#if !HAS_BIAS
  const _Float16 *BIAS = nullptr;
#endif
  const int tid = DNX_TID;
  const int wv = tid >> 6;
  const int lane = tid & 63;
  const int x0 = DNX_BID_X * TW;
  const int y0 = DNX_BID_Y * TH;
  const int kt = DNX_BID_Z; // output-channel tile

  float16v acc[KB][RPW];
#pragma unroll
  for (int kb = 0; kb < KB; ++kb)
#pragma unroll
    for (int j = 0; j < RPW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        acc[kb][j][i] = 0.0f;

  // packed filter: [kt][chunk][tap][KT][len(chunk)]
  const _Float16 *wbase = FILT + (size_t)kt * 9 * KT * CPAD;
  Staged st;
  if (NCHUNK > 1 || TAIL == CK)
    fetch_chunk<CK>(A, B, wbase, st, 0, y0, x0, pc, tid);
  else
    fetch_chunk<TAIL>(A, B, wbase, st, 0, y0, x0, pc, tid);
  for (int chunk = 0; chunk < NCHUNK; ++chunk) {
    const bool fullNow = (TAIL == CK) || (chunk < NCHUNK - 1);
    if (fullNow)
      commit_chunk<CK>(st, sIn, sW, tid);
    else
      commit_chunk<TAIL>(st, sIn, sW, tid);
    DNX_SYNC();
    if (chunk + 1 < NCHUNK) { // loads for the next chunk fly during the MFMAs below
      const int c1 = (chunk + 1) * CK;
      const _Float16 *wnext = wbase + (size_t)9 * KT * c1;
      if (TAIL == CK || chunk + 1 < NCHUNK - 1)
        fetch_chunk<CK>(A, B, wnext, st, c1, y0, x0, pc, tid);
      else
        fetch_chunk<TAIL>(A, B, wnext, st, c1, y0, x0, pc, tid);
    }
    if (fullNow)
      mma_chunk<CK, CKP>(sIn, sW, 0, acc, wv, lane);
    else
      mma_chunk<TAIL, CKP>(sIn, sW, 0, acc, wv, lane);
    DNX_SYNC();
  }
  store_tile(acc, OUT, BIAS, y0, x0, kt, wv, lane, pc);
}
