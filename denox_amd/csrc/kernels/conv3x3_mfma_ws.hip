// conv3x3_mfma_ws.hip -- weight-stationary variant of the fused 3x3 convolution
// (same operation and compile-time interface as conv3x3_mfma.hip, see conv_common.h).
//
// The launch is persistent: GRID workgroups, one per compute unit, each keeps the whole
// 9 x KT x CPAD weight slice of its output-channel tile in LDS for its lifetime and walks
// over many (WAVES*RPW) x 32 pixel tiles.  Only input halos stream: CK channels at a time
// through two LDS buffers, the loads of step i+1 issued into registers before the matrix
// work of step i, one barrier per step.  Compared with streaming the weights per tile this
// removes most L2 reads, most LDS writes and most address arithmetic of the inner loop.
//
// Workgroup b serves XCD b % 8 (workgroups are dealt round-robin to the 8 XCDs), and each
// XCD walks its own contiguous band of tiles so that neighbouring halos meet in one L2.
//   SLOTS   workgroups per (XCD, output-channel tile); GRID = 8 * NKT * SLOTS
#include "conv_common.h"

#ifndef KERNEL_NAME
#define KERNEL_NAME conv3x3_mfma_ws
#endif

#define NKT (KOUTP / KT)
#define CPADP (CPAD + 8)
#define NV_IN ((HALO_PIX * (CK / 8) + NT - 1) / NT)
#define NXCD 8

template <int L>
__device__ DNX_INLINE void
fetch_halo(const _Float16 *__restrict__ A, const _Float16 *__restrict__ B, uint4v (&st)[NV_IN], int c0, int y0, int x0,
           const PushConstants &pc, int tid) {
  constexpr int VPP = L / 8;
#pragma unroll
  for (int it = 0; it < NV_IN; ++it) {
    const int i = tid + it * NT;
    uint4v val = {0u, 0u, 0u, 0u};
    if (i < HALO_PIX * VPP)
      val = load_halo_vec<L>(A, B, i, c0, y0, x0, pc);
    st[it] = val;
  }
}

template <int L>
__device__ DNX_INLINE void commit_halo(const uint4v (&st)[NV_IN], _Float16 *sIn, int tid) {
  constexpr int VPP = L / 8;
#pragma unroll
  for (int it = 0; it < NV_IN; ++it) {
    const int i = tid + it * NT;
    if (i < HALO_PIX * VPP) {
      const int pix = i / VPP;
      const int v = i - pix * VPP;
      *reinterpret_cast<uint4v *>(sIn + pix * CKP + v * 8) = st[it];
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
  __shared__ __attribute__((aligned(16))) _Float16 sW[9 * KT * CPADP];
  __shared__ __attribute__((aligned(16))) _Float16 sIn[2][HALO_PIX * CKP];
#if CB == 0
  const _Float16 *B = nullptr;
#endif
#if !HAS_BIAS
  const _Float16 *BIAS = nullptr;
#endif
  const int tid = DNX_TID;
  const int wv = tid >> 6;
  const int lane = tid & 63;

  const int b = DNX_BID_X;
  const int xcd = b % NXCD;
  const int q = b / NXCD;
  const int kt = q % NKT;
  const int slot = q / NKT;
  const int tilesX = (pc.IN_W + TW - 1) / TW;
  const int tilesY = (pc.IN_H + TH - 1) / TH;
  const int numTiles = tilesX * tilesY;
  const int perXcd = (numTiles + NXCD - 1) / NXCD;
  const int first = xcd * perXcd;
  int last = first + perXcd;
  last = last < numTiles ? last : numTiles;
  int tile = first + slot;
  if (tile >= last)
    return; // uniform for the workgroup: nothing was staged yet

  // ---- resident weights: global [tap][KT][CPAD] (one chunk = whole reduction) -> LDS rows of CPADP ----
  {
    const _Float16 *wsrc = FILT + (size_t)kt * 9 * KT * CPAD;
    constexpr int VPR = CPAD / 8;
    for (int i = tid; i < 9 * KT * VPR; i += NT) {
      const int row = i / VPR;
      const int v = i - row * VPR;
      *reinterpret_cast<uint4v *>(sW + row * CPADP + v * 8) = ld16(wsrc + (size_t)i * 8);
    }
  }

  uint4v st[NV_IN];
  int ty = tile / tilesX, tx = tile - ty * tilesX;
  if (NCHUNK > 1 || TAIL == CK)
    fetch_halo<CK>(A, B, st, 0, ty * TH, tx * TW, pc, tid);
  else
    fetch_halo<TAIL>(A, B, st, 0, ty * TH, tx * TW, pc, tid);
  int buf = 0;
  while (true) {
    const int y0 = ty * TH, x0 = tx * TW;
    const int ntile = tile + SLOTS;
    const bool more = ntile < last;
    const int nty = ntile / tilesX, ntx = ntile - nty * tilesX;

    float16v acc[KB][RPW];
#pragma unroll
    for (int kb = 0; kb < KB; ++kb)
#pragma unroll
      for (int j = 0; j < RPW; ++j)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          acc[kb][j][i] = 0.0f;

    for (int chunk = 0; chunk < NCHUNK; ++chunk) {
      const bool fullNow = (TAIL == CK) || (chunk < NCHUNK - 1);
      if (fullNow)
        commit_halo<CK>(st, sIn[buf], tid);
      else
        commit_halo<TAIL>(st, sIn[buf], tid);
      // One barrier per step: buffer `buf` was last read two steps ago, and every wave
      // has passed the barrier of the step in between since then.
      DNX_SYNC();
      if (chunk + 1 < NCHUNK) {
        const int c1 = (chunk + 1) * CK;
        if (TAIL == CK || chunk + 1 < NCHUNK - 1)
          fetch_halo<CK>(A, B, st, c1, y0, x0, pc, tid);
        else
          fetch_halo<TAIL>(A, B, st, c1, y0, x0, pc, tid);
      } else if (more) {
        if (NCHUNK > 1 || TAIL == CK)
          fetch_halo<CK>(A, B, st, 0, nty * TH, ntx * TW, pc, tid);
        else
          fetch_halo<TAIL>(A, B, st, 0, nty * TH, ntx * TW, pc, tid);
      }
      if (fullNow)
        mma_chunk<CK, CPADP>(sIn[buf], sW, chunk * CK, acc, wv, lane);
      else
        mma_chunk<TAIL, CPADP>(sIn[buf], sW, chunk * CK, acc, wv, lane);
      buf ^= 1;
    }
    store_tile(acc, OUT, BIAS, y0, x0, kt, wv, lane, pc);
    if (!more)
      break;
    tile = ntile;
    ty = nty;
    tx = ntx;
  }
}
