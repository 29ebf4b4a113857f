// conv3x3_upfold.hip -- 3x3 convolution over concat(upsample2x(A), B) with the upsample folded into the weights.
//
// A 3x3 convolution over a 2x nearest-upsampled image reads, for the output pixel (2y+a, 2x+b), only the 2x2
// low-resolution neighbourhood rows {y+a-1, y+a} x columns {x+b-1, x+b}: the three taps of a row (column) fall on
// two source rows (columns), two of them on the same one.  Summing the weights of coinciding taps on the host gives,
// per parity class (a, b), a 2x2 convolution of the low-resolution source -- 4 taps instead of 9 for the upsampled
// channels, the same result up to one rounding of the summed weights to binary16.  The second source B (full
// resolution, the skip connection) keeps its 9 taps, read at every other pixel.
//
// One workgroup computes one class (a, b) for KT output channels: out[2y+a, 2x+b, :] for the low-resolution tile
// y in [yl0, yl0 + WAVES*RPW), x in [xl0, xl0 + 32).  Its folded weights (4 x KT x CAP for A, 9 x KT x CBP for B)
// stay in LDS (persistent launch, bands of tiles per XCD as in conv3x3_mfma_ws.hip).  Per tile there are two steps,
// each behind one barrier: all channels of the A halo ((TLH+1) x 33 low-resolution pixels), then all channels of the
// B halo ((2 TLH+1) x 65 full-resolution pixels, stored de-interleaved by column parity so that "every other
// pixel" is consecutive in LDS).  Loads for the next tile's halos are issued right after a halo is written to LDS.
//
// Compile-time interface: conv_common.h (CA, CB, KOUT, KT, ACT, HAS_BIAS, WAVES, RPW, PADB, SLOTS; UPA = 1, MF = 32,
// no POOL / CROP / PADA) plus the layout of the packed weights: [class][kt][A taps ty*2+tx][KT][CAP][B taps r*3+s][KT][CBP].
#include "conv_common.h"

#ifndef KERNEL_NAME
#define KERNEL_NAME conv3x3_upfold
#endif
static_assert(UPA == 1 && MF == 32 && !POOL && !CROP && !PADA && KR == 3 && KS == 3 && PY == 1 && PX == 1 && SY == 1 && SX == 1, "upsample-folded variant");
static_assert(CA % 8 == 0 && (CB == 0 || CB >= 8), "whole 8-channel vectors of A; at least one whole vector of B");

#define NKT (KOUTP / KT)
#ifndef NXCD
#define NXCD 8 // accelerator dies, each with an L2 of its own; the host sizes the grid with the same number
#endif
#define CAP ((CA + 15) / 16 * 16)
#define CBP ((CB + 15) / 16 * 16)
#define APITCH (CAP + 8)
#define BWP (CBP + 8) // pitch of the B weights
#ifndef BPITCH
#define BPITCH (CBP + 8) // pitch of a B halo pixel (CBP: no padding, where LDS is short)
#endif
#define TLH (WAVES * RPW)
#define AH (TLH + 1)
#define AW 33
#define BH (2 * TLH + 1)
#define BW 65
#define VA (CAP / 8)
#define VB (CBP / 8)
#define NVA ((AH * AW * VA + NT - 1) / NT)
#define NVB (CB > 0 ? (BH * BW * VB + NT - 1) / NT : 0)

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
  __shared__ __attribute__((aligned(16))) _Float16 sWA[4 * KT * APITCH];
  __shared__ __attribute__((aligned(16))) _Float16 sWB[CB > 0 ? 9 * KT * BWP : 8];
  __shared__ __attribute__((aligned(16))) _Float16 sA[AH * AW * APITCH];
  __shared__ __attribute__((aligned(16))) _Float16 sB[CB > 0 ? BH * BW * BPITCH : 8];
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
  const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16 *>(A), 0, (int)srcs.bytesA, 0x00020000);
  const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16 *>(CB > 0 ? B : A), 0, (int)(CB > 0 ? srcs.bytesB : 0u), 0x00020000);
  const int wv = tid >> 6;
  const int lane = tid & 63;
  const int l32 = lane & 31;
  const int kq = (lane >> 5) * 8;

  const int bidx = DNX_BID_X;
  const int xcd = bidx % NXCD;
  const int q = bidx / NXCD;
  const int cls = q % 4;         // parity class: a = row parity, b = column parity of the output pixels
  const int kt = (q / 4) % NKT;
  const int slot = q / (4 * NKT);
  const int ca = cls >> 1, cb = cls & 1;
  const int WL = (int)(pc.IN_W >> 1), HL = (int)(pc.IN_H >> 1);
  const int tilesX = (WL + 31) / 32, tilesY = (HL + TLH - 1) / TLH;
  const int numTiles = tilesX * tilesY;
  const int perXcd = (numTiles + NXCD - 1) / NXCD;
  const int first = xcd * perXcd;
  int last = first + perXcd;
  last = last < numTiles ? last : numTiles;
  int tile = first + slot;
  if (tile >= last)
    return; // uniform for the workgroup
  const bool rev = (pc.FLAGS & 1u) != 0;
  auto tileY = [&](int t) { return ((rev ? numTiles - 1 - t : t) / tilesX) * TLH; }; // low-resolution coordinates
  auto tileX = [&](int t) { return ((rev ? numTiles - 1 - t : t) % tilesX) * 32; };

  { // resident weights of this (class, kt)
    const _Float16 *w = FILT + (size_t)(cls * NKT + kt) * KT * (4 * CAP + 9 * CBP);
    for (int i = tid; i < 4 * KT * VA; i += NT) {
      const int row = i / VA, v = i - row * VA;
      *reinterpret_cast<uint4v *>(sWA + row * APITCH + v * 8) = ld16(w + (size_t)i * 8);
    }
#if CB > 0
    w += 4 * KT * CAP;
    for (int i = tid; i < 9 * KT * VB; i += NT) {
      const int row = i / VB, v = i - row * VB;
      *reinterpret_cast<uint4v *>(sWB + row * BWP + v * 8) = ld16(w + (size_t)i * 8);
    }
#endif
  }

  // What does not change from tile to tile is computed once per thread: where each of its halo vectors goes in LDS,
  // its row / column inside the halo and its byte offset relative to the halo's first pixel.
  uint4v ga[NVA];
  int aLds[NVA], aYX[NVA], aRel[NVA];
#pragma unroll
  for (int it = 0; it < NVA; ++it) {
    const int i = tid + it * NT;
    const int pix = i / VA, v = i - pix * VA;
    const int hy = pix / AW, hx = pix - hy * AW;
    // every vector of the CAP staged channels gets a slot: those past CA are stored as zeros (their weights are zero, but
    // what LDS held before is not, and 0 * NaN is NaN)
    aLds[it] = i < AH * AW * VA ? pix * APITCH + v * 8 : -1;
    aYX[it] = (hy << 16) | hx;
    aRel[it] = ((hy * WL + hx) * CA + v * 8) * 2;
  }
  // loads of the A halo of low-resolution tile (yl0, xl0): rows yl0 + ca - 1 .., columns xl0 + cb - 1 ..
  auto issueA = [&](int t) {
    const bool live = t < last;
    const int yb = tileY(live ? t : tile) + ca - 1, xb = tileX(live ? t : tile) + cb - 1;
    const int base = (yb * WL + xb) * CA * 2;
#pragma unroll
    for (int it = 0; it < NVA; ++it) {
      const int yl = yb + (aYX[it] >> 16), xl = xb + (aYX[it] & 0xFFFF);
      const bool ok = live && aLds[it] >= 0 && aLds[it] % APITCH < CA && yl >= 0 && yl < HL && xl >= 0 && xl < WL;
      ga[it] = __builtin_amdgcn_raw_buffer_load_b128(ra, ok ? (unsigned)(base + aRel[it]) : NO_LOAD, 0, LOAD_AUX);
    }
  };
  auto commitA = [&]() {
#pragma unroll
    for (int it = 0; it < NVA; ++it)
      if (aLds[it] >= 0)
        *reinterpret_cast<uint4v *>(sA + aLds[it]) = ga[it];
  };
#if CB > 0
  uint4v gb[NVB];
  int bLds[NVB], bYX[NVB], bRel[NVB];
#pragma unroll
  for (int it = 0; it < NVB; ++it) {
    const int i = tid + it * NT;
    const int pix = i / VB, v = i - pix * VB;
    const int hy = pix / BW, hx = pix - hy * BW;
    const int cc = v * 8;
    const int chan = (CB % 8 == 0 || cc + 8 <= CB) ? cc : CB - 8; // the partial last vector ends at the last channel
    // columns de-interleaved by parity: even columns first (33 of them), then the odd ones
    bLds[it] = i < BH * BW * VB ? (hy * BW + (hx & 1) * 33 + (hx >> 1)) * BPITCH + cc : -1; // vectors past CB: stored as zeros
    bYX[it] = (hy << 16) | hx;
#if PADB
    bRel[it] = chan * 2;
#else
    bRel[it] = ((hy * (int)pc.IN_W + hx) * CB + chan) * 2;
#endif
  }
  // loads of the B halo: full-resolution rows 2 yl0 + ca - 1 .., columns 2 xl0 + cb - 1 ..
  auto issueB = [&](int t) {
    const bool live = t < last;
    const int yb = 2 * tileY(live ? t : tile) + ca - 1, xb = 2 * tileX(live ? t : tile) + cb - 1;
#if !PADB
    const int base = (yb * (int)pc.IN_W + xb) * CB * 2;
#endif
#pragma unroll
    for (int it = 0; it < NVB; ++it) {
      const int gy = yb + (bYX[it] >> 16), gx = xb + (bYX[it] & 0xFFFF);
      const bool ok = live && bLds[it] >= 0 && bLds[it] % BPITCH < CB && gy >= 0 && gy < (int)pc.IN_H && gx >= 0 && gx < (int)pc.IN_W;
#if PADB
      const int sy = clampi(gy - (int)pc.PAD_T, 0, (int)pc.SRC_H - 1), sx = clampi(gx - (int)pc.PAD_L, 0, (int)pc.SRC_W - 1);
      const unsigned off = (unsigned)((sy * (int)pc.SRC_W + sx) * CB * 2 + bRel[it]);
#else
      const unsigned off = (unsigned)(base + bRel[it]);
#endif
      gb[it] = __builtin_amdgcn_raw_buffer_load_b128(rb, ok ? off : NO_LOAD, 0, LOAD_AUX);
    }
  };
  auto commitB = [&]() {
#pragma unroll
    for (int it = 0; it < NVB; ++it)
      if (bLds[it] >= 0) {
        uint4v val = gb[it];
        if (CB % 8 != 0) {
          const uint4v sh = shr_halves<(8 - CB % 8) % 8>(val);
          const bool part = (bLds[it] % BPITCH) + 8 > CB; // the vector's first channel is its LDS offset inside the pixel
#pragma unroll
          for (int e = 0; e < 4; ++e) val[e] = part ? sh[e] : val[e];
        }
        *reinterpret_cast<uint4v *>(sB + bLds[it]) = val;
      }
  };
#endif

  Acc acc;
  Packed done;
  int dtile = 0;
  bool pend = false;
  issueA(tile);
#if CB > 0
  __builtin_amdgcn_sched_barrier(0);
  issueB(tile);
#endif
  stage_bias(sBias, BIAS, kt, tid); // (behind the first halos' loads, so that it does not cost a memory round trip of its own)
  for (; tile < last; tile += SLOTS) {
    // ---- step A: the folded 2x2 taps over the low-resolution source
    commitA();
    DNX_SYNC();
    init_acc(acc, sBias, lane);
    if (pend) { // the previous tile's stores, in front of this step's loads
      store_packed(done, out, 2 * tileY(dtile) + ca, 2 * tileX(dtile) + cb, kt, wv, lane, pc, 0, 1, 2, 2);
      pend = false;
    }
    issueA(tile + SLOTS);
#pragma unroll
    for (int ks = 0; ks < CAP / 16; ++ks) {
      const int kk = ks * 16 + kq;
#pragma unroll
      for (int tx = 0; tx < 2; ++tx) {
        half8 px[RPW + 1];
#pragma unroll
        for (int t = 0; t < RPW + 1; ++t)
          px[t] = *reinterpret_cast<const half8 *>(sA + ((wv * RPW + t) * AW + l32 + tx) * APITCH + kk);
#pragma unroll
        for (int ty = 0; ty < 2; ++ty) {
          half8 wf[KB];
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
            wf[kb] = *reinterpret_cast<const half8 *>(sWA + ((ty * 2 + tx) * KT + kb * 32 + l32) * APITCH + kk);
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int j = 0; j < RPW; ++j)
              acc.v[kb][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[kb], px[j + ty], acc.v[kb][j], 0, 0, 0);
        }
      }
    }
#if CB > 0
    // ---- step B: the 9 taps over the full-resolution source, at every other pixel
    commitB();
    DNX_SYNC();
    issueB(tile + SLOTS);
#pragma unroll
    for (int ks = 0; ks < CBP / 16; ++ks) {
      const int kk = ks * 16 + kq;
#pragma unroll
      for (int s = 0; s < 3; ++s) {
        half8 px[2 * RPW + 1];
#pragma unroll
        for (int t = 0; t < 2 * RPW + 1; ++t)
          px[t] = *reinterpret_cast<const half8 *>(sB + ((2 * wv * RPW + t) * BW + (s & 1) * 33 + l32 + (s >> 1)) * BPITCH + kk);
#pragma unroll
        for (int r = 0; r < 3; ++r) {
          half8 wf[KB];
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
            wf[kb] = *reinterpret_cast<const half8 *>(sWB + ((r * 3 + s) * KT + kb * 32 + l32) * BWP + kk);
#pragma unroll
          for (int kb = 0; kb < KB; ++kb)
#pragma unroll
            for (int j = 0; j < RPW; ++j)
              acc.v[kb][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[kb], px[2 * j + r], acc.v[kb][j], 0, 0, 0);
        }
      }
    }
#endif
    pack_tile(acc, done);
    dtile = tile;
    pend = true;
  }
  if (pend)
    store_packed(done, out, 2 * tileY(dtile) + ca, 2 * tileX(dtile) + cb, kt, wv, lane, pc, 0, 1, 2, 2);
}
