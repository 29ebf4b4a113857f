// conv3x3_upfold_ws.hip -- 3x3 convolution over concat(upsample2x(A), B) with the upsample folded into the weights
// (conv3x3_upfold.hip: 4 taps instead of 9 for the upsampled channels), with wave specialisation and whole output rows.
//
// One workgroup computes one ROW parity a of the output for KT output channels: the rows 2y + a, all columns, of the
// low-resolution tile y in [yl0, yl0 + TLH), x in [xl0, xl0 + 32) -- 64 consecutive output pixels per row, as two
// matrix blocks (even and odd columns, parity classes (a, 0) and (a, 1)).  The folded weights of both classes and the
// 9-tap weights of B (the same for every class) stay in LDS for the workgroup's lifetime (persistent launch, bands of
// tiles per XCD as in conv3x3_mfma_ws.hip).  Both classes share the halos: A, (TLH+1) x 34 low-resolution pixels, and
// B, (2 TLH+1) x 66 full-resolution pixels, de-interleaved by column parity so that "every other pixel" is consecutive.
//
// WAVES waves only compute (LDS reads, MFMA, conversion), PW further waves do everything that touches memory.  A tile
// takes NA + 1 steps, one barrier each: NA steps of CKA channels of A and one step with all channels of B.  Every kind
// of step has an LDS buffer of its own and a register set of its own in the staging waves: while the computing waves
// multiply step k, the staging waves write the halo of step k + 1 (loaded a whole tile earlier) into the buffer that was
// last read NA steps ago, and at once issue the loads of the same step of the next tile.  The finished tile goes to
// memory through LDS as well: the computing waves leave it there as binary16 and the staging waves store it during the
// next tile's first step -- whole output rows, 1 KiB of consecutive addresses per store instruction, instead of 16
// bytes per lane at a stride of two pixels.  The 9-tap weights of B (at most 32 channels) live in registers of the
// computing waves, which is what makes room for that tile in LDS.
//
// KSP = 2 divides the work of a tile among the computing waves by output channels as well as by rows: wave w takes the 32
// channels w % 2 of the 64 and the RPW rows of row group w / 2 (KSP = 1: all channels, RPW rows of group w).  A weight
// fragment read from LDS then feeds RPW = 2 matrix instructions instead of one, a pixel fragment as many as before:
// 17 instead of 22 LDS reads per 16 matrix instructions in the steps over A, whose pace the LDS read rate sets.
//
// Compile-time interface: as conv3x3_upfold.hip, plus PW (staging waves) and CKA (channels of A per step, divides CAP);
// 8 <= CB <= 32 (its 9-tap weights must fit the registers); KT = 32 or 64 and KOUT a multiple of KT; the result 16-byte aligned (OVEC).  Packed weights as there:
// [class a*2+b][kt][A taps ty*2+tx][KT][CAP][B taps r*3+s][KT][CBP].
#include "conv_common.h"

#ifndef KERNEL_NAME
#define KERNEL_NAME conv3x3_upfold_ws
#endif
static_assert(UPA == 1 && MF == 32 && !POOL && !CROP && !PADA && KR == 3 && KS == 3 && PY == 1 && PX == 1 && SY == 1 && SX == 1, "upsample-folded variant");
static_assert(CA % 8 == 0 && CB >= 8 && PW > 0, "whole 8-channel vectors of A; a second source with at least one whole vector; staging waves");

#define NKT (KOUTP / KT)
#ifndef NXCD
#define NXCD 8 // accelerator dies, each with an L2 of its own; the host sizes the grid with the same number
#endif
#define CAP ((CA + 15) / 16 * 16)
#define CBP ((CB + 15) / 16 * 16)
#ifndef CKA
#define CKA CAP
#endif
static_assert(CAP % CKA == 0 && CKA % 16 == 0, "whole steps");
#ifndef KSP
#define KSP 1
#endif
#define KBW (KB / KSP) // 32-channel blocks of the result per computing wave
static_assert(KB % KSP == 0 && WAVES % KSP == 0, "whole blocks and whole row groups per wave");
static_assert(9 * (CBP / 16) * KBW * 4 <= 96, "the weights of B are kept in registers: 9 taps x channel steps x output blocks fragments");
static_assert((KT == 32 || KT == 64) && KOUT % KT == 0 && OVEC && OPITCH % 8 == 0 && !LAYOUT_OUT && !LAYIN, "whole 16-byte slots of a pixel-major result");
#define NA (CAP / CKA)
#define WAP (CAP + 8)    // pitch of the A weights
#define APITCH (CKA + 8) // pitch of a staged A pixel
#define BWP (CBP + 8)    // pitch of the B weights
#ifndef BPITCH
#define BPITCH (CBP + 8) // pitch of a B halo pixel (CBP: no padding, where LDS is short)
#endif
#define TLH (WAVES / KSP * RPW)
#define AH (TLH + 1)
#define AW 34
#define BH (2 * TLH + 1)
#define BW 66
#define VA (CKA / 8)
#define VB (CBP / 8)
#define NSTG (PW * 64)
#define NVA ((AH * AW * VA + NSTG - 1) / NSTG)
#define NVB ((BH * BW * VB + NSTG - 1) / NSTG)
#define SPP (KT / 8)                                   // 16-byte slots of one output pixel
#define NVO ((TLH * 64 * SPP + NSTG - 1) / NSTG)       // slots of the finished tile per staging thread
// The finished tile in LDS, in 16-byte slots: [row][pixel pair][2 * SPP slots], the slot index inside a pair XOR-ed with
// the pair's index.  A computing lane holds pixels 2 l + b: the 16 lanes of one LDS pass write 16 different pairs, and
// the XOR spreads them over all banks; 16 consecutive staging lanes read the 16 slots of one pair, a permutation of them.
#define OUT_SLOT(row, pix, slot) ((((row) * 32 + ((pix) >> 1)) * (2 * SPP)) + (((((pix) & 1) * SPP) + (slot)) ^ (((pix) >> 1) & (2 * SPP - 1))))

extern "C" __global__ DNX_LAUNCH_BOUNDS(NT) void KERNEL_NAME(
    const _Float16 *__restrict__ A, const _Float16 *__restrict__ B, _Float16 *__restrict__ OUT, const _Float16 *__restrict__ FILT,
#if HAS_BIAS
    const _Float16 *__restrict__ BIAS,
#endif
    PushConstants pc) {
  __shared__ __attribute__((aligned(16))) _Float16 sWA[2][4 * KT * WAP]; // column parity b = 0, 1
  __shared__ __attribute__((aligned(16))) _Float16 sA[NA][AH * AW * APITCH + 8]; // + a slot for the vectors of threads with nothing to stage
  __shared__ __attribute__((aligned(16))) _Float16 sB[BH * BW * BPITCH + 8];
  __shared__ uint4v sOut[TLH * 64 * SPP];
  __shared__ __attribute__((aligned(16))) bias_t sBias[KT];
#if !HAS_BIAS
  const _Float16 *BIAS = nullptr;
#endif
  const int tid = DNX_TID;
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6); // wave-uniform: roles branch on it
  const int lane = tid & 63;

  const int bidx = DNX_BID_X;
  const int xcd = bidx % NXCD;
  const int q = bidx / NXCD;
  const int ca = q % 2; // row parity of this workgroup's output rows
  const int kt = (q / 2) % NKT;
  const int slot = q / (2 * NKT);
  const int WL = (int)(pc.IN_W >> 1), HL = (int)(pc.IN_H >> 1);
  const int tilesX = (WL + 31) / 32, tilesY = (HL + TLH - 1) / TLH;
  const int numTiles = tilesX * tilesY;
  const int perXcd = (numTiles + NXCD - 1) / NXCD;
  const int first = xcd * perXcd;
  int last = first + perXcd;
  last = last < numTiles ? last : numTiles;
  const int tile0 = first + slot;
  if (tile0 >= last)
    return; // uniform for the workgroup
  const int myTiles = (last - tile0 + SLOTS - 1) / SLOTS;
  const bool rev = (pc.FLAGS & 1u) != 0;
  auto tileY = [&](int t) { return ((rev ? numTiles - 1 - t : t) / tilesX) * TLH; }; // low-resolution coordinates
  auto tileX = [&](int t) { return ((rev ? numTiles - 1 - t : t) % tilesX) * 32; };

  // Resident weights of the classes (ca, 0) and (ca, 1) of this kt and the bias, by all waves: every load of a thread is in flight before
  // the first is waited for, and the staging waves have asked for the first tile's halos before that (see their branch) -- one memory
  // round trip in front of the first step instead of one per portion the compiler happened to unroll.
  auto stage_weights_and_bias = [&]() {
    constexpr int VWA = CAP / 8, NW = 4 * KT * VWA, PER = (NW + NT - 1) / NT;
    static_assert(2 * PER <= 32, "weight vectors per thread");
    uint4v wreg[2][PER];
#if HAS_BIAS
    static_assert(KT <= NT, "one bias value per thread");
    const _Float16 bias = BIAS[kt * KT + (tid < KT ? tid : 0)];
#endif
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      const _Float16 *w = FILT + (size_t)((ca * 2 + b) * NKT + kt) * KT * (4 * CAP + 9 * CBP);
#pragma unroll
      for (int k = 0; k < PER; ++k) {
        const int i = tid + k * NT;
        wreg[b][k] = ld16(w + (size_t)(i < NW ? i : NW - 1) * 8);
      }
    }
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int k = 0; k < PER; ++k) {
        const int i = tid + k * NT;
        const int row = i / VWA, v = i - row * VWA;
        if (i < NW)
          *reinterpret_cast<uint4v *>(sWA[b] + row * WAP + v * 8) = wreg[b][k];
      }
#if HAS_BIAS
    if (tid < KT)
      sBias[tid] = (float)bias;
#endif
  };

  if (wv >= WAVES) {
    // ---- staging waves ---------------------------------------------------------------------------------------
    const int st = tid - WAVES * 64;
    const OutBuf out = out_buffer(OUT, pc);
    const Sources srcs = make_sources(A, B, pc);
    const __amdgpu_buffer_rsrc_t ra = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16 *>(A), 0, (int)srcs.bytesA, 0x00020000);
    const __amdgpu_buffer_rsrc_t rb = __builtin_amdgcn_make_buffer_rsrc(const_cast<_Float16 *>(B), 0, (int)srcs.bytesB, 0x00020000);
    // What does not change from tile to tile, per vector of this thread: its place in LDS, its row / column inside
    // the halo and its byte offset relative to the halo's first pixel.
    uint4v ga[NA][NVA];
    int aLds[NVA], aYX[NVA], aRel[NVA];
#pragma unroll
    for (int it = 0; it < NVA; ++it) {
      const int i = st + it * NSTG;
      const int pix = i / VA, v = i - pix * VA;
      const int hy = pix / AW, hx = pix - hy * AW;
      aLds[it] = i < AH * AW * VA ? pix * APITCH + v * 8 : -1; // -1: past the halo (loads nothing, writes the spare slot)
      aYX[it] = (hy << 16) | hx;
      aRel[it] = ((hy * WL + hx) * CA + v * 8) * 2;
    }
    uint4v gb[NVB];
    int bLds[NVB], bYX[NVB], bRel[NVB];
#pragma unroll
    for (int it = 0; it < NVB; ++it) {
      const int i = st + it * NSTG;
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
    // loads of step `kind` (A chunk 0 .. NA-1, or NA: the B halo) of this workgroup's n-th tile; past the last tile
    // the same number of loads is issued and none of them reads memory
    auto issue = [&](int kind, int n) {
      const bool live = n < myTiles;
      const int t = live ? tile0 + n * SLOTS : tile0;
      if (kind < NA) {
        const int yb = tileY(t) + ca - 1, xb = tileX(t) - 1; // rows yl0 + ca - 1 .., columns xl0 - 1 ..
        const int base = ((yb * WL + xb) * CA + kind * CKA) * 2;
#pragma unroll
        for (int c = 0; c < NA; ++c)
          if (c == kind) {
#pragma unroll
            for (int it = 0; it < NVA; ++it) {
              const int yl = yb + (aYX[it] >> 16), xl = xb + (aYX[it] & 0xFFFF);
              // channels past CA are staged as zeros (their weights are zero, but 0 * NaN is NaN)
              const bool ok = live && aLds[it] >= 0 && c * CKA + aLds[it] % APITCH < CA && yl >= 0 && yl < HL && xl >= 0 && xl < WL;
              ga[c][it] = __builtin_amdgcn_raw_buffer_load_b128(ra, ok ? (unsigned)(base + aRel[it]) : NO_LOAD, 0, LOAD_AUX);
            }
          }
      } else {
        const int yb = 2 * tileY(t) + ca - 1, xb = 2 * tileX(t) - 1; // full-resolution rows 2 yl0 + ca - 1 .., columns 2 xl0 - 1 ..
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
      }
    };
    auto commit = [&](int kind) {
      if (kind < NA) {
#pragma unroll
        for (int c = 0; c < NA; ++c)
          if (c == kind) {
#pragma unroll
            for (int it = 0; it < NVA; ++it)
              *reinterpret_cast<uint4v *>(sA[c] + (aLds[it] >= 0 ? aLds[it] : AH * AW * APITCH)) = ga[c][it];
          }
      } else {
#pragma unroll
        for (int it = 0; it < NVB; ++it) {
            uint4v val = gb[it];
            if (CB % 8 != 0) {
              const uint4v sh = shr_halves<(8 - CB % 8) % 8>(val);
              const bool part = (bLds[it] % BPITCH) + 8 > CB; // the vector's first channel is its LDS offset inside the pixel
#pragma unroll
              for (int e = 0; e < 4; ++e) val[e] = part ? sh[e] : val[e];
            }
            *reinterpret_cast<uint4v *>(sB + (bLds[it] >= 0 ? bLds[it] : BH * BW * BPITCH)) = val;
          }
      }
    };
    // The finished tile, as the computing waves left it in LDS, goes to memory as whole rows of 64 pixels, consecutive
    // lanes storing consecutive 16 bytes.  It is read from LDS in the next tile's first step (the only interval in
    // which it is complete and not yet being rewritten) and stored in portions, one per step of that tile: a store
    // instruction waits for room in the memory pipeline, and eight of them in a row made the first step's staging work
    // longer than its matrix work while the last step's staging waves idled.  The last step takes a quarter of the
    // vectors, the steps over A share the rest.
    uint4v ov[NVO];
    auto read_tile = [&]() {
#pragma unroll
      for (int it = 0; it < NVO; ++it) {
        const int i = st + it * NSTG;
        const int r = i / (64 * SPP), rem = i - r * (64 * SPP);
        const int p = rem / SPP, sl = rem - p * SPP;
        ov[it] = sOut[i < TLH * 64 * SPP ? OUT_SLOT(r, p, sl) : 0];
      }
    };
    constexpr int NV_LAST = NVO / 4, NV_STEP = (NVO - NV_LAST + NA - 1) / NA;
    auto store_part = [&](int n, int first, int last) { // vectors [first, last) of this workgroup's n-th tile
      const int t = tile0 + n * SLOTS;
      const int yl0 = tileY(t), x0 = 2 * tileX(t);
#pragma unroll
      for (int it = 0; it < NVO; ++it) {
        if (it < first || it >= last)
          continue;
        const int i = st + it * NSTG;
        const int r = i / (64 * SPP), rem = i - r * (64 * SPP);
        const int p = rem / SPP, sl = rem - p * SPP;
        const bool ok = n >= 0 && i < TLH * 64 * SPP && yl0 + r < HL && x0 + p < (int)pc.IN_W;
        const unsigned off = ((unsigned)((2 * (yl0 + r) + ca) * (int)pc.IN_W + x0 + p) * (unsigned)OPITCH + (unsigned)(kt * KT + sl * 8)) * 2u;
        __builtin_amdgcn_raw_buffer_store_b128(ov[it], out, ok ? off : NO_STORE, 0, STORE_AUX);
      }
    };
#pragma unroll
    for (int k = 0; k <= NA; ++k) {
      issue(k, 0);
      __builtin_amdgcn_sched_barrier(0); // keep the register sets in issue order: the waits count loads in flight
    }
    stage_weights_and_bias();
    __builtin_amdgcn_sched_barrier(0);
    commit(0);
    issue(0, 1);
    for (int n = 0; n < myTiles; ++n) {
#pragma unroll
      for (int k = 0; k <= NA; ++k) {
        DNX_SYNC(); // step k of tile n starts: its buffer is complete, every other buffer is free
        const int nk = k == NA ? 0 : k + 1; // the step after this one
        const int nn = k == NA ? n + 1 : n;
        // The same instructions on every path through the loop (past the last tile the loads read nothing, what is
        // written to LDS is never read and the stores store nothing): the waits then count exactly the loads in flight.
        commit(nk);
        issue(nk, nn + 1);
        if (k == 0)
          read_tile(); // tile n - 1: complete since the barrier above, rewritten only after this tile's last barrier
        constexpr int cut = NVO - NV_LAST;
        const int first = k == NA ? cut : (k * NV_STEP < cut ? k * NV_STEP : cut);
        const int last = k == NA ? NVO : ((k + 1) * NV_STEP < cut ? (k + 1) * NV_STEP : cut);
        store_part(n - 1, first, last);
      }
    }
    DNX_SYNC(); // the last tile is in LDS
    read_tile();
    store_part(myTiles - 1, 0, NVO);
  } else {
    // ---- computing waves -------------------------------------------------------------------------------------
    stage_weights_and_bias();
    const int l32 = lane & 31;
    const int kq = (lane >> 5) * 8;
    const int rg = wv / KSP;           // row group: low-resolution rows rg * RPW .. of the tile
    const int kb0 = (wv % KSP) * KBW;  // first of this wave's 32-channel blocks
    // the 9 taps of B: the same for every class (class (ca, 0)'s copy), one matrix step of channels, in registers
    half8 wB[9][CBP / 16][KBW];
    {
      const _Float16 *w = FILT + (size_t)((ca * 2) * NKT + kt) * KT * (4 * CAP + 9 * CBP) + 4 * KT * CAP;
#pragma unroll
      for (int tap = 0; tap < 9; ++tap)
#pragma unroll
        for (int ks = 0; ks < CBP / 16; ++ks)
#pragma unroll
          for (int kb = 0; kb < KBW; ++kb)
            wB[tap][ks][kb] = *reinterpret_cast<const half8 *>(w + ((tap * KT + (kb0 + kb) * 32 + l32) * CBP + ks * 16 + kq));
    }
    Acc acc[2]; // column parity b = 0, 1; blocks kb0 .. kb0 + KBW - 1 in v[0 .. KBW - 1]
    for (int n = 0; n < myTiles; ++n) {
      // ---- the folded 2x2 taps over the low-resolution source, CKA channels per step: class (ca, b), tap (ty, tx)
      // reads low-resolution row y + ca - 1 + ty, column x + b - 1 + tx = halo column (x - xl0) + b + tx
#pragma unroll
      for (int c = 0; c < NA; ++c) {
        DNX_SYNC();
        if (c == 0) { // the staged bias is visible after the first barrier
#pragma unroll
          for (int b = 0; b < 2; ++b)
#pragma unroll
            for (int kb = 0; kb < KBW; ++kb)
#pragma unroll
              for (int j = 0; j < RPW; ++j)
#pragma unroll
                for (int i = 0; i < 16; ++i)
                  acc[b].v[kb][j][i] = HAS_BIAS ? sBias[(kb0 + kb) * 32 + (lane >> 5) * 16 + i] : 0.0f;
        }
#if SWP
        {
          // Software pipeline.  A unit is one weight fragment set: a 16-channel slice ks, a column cc = b + tx of the halo window,
          // one of the (b, tx) pairs with that sum and a row tap ty -- KBW weight reads that feed KBW * RPW matrix
          // instructions; the first unit of a column also reads the column's RPW + 1 pixel fragments.  The reads of unit
          // u + SWPD are issued in front of unit u's matrix instructions, into rings of SWPD + 1 weight sets and three pixel
          // columns (a column has at least two units, so the units u .. u + 3 touch at most three).  Left to the compiler,
          // every weight read stood right in front of the instruction that needs it, which then waited out the LDS round
          // trip: 2048 cycles of matrix work per tile took 3250.
          constexpr int SWPD = 3, NU = (CKA / 16) * 8;
          half8 px[3][RPW + 1], wf[SWPD + 1][KBW];
          auto reads = [&](int u) {
            const int ks = u >> 3, combo = (u >> 1) & 3, ty = u & 1, b = combo >> 1, tx = combo & 1, cc = b + tx;
            const int kk = ks * 16 + kq;
            if ((u & 7) == 0 || (u & 7) == 2 || (u & 7) == 6) {
#pragma unroll
              for (int t = 0; t < RPW + 1; ++t)
                px[(ks * 3 + cc) % 3][t] = *reinterpret_cast<const half8 *>(sA[c] + ((rg * RPW + t) * AW + l32 + cc) * APITCH + kk);
            }
#pragma unroll
            for (int kb = 0; kb < KBW; ++kb)
              wf[u % (SWPD + 1)][kb] = *reinterpret_cast<const half8 *>(sWA[b] + ((ty * 2 + tx) * KT + (kb0 + kb) * 32 + l32) * WAP + c * CKA + kk);
          };
#pragma unroll
          for (int u = 0; u < SWPD; ++u) reads(u);
#pragma unroll
          for (int u = 0; u < NU; ++u) {
            if (u + SWPD < NU)
              reads(u + SWPD);
            __builtin_amdgcn_sched_barrier(0);
            const int ks = u >> 3, combo = (u >> 1) & 3, ty = u & 1, b = combo >> 1, tx = combo & 1, cc = b + tx;
#pragma unroll
            for (int kb = 0; kb < KBW; ++kb)
#pragma unroll
              for (int j = 0; j < RPW; ++j)
                acc[b].v[kb][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[u % (SWPD + 1)][kb], px[(ks * 3 + cc) % 3][j + ty], acc[b].v[kb][j], 0, 0, 0);
            __builtin_amdgcn_sched_barrier(0);
          }
        }
#else
#pragma unroll
        for (int ks = 0; ks < CKA / 16; ++ks) {
          const int kk = ks * 16 + kq;
          half8 px[RPW + 1][3];
#pragma unroll
          for (int t = 0; t < RPW + 1; ++t)
#pragma unroll
            for (int cc = 0; cc < 3; ++cc)
              px[t][cc] = *reinterpret_cast<const half8 *>(sA[c] + ((rg * RPW + t) * AW + l32 + cc) * APITCH + kk);
#pragma unroll
          for (int ty = 0; ty < 2; ++ty)
#pragma unroll
            for (int tx = 0; tx < 2; ++tx)
#pragma unroll
              for (int b = 0; b < 2; ++b) {
                half8 wf[KBW];
#pragma unroll
                for (int kb = 0; kb < KBW; ++kb)
                  wf[kb] = *reinterpret_cast<const half8 *>(sWA[b] + ((ty * 2 + tx) * KT + (kb0 + kb) * 32 + l32) * WAP + c * CKA + kk);
#pragma unroll
                for (int kb = 0; kb < KBW; ++kb)
#pragma unroll
                  for (int j = 0; j < RPW; ++j)
                    acc[b].v[kb][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[kb], px[j + ty][b + tx], acc[b].v[kb][j], 0, 0, 0);
              }
        }
#endif
      }
      // ---- the 9 taps over the full-resolution source: class (ca, b), tap (r, s) reads halo row 2 (y - yl0) + r,
      // halo column 2 (x - xl0) + b + s, which the de-interleaved halo holds at [parity (b + s) & 1][(x - xl0) + (b + s) / 2]
      DNX_SYNC();
#if SWP
      {
        // a unit is one row tap r of one 16-channel slice: RPW x 4 pixel fragments (the weights are in registers) for 6 KBW RPW
        // matrix instructions; the next unit's fragments are read in front of this unit's instructions
        constexpr int NUB = (CBP / 16) * 3;
        half8 px[2][RPW][4];
        auto reads = [&](int u) {
          const int ks = u / 3, r = u % 3, kk = ks * 16 + kq;
#pragma unroll
          for (int j = 0; j < RPW; ++j)
#pragma unroll
            for (int cc = 0; cc < 4; ++cc)
              px[u & 1][j][cc] = *reinterpret_cast<const half8 *>(sB + ((2 * (rg * RPW + j) + r) * BW + (cc & 1) * 33 + l32 + (cc >> 1)) * BPITCH + kk);
        };
        reads(0);
#pragma unroll
        for (int u = 0; u < NUB; ++u) {
          if (u + 1 < NUB)
            reads(u + 1);
          __builtin_amdgcn_sched_barrier(0);
          const int ks = u / 3, r = u % 3;
#pragma unroll
          for (int s2 = 0; s2 < 3; ++s2)
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
              for (int kb = 0; kb < KBW; ++kb)
#pragma unroll
                for (int j = 0; j < RPW; ++j)
                  acc[b].v[kb][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wB[r * 3 + s2][ks][kb], px[u & 1][j][b + s2], acc[b].v[kb][j], 0, 0, 0);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
#else
#pragma unroll
      for (int ks = 0; ks < CBP / 16; ++ks) {
        const int kk = ks * 16 + kq;
#pragma unroll
        for (int r = 0; r < 3; ++r) {
          half8 px[RPW][4];
#pragma unroll
          for (int j = 0; j < RPW; ++j)
#pragma unroll
            for (int cc = 0; cc < 4; ++cc)
              px[j][cc] = *reinterpret_cast<const half8 *>(sB + ((2 * (rg * RPW + j) + r) * BW + (cc & 1) * 33 + l32 + (cc >> 1)) * BPITCH + kk);
#pragma unroll
          for (int s2 = 0; s2 < 3; ++s2)
#pragma unroll
            for (int b = 0; b < 2; ++b)
#pragma unroll
              for (int kb = 0; kb < KBW; ++kb)
#pragma unroll
                for (int j = 0; j < RPW; ++j)
                  acc[b].v[kb][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wB[r * 3 + s2][ks][kb], px[j][b + s2], acc[b].v[kb][j], 0, 0, 0);
        }
      }
#endif
      // the tile as binary16 into LDS: this lane's 16 channels kb * 32 + (lane >> 5) * 16 .. of the pixels 2 l32 + b
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int kb = 0; kb < KBW; ++kb)
#pragma unroll
          for (int j = 0; j < RPW; ++j) {
            float v[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) v[i] = acc[b].v[kb][j][i];
            const half8 done[2] = {finish8(v), finish8(v + 8)}; // activation, rounding
#pragma unroll
            for (int e = 0; e < 2; ++e)
              sOut[OUT_SLOT(rg * RPW + j, 2 * l32 + b, (kb0 + kb) * 4 + (lane >> 5) * 2 + e)] = __builtin_bit_cast(uint4v, done[e]);
          }
    }
    DNX_SYNC(); // the last tile is in LDS
  }
}
