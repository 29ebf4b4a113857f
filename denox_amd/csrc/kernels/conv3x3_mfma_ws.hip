// conv3x3_mfma_ws.hip -- weight-stationary variant of the fused 3x3 convolution
// (same operation and compile-time interface as conv3x3_mfma.hip, see conv_common.h).
//
// The launch is persistent: GRID workgroups, one per compute unit, each keeps the whole
// 9 x KT x CPAD weight slice of its output-channel tile in LDS for its lifetime and walks
// over many (WAVES*RPW) x 32 pixel tiles.  Only input halos stream: CK channels at a time
// through two LDS buffers, one barrier per step, every global load issued two steps before
// its data is written to LDS.  Compared with streaming the weights per tile this removes
// most L2 reads, most LDS writes and most address arithmetic of the inner loop.
//
//   PW = 0  every wave stages its share of the halo and then computes;
//   PW > 0  wave specialisation: WAVES waves only compute (LDS reads + MFMA + epilogue) while
//           PW further waves only stage halos, so that address arithmetic, load waits and LDS
//           writes run beside the matrix work instead of in front of it (all waves of a
//           workgroup meet at the step barrier, so inside one role nothing overlaps).
//   OSTAGE  (with PW > 0, pixel-major result, at least two steps per tile) the finished tile goes to memory through
//           LDS: the computing waves leave it there as binary16, and the staging waves store it during the next tile's
//           first step with consecutive lanes on consecutive 16 bytes -- whole pixels (KT channels), 1 KiB per store
//           instruction, instead of 16 bytes per lane at a stride of one pixel.  The computing waves then never wait
//           for memory at all.
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
#ifndef NXCD
#define NXCD 8 // accelerator dies, each with an L2 of its own; the host sizes the grid with the same number
#endif
#define NSTAGE ((PW > 0 ? PW : WAVES) * 64) // threads that stage halos
#ifndef OSTAGE
#define OSTAGE 0
#endif
#if OSTAGE
static_assert(PW > 0 && MF == 32 && NCHUNK >= 2 && !POOL && !CROP && !LAYOUT_OUT && OVEC && OPITCH % 8 == 0 && KOUT % 8 == 0, "staged result: see above");
#define SPP (KT / 8)                             // 16-byte slots of a pixel's KT channels
#define OSLOTS (SPP + 1)                         // pitch of a pixel in the staged tile: odd, so that 16 consecutive pixels start in 16 different bank groups
#define NVO ((TH * TW * SPP + NSTAGE - 1) / NSTAGE) // slots per staging thread
#endif

// The resident weights ([tap][KT][CPAD] in memory, one chunk = the whole reduction, to LDS rows of CPADP) and the bias, by all
// threads of the workgroup: every thread issues all of its loads before it waits for the first, in batches of at most WBATCH
// vectors -- one memory round trip, where a loop of load / store pairs (which the compiler unrolls six times) took one per six
// vectors, in front of a kernel whose whole run may be ten such round trips long.
#define WBATCH 24
__device__ DNX_INLINE void stage_weights_and_bias(_Float16 *sW, bias_t *sBias, const _Float16 *__restrict__ wsrc, const _Float16 *__restrict__ BIAS, int kt, int tid) {
  constexpr int VPR = CPAD / 8, N = NTAPS * KT * VPR, PER = (N + NT - 1) / NT;
#if HAS_BIAS
  static_assert(KT <= NT, "one bias value per thread");
  const _Float16 bias = BIAS[kt * KT + (tid < KT ? tid : 0)];
#endif
#pragma unroll
  for (int r0 = 0; r0 < PER; r0 += WBATCH) {
    uint4v w[WBATCH];
#pragma unroll
    for (int k = 0; k < WBATCH; ++k)
      if (r0 + k < PER) {
        const int i = tid + (r0 + k) * NT;
        w[k] = ld16(wsrc + (size_t)(i < N ? i : N - 1) * 8); // threads past the end re-read the last vector
      }
#pragma unroll
    for (int k = 0; k < WBATCH; ++k)
      if (r0 + k < PER) {
        const int i = tid + (r0 + k) * NT;
        const int row = i / VPR, v = i - row * VPR;
        if (i < N)
          *reinterpret_cast<uint4v *>(sW + row * CPADP + v * 8) = w[k];
      }
  }
#if HAS_BIAS
  if (tid < KT)
    sBias[tid] = (float)bias;
#endif
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
  __shared__ __attribute__((aligned(16))) _Float16 sW[NTAPS * KT * CPADP];
  __shared__ __attribute__((aligned(16))) _Float16 sIn[2][HALO_ELEMS];
  __shared__ __attribute__((aligned(16))) bias_t sBias[KT];
#if OSTAGE
  __shared__ uint4v sOut[TH * TW * OSLOTS];
#endif
#if CB == 0
  const _Float16 *B = nullptr;
#endif
#if !HAS_BIAS
  const _Float16 *BIAS = nullptr;
#endif
  const int tid = DNX_TID;
  const OutBuf out = out_buffer(OUT, pc);
  const Sources srcs = make_sources(A, B, pc);
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6); // wave-uniform: roles branch on it
  const int lane = tid & 63;

  const int b = DNX_BID_X;
  const int xcd = b % NXCD;
  const int q = b / NXCD;
  const int kt = q % NKT;
  const int slot = q / NKT;
  const int tilesX = (CONV_OUT_W(pc) + TW - 1) / TW;
  const int tilesY = (CONV_OUT_H(pc) + TH - 1) / TH;
  const int numTiles = tilesX * tilesY;
  const int perXcd = (numTiles + NXCD - 1) / NXCD;
  const int first = xcd * perXcd;
  int last = first + perXcd;
  last = last < numTiles ? last : numTiles;
  int tile = first + slot;
  if (tile >= last)
    return; // uniform for the workgroup: nothing was staged yet
  const bool rev = (pc.FLAGS & 1u) != 0;
  // position of the t-th tile of the walk
  auto tileY = [&](int t) { return ((rev ? numTiles - 1 - t : t) / tilesX) * TH; };
  auto tileX = [&](int t) { return ((rev ? numTiles - 1 - t : t) % tilesX) * TW; };

  // The fetch cursor walks the same sequence of steps as the compute cursor (tile by tile,
  // NCHUNK steps per tile), two steps ahead.
  typedef Halo<NSTAGE> H;
  H::Map map;
  H::Src fsrc;
  int ftile = tile, fchunk = 0;
  // Past its last tile the cursor stays where it is: the loads are issued all the same (and never used), so that
  // the number of loads in flight is the same on every path through the loop.
  auto issue = [&](H::Regs &regs) {
    H::fetch_step(srcs, regs, map, fsrc, fchunk);
    if (++fchunk == NCHUNK) {
      fchunk = 0;
      ftile += SLOTS;
      if (ftile < last)
        H::src_init(fsrc, map, tileY(ftile), tileX(ftile), pc);
    }
  };

  // The first two halos are on their way before the weights are asked for: everything a workgroup needs for its first step
  // then arrives in one round trip.
  H::Regs st0, st1;
  if (PW == 0 || wv >= WAVES) {
    H::map_init(map, PW > 0 ? tid - WAVES * 64 : tid);
    H::src_init(fsrc, map, tileY(ftile), tileX(ftile), pc);
    issue(st0); // step 0
    __builtin_amdgcn_sched_barrier(0); // keep the two sets in issue order: the waits count loads in flight
    issue(st1); // step 1
    __builtin_amdgcn_sched_barrier(0);
  }
  stage_weights_and_bias(sW, sBias, FILT + (size_t)kt * NTAPS * KT * CPAD, BIAS, kt, tid);

#if PW == 0
  Acc acc;
  // The finished tile, converted.  Its stores go out in NPARTS portions during the steps of the next tile: a
  // burst of all stores of all waves at once would hold the waves up at the store queue while nothing multiplies.
  constexpr int NPARTS = NCHUNK < OROWS ? NCHUNK : OROWS; // whole output rows per portion
  Packed done;
  int dtile = 0, dpart = 0;
  bool pend = false;
  auto store_part = [&]() {
#pragma unroll
    for (int p = 0; p < NPARTS; ++p)
      if (dpart == p)
        store_packed(done, out, tileY(dtile), tileX(dtile), kt, wv, lane, pc, p, NPARTS);
    if (++dpart == NPARTS)
      pend = false;
  };
#if PP
  // Two-phase schedule.  The waves form two groups that every SIMD holds in equal parts ((wave / 4) % 2).  A step has
  // two phases with a barrier after each: in the first, group A multiplies step k while group B does everything
  // else (converting and storing finished tiles, writing its share of halo k+1 to LDS, issuing loads); in the second
  // the roles swap.  The matrix pipe then always has one group feeding it, instead of idling while all waves stage,
  // convert or wait at the same time.  Halo k+1 goes to the buffer that held halo k-1, which both groups finished
  // reading before the phase in which the first share is written.
  static_assert(WAVES % 8 == 0, "two wave groups on four SIMDs");
  const bool groupB = ((wv >> 2) & 1) != 0;
  int cchunk = 0, commitChunk = 0;
  auto mma = [&](int buf) { mma_step<CPADP>(sIn[buf], sW, cchunk * CK, acc, wv, lane, cchunk); };
  auto post = [&]() { // after this wave's matrix work of a step
    if (++cchunk == NCHUNK) {
      pack_tile(acc, done);
      init_acc(acc, sBias, lane);
      dtile = tile;
      dpart = 0;
      pend = tile < last; // false in the spare step
      cchunk = 0;
      tile += SLOTS;
    }
  };
  auto stage = [&](H::Regs &regs, int buf) { // this wave's share of the next halo, and the refill of the register set
    if (pend)
      store_part();
    H::commit_step(regs, sIn[buf], map, commitChunk);
    if (++commitChunk == NCHUNK)
      commitChunk = 0;
    issue(regs);
  };
  stage(st0, 0); // halo 0, by all waves
  DNX_SYNC();
  init_acc(acc, sBias, lane); // the staged bias is visible from here on
  if (!groupB) {
    do {
      mma(0); DNX_SYNC(); post(); stage(st1, 1); DNX_SYNC();
      mma(1); DNX_SYNC(); post(); stage(st0, 0); DNX_SYNC();
    } while (tile < last);
  } else {
    do {
      stage(st1, 1); DNX_SYNC(); mma(0); DNX_SYNC(); post();
      stage(st0, 0); DNX_SYNC(); mma(1); DNX_SYNC(); post();
    } while (tile < last);
  }
#else
  int cchunk = 0, buf = 0;
  auto step = [&](H::Regs &regs) {
    H::commit_step(regs, sIn[buf], map, cchunk);
    // One barrier per step: buffer `buf` was last read two steps ago, and every wave
    // has passed the barrier of the step in between since then.
    DNX_SYNC();
    if (cchunk == 0)
      init_acc(acc, sBias, lane);
    // A portion of the previous tile's stores, in front of this step's loads: when a later step waits for those
    // loads, it counts back over at most these stores, which are old by then.
    if (pend)
      store_part();
    issue(regs); // refill this register set: the step after next
    mma_step<CPADP>(sIn[buf], sW, cchunk * CK, acc, wv, lane, cchunk);
    buf ^= 1;
    if (++cchunk == NCHUNK) {
      pack_tile(acc, done);
      dtile = tile;
      dpart = 0;
      pend = tile < last; // false in the spare step below
      cchunk = 0;
      tile += SLOTS;
    }
  };
  // The loop always runs both steps, so that it has one entry and one back edge with the same loads in flight on
  // both: the compiler then waits for exactly the register set a step needs.  When the last tile ends after the
  // first step, the second one is a spare: it stages and multiplies stale data and stores nothing.
  do {
    step(st0);
    step(st1);
  } while (tile < last);
#endif
#pragma unroll
  for (int p = 0; p < NPARTS; ++p)
    if (pend)
      store_part();
#else
  // number of steps this workgroup runs: both roles execute exactly one barrier per step
  const int myTiles = (last - tile + SLOTS - 1) / SLOTS;
  const int steps = myTiles * NCHUNK;
  if (wv >= WAVES) {
    // ---- staging waves: step g's halo is written to sIn[g & 1] during step g - 1 ----
    int cchunk = 0; // chunk index of the step being committed
    auto commit = [&](H::Regs &regs, int g) {
      H::commit_step(regs, sIn[g & 1], map, cchunk);
      if (++cchunk == NCHUNK)
        cchunk = 0;
    };
#if OSTAGE
    // the n-th tile of this workgroup, as the computing waves left it in LDS
    const int stid = tid - WAVES * 64;
    auto store_staged = [&](int n) {
      const int t = tile + n * SLOTS;
      const int y0 = tileY(t), x0 = tileX(t);
#pragma unroll
      for (int it = 0; it < NVO; ++it) {
        const int i = stid + it * NSTAGE;
        const int p = i / SPP, sl = i - p * SPP; // pixel of the tile (row-major), slot of the pixel
        const int y = y0 + p / TW, x = x0 + p % TW;
        const bool ok = i < TH * TW * SPP && y < (int)CONV_OUT_H(pc) && x < (int)CONV_OUT_W(pc) && kt * KT + sl * 8 < KOUT;
        const uint4v v = sOut[i < TH * TW * SPP ? p * OSLOTS + sl : 0];
        const unsigned off = ((unsigned)(y * (int)CONV_OUT_W(pc) + x) * (unsigned)OPITCH + (unsigned)(kt * KT + sl * 8)) * 2u;
        __builtin_amdgcn_raw_buffer_store_b128(v, out, ok ? off : NO_STORE, 0, STORE_AUX);
      }
    };
#endif
    commit(st0, 0);
    issue(st0);         // step 2
    for (int g = 0; g < steps; g += 2) {
      DNX_SYNC();       // step g starts: sIn[g & 1] is complete, sIn[(g + 1) & 1] is free
      if (g + 1 < steps) {
        commit(st1, g + 1);
        issue(st1);     // step g + 3
      }
#if OSTAGE
      if (g > 0 && g % NCHUNK == 0)
        store_staged(g / NCHUNK - 1); // complete since the barrier above; rewritten after the last barrier of this tile
#endif
      if (g + 1 >= steps)
        break;
      DNX_SYNC();       // step g + 1 starts
      if (g + 2 < steps) {
        commit(st0, g + 2);
        issue(st0);     // step g + 4
      }
#if OSTAGE
      if ((g + 1) % NCHUNK == 0)
        store_staged((g + 1) / NCHUNK - 1);
#endif
    }
#if OSTAGE
    DNX_SYNC();         // the last tile is in LDS
    store_staged(myTiles - 1);
#endif
  } else {
    // ---- computing waves ----
    Acc acc;
    int cchunk = 0;
    for (int g = 0; g < steps; ++g) {
      DNX_SYNC();
      if (cchunk == 0)
        init_acc(acc, sBias, lane);
      mma_step<CPADP>(sIn[g & 1], sW, cchunk * CK, acc, wv, lane, cchunk);
      if (++cchunk == NCHUNK) {
#if OSTAGE
        // the tile as binary16 into LDS: this lane's 16 channels kb * 32 + (lane >> 5) * 16 .. of pixel (wv * RPW + j, lane & 31)
        Packed pk;
        pack_tile(acc, pk);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int j = 0; j < RPW; ++j)
#pragma unroll
            for (int e = 0; e < 2; ++e)
              sOut[((wv * RPW + j) * TW + (lane & 31)) * OSLOTS + kb * 4 + (lane >> 5) * 2 + e] = __builtin_bit_cast(uint4v, pk.o[kb][j][e]);
#else
        store_tile(acc, out, tileY(tile), tileX(tile), kt, wv, lane, pc);
#endif
        cchunk = 0;
        tile += SLOTS;
      }
    }
#if OSTAGE
    DNX_SYNC(); // the last tile is in LDS
#endif
  }
#endif
}
