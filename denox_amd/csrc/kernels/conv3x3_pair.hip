// conv3x3_pair.hip -- two consecutive 3x3 convolutions in one dispatch:
//
//   mid[y,x,k] = act1(bias1[k] + sum_{r,s,c} src[y+r-1, x+s-1, c] * W1[k,c,r,s])      (K1 <= 32 channels, binary16)
//   out[y,x,k] = act (bias [k] + sum_{r,s,c} mid[y+r-1, x+s-1, c] * W2[k,c,r,s])      (KOUT <= 32 channels)
//
// with `src` assembled by the loader of conv_common.h (concat, 2x upsample, replicate pad of a source) and the result
// optionally reduced by a 2x2 max pool or cropped, exactly as in the single-convolution kernels.  `mid` never leaves
// the compute unit: where a thin full-resolution layer feeds another one, writing and re-reading that tensor is most
// of both layers' time.  The reference fuses for the same reason -- to skip a tensor's round trip through memory --
// in its concat+conv shader (compiler/src/denox/compiler/implement/shaders/conv/ConcatConvCMShader.cpp:760-965).
//
// Geometry.  The image is cut into vertical strips of SWO = 30 output columns, each strip into segments of rows; one
// persistent workgroup walks down one segment in steps of IH = WAVES*RPW rows.  In step k it
//   1. computes IH rows x 32 columns of `mid` (columns xs-1 .. xs+30 of strip xs) on the matrix cores from a staged
//      (IH+2) x 34 input halo, CK channels per LDS stage, weights W1 resident in LDS,
//   2. rounds them to binary16 (bias, activation; zero outside the image, which is the second convolution's padding)
//      and writes them into a ring of rows in LDS: the last two rows of step k-1 stay, so no row of `mid` is computed
//      twice along a segment (two rows at each segment's start are the only vertical overlap),
//   3. and, one barrier later -- in the same barrier interval as the first channel chunk of step k+1 -- computes IH x 32
//      outputs of the second convolution from the ring (rows lag two behind), of which the 30 inner columns are valid,
//      and stores them.  The second convolution's weights live in registers (9 taps x 32 channels of one row per lane).
// One barrier per channel chunk is all the synchronisation there is: between two barriers every wave runs its own
// sequence of second convolution, stores, first convolution and ring writes, so the waves that share a SIMD drift apart
// and one's conversions and stores overlap the other's matrix instructions.  With a single chunk per step the ring holds
// 2 IH + 2 rows (step k+1 is written while step k is read), otherwise IH + 2.
// Lanes 30 and 31 of the second convolution read two pixels past their ring row and compute garbage that is never
// stored; every output column of a matrix instruction depends on its own pixel only.
//
// Compile-time interface: everything conv_common.h takes describes the first convolution's sources (CA, CB, UPA,
// PADA, PADB, CK) and the second convolution's result (KOUT, ACT, HAS_BIAS, POOL, CROP, OPITCH); in addition
//   K1, ACT1, ALPHA1, HAS_BIAS1   output channels, activation and bias of the first convolution
//   TAPM                          1: the second convolution has so few output channels (3 KOUT <= 15) that its three filter
//                                 columns ride in the matrix rows (see below); not combined with POOL
//   SLOTS, NXCD                   the grid is NXCD * SLOTS persistent workgroups
//   PW                            0: every wave stages its share of the halo and computes; > 0: WAVES waves only compute
//                                 and PW further waves only move halos from memory to LDS (as in conv3x3_mfma_ws.hip)
//   W1REG                         1: the first convolution's weights live in registers of the computing waves as well
//                                 (9 taps x CPAD / 16 fragments), not in LDS.  With 32 output channels a weight fragment
//                                 serves RPW matrix instructions only, so reading it from LDS is 3 of the 7 LDS reads per
//                                 6 instructions, and the LDS read rate, not the matrix pipe, sets the pace of such layers
//   C2STAGE                       1 (needs PW == WAVES): the second convolution, its epilogue and its stores run on the staging
//                                 waves, which otherwise wait for memory most of the time: staging wave i does for the rows
//                                 of computing wave i, in the first chunk of step k + 1, what that wave would do itself.  A
//                                 computing wave then issues nothing but the first convolution's LDS reads, matrix
//                                 instructions and ring writes, and the latencies of the second convolution's epilogue
//                                 (cross-lane sums, conversions, narrow stores) overlap the matrix work of the wave that
//                                 shares its SIMD instead of preceding it
// KT is 32 for both convolutions.
#include "conv_common.h"

#ifndef KERNEL_NAME
#define KERNEL_NAME conv3x3_pair
#endif
#ifndef NXCD
#define NXCD 8
#endif
#ifndef ACT1
#define ACT1 0
#endif
#ifndef ALPHA1
#define ALPHA1 0.0f
#endif
#ifndef HAS_BIAS1
#define HAS_BIAS1 0
#endif
#ifndef TAPM
#define TAPM 0
#endif
#ifndef W1REG
#define W1REG 0
#endif
#ifndef C2STAGE
#define C2STAGE 0
#endif
#ifndef NBUF
#define NBUF 2 // halo buffers.  3 (with DLDS): the loads of chunk c + 2 are issued while chunk c is multiplied, a whole chunk earlier
#endif
static_assert(NBUF == 2 || (NBUF == 3 && DLDS), "a third halo buffer serves loads that go straight into LDS");
// Where the registers allow it, a convolution's accumulators start from its bias held in registers (see load_bias_regs);
// where the first convolution's weights fill the register file they start from the bias staged in LDS.
#define BIAS1REG (!W1REG)
#define BIAS2REG (!(W1REG && (!C2STAGE || DLDS)))
static_assert(!C2STAGE || PW == WAVES, "second convolution on the staging waves: one staging wave per computing wave");
static_assert(!TAPM || (3 * KOUT <= 15 && !POOL), "filter columns in the matrix rows: at most 5 output channels, no pooling");

static_assert(MF == 32 && KT == 32 && KB == 1, "one 32-channel block per convolution");
static_assert(KR == 3 && KS == 3 && SY == 1 && SX == 1 && PY == 1 && PX == 1, "3x3, stride 1, extent-preserving");
static_assert(K1 <= 32 && KOUT <= 32 && PP == 0, "unsupported variant");

#define CPADP (CPAD + 8)
#define IH TH             // rows of `mid` per step
#define IW 32             // columns of `mid` per step
#define SWO (IW - 2)      // output columns per strip
#define NS (NCHUNK == 1 ? 2 * IH + 2 : IH + 2) // rows in the ring
#define C2PAD 32          // channels of `mid` as the second convolution reduces over them (K1 padded)
#define C2P (C2PAD + 8)   // pixel pitch of the ring in halves: an odd multiple of 16 bytes
#define GRID (NXCD * SLOTS)

__device__ DNX_INLINE half8 finish8_first(const float *v) {
  half8 h;
#if ACT1 == 1
#pragma unroll
  for (int i = 0; i < 8; ++i) h[i] = (_Float16)v[i];
  const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  return __builtin_elementwise_max(h, zero);
#elif ACT1 == 2
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const float av = ALPHA1 * v[i];
    h[i] = (_Float16)(v[i] > av ? v[i] : av);
  }
  return h;
#else
#pragma unroll
  for (int i = 0; i < 8; ++i) h[i] = (_Float16)v[i];
  return h;
#endif
}

// (W1REG: no registers left for the first convolution's bias; its accumulators start from the bias staged in LDS)
__device__ DNX_INLINE void init_acc_first(Acc &acc, const bias_t *sBias1, int lane) {
  const int hsel = lane >> 5;
#pragma unroll
  for (int j = 0; j < RPW; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i)
#if HAS_BIAS1
      acc.v[0][j][i] = sBias1[hsel * 16 + i];
#else
      acc.v[0][j][i] = 0.0f;
#endif
}

// The bias of a convolution as an accumulator-shaped register set: lane's 16 output channels (lane >> 5) * 16 + i.  The first
// matrix instruction into each accumulator of a step takes it as its addend, so no pass over the accumulators starts a step
// (vector ALU instructions are not free beside matrix instructions here: what a wave issues between them delays them).
__device__ DNX_INLINE float16v load_bias_regs(const _Float16 *__restrict__ bias, bool has, int lane) {
  float16v b;
#pragma unroll
  for (int i = 0; i < 16; ++i) b[i] = has ? (float)bias[(lane >> 5) * 16 + i] : 0.0f;
  return b;
}

// The wave's RPW finished rows of `mid` -> ring.  acc.v[0][j] holds, for row j of the wave and pixel lane & 31, the 16
// channels (lane >> 5) * 16 + i.  slot0: ring row of the step's first row; (m0, xm0): image position of the step's
// first `mid` pixel.
__device__ DNX_INLINE void
store_mid(const Acc &acc, _Float16 *sMid, int slot0, int m0, int xm0, int H, int W, int wv, int lane) {
  const int l32 = lane & 31;
  const int x = xm0 + l32;
#pragma unroll
  for (int j = 0; j < RPW; ++j) {
    const int row = wv * RPW + j;
    int slot = slot0 + row;
    slot = slot >= NS ? slot - NS : slot;
    const int m = m0 + row;
    const bool inside = m >= 0 && m < H && x >= 0 && x < W;
    float v[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) v[i] = acc.v[0][j][i];
    uint4v lo = __builtin_bit_cast(uint4v, finish8_first(v)), hi = __builtin_bit_cast(uint4v, finish8_first(v + 8));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      lo[i] = inside ? lo[i] : 0u;
      hi[i] = inside ? hi[i] : 0u;
    }
    _Float16 *dst = sMid + (slot * IW + l32) * C2P + (lane >> 5) * 16;
    *reinterpret_cast<uint4v *>(dst) = lo;
    *reinterpret_cast<uint4v *>(dst + 8) = hi;
  }
}

// The second convolution's weights, in registers for the whole kernel: fragment [tap][ks] of weight row lane & 31
// (global layout [tap][32 rows][C2PAD]).
//
// TAPM.  A second convolution with KOUT <= 5 output channels would leave 27 of the 32 matrix rows idle.  Instead, matrix
// row (s, k) holds filter column s of output channel k (global layout [r][32 rows][C2PAD], row order as the epilogue's
// channel order): one instruction per filter row r then yields, for every ring pixel p, the three partial sums
// T[s][k][p] = sum_c W2[k][c][r][s] * mid[.][p][c], and out[k][x] = T[0][k][x] + T[1][k][x+1] + T[2][k][x+2] is finished
// with two cross-lane reads per channel.  3 instead of 9 matrix instructions per output row and 16-channel slice, and a
// third of the LDS reads (no shifted copies of the pixel fragments).
#if TAPM
#define W2TAPS 3
#else
#define W2TAPS NTAPS
#endif
struct SecondWeights {
  half8 w[W2TAPS][C2PAD / 16];
};
__device__ DNX_INLINE void load_second_weights(SecondWeights &sw, const _Float16 *__restrict__ FILT2, int lane) {
  const int l32 = lane & 31, kq = (lane >> 5) * 8;
#pragma unroll
  for (int tap = 0; tap < W2TAPS; ++tap)
#pragma unroll
    for (int ks = 0; ks < C2PAD / 16; ++ks)
      sw.w[tap][ks] = __builtin_bit_cast(half8, ld16(FILT2 + (size_t)(tap * 32 + l32) * C2PAD + ks * 16 + kq));
}

// Both matrix loops below are software-pipelined by hand: a "group" is one filter column s of one 16-channel slice, i.e.
// PXROWS pixel fragments (and, for the first convolution, three weight fragments) feeding 3 * RPW matrix instructions; the
// LDS reads of group g + 1 are issued in front of the matrix instructions of group g, and scheduling barriers keep that
// order.  Left to the compiler, every read was issued right in front of the instruction that needs it, so each pair of
// matrix instructions waited out a full LDS round trip.

// Second convolution: 9 taps x (C2PAD / 16) reduction steps from the ring.  rslot0: ring row that holds `mid` row
// (first output row of the step) - 1.
// BIAS2REG: the accumulators start from `bias`; else they hold their start values already
__device__ DNX_INLINE void mma_mid(const _Float16 *sMid, int rslot0, const SecondWeights &sw, Acc &acc, const float16v &bias, int wv, int lane) {
  const int l32 = lane & 31;
  const int kq = (lane >> 5) * 8;
  lds_half_t *pr[PXROWS];
#pragma unroll
  for (int hr = 0; hr < PXROWS; ++hr) {
    int slot = rslot0 + wv * RPW + hr;
    slot = slot >= NS ? slot - NS : slot;
    pr[hr] = lds_opaque(sMid + (slot * IW + l32) * C2P + kq);
  }
#if TAPM
  constexpr int NG = C2PAD / 16; // a group: one 16-channel slice, all filter columns at once
#else
  constexpr int NG = 3 * (C2PAD / 16);
#endif
  half8 px[2][PXROWS];
  auto load = [&](int g) {
    const int s = TAPM ? 0 : g / (C2PAD / 16), ks = TAPM ? g : g % (C2PAD / 16);
#pragma unroll
    for (int hr = 0; hr < PXROWS; ++hr)
      px[g & 1][hr] = *reinterpret_cast<lds_half8_t *>(pr[hr] + s * C2P + ks * 16);
  };
  load(0);
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const int s = TAPM ? 0 : g / (C2PAD / 16), ks = TAPM ? g : g % (C2PAD / 16);
    if (g + 1 < NG)
      load(g + 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
      for (int j = 0; j < RPW; ++j)
        acc.v[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(sw.w[TAPM ? r : r * 3 + s][ks], px[g & 1][j + r], (BIAS2REG && g == 0 && r == 0) ? bias : acc.v[0][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }
}

#if TAPM
// Epilogue of the TAPM form: lane x of the lower half adds the partial sums of filter columns 1 and 2 held by lanes
// x + 1 and x + 2 (registers KOUT + k and 2 KOUT + k) to its own (register k), then activation and rounding.  The
// neighbours' values arrive by DPP wave shifts (a vector ALU operand modifier); as LDS permutes each of them was a
// round trip through the LDS queue that the sum had to wait for.
__device__ DNX_INLINE float from_next_lane(float v) { // lane i: v of lane i + 1 (wave_shl:1); lane 63: 0
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), 0x130, 0xf, 0xf, true));
}
__device__ DNX_INLINE void pack_tapm(const Acc &acc, Packed &pk) {
#pragma unroll
  for (int j = 0; j < RPW; ++j) {
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      float v = 0.0f;
      if (i < KOUT) {
        const float p1 = acc.v[0][j][KOUT + i], p2 = acc.v[0][j][2 * KOUT + i]; // (a vector element is no object: copy it before reinterpreting its bits)
        v = (acc.v[0][j][i] + from_next_lane(p1)) + from_next_lane(from_next_lane(p2));
      }
      pk.o[0][j][i >> 3][i & 7] = finish1(v);
    }
  }
}
#endif

// First convolution, one chunk of L channels: as mma_chunk of conv_common.h (32 weight rows, pitch WPITCH; halo pitch CKP),
// pipelined as described above.
// FIRST: the accumulators start from `bias` (their contents are not read).
template <int L, int WPITCH, bool FIRST>
__device__ DNX_INLINE void mma_first(const _Float16 *sIn, const _Float16 *sW, int wofs, Acc &acc, const float16v &bias, int wv, int lane) {
  const int l32 = lane & 31;
  const int kq = (lane >> 5) * 8;
#if HROTL
  PxBase pxb;
  px_base_init(pxb, sIn, wv * RPW, lane);
#else
  lds_half_t *pxb = lds_opaque(sIn + (wv * RPW * HALO_W + l32) * CKP + kq);
#endif
  lds_half_t *wb = lds_opaque(sW + l32 * WPITCH + wofs + kq);
  constexpr int NG = 3 * (L / 16);
  half8 px[2][PXROWS], wf[2][3];
  auto load = [&](int g) {
    const int s = g / (L / 16), ks = g % (L / 16);
#pragma unroll
    for (int hr = 0; hr < PXROWS; ++hr)
#if HROTL
      px[g & 1][hr] = PX_READ(pxb, hr, s, ks);
#else
      px[g & 1][hr] = *reinterpret_cast<lds_half8_t *>(pxb + (hr * HALO_W + s) * CKP + ks * 16);
#endif
#pragma unroll
    for (int r = 0; r < 3; ++r)
      wf[g & 1][r] = *reinterpret_cast<lds_half8_t *>(wb + ((r * 3 + s) * 32) * WPITCH + ks * 16);
  };
  load(0);
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    if (g + 1 < NG)
      load(g + 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
      for (int j = 0; j < RPW; ++j)
        acc.v[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[g & 1][r], px[g & 1][j + r], (FIRST && g == 0 && r == 0) ? bias : acc.v[0][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }
}

#if W1REG
// The first convolution's weights in registers: fragment [tap][16-channel slice] of weight row lane & 31 (global layout
// [tap][32 rows][CPAD]).
struct FirstWeights {
  half8 w[NTAPS][CPAD / 16];
};
__device__ DNX_INLINE void load_first_weights(FirstWeights &fw, const _Float16 *__restrict__ FILT1, int lane) {
  const int l32 = lane & 31, kq = (lane >> 5) * 8;
#pragma unroll
  for (int tap = 0; tap < NTAPS; ++tap)
#pragma unroll
    for (int ks = 0; ks < CPAD / 16; ++ks)
      fw.w[tap][ks] = __builtin_bit_cast(half8, ld16(FILT1 + (size_t)(tap * 32 + l32) * CPAD + ks * 16 + kq));
}

// mma_first with the weights from registers; CHUNK (compile-time) selects the 16-channel slices CHUNK * CK / 16 ...
template <int L, int CHUNK>
__device__ DNX_INLINE void mma_first_reg(const _Float16 *sIn, const FirstWeights &fw, Acc &acc, int wv, int lane) {
  const int l32 = lane & 31;
  const int kq = (lane >> 5) * 8;
#if HROTL
  PxBase pxb;
  px_base_init(pxb, sIn, wv * RPW, lane);
#else
  lds_half_t *pxb = lds_opaque(sIn + (wv * RPW * HALO_W + l32) * CKP + kq);
#endif
  constexpr int NG = 3 * (L / 16);
  half8 px[2][PXROWS];
  auto load = [&](int g) {
    const int s = g / (L / 16), ks = g % (L / 16);
#pragma unroll
    for (int hr = 0; hr < PXROWS; ++hr)
#if HROTL
      px[g & 1][hr] = PX_READ(pxb, hr, s, ks);
#else
      px[g & 1][hr] = *reinterpret_cast<lds_half8_t *>(pxb + (hr * HALO_W + s) * CKP + ks * 16);
#endif
  };
  load(0);
#pragma unroll
  for (int g = 0; g < NG; ++g) {
    const int s = g / (L / 16), ks = g % (L / 16);
    if (g + 1 < NG)
      load(g + 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int r = 0; r < 3; ++r)
#pragma unroll
      for (int j = 0; j < RPW; ++j)
        acc.v[0][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(fw.w[r * 3 + s][CHUNK * (CK / 16) + ks], px[g & 1][j + r], acc.v[0][j], 0, 0, 0);
    __builtin_amdgcn_sched_barrier(0);
  }
}

// chunk `cchunk` of a step, found by comparison: the register file is indexed by constants only
template <int C>
__device__ DNX_INLINE void mma_first_reg_chunk(int cchunk, const _Float16 *sIn, const FirstWeights &fw, Acc &acc, int wv, int lane) {
  if constexpr (C < NCHUNK) {
    if (cchunk == C)
      mma_first_reg<(TAIL == CK || C < NCHUNK - 1) ? CK : TAIL, C>(sIn, fw, acc, wv, lane);
    else
      mma_first_reg_chunk<C + 1>(cchunk, sIn, fw, acc, wv, lane);
  }
}
#endif

// Stores the step's outputs: rows ob + wave * RPW + r, columns xs + (lane & 31); only the SWO inner columns and the
// rows in [ylo, yhi) belong to this step (the rest is another step's, or garbage).
__device__ DNX_INLINE void
store_pair(const Packed &pk, OutBuf out, int ob, int xs, int ylo, int yhi, int wv, int lane, const PushConstants &pc) {
  const unsigned W = CONV_OUT_W(pc), H = CONV_OUT_H(pc);
  const unsigned plane = LAYOUT_OUT ? out_plane_bytes(pc) : 0u;
  const int l32 = lane & 31;
  const int x = xs + l32;
  const int chb = (lane >> 5) * 16;
#pragma unroll
  for (int r = 0; r < OROWS; ++r) {
#if POOL
    const int y = ob + wv * RPW + 2 * r; // first row of the pooled pair; segment borders are even
    const unsigned WP = W >> 1, HP = H >> 1;
    const unsigned py = (unsigned)(y < 0 ? 0 : y) >> 1, px = (unsigned)x >> 1;
    const bool ok = (l32 & 1) == 0 && l32 < SWO && y >= ylo && y < yhi && py < HP && px < WP;
    store16(out, ok, py * WP + px, pk.o[0][r], chb, plane);
#else
    const int y = ob + wv * RPW + r;
    const bool mine = l32 < SWO && (!TAPM || lane < 32) && y >= ylo && y < yhi && x < (int)W && y < (int)H;
#if CROP
    const int oy = y - (int)pc.CROP_T, ox = x - (int)pc.CROP_L;
    store16(out, mine && oy >= 0 && oy < (int)pc.OUT_H && ox >= 0 && ox < (int)pc.OUT_W, (unsigned)oy * pc.OUT_W + (unsigned)ox, pk.o[0][r], chb, plane);
#else
    store16(out, mine, (unsigned)(y < 0 ? 0 : y) * W + (unsigned)x, pk.o[0][r], chb, plane);
#endif
#endif
  }
}

extern "C" __global__ DNX_LAUNCH_BOUNDS(NT) void KERNEL_NAME(
    const _Float16 *__restrict__ A,
#if CB > 0
    const _Float16 *__restrict__ B,
#endif
    _Float16 *__restrict__ OUT, const _Float16 *__restrict__ FILT1,
#if HAS_BIAS1
    const _Float16 *__restrict__ BIAS1,
#endif
    const _Float16 *__restrict__ FILT2,
#if HAS_BIAS
    const _Float16 *__restrict__ BIAS2,
#endif
    PushConstants pc) {
#if !W1REG
  __shared__ __attribute__((aligned(16))) _Float16 sW1[NTAPS * 32 * CPADP];
#else
  __shared__ __attribute__((aligned(16))) bias_t sBias1[32];
#endif
#if !BIAS2REG
  __shared__ __attribute__((aligned(16))) bias_t sBias2[32];
#endif
  __shared__ __attribute__((aligned(16))) _Float16 sIn[NBUF][HALO_ELEMS];
  __shared__ __attribute__((aligned(16))) _Float16 sMid[(NS * IW + 2) * C2P];
#if CB == 0
  const _Float16 *B = nullptr;
#endif
  const int tid = DNX_TID;
  const OutBuf out = out_buffer(OUT, pc);
  const Sources srcs = make_sources(A, B, pc);
  const int wv = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int lane = tid & 63;

  // ---- work units: (strip, segment) pairs, dealt so that neighbouring strips meet in one XCD's L2 ----
  const int Wc = (int)CONV_OUT_W(pc), Hc = (int)CONV_OUT_H(pc);
  if (Wc <= 0 || Hc <= 0)
    return;
  const int nstrips = (Wc + SWO - 1) / SWO;
  const int n0 = GRID / nstrips > 1 ? GRID / nstrips : 1;            // segments per strip aimed at
  const int L = (((Hc + n0 - 1) / n0 + 2) + IH - 1) / IH * IH;       // rows of `mid` per segment, whole steps
  const int nseg = (Hc + (L - 2) - 1) / (L - 2);                     // a segment yields L - 2 output rows
  const int units = nstrips * nseg;
  const int b = DNX_BID_X;
  int unit = (b % NXCD) * SLOTS + b / NXCD;
  if (unit >= units)
    return; // uniform for the workgroup: nothing was staged yet
  struct Geo { int xs, ys, ye, steps; };
  auto geometry = [&](int u) {
    Geo g;
    const int strip = u / nseg, seg = u - strip * nseg;
    g.xs = strip * SWO;
    g.ys = seg * (L - 2);
    g.ye = g.ys + L - 2 < Hc ? g.ys + L - 2 : Hc;
    g.steps = (g.ye - g.ys + 2 + IH - 1) / IH;
    return g;
  };

  // ---- resident weights and biases.  What goes to LDS is loaded here and written there by publish_resident(), which every role
  // calls once it has asked for its first halos (and before its first barrier): written at once, each of these small pieces cost
  // the kernel a memory round trip of its own in front of everything else. ----
#if !BIAS2REG && HAS_BIAS
  const _Float16 stagedBias2 = BIAS2[tid & 31];
#endif
#if W1REG
#if HAS_BIAS1
  const _Float16 stagedBias1 = BIAS1[tid & 31];
#endif
  static_assert(PW > 0, "weights in registers: computing waves that hold nothing else");
  FirstWeights w1;
  if (wv < WAVES)
    load_first_weights(w1, FILT1, lane);
#else
  constexpr int VPR1 = CPAD / 8, NW1 = NTAPS * 32 * VPR1, PER1 = (NW1 + NT - 1) / NT; // global [tap][32 rows][CPAD] -> LDS rows of CPADP
  uint4v stagedW1[PER1];
#pragma unroll
  for (int k = 0; k < PER1; ++k) {
    const int i = tid + k * NT;
    stagedW1[k] = ld16(FILT1 + (size_t)(i < NW1 ? i : NW1 - 1) * 8);
  }
#endif
  auto publish_resident = [&]() {
#if !BIAS2REG && HAS_BIAS
    if (tid < 32) sBias2[tid] = (float)stagedBias2;
#endif
#if W1REG
#if HAS_BIAS1
    if (tid < 32) sBias1[tid] = (float)stagedBias1;
#endif
#else
#pragma unroll
    for (int k = 0; k < PER1; ++k) {
      const int i = tid + k * NT;
      const int row = i / VPR1, v = i - row * VPR1;
      if (i < NW1)
        *reinterpret_cast<uint4v *>(sW1 + row * CPADP + v * 8) = stagedW1[k];
    }
#endif
  };
  SecondWeights w2;
  if (!C2STAGE || wv >= WAVES) // (with C2STAGE the computing waves never touch them: dead there, no registers)
    load_second_weights(w2, FILT2, lane);
#if !W1REG
#if HAS_BIAS1
  const float16v bias1 = load_bias_regs(BIAS1, true, lane);
#else
  const float16v bias1 = load_bias_regs(nullptr, false, lane);
#endif
#endif
#if BIAS2REG && HAS_BIAS
  const float16v bias2 = load_bias_regs(BIAS2, true, lane);
#else
  const float16v bias2 = load_bias_regs(nullptr, false, lane); // (zeros, or unused)
#endif

  // ---- the fetch cursor walks the same sequence of (unit, step, channel chunk) as the compute cursor, two chunks ahead.
  // Every unit has one step more than it has rows for: the last one only drains the second convolution, its loads are
  // aimed past the end of the sources (they return zeros without touching memory) and its matrix work is skipped. ----
  Geo fg = geometry(unit);
  int funit = unit, fk = 0, fchunk = 0;
  typedef Halo<(PW > 0 ? PW : WAVES) * 64> H;
  H::Map map;
  H::Src fsrc;
  H::map_init(map, PW > 0 ? tid - WAVES * 64 : tid); // (computing waves of the specialised variant never use it)
#if SRC_UNIFORM
  H::Cols fcols; // the column part of the offsets: one strip, one set of columns
  H::cols_init(fcols, PW > 0 ? tid - WAVES * 64 : tid, fg.xs - 1, pc);
#endif
  auto aim = [&]() { // source offsets of the fetch cursor's step; a drain step (or none) reads nothing
    const bool real = funit < units && fk < fg.steps;
#if SRC_UNIFORM
    H::rows_init(fsrc, fcols, map, real ? fg.ys - 1 + fk * IH : -0x10000, pc);
#else
    H::src_init(fsrc, map, real ? fg.ys - 1 + fk * IH : -0x10000, fg.xs - 1, pc);
#endif
  };
  // Past the last step the cursor stays where it is: the loads are issued all the same (and never used), so that the
  // number of loads in flight is the same on every path through the loop.
  auto issue = [&](H::Regs &regs) {
    if (fchunk == 0)
      aim(); // (here rather than after the cursor has moved: the offsets then live in registers only until the loads are out)
    H::fetch_step(srcs, regs, map, fsrc, fchunk);
    if (++fchunk == NCHUNK) {
      fchunk = 0;
      if (funit < units && ++fk > fg.steps) {
        fk = 0;
        funit += GRID;
        if (funit < units) {
          fg = geometry(funit);
#if SRC_UNIFORM
          H::cols_init(fcols, PW > 0 ? tid - WAVES * 64 : tid, fg.xs - 1, pc);
#endif
        }
      }
    }
  };
#if DLDS
  // the halo of the fetch cursor's chunk straight into `dst`, and the cursor one chunk on (as issue() above)
  auto dma = [&](_Float16 *dst) {
    if (fchunk == 0)
      aim();
    H::dma_step(srcs, dst, map, fsrc, fchunk, wv - WAVES);
    if (++fchunk == NCHUNK) {
      fchunk = 0;
      if (funit < units && ++fk > fg.steps) {
        fk = 0;
        funit += GRID;
        if (funit < units) {
          fg = geometry(funit);
          H::cols_init(fcols, tid - WAVES * 64, fg.xs - 1, pc);
        }
      }
    }
  };
#endif

  Geo g = geometry(unit);
  int k = 0, cchunk = 0, buf = 0;
  int wslot = 0; // ring row that takes the first `mid` row of step k
  Acc acc;       // the first convolution's accumulators during a step's chunks, the second's in between
  // outputs of step k - 1, in the first chunk of step k: its `mid` rows and the two before them are in the ring.
  // rw: the wave whose rows these are
  // (the store of a step's outputs can be put off: its arguments)
  struct PairStore { Packed pk; int ob, xs, ylo, yhi, rw; bool valid; };
  auto second_compute = [&](int rw, PairStore &ps) {
    ps.valid = cchunk == 0 && unit < units && k > 0; // (unit >= units: a spare chunk behind the last step)
    if (ps.valid) {
#if !BIAS2REG
      init_acc(acc, sBias2, lane);
#endif
      int rslot = wslot - IH - 2;
      rslot = rslot < 0 ? rslot + NS : rslot;
      rslot = rslot < 0 ? rslot + NS : rslot;
      mma_mid(sMid, rslot, w2, acc, bias2, rw, lane);
#if TAPM
      pack_tapm(acc, ps.pk);
#else
      pack_tile(acc, ps.pk);
#endif
      ps.ob = g.ys + (k - 1) * IH - 2; ps.xs = g.xs; ps.ylo = g.ys; ps.yhi = g.ye; ps.rw = rw;
    }
  };
  auto second_store = [&](const PairStore &ps) {
    if (ps.valid)
      store_pair(ps.pk, out, ps.ob, ps.xs, ps.ylo, ps.yhi, ps.rw, lane, pc);
  };
  auto second = [&](int rw) {
    PairStore ps;
    second_compute(rw, ps);
    second_store(ps);
  };
  // what the computing side does in one chunk, after the barrier that published the chunk's halo
  auto compute = [&]() {
#if !C2STAGE
    second(wv);
#endif
#if W1REG
    if (cchunk == 0)
      init_acc_first(acc, sBias1, lane);
#endif
  };
  // moves the cursor (unit, k, cchunk, wslot) one chunk on
  auto advance = [&]() {
    if (++cchunk == NCHUNK) {
      cchunk = 0;
      wslot += IH;
      wslot = wslot >= NS ? wslot - NS : wslot;
      if (unit < units && ++k > g.steps) { // the drain step is done: next unit
        k = 0;
        wslot = 0;
        unit += GRID;
        if (unit < units)
          g = geometry(unit);
      }
    }
  };
  auto multiply = [&]() {
    const bool alive = unit < units;
    const bool real = alive && k < g.steps;
    if (real) {
#if W1REG
      mma_first_reg_chunk<0>(cchunk, sIn[buf], w1, acc, wv, lane);
#else
      if (cchunk == 0)
        mma_first<(NCHUNK > 1 ? CK : TAIL), CPADP, true>(sIn[buf], sW1, 0, acc, bias1, wv, lane);
      else if (TAIL == CK || cchunk < NCHUNK - 1)
        mma_first<CK, CPADP, false>(sIn[buf], sW1, cchunk * CK, acc, bias1, wv, lane);
      else
        mma_first<TAIL, CPADP, false>(sIn[buf], sW1, cchunk * CK, acc, bias1, wv, lane);
#endif
    }
    buf = buf == NBUF - 1 ? 0 : buf + 1;
    if (real && cchunk == NCHUNK - 1)
      store_mid(acc, sMid, wslot, g.ys - 1 + k * IH, g.xs - 1, Hc, Wc, wv, lane);
    advance();
  };
#if PW == 0
  auto step = [&](H::Regs &regs) {
    H::commit_step(regs, sIn[buf], map, cchunk);
    // One barrier per chunk: buffer `buf` was last read two chunks ago, and every wave has passed the barrier of the
    // chunk in between since then.  The first barrier of a step also publishes the `mid` rows the previous step wrote.
    DNX_SYNC();
    compute();
    issue(regs); // refill this register set: the chunk after next
    multiply();
  };
  H::Regs st0, st1;
  issue(st0);
  __builtin_amdgcn_sched_barrier(0); // keep the two sets in issue order: the waits count loads in flight
  issue(st1);
  __builtin_amdgcn_sched_barrier(0);
  publish_resident();
  // The loop always runs two chunks, so that it has one entry and one back edge with the same loads in flight on both.
  // When the last step ends after the first of them, the second is a spare: it multiplies nothing and stores nothing.
  do {
    step(st0);
    step(st1);
  } while (unit < units);
#else
  // chunks this workgroup runs: both roles execute exactly one barrier per chunk
  int chunks = 0;
  for (int u = unit; u < units; u += GRID)
    chunks += (geometry(u).steps + 1) * NCHUNK;
  if (wv >= WAVES) {
#if DLDS
    // ---- staging waves, halos straight into LDS: chunk c + 1's loads are issued right after the barrier that starts chunk c
    // (all waves have left sIn[(c + 1) & 1] by then) and have to land before the barrier that starts chunk c + 1.  With
    // C2STAGE the second convolution's outputs are stored one chunk late, in front of the next loads: the wait for those
    // loads then never waits for stores that have only just been issued. ----
    dma(sIn[0]); // chunk 0
#if NBUF == 3
    dma(sIn[1]); // chunk 1
#endif
    publish_resident();
    H::dma_wait();
#if C2STAGE
    PairStore pend;
    pend.valid = false;
#endif
    int nb = NBUF - 1; // buffer of the chunk whose loads are issued next
    for (int c = 0; c < chunks; ++c) {
      DNX_SYNC(); // chunk c starts: its halo is complete, the buffer chunk c - 1 used is free
#if C2STAGE
      second_store(pend);
#endif
      // (past the last chunk the loads are issued all the same, aimed outside the image: the wait below counts them)
      dma(sIn[nb]);
      nb = nb == NBUF - 1 ? 0 : nb + 1;
#if C2STAGE
      __builtin_amdgcn_s_setprio(1);
      second_compute(wv - WAVES, pend);
      __builtin_amdgcn_s_setprio(0);
      advance();
#endif
#if NBUF == 3
      // The next chunk's halo was requested one chunk ago: everything but the loads just issued has to have landed.  Loads and
      // stores complete in the order they were issued, and this interval's stores precede its loads.
      H::dma_wait_all_but_last();
#else
      H::dma_wait();
#endif
    }
#if C2STAGE
    second_store(pend);
#endif
#else
    // ---- staging waves: chunk c's halo is written to sIn[c & 1] during chunk c - 1 ----
    H::Regs st0, st1;
    int commitChunk = 0; // channel chunk of the halo being written
    auto commit = [&](H::Regs &regs, int c) {
      H::commit_step(regs, sIn[c & 1], map, commitChunk);
      if (++commitChunk == NCHUNK)
        commitChunk = 0;
    };
    issue(st0);   // chunk 0
    __builtin_amdgcn_sched_barrier(0);
    issue(st1);   // chunk 1
    __builtin_amdgcn_sched_barrier(0);
    publish_resident();
    commit(st0, 0);
    issue(st0);   // chunk 2
    // with C2STAGE: the second convolution of the step the cursor (unit, k, ...) has just left, for the rows of
    // computing wave wv - WAVES, after the chunk's memory work is under way
    auto rest = [&]() {
#if C2STAGE
      // (a raised wave priority for this part: its dozen matrix instructions compete with the computing wave's stream
      // for the pipe, and the step ends when this wave is done: 2 - 3 % per launch)
      __builtin_amdgcn_s_setprio(1);
      second(wv - WAVES);
      __builtin_amdgcn_s_setprio(0);
      advance();
#endif
    };
    for (int c = 0; c < chunks; c += 2) {
      DNX_SYNC(); // chunk c starts: sIn[c & 1] is complete, the other buffer is free
      if (c + 1 < chunks) {
        commit(st1, c + 1);
        issue(st1); // chunk c + 3
      }
      rest();
      if (c + 1 >= chunks)
        break;
      DNX_SYNC(); // chunk c + 1 starts
      if (c + 2 < chunks) {
        commit(st0, c + 2);
        issue(st0); // chunk c + 4
      }
      rest();
    }
#endif
  } else {
    // ---- computing waves ----
    publish_resident();
    for (int c = 0; c < chunks; ++c) {
      DNX_SYNC();
      compute();
      multiply();
    }
  }
#endif
}
