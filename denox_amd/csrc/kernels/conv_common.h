// Shared pieces of the conv3x3 MFMA kernels: the compile-time interface, the
// source loader (concat / upsample / replicate-pad folded into the addressing)
// and the epilogue (bias, activation, rounding, 2x2 max pool or crop, store).
//
//   out[y,x,k] = act(bias[k] + sum_{r,s,c} src[y*SY+r-PY, x*SX+s-PX, c] * W[k,c,r,s])   (zero outside the image; KR x KS taps)
//   src[y,x,c] = c < CA ? A'[y,x,c] : B'[y,x,c-CA]
//   A' = UPA ? A[y/2, x/2] : (PADA ? A[clamp(y-PAD_T), clamp(x-PAD_L)] : A[y,x]),   B' likewise with PADB
//
// Definitions every variant is compiled with:
//   CA, CB      channels of source A / source B (CB = 0: single source)
//   UPA         1: A is stored at half resolution and read at (y>>1, x>>1)
//   PADA, PADB  1: that source is stored un-padded (SRC_H x SRC_W) and read through a
//               replicate pad with offsets (PAD_T, PAD_L); IN_H x IN_W is the padded extent
//   KOUT        output channels;  KT: output channels per workgroup (multiple of 32)
//   ACT         0 none, 1 ReLU, 2 LeakyReLU(ALPHA);   HAS_BIAS 0/1
//   POOL        1: store max over 2x2 output windows at (y/2, x/2) only
//   CROP        1: store only rows/cols inside [CROP_T, CROP_T+OUT_H) x [CROP_L, CROP_L+OUT_W)
//   OPITCH      channels between consecutive output pixels (default KOUT).  Larger when the output is the channel
//               range of a wider tensor -- a concat whose sources are written in place; OUT then points at the
//               first channel of the range.  OVEC 0: that range is not 16-byte aligned, store element by element
//   WAVES, RPW  computing waves per workgroup, output rows per wave -> tile = (WAVES*RPW) x 32 pixels
//   CK          input channels staged in LDS per step (multiple of 16)
//   LAYIN       1: the sources are stored channel-block-major (CHWC8: [C/8][H][W][8], the reference's second activation layout,
//               common/src/denox/memory/tensor/ActivationLayout.hpp:37-66) instead of pixel-major (HWC); needs CA % 8 == 0,
//               CB % 8 == 0 and every LDS step inside one source
//   LAYOUT_OUT  1: the result is stored CHWC8; needs KOUT % 8 == 0 and OPITCH == KOUT
//
// Mapping onto v_mfma_f32_32x32x16_f16: the weights are the M operand (32 output
// channels per block, rows permuted so that each lane ends up with 16 consecutive
// channels), 32 consecutive pixels of one image row are the N operand, and the
// reduction runs over (tap, input channel) in steps of 16 channels.
#include "prelude.h"
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef unsigned short ushort_t;

#ifndef ALPHA
#define ALPHA 0.0f
#endif
#ifndef PADA
#define PADA 0
#endif
#ifndef PADB
#define PADB 0
#endif
#ifndef CROP
#define CROP 0
#endif
#ifndef OPITCH
#define OPITCH KOUT
#endif
#ifndef OVEC
#define OVEC 1
#endif
#ifndef LAYIN
#define LAYIN 0
#endif
#ifndef LAYOUT_OUT
#define LAYOUT_OUT 0
#endif

// Matrix-core shape: MF = 32 -> v_mfma_f32_32x32x16_f16 (32 output channels x 32 pixels per block, 16 input
// channels per step), MF = 16 -> v_mfma_f32_16x16x32_f16 (16 x 16 per block, 32 input channels per step; XB blocks
// side by side in x).  The 16-wide shape wastes less on output-channel counts like 48, 80, 112 or 3 and makes
// smaller tiles for low-resolution layers; the 32-wide shape pads input channels less (73 -> 80 instead of 96).
// Filter extent KR x KS (odd; the convolution keeps the image extent: zero padding (KR-1)/2, (KS-1)/2, stride 1).
#ifndef KR
#define KR 3
#endif
#ifndef KS
#define KS 3
#endif
#define NTAPS (KR * KS)
// Zero padding PY x PX (default: the image extent is kept for odd filters) and stride SY x SX (default 1):
// out[y, x] = sum in[y * SY + r - PY, x * SX + s - PX] * w[r, s]; output extent (IN + 2 P - K) / S + 1
// (direct_conv.comp:209-212,304-311 of the reference take STRIDE_* and PADDING_* the same way).
#ifndef PY
#define PY ((KR - 1) / 2)
#endif
#ifndef PX
#define PX ((KS - 1) / 2)
#endif
#ifndef SY
#define SY 1
#endif
#ifndef SX
#define SX 1
#endif
// extent of the convolution's own output (before POOL / CROP); folds to IN_W / IN_H for the default padding and stride
#define CONV_OUT_W(pc) (((pc).IN_W + 2u * PX - KS) / SX + 1u)
#define CONV_OUT_H(pc) (((pc).IN_H + 2u * PY - KR) / SY + 1u)
#ifndef MF
#define MF 32
#endif
#ifndef XB
#define XB 1
#endif
#define KSTEP (MF == 32 ? 16 : 32) // input channels per matrix instruction
#define CIN (CA + CB)
#define CPAD (((CIN) + KSTEP - 1) / KSTEP * KSTEP)
#define NCHUNK ((CPAD + CK - 1) / CK)
#define TAIL (CPAD - (NCHUNK - 1) * CK)
#define TW (MF == 32 ? 32 : 16 * XB)
#define TH (WAVES * RPW)
#define HALO_W ((TW - 1) * SX + KS)
#define HALO_H ((TH - 1) * SY + KR)
#define PXROWS ((RPW - 1) * SY + KR) // halo rows one wave's RPW output rows read
#define HALO_PIX (HALO_W * HALO_H)
#define CKP (CK + 8)
#define KB (KT / MF)
#ifndef LOAD_AUX
#define LOAD_AUX 0 // cache policy bits of the halo loads through buffer resources (bit 1: non-temporal)
#endif
#ifndef STORE_AUX
#define STORE_AUX 0 // cache policy bits of the output stores (bit 1: non-temporal)
#endif
#ifndef PP
#define PP 0 // 1: two-phase schedule of the weight-stationary kernel (wave groups alternate matrix work and everything else)
#endif
#ifndef PW
#define PW 0 // extra waves that only stage halos (weight-stationary kernel)
#endif
#define NT ((WAVES + PW) * 64)
#define KOUTP (((KOUT) + MF - 1) / MF * MF)
// DLDS 1: halos go from memory straight into LDS (buffer_load_dwordx4 ... lds, new with gfx950) instead of through registers
// of the staging waves.  The hardware writes the 64 lanes of such a load to 64 consecutive 16-byte slots, so the slot a
// vector lands in is fixed by who loads it: staging thread t's it-th load fills slot t + it * (staging threads).  What each
// lane is free to choose is WHICH vector it loads into its slot.  The staged halo stays pixel-major without padding (G = CK / 8
// slots per pixel), and slot P * G + r of pixel P receives channel group (r - P / (8 / G)) mod G: a rotation that puts the same
// channel group of 8 consecutive pixels into 8 different 16-byte bank groups, so the matrix loop's fragment reads stay free of
// bank conflicts, while the G lanes of a pixel still read one contiguous piece of memory.  Needs staging waves, whole
// 8-channel groups and every LDS step inside one source.
#ifndef DLDS
#define DLDS 0
#endif
// HROT 1: the same rotated, unpadded halo layout with the halo still staged through registers (the staging threads write each
// vector to its rotated slot themselves).  A pixel then takes CK / 8 slots instead of CK / 8 + 1: halos of 32 channels fit
// where the padded form allowed 16, which halves the barriers per tile.
#ifndef HROT
#define HROT 0
#endif
#define HROTL (DLDS || HROT)                                               // the rotated layout is in use
#define DG (CK / 8)                                                        // 16-byte slots per staged pixel
#define DD (8 / DG)                                                        // pixels that share a 128-byte row of LDS
#if DLDS
#define HALO_SLOTS (((HALO_PIX * DG + PW * 64 - 1) / (PW * 64)) * (PW * 64)) // whole loads of all staging threads
#define HALO_ELEMS (HALO_SLOTS * 8)
#elif HROT
#define HALO_ELEMS (HALO_PIX * DG * 8)
#else
#define HALO_ELEMS (HALO_PIX * CKP)
#endif
// SWP 1: the matrix loop reads the fragments of the next group of matrix instructions while it issues the current group's,
// one LDS read behind each instruction, in an order that scheduling barriers pin (32 x 32 x 16 shape).
#ifndef SWP
#define SWP 0
#endif

struct PushConstants {
  unsigned int IN_W;
  unsigned int IN_H;
#if PADA || PADB
  unsigned int SRC_W, SRC_H, PAD_L, PAD_T;
#endif
#if CROP
  unsigned int OUT_W, OUT_H, CROP_L, CROP_T;
#endif
  // bit 0: walk the tiles in reverse order.  Consecutive layers alternate, so a layer starts
  // where its producer just finished and finds that part of its input still in the
  // memory-side cache.
  unsigned int FLAGS;
};

__device__ DNX_INLINE uint4v ld16(const _Float16 *p) {
  return *reinterpret_cast<const uint4v *>(p);
}

__device__ DNX_INLINE int clampi(int v, int lo, int hi) { return v < lo ? lo : (v > hi ? hi : v); }

// An LDS address the optimiser must take as it is.  A fragment read is `base that changes per step + per-lane part +
// compile-time constant`; left alone, the compiler sums the per-lane part and each constant once, outside the step
// loop (they do not change there), keeps 20-odd registers of such sums and adds the step's base to every one of them
// again in every step -- one vector add per LDS read, in a loop whose matrix instructions wait for exactly those
// slots.  With the step's base + per-lane part made opaque, the constants stay what the LDS instructions have a
// field for: immediate offsets.
typedef __attribute__((address_space(3))) const _Float16 lds_half_t;
typedef __attribute__((address_space(3))) const half8 lds_half8_t;
typedef __attribute__((address_space(3))) void lds_void_t;
__device__ DNX_INLINE lds_half_t *lds_opaque(const _Float16 *p) {
  unsigned a = (unsigned)(size_t)(lds_half_t *)p;
  __asm__ volatile("" : "+v"(a));
  return (lds_half_t *)(size_t)a;
}

// Element offsets of full-resolution pixel (gy, gx) inside A and B.
__device__ DNX_INLINE void src_offsets(int gy, int gx, const PushConstants &pc, size_t &pa, size_t &pb) {
  const unsigned W = pc.IN_W;
#if PADA
  const int ay = clampi(gy - (int)pc.PAD_T, 0, (int)pc.SRC_H - 1), ax = clampi(gx - (int)pc.PAD_L, 0, (int)pc.SRC_W - 1);
  const unsigned WA = pc.SRC_W;
#else
  const int ay = UPA ? (gy >> 1) : gy, ax = UPA ? (gx >> 1) : gx;
  const unsigned WA = UPA ? (W >> 1) : W;
#endif
#if PADB
  const int by = clampi(gy - (int)pc.PAD_T, 0, (int)pc.SRC_H - 1), bx = clampi(gx - (int)pc.PAD_L, 0, (int)pc.SRC_W - 1);
  const unsigned WB = pc.SRC_W;
#else
  const int by = gy, bx = gx;
  const unsigned WB = W;
#endif
  // element offset of the pixel's first channel; in the block-major layout a pixel of one 8-channel plane is 8 elements
  pa = ((size_t)ay * WA + (size_t)ax) * (LAYIN ? 8 : CA);
  pb = ((size_t)by * WB + (size_t)bx) * (LAYIN ? 8 : (CB > 0 ? CB : 1));
}

typedef uint4v __attribute__((aligned(2))) uint4v_u; // global memory is accessed in unaligned mode

// 128-bit value shifted right by K halves (zero fill), K a compile-time constant.
template <int K>
__device__ DNX_INLINE uint4v shr_halves(uint4v v) {
  constexpr int Q = (K * 16) / 32, Bt = (K * 16) % 32;
  uint4v r;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const unsigned lo = (i + Q < 4) ? v[(i + Q) & 3] : 0u;
    const unsigned hi = (i + Q + 1 < 4) ? v[(i + Q + 1) & 3] : 0u;
    r[i] = Bt == 0 ? lo : ((lo >> Bt) | (hi << (32 - Bt)));
  }
  return r;
}

// Channels [cc, cc+8) of one pixel of a C-channel source (cc a multiple of 8, cc < C);
// channels past C read as zero.  Any C >= 8 is read with one 16-byte load: the last,
// partial vector is fetched so that it ends at the pixel's last channel and shifted down,
// which keeps every access inside the tensor.
template <int C>
__device__ DNX_INLINE uint4v load_pixel8(const _Float16 *__restrict__ src, size_t pix, int cc) {
  if (C % 8 == 0) {
    return ld16(src + pix + cc);
  } else if (C >= 8) {
    const bool full = cc + 8 <= C;
    const uint4v v = *reinterpret_cast<const uint4v_u *>(src + pix + (full ? cc : C - 8));
    return full ? v : shr_halves<8 - C % 8>(v);
  } else {
    half8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e)
      v[e] = (cc + e < C) ? src[pix + cc + e] : (_Float16)0.0f;
    return __builtin_bit_cast(uint4v, v);
  }
}

// Eight consecutive channels [cc, cc+8) of the concatenated source at the pixel whose
// element offsets are (pa, pb); channels past CIN read as zero.
__device__ DNX_INLINE uint4v
load_src8(const _Float16 *__restrict__ A, const _Float16 *__restrict__ B, size_t pa, size_t pb, int cc) {
  if (CA % 8 == 0 || CB == 0) {
    // every 8-vector lies in one source
    if (cc < CA)
      return load_pixel8<CA>(A, pa, cc);
    if (CB > 0 && cc < CIN)
      return load_pixel8<(CB > 0 ? CB : 8)>(B, pb, cc - CA);
    return uint4v{0u, 0u, 0u, 0u};
  } else {
    // a vector may straddle the A | B boundary: assemble it element by element
    half8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int ch = cc + e;
      _Float16 x = (_Float16)0.0f;
      if (ch < CA)
        x = A[pa + ch];
      else if (ch < CIN)
        x = B[pb + (ch - CA)];
      v[e] = x;
    }
    return __builtin_bit_cast(uint4v, v);
  }
}

// When every 8-channel vector lies in one source and no source is narrower than 8 channels, a vector is one
// 16-byte load whatever the lane: the address is selected (never branched on) and the fix-up of a partial last
// vector and the zero fill happen when the value is written to LDS.  Every lane then issues the same number of
// loads in every step, so the compiler can wait for exactly the loads a step needs and leave younger ones in flight.
#define VEC_SRC ((CA % 8 == 0 || CB == 0) && CA >= 8 && (CB == 0 || CB >= 8))

__device__ DNX_INLINE const _Float16 *
src8_ptr(const _Float16 *__restrict__ A, const _Float16 *__restrict__ B, size_t pa, size_t pb, int cc) {
  const int rel = cc - CA;
  const _Float16 *qa = A + pa + ((CA % 8 == 0 || cc + 8 <= CA) ? cc : CA - 8);
  const _Float16 *qb = B + pb + ((CB % 8 == 0 || rel + 8 <= CB) ? rel : CB - 8);
  return (CB > 0 && cc >= CA) ? qb : qa;
}

__device__ DNX_INLINE uint4v src8_fix(uint4v v, int cc) {
  if (CA % 8 != 0) { // single source: its last vector was loaded so that it ends at the last channel
    const uint4v sh = shr_halves<(8 - CA % 8) % 8>(v);
    const bool part = cc < CA && cc + 8 > CA;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = part ? sh[i] : v[i];
  }
  if (CB > 0 && CB % 8 != 0) {
    const uint4v sh = shr_halves<(8 - CB % 8) % 8>(v);
    const bool part = cc >= CA && cc - CA + 8 > CB;
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = part ? sh[i] : v[i];
  }
  return v;
}

template <bool WIDE> struct MaskType { typedef unsigned int type; };
template <> struct MaskType<true> { typedef unsigned long long type; };

// When, in addition, every step of CK channels lies in one source, the step's loads go through that source's buffer
// resource with 32-bit byte offsets: one add per load, and a lane with nothing to load (halo pixel outside the image,
// padding channel) passes an offset past the end and gets zeros from the hardware.
#define SRC_UNIFORM (VEC_SRC && (CB == 0 || CA % CK == 0))
static_assert(!LAYIN || (SRC_UNIFORM && CA % 8 == 0 && CB % 8 == 0), "block-major sources: whole 8-channel groups, every LDS step inside one source");
#define NO_LOAD 0xFFFFF000u // past the end of every tensor this code accepts; stays past it when a channel offset is added
static_assert(2 * CPAD + 16 < 4096, "channel offsets must not wrap the no-access offset");

struct Sources {
  const _Float16 *A, *B;
  unsigned bytesA, bytesB;
  unsigned planeA, planeB; // bytes of one 8-channel plane (block-major layout)
};

__device__ DNX_INLINE Sources make_sources(const _Float16 *A, const _Float16 *B, const PushConstants &pc) {
  Sources s;
  s.A = A;
  s.B = B;
#if PADA
  const unsigned pixA = pc.SRC_W * pc.SRC_H;
#else
  const unsigned pixA = UPA ? (pc.IN_W >> 1) * (pc.IN_H >> 1) : pc.IN_W * pc.IN_H;
#endif
#if PADB
  const unsigned pixB = pc.SRC_W * pc.SRC_H;
#else
  const unsigned pixB = pc.IN_W * pc.IN_H;
#endif
  s.bytesA = pixA * (unsigned)CA * 2u;
  s.bytesB = pixB * (unsigned)CB * 2u;
  s.planeA = pixA * 16u;
  s.planeB = pixB * 16u;
  return s;
}

// ---- halo staging ---------------------------------------------------------------------
// The (TH+2) x 34 pixel halo of one reduction step is moved by NTH threads, 16 bytes
// (8 channels) per access.  Vector i = t + it*NTH covers pixel i / (CK/8), channel group
// i % (CK/8) (block-major sources: channel group i / HALO_PIX, pixel i % HALO_PIX).  What does not change between steps is computed once: the LDS slot of each
// of a thread's vectors (HaloMap, per kernel) and the element offsets of its pixels in
// the sources (HaloSrc, per tile).
#define VPPK (CK / 8)

template <int NTH>
struct Halo {
  static constexpr int NV = (HALO_PIX * VPPK + NTH - 1) / NTH;
  struct Map {
    int lds[NV]; // element offset inside the staged halo, -1: no such vector
    int hy[NV], hx[NV], v8[NV];
  };
  struct Src {
    // offsets of the pixel in A and B.  SRC_UNIFORM: in bytes, NO_LOAD outside the image; else in elements,
    // pa < 0 outside the image (reads as zero)
    int pa[NV], pb[NV];
  };
  static_assert(NV <= 64, "halo share of one thread too large");
  typedef typename MaskType<(NV > 32)>::type Mask;
  struct Regs {
    uint4v v[NV];
    Mask ok; // bit it: vector it holds image data (clear: it reads as zero)
  };

  static __device__ DNX_INLINE void map_init(Map &m, int t) {
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int i = t + it * NTH;
#if LAYIN && !DLDS
      // block-major sources: consecutive lanes take consecutive pixels of one 8-channel plane (16 consecutive bytes each)
      const int v = i / HALO_PIX;
      const int pix = i - v * HALO_PIX;
#else
      const int pix = i / VPPK;
      const int v = i - pix * VPPK;
#endif
      m.hy[it] = pix / HALO_W;
      m.hx[it] = pix - m.hy[it] * HALO_W;
#if DLDS
      // slot i = pix * DG + v is where the hardware puts this lane's load; the channel group that belongs there
      m.v8[it] = ((v - pix / DD) & (DG - 1)) * 8;
      m.lds[it] = i < HALO_PIX * VPPK ? i * 8 : -1;
#elif HROT
      m.v8[it] = v * 8;
      m.lds[it] = i < HALO_PIX * VPPK ? (pix * DG + ((v + pix / DD) & (DG - 1))) * 8 : -1;
#else
      m.v8[it] = v * 8;
      m.lds[it] = i < HALO_PIX * VPPK ? pix * CKP + v * 8 : -1;
#endif
    }
  }

  static __device__ DNX_INLINE void src_init(Src &s, const Map &m, int y0, int x0, const PushConstants &pc) {
#if SRC_UNIFORM
    // Byte offsets below 4 GiB (a buffer resource addresses no more), in 32-bit arithmetic and without a branch: the
    // coordinates of a pixel outside the image are clamped (or shifted) like any other and the result replaced.
    const unsigned W = pc.IN_W;
    constexpr unsigned pixA = LAYIN ? 16 : CA * 2, pixB = LAYIN ? 16 : (CB > 0 ? CB : 1) * 2;
#if PADA
    const unsigned rowA = pc.SRC_W * pixA;
#else
    const unsigned rowA = (UPA ? (W >> 1) : W) * pixA;
#endif
#if PADB
    const unsigned rowB = pc.SRC_W * pixB;
#else
    const unsigned rowB = W * pixB;
#endif
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int gy = y0 * SY + m.hy[it] - PY; // (y0, x0): the tile's first output pixel
      const int gx = x0 * SX + m.hx[it] - PX;
      const bool inside = m.lds[it] >= 0 && gy >= 0 && gy < (int)pc.IN_H && gx >= 0 && gx < (int)pc.IN_W;
#if PADA
      const int ay = clampi(gy - (int)pc.PAD_T, 0, (int)pc.SRC_H - 1), ax = clampi(gx - (int)pc.PAD_L, 0, (int)pc.SRC_W - 1);
#else
      const int ay = UPA ? (gy >> 1) : gy, ax = UPA ? (gx >> 1) : gx;
#endif
#if PADB
      const int by = clampi(gy - (int)pc.PAD_T, 0, (int)pc.SRC_H - 1), bx = clampi(gx - (int)pc.PAD_L, 0, (int)pc.SRC_W - 1);
#else
      const int by = gy, bx = gx;
#endif
      s.pa[it] = inside ? (int)((unsigned)ay * rowA + (unsigned)ax * pixA) : (int)NO_LOAD;
      s.pb[it] = inside ? (int)((unsigned)by * rowB + (unsigned)bx * pixB) : (int)NO_LOAD;
    }
#else
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int gy = y0 * SY + m.hy[it] - PY; // (y0, x0): the tile's first output pixel
      const int gx = x0 * SX + m.hx[it] - PX;
      size_t pa = 0, pb = 0;
      const bool inside = m.lds[it] >= 0 && gy >= 0 && gy < (int)pc.IN_H && gx >= 0 && gx < (int)pc.IN_W;
      if (inside)
        src_offsets(gy, gx, pc, pa, pb);
      s.pa[it] = inside ? (int)pa : -1;
      s.pb[it] = (int)pb;
    }
#endif
  }

#if SRC_UNIFORM
  // src_init in two parts, for a kernel that walks down a strip of tiles: the column of a vector's pixel, and with it
  // everything src_init derives from gx, stays the same from tile to tile.  cols_init computes that part once per strip
  // (byte offset of the column inside a source row, -1: no such vector or a column outside the image); rows_init adds
  // the row: half a dozen 32-bit instructions per vector and no branch, where src_init takes some twenty with 64-bit
  // multiplies -- instructions that a staging wave has to get issued between the matrix instructions of the
  // computing wave on its SIMD.  Offsets are bytes below 4 GiB (the buffer resources address no more).
  struct Cols {
    int ca[NV], cb[NV];
  };
  // (t: the thread's index among the NTH, as for map_init; the halo column is derived again rather than kept in the
  // map, whose hx then occupies no registers in a kernel that never calls src_init)
  static __device__ DNX_INLINE void cols_init(Cols &c, int t, int x0, const PushConstants &pc) {
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int i = t + it * NTH;
#if LAYIN && !DLDS
      const int pix = i % HALO_PIX;
#else
      const int pix = i / VPPK;
#endif
      const int gx = x0 * SX + pix % HALO_W - PX;
      const bool inside = i < HALO_PIX * VPPK && gx >= 0 && gx < (int)pc.IN_W;
#if PADA
      const int ax = clampi(gx - (int)pc.PAD_L, 0, (int)pc.SRC_W - 1);
#else
      const int ax = UPA ? (gx >> 1) : gx;
#endif
#if PADB
      const int bx = clampi(gx - (int)pc.PAD_L, 0, (int)pc.SRC_W - 1);
#else
      const int bx = gx;
#endif
      c.ca[it] = inside ? ax * (LAYIN ? 16 : CA * 2) : -1;
      c.cb[it] = inside ? bx * (LAYIN ? 16 : (CB > 0 ? CB : 1) * 2) : -1;
    }
  }
  static __device__ DNX_INLINE void rows_init(Src &s, const Cols &c, const Map &m, int y0, const PushConstants &pc) {
    const unsigned W = pc.IN_W;
#if PADA
    const unsigned rowA = pc.SRC_W * (unsigned)(LAYIN ? 16 : CA * 2);
#else
    const unsigned rowA = (UPA ? (W >> 1) : W) * (unsigned)(LAYIN ? 16 : CA * 2);
#endif
#if PADB
    const unsigned rowB = pc.SRC_W * (unsigned)(LAYIN ? 16 : (CB > 0 ? CB : 1) * 2);
#else
    const unsigned rowB = W * (unsigned)(LAYIN ? 16 : (CB > 0 ? CB : 1) * 2);
#endif
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int gy = y0 * SY + m.hy[it] - PY;
      const bool inside = gy >= 0 && gy < (int)pc.IN_H && c.ca[it] >= 0;
#if PADA
      const int ay = clampi(gy - (int)pc.PAD_T, 0, (int)pc.SRC_H - 1);
#else
      const int ay = UPA ? (gy >> 1) : gy;
#endif
#if PADB
      const int by = clampi(gy - (int)pc.PAD_T, 0, (int)pc.SRC_H - 1);
#else
      const int by = gy;
#endif
      s.pa[it] = inside ? (int)((unsigned)ay * rowA + (unsigned)c.ca[it]) : (int)NO_LOAD;
      s.pb[it] = inside ? (int)((unsigned)by * rowB + (unsigned)c.cb[it]) : (int)NO_LOAD;
    }
  }
#endif

  // Issue the loads of the L channels starting at c0 into registers ...
  template <int L>
  static __device__ DNX_INLINE void fetch(const Sources &src, Regs &st, const Map &m, const Src &s, int c0) {
#if SRC_UNIFORM
    st.ok = 0;
    // One stream of load instructions whichever the source (no branch: the waits for these loads are counted),
    // with the source's base, size and channel count selected by scalar conditions.
    const bool fromA = CB == 0 || c0 < CA; // the same for all lanes
    const int cs = fromA ? CA : CB;        // channels of the step's source
    const int cbase = fromA ? 0 : CA;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16 *>(fromA ? src.A : src.B), 0, (int)(fromA ? src.bytesA : src.bytesB), 0x00020000);
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int rel = c0 + m.v8[it] - cbase;
      const int chan = ((CA % 8 == 0 && CB % 8 == 0) || rel + 8 <= cs) ? rel : cs - 8;
      const unsigned pixoff = (unsigned)(fromA ? s.pa[it] : s.pb[it]);
#if LAYIN
      // 8-channel group chan / 8 lives in its own plane; a pixel outside the image must stay outside whatever is added
      unsigned off = pixoff + (unsigned)(chan >> 3) * (fromA ? src.planeA : src.planeB);
      off = pixoff == NO_LOAD ? NO_LOAD : off;
#else
      unsigned off = pixoff + 2u * (unsigned)chan;
#endif
      off = (m.v8[it] < L && rel < cs) ? off : NO_LOAD;
      st.v[it] = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, LOAD_AUX);
    }
#else
    const _Float16 *__restrict__ A = src.A;
    const _Float16 *__restrict__ B = src.B;
    Mask ok = 0;
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int cc = c0 + m.v8[it];
#if VEC_SRC
      const bool act = s.pa[it] >= 0 && m.v8[it] < L && cc < CIN;
      const _Float16 *p = src8_ptr(A, B, (size_t)s.pa[it], (size_t)s.pb[it], cc);
      st.v[it] = *reinterpret_cast<const uint4v_u *>(act ? p : A); // idle lanes re-read the first pixel
      ok |= act ? (Mask)1 << it : (Mask)0;
#else
      uint4v val = {0u, 0u, 0u, 0u};
      if (s.pa[it] >= 0 && m.v8[it] < L)
        val = load_src8(A, B, (size_t)s.pa[it], (size_t)s.pb[it], cc);
      st.v[it] = val;
#endif
    }
    st.ok = ok;
#endif
  }

#if DLDS
  // The same loads with LDS as their destination: thread t's it-th vector lands in slot t + it * NTH of `dst` (64 consecutive
  // slots per wave and load), zeros where fetch() would have produced zeros.  No wave may read `dst` before these loads have
  // been waited for (dma_wait) and a barrier has passed.
  template <int L>
  static __device__ DNX_INLINE void dma(const Sources &src, _Float16 *dst, const Map &m, const Src &s, int c0, int wave) {
    const bool fromA = CB == 0 || c0 < CA; // the same for all lanes
    const int cs = fromA ? CA : CB;
    const int cbase = fromA ? 0 : CA;
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<_Float16 *>(fromA ? src.A : src.B), 0, (int)(fromA ? src.bytesA : src.bytesB), 0x00020000);
#pragma unroll
    for (int it = 0; it < NV; ++it) {
      const int rel = c0 + m.v8[it] - cbase;
      const unsigned pixoff = (unsigned)(fromA ? s.pa[it] : s.pb[it]);
#if LAYIN
      unsigned off = pixoff + (unsigned)(rel >> 3) * (fromA ? src.planeA : src.planeB);
      off = pixoff == NO_LOAD ? NO_LOAD : off;
#else
      unsigned off = pixoff + 2u * (unsigned)rel;
#endif
      off = (m.lds[it] >= 0 && m.v8[it] < L && rel < cs) ? off : NO_LOAD;
      __builtin_amdgcn_raw_ptr_buffer_load_lds(rsrc, (lds_void_t *)(dst + (wave * 64 + it * NTH) * 8), 16, off, 0, 0, LOAD_AUX);
    }
  }
  static __device__ DNX_INLINE void dma_step(const Sources &src, _Float16 *dst, const Map &m, const Src &s, int chunk, int wave) {
    if (TAIL == CK || chunk < NCHUNK - 1)
      dma<CK>(src, dst, m, s, chunk * CK, wave);
    else
      dma<TAIL>(src, dst, m, s, chunk * CK, wave);
  }
  // every load of this wave has arrived (in front of the barrier that publishes the halo)
  static __device__ DNX_INLINE void dma_wait() { __asm__ volatile("s_waitcnt vmcnt(0)" ::: "memory"); }
  // ... every load and store older than the NV loads of the last dma() call has (memory instructions complete in issue order)
  static __device__ DNX_INLINE void dma_wait_all_but_last() {
    static_assert(NV <= 63, "the counter's field");
    __asm__ volatile("s_waitcnt vmcnt(%0)" ::"n"(NV) : "memory");
  }
#endif

  // ... and write them to the staged halo.
  template <int L>
  static __device__ DNX_INLINE void commit(const Regs &st, _Float16 *sIn, const Map &m, int c0) {
#pragma unroll
    for (int it = 0; it < NV; ++it)
      if (m.lds[it] >= 0 && m.v8[it] < L) {
        uint4v v = st.v[it];
#if VEC_SRC
        v = src8_fix(v, c0 + m.v8[it]);
#if !SRC_UNIFORM // (with SRC_UNIFORM the hardware already returned zeros where nothing was to be read)
        const bool keep = ((st.ok >> it) & 1) != 0;
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = keep ? v[i] : 0u;
#endif
#endif
        *reinterpret_cast<uint4v *>(sIn + m.lds[it]) = v;
      }
  }

  // fetch / commit of step `chunk` of a tile, whichever length that step has
  static __device__ DNX_INLINE void
  fetch_step(const Sources &src, Regs &st, const Map &m, const Src &s, int chunk) {
    if (TAIL == CK || chunk < NCHUNK - 1)
      fetch<CK>(src, st, m, s, chunk * CK);
    else
      fetch<TAIL>(src, st, m, s, chunk * CK);
  }
  static __device__ DNX_INLINE void commit_step(const Regs &st, _Float16 *sIn, const Map &m, int chunk) {
    if (TAIL == CK || chunk < NCHUNK - 1)
      commit<CK>(st, sIn, m, chunk * CK);
    else
      commit<TAIL>(st, sIn, m, chunk * CK);
  }
};

#if DLDS
static_assert(SRC_UNIFORM && CA % 8 == 0 && CB % 8 == 0 && PW > 0, "halos straight into LDS: see DLDS above");
#endif
#if HROTL
static_assert(MF == 32 && SX == 1 && SY == 1 && CK >= 16 && CK <= 64 && (DG & (DG - 1)) == 0, "rotated halo layout: 16, 32 or 64 channels per step, stride 1");
// Reading side of the rotated layout.  A pixel fragment of the matrix loop is channel group 2 ks + kh (kh: the lane's k half) of pixel
// u + c, where u = (first halo row of the wave) * HALO_W + (lane & 31) belongs to the lane and c = hr * HALO_W + s is a
// compile-time constant.  Its slot is (u + c) * DG + ((2 ks + kh + (u + c) / DD) mod DG); the rotation splits into a part of
// the lane, which depends on c only through a = c % DD (a carry) and k = (2 ks + c / DD) mod DG, and the constant c * DG.
// So a lane keeps DD * DG = 8 base addresses and every read is `base[a][k] + immediate`.
struct PxBase {
  lds_half_t *b[DD][DG];
};
__device__ DNX_INLINE void px_base_init(PxBase &pb, const _Float16 *sIn, int row0, int lane) {
  const int u = row0 * HALO_W + (lane & 31), kh = lane >> 5;
#pragma unroll
  for (int a = 0; a < DD; ++a)
#pragma unroll
    for (int k = 0; k < DG; ++k) {
      const int rot = (kh + u / DD + ((u % DD + a) >= DD ? 1 : 0) + k) & (DG - 1);
      pb.b[a][k] = lds_opaque(sIn + (u * DG + rot) * 8);
    }
}
#define PX_READ(pb, hr, s, ks) \
  (*reinterpret_cast<lds_half8_t *>((pb).b[((hr) * HALO_W + (s)) % DD][(2 * (ks) + ((hr) * HALO_W + (s)) / DD) & (DG - 1)] + ((hr) * HALO_W + (s)) * DG * 8))
#endif

__device__ DNX_INLINE float apply_act(float v) {
#if ACT == 1
  return v > 0.0f ? v : 0.0f;
#elif ACT == 2
  const float av = ALPHA * v;
  return v > av ? v : av;
#else
  return v;
#endif
}

// Activation and the one rounding fp32 -> binary16 of an accumulator (the bias is in it already, see init_acc).
// ReLU commutes with the rounding -- both keep sign and zero -- so it is applied to the rounded values, where one
// instruction handles two channels; LeakyReLU multiplies and therefore stays in fp32.
__device__ DNX_INLINE _Float16 finish1(float v) {
#if ACT == 1
  return __builtin_fmaxf16((_Float16)v, (_Float16)0.0f);
#else
  return (_Float16)apply_act(v);
#endif
}
__device__ DNX_INLINE half8 finish8(const float *v) {
  half8 h;
#if ACT == 1
#pragma unroll
  for (int i = 0; i < 8; ++i) h[i] = (_Float16)v[i];
  const half8 zero = {0, 0, 0, 0, 0, 0, 0, 0};
  return __builtin_elementwise_max(h, zero);
#else
#pragma unroll
  for (int i = 0; i < 8; ++i) h[i] = (_Float16)apply_act(v[i]);
  return h;
#endif
}

__device__ DNX_INLINE ushort_t dpp_xor1(ushort_t v) {
  // quad_perm [1,0,3,2]: exchange with the neighbouring lane
  return (ushort_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true);
}
// The 2x2 maximum of a pooled result: the rows are two accumulators of this lane, the columns this lane and its
// neighbour.  Bias, ReLU and the rounding to binary16 never decrease when their argument grows, so the largest of the
// four sums finished once is the largest of the four finished values: two instructions per window and one conversion,
// where finishing all four and comparing the halves took a dozen.  (LeakyReLU with a negative slope is not monotonic:
// it keeps the element-wise form.)
#define POOL_MAX_FIRST (POOL && ACT <= 1)
__device__ DNX_INLINE float pool_max(float top, float bottom) {
  // The median of (x, y, +inf) is the larger of x and y in one instruction; fmaxf first quiets both operands, three
  // instructions -- and the compiler turns a median with a constant infinity back into that, so the infinity is a
  // register whose value it cannot see.
  float inf = __builtin_inff();
  asm("" : "+v"(inf));
  const float a = __builtin_amdgcn_fmed3f(top, bottom, inf);
  const float n = __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, a), 0xB1, 0xF, 0xF, true));
  return __builtin_amdgcn_fmed3f(a, n, inf);
}

// ---- output stores ---------------------------------------------------------------------
// The output is written through a buffer resource: a lane that has nothing to store (pixel outside the image or the
// crop window, odd lane of a pooled pair, channel past KOUT) passes an offset past the end and the hardware drops
// its part of the store.  No branch surrounds a store, so every wave issues the same number of them per tile.
typedef __amdgpu_buffer_rsrc_t OutBuf;
#define NO_STORE 0xFFFFF000u // beyond every output this code accepts (byte sizes are limited to below this value)

__device__ DNX_INLINE OutBuf out_buffer(_Float16 *OUT, const PushConstants &pc) {
#if POOL
  const unsigned w = CONV_OUT_W(pc) >> 1, h = CONV_OUT_H(pc) >> 1;
#elif CROP
  const unsigned w = pc.OUT_W, h = pc.OUT_H;
#else
  const unsigned w = CONV_OUT_W(pc), h = CONV_OUT_H(pc);
#endif
  // the last pixel ends after its KOUT channels, not after a whole pitch: the rest belongs to another tensor's range
  const unsigned pixels = w * h;
  return __builtin_amdgcn_make_buffer_rsrc(OUT, 0, (int)(pixels ? ((pixels - 1u) * (unsigned)OPITCH + (unsigned)KOUT) * 2u : 0u), 0x00020000);
}

// bytes of one 8-channel plane of the result (block-major layout)
__device__ DNX_INLINE unsigned out_plane_bytes(const PushConstants &pc) {
#if POOL
  return (CONV_OUT_W(pc) >> 1) * (CONV_OUT_H(pc) >> 1) * 16u;
#elif CROP
  return pc.OUT_W * pc.OUT_H * 16u;
#else
  return CONV_OUT_W(pc) * CONV_OUT_H(pc) * 16u;
#endif
}
static_assert(!LAYOUT_OUT || (KOUT % 8 == 0 && OPITCH == KOUT), "block-major result: whole 8-channel groups, a tensor of its own");

// 16 consecutive channels starting at chb of the pixel with linear index `pix`; plane: out_plane_bytes() (block-major results only)
__device__ DNX_INLINE void store16(OutBuf out, bool ok, unsigned pix, const half8 (&o)[2], int chb, unsigned plane = 0) {
#if LAYOUT_OUT
  const unsigned offb = (unsigned)(chb >> 3) * plane + pix * 16u; // the two 8-channel groups go to consecutive planes
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, o[0]), out, (ok && chb < KOUT) ? offb : NO_STORE, 0, STORE_AUX);
  __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, o[1]), out, (ok && chb + 8 < KOUT) ? offb + plane : NO_STORE, 0, STORE_AUX);
  return;
#endif
  const unsigned off = (pix * (unsigned)OPITCH + (unsigned)chb) * 2u;
  if (KOUT % 16 == 0 && OPITCH % 8 == 0 && OVEC) {
    const unsigned o0 = (ok && chb < KOUT) ? off : NO_STORE;
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, o[0]), out, o0, 0, STORE_AUX);
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, o[1]), out, o0 + 16u, 0, STORE_AUX);
  } else if (KOUT % 8 == 0 && OPITCH % 8 == 0 && OVEC) {
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, o[0]), out, (ok && chb < KOUT) ? off : NO_STORE, 0, STORE_AUX);
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, o[1]), out, (ok && chb + 8 < KOUT) ? off + 16u : NO_STORE, 0, STORE_AUX);
  } else {
#pragma unroll
    for (int i = 0; i < (KOUT < 16 ? KOUT : 16); ++i) {
      const _Float16 h = o[i >> 3][i & 7]; // a vector element is no object: copy it before reinterpreting its bits
      __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(ushort_t, h), out, (ok && chb + i < KOUT) ? off + 2u * i : NO_STORE, 0, STORE_AUX);
    }
  }
}

// The KT bias values of a workgroup's output channels are staged in LDS once, as fp32 (the global buffer is
// zero-padded to KOUTP).  Visible after the first barrier: every tile's accumulators start from them (init_acc), as the
// reference loads the bias straight into its accumulators (direct_conv_cm.comp:175-192), so the epilogue adds nothing.
typedef float bias_t;
__device__ DNX_INLINE void stage_bias(bias_t *sBias, const _Float16 *__restrict__ BIAS, int kt, int tid) {
#if HAS_BIAS
  for (int i = tid; i < KT; i += NT)
    sBias[i] = (float)BIAS[kt * KT + i];
#endif
}

#if MF == 32
// ---- 32 x 32 x 16 shape ----------------------------------------------------------------------------------
struct Acc {
  float16v v[KB][RPW];
};

// Epilogue of one wave in two parts, so that a persistent kernel can convert a finished tile at once and issue
// its stores later, after the next loads.  acc[kb][j] holds, for output row y0 + wv*RPW + j and pixel
// x0 + (lane & 31), the 16 channels kt*KT + kb*32 + (lane >> 5)*16 + i.
#define OROWS (POOL ? RPW / 2 : RPW) // output rows a wave stores per tile
struct Packed {
  half8 o[KB][OROWS][2];
};

// activation, rounding to fp16 and (POOL) the 2x2 maximum
__device__ DNX_INLINE void pack_tile(const Acc &acc, Packed &pk) {
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
#if POOL
#pragma unroll
    for (int j = 0; j < RPW; j += 2) {
#if POOL_MAX_FIRST
      float m[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) m[i] = pool_max(acc.v[kb][j][i], acc.v[kb][j + 1][i]);
      pk.o[kb][j >> 1][0] = finish8(m);
      pk.o[kb][j >> 1][1] = finish8(m + 8);
#else
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const _Float16 v0 = finish1(acc.v[kb][j][i]);
        const _Float16 v1 = finish1(acc.v[kb][j + 1][i]);
        const _Float16 n0 = __builtin_bit_cast(_Float16, dpp_xor1(__builtin_bit_cast(ushort_t, v0)));
        const _Float16 n1 = __builtin_bit_cast(_Float16, dpp_xor1(__builtin_bit_cast(ushort_t, v1)));
        // window order (0,0) (0,1) (1,0) (1,1); replace only on strictly greater
        _Float16 m = v0;
        m = n0 > m ? n0 : m;
        m = v1 > m ? v1 : m;
        m = n1 > m ? n1 : m;
        pk.o[kb][j >> 1][i >> 3][i & 7] = m;
      }
#endif
    }
#else
#pragma unroll
    for (int j = 0; j < RPW; ++j) {
      float v[16];
#pragma unroll
      for (int i = 0; i < 16; ++i) v[i] = acc.v[kb][j][i];
      pk.o[kb][j][0] = finish8(v);
      pk.o[kb][j][1] = finish8(v + 8);
    }
#endif
  }
}

// Stores the output rows r with r % nparts == part (all of them with nparts = 1).  All channels of a pixel go out
// together: a 128-byte line that is filled in two portions far apart in time is written to memory twice.
__device__ DNX_INLINE void
store_packed(const Packed &pk, OutBuf out, int y0, int x0, int kt, int wv, int lane, const PushConstants &pc, int part = 0, int nparts = 1,
             int ystep = 1, int xstep = 1) { // (steps of 2: a kernel that computes every other row / column of the output)
  const unsigned W = CONV_OUT_W(pc), H = CONV_OUT_H(pc);
  const unsigned plane = LAYOUT_OUT ? out_plane_bytes(pc) : 0u;
  const int l32 = lane & 31;
  const int x = x0 + l32 * xstep;
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
    const int chb = kt * KT + kb * 32 + (lane >> 5) * 16; // first of this lane's 16 channels
#pragma unroll
    for (int r = 0; r < OROWS; ++r) {
      if (r % nparts != part)
        continue;
#if POOL
      const unsigned WP = W >> 1, HP = H >> 1;
      const unsigned py = (unsigned)(y0 + wv * RPW + 2 * r) >> 1, px = (unsigned)x >> 1;
      store16(out, (l32 & 1) == 0 && py < HP && px < WP, py * WP + px, pk.o[kb][r], chb, plane);
#else
      const int y = y0 + (wv * RPW + r) * ystep;
#if CROP
      const int oy = y - (int)pc.CROP_T, ox = x - (int)pc.CROP_L;
      store16(out, y < (int)H && x < (int)W && oy >= 0 && oy < (int)pc.OUT_H && ox >= 0 && ox < (int)pc.OUT_W,
              (unsigned)oy * pc.OUT_W + (unsigned)ox, pk.o[kb][r], chb, plane);
#else
      store16(out, y < (int)H && x < (int)W, (unsigned)y * W + (unsigned)x, pk.o[kb][r], chb, plane);
#endif
#endif
    }
  }
}

// 9 taps x (L/16) reduction steps from one staged halo (row pitch CKP halves, or the rotated layout) and
// a weight slice whose rows are WPITCH halves apart; `wofs` selects the channel
// offset of this chunk inside a weight row.
template <int L, int WPITCH>
__device__ DNX_INLINE void
mma_chunk(const _Float16 *sIn, const _Float16 *sW, int wofs, Acc &acc, int wv, int lane) {
  const int l32 = lane & 31;
  const int kq = (lane >> 5) * 8;
#if HROTL
  PxBase pxb;
  px_base_init(pxb, sIn, wv * RPW, lane);
  auto px_read = [&](int hr, int s, int ks) { return PX_READ(pxb, hr, s, ks); };
#else
  lds_half_t *pxb = lds_opaque(sIn + (wv * RPW * SY * HALO_W + l32 * SX) * CKP + kq);
  auto px_read = [&](int hr, int s, int ks) { return *reinterpret_cast<lds_half8_t *>(pxb + (hr * HALO_W + s) * CKP + ks * 16); };
#endif
  lds_half_t *wb = lds_opaque(sW + l32 * WPITCH + wofs + kq);
  auto w_read = [&](int r, int kb, int s, int ks) { return *reinterpret_cast<lds_half8_t *>(wb + ((r * KS + s) * KT + kb * 32) * WPITCH + ks * 16); };
#if SWP
  // A group is one filter column s of one 16-channel slice: PXROWS pixel fragments and KR * KB weight fragments feed
  // KR * KB * RPW matrix instructions.  Left to the compiler, each read was issued right in front of the instruction that
  // needs it, and every few instructions waited out an LDS round trip.
  static_assert(SY == 1, "the pipelined matrix loop reads every halo row");
  constexpr int NG = KS * (L / 16), NREAD = PXROWS + KR * KB, NMMA = KR * KB * RPW;
  half8 px[2][PXROWS], wf[2][KR][KB];
  auto read_one = [&](int g, int i) { // read i of group g
    const int s = g / (L / 16), ks = g % (L / 16);
    if (i < PXROWS)
      px[g & 1][i] = px_read(i, s, ks);
    else
      wf[g & 1][(i - PXROWS) / KB][(i - PXROWS) % KB] = w_read((i - PXROWS) / KB, (i - PXROWS) % KB, s, ks);
  };
#pragma unroll
  for (int i = 0; i < NREAD; ++i) read_one(0, i);
#pragma unroll
  for (int g = 0; g < NG; ++g) {
#pragma unroll
    for (int i = 0; i < (NMMA > NREAD ? NMMA : NREAD); ++i) {
      if (g + 1 < NG && i < NREAD)
        read_one(g + 1, i);
      __builtin_amdgcn_sched_barrier(0);
      if (i < NMMA) {
        const int r = i / (KB * RPW), kb = (i / RPW) % KB, j = i % RPW;
        acc.v[kb][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[g & 1][r][kb], px[g & 1][j + r], acc.v[kb][j], 0, 0, 0);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
#else
#pragma unroll
  for (int s = 0; s < KS; ++s) {
#pragma unroll
    for (int ks = 0; ks < L / 16; ++ks) {
      half8 px[PXROWS];
#pragma unroll
      for (int hr = 0; hr < PXROWS; ++hr)
        if (SY == 1 || hr % SY < KR) // with a stride larger than the filter some halo rows are never read
          px[hr] = px_read(hr, s, ks);
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        half8 wf[KB];
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
          wf[kb] = w_read(r, kb, s, ks);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int j = 0; j < RPW; ++j)
            acc.v[kb][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(wf[kb], px[j * SY + r], acc.v[kb][j], 0, 0, 0);
      }
    }
  }
#endif
}

// Start of a tile: every accumulator holds the bias of its output channel (zero without one).  Reads the staged bias,
// so it runs after a barrier that follows stage_bias.
__device__ DNX_INLINE void init_acc(Acc &acc, const bias_t *sBias, int lane) {
  const int hsel = lane >> 5;
#pragma unroll
  for (int kb = 0; kb < KB; ++kb)
#pragma unroll
    for (int j = 0; j < RPW; ++j)
#pragma unroll
      for (int i = 0; i < 16; ++i)
#if HAS_BIAS
        acc.v[kb][j][i] = sBias[kb * 32 + hsel * 16 + i];
#else
        acc.v[kb][j][i] = 0.0f;
#endif
}

#else
// ---- 16 x 16 x 32 shape ----------------------------------------------------------------------------------
// acc.v[kb][j][xb] holds, for output row y0 + wv*RPW + j and pixel x0 + xb*16 + (lane & 15), four channels of
// 16-channel block kb.  Blocks are paired (kb = 2p, 2p+1) and their rows permuted on the host so that lane group
// g = lane >> 4 owns the 8 consecutive channels 32p + 8g .. + 7 (one 16-byte store); an unpaired last block
// gives 4 consecutive channels 16kb + 4g .. + 3.
struct Acc {
  float4v v[KB][RPW][XB];
};

// n = 8 or 4 consecutive channels starting at chb of the pixel with linear index `pix`
__device__ DNX_INLINE void store_vec(OutBuf out, bool ok, unsigned pix, const _Float16 (&o)[8], int chb, int n, unsigned plane = 0) {
#if LAYOUT_OUT
  const unsigned off = (unsigned)(chb >> 3) * plane + pix * 16u + (unsigned)(chb & 7) * 2u; // n = 8: a whole group; n = 4: half of one
#else
  const unsigned off = (pix * (unsigned)OPITCH + (unsigned)chb) * 2u;
#endif
  if (KOUT % 8 == 0 && OPITCH % 8 == 0 && OVEC && n == 8) {
    half8 h;
#pragma unroll
    for (int i = 0; i < 8; ++i) h[i] = o[i];
    __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, h), out, (ok && chb < KOUT) ? off : NO_STORE, 0, STORE_AUX);
  } else {
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (i < n)
        __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(ushort_t, o[i]), out, (ok && chb + i < KOUT) ? off + 2u * i : NO_STORE, 0, STORE_AUX);
  }
}

#define OROWS (POOL ? RPW / 2 : RPW) // output rows a wave stores per tile
#define KPAIRS ((KB + 1) / 2)
struct Packed {
  _Float16 o[KPAIRS][XB][OROWS][8];
};

// activation, rounding to fp16 and (POOL) the 2x2 maximum
__device__ DNX_INLINE void pack_tile(const Acc &acc, Packed &pk) {
#pragma unroll
  for (int kp = 0; kp < KPAIRS; ++kp) {
    const bool paired = 2 * kp + 1 < KB;
    const int n = paired ? 8 : 4;
#pragma unroll
    for (int xb = 0; xb < XB; ++xb) {
#pragma unroll
      for (int r = 0; r < OROWS; ++r) {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const int kb = 2 * kp + (i >> 2) < KB ? 2 * kp + (i >> 2) : 0;
          _Float16 m = (_Float16)0.0f;
          if (i < n) {
#if POOL_MAX_FIRST
            m = finish1(pool_max(acc.v[kb][2 * r][xb][i & 3], acc.v[kb][2 * r + 1][xb][i & 3]));
#elif POOL
            const _Float16 v0 = finish1(acc.v[kb][2 * r][xb][i & 3]);
            const _Float16 v1 = finish1(acc.v[kb][2 * r + 1][xb][i & 3]);
            const _Float16 n0 = __builtin_bit_cast(_Float16, dpp_xor1(__builtin_bit_cast(ushort_t, v0)));
            const _Float16 n1 = __builtin_bit_cast(_Float16, dpp_xor1(__builtin_bit_cast(ushort_t, v1)));
            m = v0; // window order (0,0) (0,1) (1,0) (1,1); replace only on strictly greater
            m = n0 > m ? n0 : m;
            m = v1 > m ? v1 : m;
            m = n1 > m ? n1 : m;
#else
            m = finish1(acc.v[kb][r][xb][i & 3]);
#endif
          }
          pk.o[kp][xb][r][i] = m;
        }
      }
    }
  }
}

// Stores the output rows r with r % nparts == part (all of them with nparts = 1).  All channels of a pixel go out
// together: a 128-byte line that is filled in two portions far apart in time is written to memory twice.
__device__ DNX_INLINE void
store_packed(const Packed &pk, OutBuf out, int y0, int x0, int kt, int wv, int lane, const PushConstants &pc, int part = 0, int nparts = 1) {
  const unsigned W = CONV_OUT_W(pc), H = CONV_OUT_H(pc);
  const unsigned plane = LAYOUT_OUT ? out_plane_bytes(pc) : 0u;
  const int l16 = lane & 15;
  const int g = lane >> 4;
#pragma unroll
  for (int kp = 0; kp < KPAIRS; ++kp) {
    const bool paired = 2 * kp + 1 < KB;
    const int n = paired ? 8 : 4;
    const int chb = kt * KT + (paired ? 32 * kp + 8 * g : 16 * (2 * kp) + 4 * g);
#pragma unroll
    for (int xb = 0; xb < XB; ++xb) {
      const int x = x0 + xb * 16 + l16;
#pragma unroll
      for (int r = 0; r < OROWS; ++r) {
        if (r % nparts != part)
          continue;
#if POOL
        const unsigned WP = W >> 1, HP = H >> 1;
        const unsigned py = (unsigned)(y0 + wv * RPW + 2 * r) >> 1, px = (unsigned)x >> 1;
        store_vec(out, (l16 & 1) == 0 && py < HP && px < WP, py * WP + px, pk.o[kp][xb][r], chb, n, plane);
#else
        const int y = y0 + wv * RPW + r;
#if CROP
        const int oy = y - (int)pc.CROP_T, ox = x - (int)pc.CROP_L;
        store_vec(out, y < (int)H && x < (int)W && oy >= 0 && oy < (int)pc.OUT_H && ox >= 0 && ox < (int)pc.OUT_W,
                  (unsigned)oy * pc.OUT_W + (unsigned)ox, pk.o[kp][xb][r], chb, n, plane);
#else
        store_vec(out, y < (int)H && x < (int)W, (unsigned)y * W + (unsigned)x, pk.o[kp][xb][r], chb, n, plane);
#endif
#endif
      }
    }
  }
}

// 9 taps x (L/32) reduction steps; lane = (pixel or weight row) lane & 15, k group lane >> 4.
template <int L, int WPITCH>
__device__ DNX_INLINE void
mma_chunk(const _Float16 *sIn, const _Float16 *sW, int wofs, Acc &acc, int wv, int lane) {
  const int l16 = lane & 15;
  const int kq = (lane >> 4) * 8;
  lds_half_t *pxb = lds_opaque(sIn + (wv * RPW * SY * HALO_W + l16 * SX) * CKP + kq);
  lds_half_t *wb = lds_opaque(sW + l16 * WPITCH + wofs + kq);
#pragma unroll
  for (int s = 0; s < KS; ++s) {
#pragma unroll
    for (int ks = 0; ks < L / 32; ++ks) {
      half8 px[PXROWS][XB];
#pragma unroll
      for (int hr = 0; hr < PXROWS; ++hr)
#pragma unroll
        for (int xb = 0; xb < XB; ++xb)
          if (SY == 1 || hr % SY < KR)
            px[hr][xb] = *reinterpret_cast<lds_half8_t *>(pxb + (hr * HALO_W + xb * 16 * SX + s) * CKP + ks * 32);
#pragma unroll
      for (int r = 0; r < KR; ++r) {
        half8 wf[KB];
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
          wf[kb] = *reinterpret_cast<lds_half8_t *>(wb + ((r * KS + s) * KT + kb * 16) * WPITCH + ks * 32);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int j = 0; j < RPW; ++j)
#pragma unroll
            for (int xb = 0; xb < XB; ++xb)
              acc.v[kb][j][xb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(wf[kb], px[j * SY + r][xb], acc.v[kb][j][xb], 0, 0, 0);
      }
    }
  }
}

// Start of a tile: every accumulator holds the bias of its output channel (zero without one); the channel of
// acc.v[kb][..][..][e] is the one pack_tile / store_packed assign to it.  Runs after a barrier that follows stage_bias.
__device__ DNX_INLINE void init_acc(Acc &acc, const bias_t *sBias, int lane) {
  const int g = lane >> 4;
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
    const int kp = kb >> 1;
    const bool paired = 2 * kp + 1 < KB;
    const int chl = paired ? 32 * kp + 8 * g + 4 * (kb & 1) : 16 * kb + 4 * g;
#pragma unroll
    for (int j = 0; j < RPW; ++j)
#pragma unroll
      for (int xb = 0; xb < XB; ++xb)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#if HAS_BIAS
          acc.v[kb][j][xb][i] = sBias[chl + i];
#else
          acc.v[kb][j][xb][i] = 0.0f;
#endif
  }
}
#endif // MF

__device__ DNX_INLINE void
store_tile(const Acc &acc, OutBuf out, int y0, int x0, int kt, int wv, int lane, const PushConstants &pc) {
  Packed pk;
  pack_tile(acc, pk);
  store_packed(pk, out, y0, x0, kt, wv, lane, pc);
}

// mma_chunk for step `chunk` of a tile, whichever length that step has
template <int WPITCH>
__device__ DNX_INLINE void
mma_step(const _Float16 *sIn, const _Float16 *sW, int wofs, Acc &acc, int wv, int lane, int chunk) {
  if (TAIL == CK || chunk < NCHUNK - 1)
    mma_chunk<CK, WPITCH>(sIn, sW, wofs, acc, wv, lane);
  else
    mma_chunk<TAIL, WPITCH>(sIn, sW, wofs, acc, wv, lane);
}

