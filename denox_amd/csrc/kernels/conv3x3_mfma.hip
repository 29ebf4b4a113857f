// conv3x3_mfma.hip -- fused 3x3 convolution (stride 1, zero padding 1) as an fp16
// implicit GEMM on CDNA4 matrix cores, fp32 accumulation.
//
// Replaces the reference's three conv shaders
//   compiler/src/denox/compiler/implement/shaders/conv/direct_conv.comp:82-775
//   compiler/src/denox/compiler/implement/shaders/conv/direct_conv_cm.comp:119-1568
//   compiler/src/denox/compiler/implement/shaders/conv/concat_conv_cm.comp:1043-1128
// and, through compile-time switches, also absorbs a 2x nearest upsample of the
// first source, a channel concat of two sources and a 2x2 max pool of the result.
//
//   out[y,x,k] = act(bias[k] + sum_{r,s,c} src[y+r-1, x+s-1, c] * W[k,c,r,s])
//   src[.., c] = c < CA ? A[(UPA ? y/2,x/2 : y,x), c] : B[y, x, c-CA]
//
// The source is compiled at model-compile time with these definitions:
//   CA, CB      channels of source A / source B (CB = 0: single source)
//   UPA         1: A is stored at half resolution and read at (y>>1, x>>1)
//   KOUT        output channels
//   KT          output channels handled per workgroup (multiple of 32)
//   ACT         0 none, 1 ReLU, 2 LeakyReLU(ALPHA)
//   POOL        1: store max over 2x2 output windows at (y/2, x/2) only
//   HAS_BIAS    0/1
//   WAVES, RPW  waves per workgroup, output rows per wave -> tile = (WAVES*RPW) x 32 pixels
//   CK          input channels staged in LDS per step (multiple of 16)
//
// Mapping onto v_mfma_f32_32x32x16_f16: the weights are the M operand (32 output
// channels per block, rows permuted so that each lane ends up with 16 consecutive
// channels), 32 consecutive pixels of one image row are the N operand, and the
// reduction runs over (tap, input channel) in steps of 16 channels.
//
// LDS holds one (TH+2) x 34 pixel halo of CK channels and the 9 x KT x CK weight
// slice for those channels; rows are padded by 8 halves so that consecutive
// pixels / weight rows start in different 16-byte bank groups.

#include "prelude.h"
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float16v __attribute__((ext_vector_type(16)));
typedef unsigned int uint4v __attribute__((ext_vector_type(4)));
typedef unsigned short ushort_t;

#ifndef ALPHA
#define ALPHA 0.0f
#endif

#define CIN (CA + CB)
#define CPAD (((CIN) + 15) / 16 * 16)
#define NCHUNK ((CPAD + CK - 1) / CK)
#define TAIL (CPAD - (NCHUNK - 1) * CK)
#define TW 32
#define TH (WAVES * RPW)
#define HALO_W (TW + 2)
#define HALO_H (TH + 2)
#define HALO_PIX (HALO_W * HALO_H)
#define CKP (CK + 8)
#define KB (KT / 32)
#define NT (WAVES * 64)
#define KOUTP (((KOUT) + 31) / 32 * 32)

// The entry point is named per variant (KERNEL_NAME) so that profilers tell variants apart.
#ifndef KERNEL_NAME
#define KERNEL_NAME conv3x3_mfma
#endif
struct PushConstants {
  unsigned int IN_W;
  unsigned int IN_H;
};

__device__ DNX_INLINE uint4v ld16(const _Float16 *p) {
  return *reinterpret_cast<const uint4v *>(p);
}

// Eight consecutive channels [cc, cc+8) of the (virtual, concatenated) source at
// full-resolution pixel (gy, gx); channels past CIN read as zero.
__device__ DNX_INLINE uint4v
load_src8(const _Float16 *__restrict__ A, const _Float16 *__restrict__ B,
          int gy, int gx, int cc, unsigned W) {
  const unsigned WA = UPA ? (W >> 1) : W;
  const int ay = UPA ? (gy >> 1) : gy;
  const int ax = UPA ? (gx >> 1) : gx;
  const size_t pa = ((size_t)ay * WA + (size_t)ax) * CA;
  const size_t pb = ((size_t)gy * W + (size_t)gx) * (CB > 0 ? CB : 1);
  if ((CA % 8 == 0) && (CB % 8 == 0)) {
    if (cc < CA)
      return ld16(A + pa + cc);
    if (CB > 0 && cc < CIN)
      return ld16(B + pb + (cc - CA));
    return uint4v{0u, 0u, 0u, 0u};
  } else {
    if ((CA % 8 == 0) && cc + 8 <= CA)
      return ld16(A + pa + cc);
    half8 v;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int ch = cc + e;
      _Float16 x = (_Float16)0.0f;
      if (ch < CA)
        x = A[pa + ch];
      else if (CB > 0 && ch < CIN)
        x = B[pb + (ch - CA)];
      v[e] = x;
    }
    return __builtin_bit_cast(uint4v, v);
  }
}

// Staging is split in two so that the global loads of the next chunk are in
// flight while the matrix cores work on the current one: fetch_chunk issues the
// loads into registers, commit_chunk writes them to LDS after the barrier.
#define NV_IN ((HALO_PIX * (CK / 8) + NT - 1) / NT)
#define NV_W ((9 * KT * (CK / 8) + NT - 1) / NT)

struct Staged {
  uint4v in[NV_IN];
  uint4v w[NV_W];
};

template <int L>
__device__ DNX_INLINE void
fetch_chunk(const _Float16 *__restrict__ A, const _Float16 *__restrict__ B,
            const _Float16 *__restrict__ wchunk, Staged &st, int c0, int y0,
            int x0, unsigned W, unsigned H, int tid) {
  constexpr int VPP = L / 8; // 16-byte vectors per pixel
#pragma unroll
  for (int it = 0; it < NV_IN; ++it) {
    const int i = tid + it * NT;
    uint4v val = {0u, 0u, 0u, 0u};
    if (i < HALO_PIX * VPP) {
      const int pix = i / VPP;
      const int v = i - pix * VPP;
      const int hy = pix / HALO_W;
      const int hx = pix - hy * HALO_W;
      const int gy = y0 + hy - 1;
      const int gx = x0 + hx - 1;
      if (gy >= 0 && gy < (int)H && gx >= 0 && gx < (int)W)
        val = load_src8(A, B, gy, gx, c0 + v * 8, W);
    }
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
__device__ DNX_INLINE void commit_chunk(const Staged &st, _Float16 *sIn,
                                        _Float16 *sW, int tid) {
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

template <int L>
__device__ DNX_INLINE void
mma_chunk(const _Float16 *sIn, const _Float16 *sW, float16v (&acc)[KB][RPW],
          int wv, int lane) {
  const int l32 = lane & 31;
  const int kq = (lane >> 5) * 8;
#pragma unroll
  for (int s = 0; s < 3; ++s) {
#pragma unroll
    for (int ks = 0; ks < L / 16; ++ks) {
      const int kk = ks * 16 + kq;
      half8 px[RPW + 2];
#pragma unroll
      for (int hr = 0; hr < RPW + 2; ++hr)
        px[hr] = *reinterpret_cast<const half8 *>(
            sIn + ((wv * RPW + hr) * HALO_W + l32 + s) * CKP + kk);
#pragma unroll
      for (int r = 0; r < 3; ++r) {
        half8 wf[KB];
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
          wf[kb] = *reinterpret_cast<const half8 *>(
              sW + (((r * 3 + s) * KT) + kb * 32 + l32) * CKP + kk);
#pragma unroll
        for (int kb = 0; kb < KB; ++kb)
#pragma unroll
          for (int j = 0; j < RPW; ++j)
            acc[kb][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                wf[kb], px[j + r], acc[kb][j], 0, 0, 0);
      }
    }
  }
}

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

__device__ DNX_INLINE ushort_t dpp_xor1(ushort_t v) {
  // quad_perm [1,0,3,2]: exchange with the neighbouring lane
  return (ushort_t)__builtin_amdgcn_mov_dpp((int)v, 0xB1, 0xF, 0xF, true);
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
  const unsigned W = pc.IN_W, H = pc.IN_H;
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
    fetch_chunk<CK>(A, B, wbase, st, 0, y0, x0, W, H, tid);
  else
    fetch_chunk<TAIL>(A, B, wbase, st, 0, y0, x0, W, H, tid);
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
        fetch_chunk<CK>(A, B, wnext, st, c1, y0, x0, W, H, tid);
      else
        fetch_chunk<TAIL>(A, B, wnext, st, c1, y0, x0, W, H, tid);
    }
    if (fullNow)
      mma_chunk<CK>(sIn, sW, acc, wv, lane);
    else
      mma_chunk<TAIL>(sIn, sW, acc, wv, lane);
    DNX_SYNC();
  }

  // ---- epilogue: bias, activation, rounding to binary16, (pool,) store ----
  const int l32 = lane & 31;
  const int hsel = lane >> 5;
  const int x = x0 + l32;
#pragma unroll
  for (int kb = 0; kb < KB; ++kb) {
    const int chb = kt * KT + kb * 32 + hsel * 16; // first of this lane's 16 channels
    float bias[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
#if HAS_BIAS
      bias[i] = (float)BIAS[chb + i]; // bias buffer is zero-padded to KOUTP
#else
      bias[i] = 0.0f;
#endif
    }
#if POOL
    const unsigned WP = W >> 1, HP = H >> 1;
#pragma unroll
    for (int j = 0; j < RPW; j += 2) {
      const int y = y0 + wv * RPW + j;
      half8 o[2];
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const _Float16 v0 = (_Float16)apply_act(acc[kb][j][i] + bias[i]);
        const _Float16 v1 = (_Float16)apply_act(acc[kb][j + 1][i] + bias[i]);
        const _Float16 n0 = __builtin_bit_cast(_Float16, dpp_xor1(__builtin_bit_cast(ushort_t, v0)));
        const _Float16 n1 = __builtin_bit_cast(_Float16, dpp_xor1(__builtin_bit_cast(ushort_t, v1)));
        // window order (0,0) (0,1) (1,0) (1,1); replace only on strictly greater
        _Float16 m = v0;
        m = n0 > m ? n0 : m;
        m = v1 > m ? v1 : m;
        m = n1 > m ? n1 : m;
        o[i >> 3][i & 7] = m;
      }
      const unsigned py = (unsigned)y >> 1, px = (unsigned)x >> 1;
      if ((l32 & 1) == 0 && py < HP && px < WP) {
        _Float16 *dst = OUT + ((size_t)py * WP + px) * KOUT + chb;
        if (KOUT % 16 == 0) {
          if (chb < KOUT) {
            *reinterpret_cast<half8 *>(dst) = o[0];
            *reinterpret_cast<half8 *>(dst + 8) = o[1];
          }
        } else {
#pragma unroll
          for (int i = 0; i < 16; ++i)
            if (chb + i < KOUT)
              dst[i] = o[i >> 3][i & 7];
        }
      }
    }
#else
#pragma unroll
    for (int j = 0; j < RPW; ++j) {
      const int y = y0 + wv * RPW + j;
      half8 o[2];
#pragma unroll
      for (int i = 0; i < 16; ++i)
        o[i >> 3][i & 7] = (_Float16)apply_act(acc[kb][j][i] + bias[i]);
      if (y < (int)H && x < (int)W) {
        _Float16 *dst = OUT + ((size_t)y * W + x) * KOUT + chb;
        if (KOUT % 16 == 0) {
          if (chb < KOUT) {
            *reinterpret_cast<half8 *>(dst) = o[0];
            *reinterpret_cast<half8 *>(dst + 8) = o[1];
          }
        } else {
#pragma unroll
          for (int i = 0; i < 16; ++i)
            if (chb + i < KOUT)
              dst[i] = o[i >> 3][i & 7];
        }
      }
    }
#endif
  }
}
