/*
 * denox_oracle.c -- CPU restatement of the denox layer semantics.
 *
 * TEST INFRASTRUCTURE ONLY.  This file is the checker for the HIP path: it is
 * compiled into oracle/_build/libdenox_oracle.so and may be loaded by tests/,
 * by __graft_entry__.smoke() and by the cpu_baseline leg of bench.py, and by
 * nothing else.  No product code path links, imports or falls back to it.
 *
 * Every function cites the reference file it restates (paths relative to the
 * reference checkout).  The reference kernels are GLSL compute shaders that
 * only run through a Vulkan driver, so nothing here is compiled from the
 * reference; the functions are pinned by tests/test_oracle_*.py against
 * library routines (torch.nn.functional in fp32), closed forms and brute
 * force.  Pinning status per function:
 *
 *   dnxo_f32_to_f16 / dnxo_f16_to_f32      pinned: numpy float16 casts, all 65536 patterns
 *   dnxo_conv2d_hwc                        pinned: F.conv2d fp32, identity tap, all-ones, fp64 brute force
 *   dnxo_maxpool_hwc_f16                   pinned: F.max_pool2d, membership invariant
 *   dnxo_avgpool_hwc_f16                   pinned: F.avg_pool2d (exact on 2x2 windows, <= 1 ulp otherwise), constant input
 *   dnxo_upsample_nearest_hwc_f16          pinned: F.interpolate(mode="nearest")
 *   dnxo_concat_hwc_f16 / dnxo_copy_channels_hwc_f16   pinned: torch.cat
 *   dnxo_pad_replicate_hwc_f16             pinned: F.pad(mode="replicate")
 *   dnxo_pad_zero_hwc_f16                  pinned: F.pad(mode="constant", value=0)
 *   dnxo_slice_hwc_f16                     pinned: tensor slicing
 *   dnxo_activation_f16                    pinned: F.relu / F.leaky_relu on fp16
 *   dnxo_layout_index / dnxo_relayout_f16  pinned: permute/reshape round trips
 *   dnxo_symir_eval                        pinned: hand-built programs with known values
 *
 * Arithmetic contract (what the HIP path is compared with):
 *   - activations and weights are IEEE binary16 in memory;
 *   - a conv accumulates in fp32 (the comparison target is an fp32 evaluation),
 *     adds the bias, applies the activation, and only then rounds to binary16
 *     (round-to-nearest-even) when store_f16 is set;
 *   - pool / upsample / concat / pad / slice move or compare binary16 bit
 *     patterns and are exact.
 */
#include <stdint.h>
#include <stddef.h>
#include <string.h>
#include <math.h>

#if defined(_OPENMP)
#include <omp.h>
#endif

#define DNXO_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------- */
/* binary16 <-> binary32.                                                     */
/* The reference's host conversion (common/src/denox/memory/dtype/f16.cpp:6-20)
 * truncates the mantissa and flushes subnormals; that is a property of its
 * weight import from fp32 ONNX files only.  Tensors here are generated in
 * binary16 directly, so the oracle uses the IEEE round-to-nearest-even
 * conversion a GPU performs when it stores an fp32 accumulator as fp16.      */

DNXO_API float dnxo_f16_to_f32(uint16_t h) {
  uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else { /* subnormal: normalise */
      int e = -1;
      do {
        man <<= 1;
        e++;
      } while ((man & 0x400u) == 0);
      man &= 0x3FFu;
      bits = sign | ((uint32_t)(127 - 15 - e) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + (127 - 15)) << 23) | (man << 13);
  }
  float f;
  memcpy(&f, &bits, 4);
  return f;
}

DNXO_API uint16_t dnxo_f32_to_f16(float f) {
  uint32_t x;
  memcpy(&x, &f, 4);
  uint32_t sign = (x >> 16) & 0x8000u;
  uint32_t ax = x & 0x7FFFFFFFu;
  if (ax >= 0x7F800000u) { /* inf / nan */
    if (ax > 0x7F800000u)
      return (uint16_t)(sign | 0x7E00u | ((ax >> 13) & 0x3FFu));
    return (uint16_t)(sign | 0x7C00u);
  }
  if (ax >= 0x477FF000u) { /* >= 65520 rounds to inf */
    return (uint16_t)(sign | 0x7C00u);
  }
  if (ax < 0x33000001u) { /* <= 2^-25 rounds to zero (ties-to-even at exactly 2^-25) */
    return (uint16_t)sign;
  }
  int32_t e = (int32_t)(ax >> 23) - 127;
  uint32_t m = (ax & 0x7FFFFFu) | 0x800000u; /* 24-bit significand */
  uint32_t shift;
  uint32_t hexp;
  if (e < -14) { /* subnormal result */
    shift = (uint32_t)(13 + (-14 - e));
    hexp = 0;
  } else {
    shift = 13;
    hexp = (uint32_t)(e + 15);
  }
  uint32_t q = m >> shift;
  uint32_t rem = m & ((1u << shift) - 1u);
  uint32_t half = 1u << (shift - 1);
  if (rem > half || (rem == half && (q & 1u)))
    q++;
  /* q carries the implicit bit for normals: adding (hexp-1)<<10 folds it in
   * and lets a mantissa overflow carry into the exponent. */
  uint32_t out;
  if (hexp == 0)
    out = q; /* may become 0x400 = smallest normal, which is correct */
  else
    out = ((hexp - 1) << 10) + q;
  return (uint16_t)(sign | out);
}

DNXO_API void dnxo_f16_to_f32_array(const uint16_t *src, float *dst, size_t n) {
  for (size_t i = 0; i < n; ++i)
    dst[i] = dnxo_f16_to_f32(src[i]);
}

DNXO_API void dnxo_f32_to_f16_array(const float *src, uint16_t *dst, size_t n) {
  for (size_t i = 0; i < n; ++i)
    dst[i] = dnxo_f32_to_f16(src[i]);
}

/* ------------------------------------------------------------------------- */
/* Activation layouts: common/src/denox/memory/tensor/ActivationLayout.hpp:37-66
 *   HWC   : h*(W*C) + w*C + c
 *   CHW   : c*(H*W) + h*W + w
 *   CHWC8 : (c>>3)*(H*W*8) + h*(W*8) + w*8 + (c&7)      (C % 8 == 0)          */
enum { DNXO_LAYOUT_HWC = 0, DNXO_LAYOUT_CHW = 1, DNXO_LAYOUT_CHWC8 = 2 };

DNXO_API int64_t dnxo_layout_index(int layout, int64_t H, int64_t W, int64_t C,
                                   int64_t h, int64_t w, int64_t c) {
  switch (layout) {
  case DNXO_LAYOUT_HWC:
    return h * (W * C) + w * C + c;
  case DNXO_LAYOUT_CHW:
    return c * (H * W) + h * W + w;
  case DNXO_LAYOUT_CHWC8:
    return (c >> 3) * (H * W * 8) + h * (W * 8) + (w * 8) + (c & 7);
  default:
    return -1;
  }
}

DNXO_API int dnxo_relayout_f16(const uint16_t *src, int src_layout,
                               uint16_t *dst, int dst_layout, int64_t H,
                               int64_t W, int64_t C) {
  if ((src_layout == DNXO_LAYOUT_CHWC8 || dst_layout == DNXO_LAYOUT_CHWC8) &&
      (C % 8) != 0)
    return -1;
  for (int64_t h = 0; h < H; ++h)
    for (int64_t w = 0; w < W; ++w)
      for (int64_t c = 0; c < C; ++c)
        dst[dnxo_layout_index(dst_layout, H, W, C, h, w, c)] =
            src[dnxo_layout_index(src_layout, H, W, C, h, w, c)];
  return 0;
}

/* ------------------------------------------------------------------------- */
/* Convolution.
 * compiler/src/denox/compiler/implement/shaders/conv/direct_conv.comp:82-775:
 *   out[y,x,k] = act(bias[k] + sum_{r,s,c} in[y*sy + r - py, x*sx + s - px, c] * W[k,c,r,s])
 * with taps outside the image contributing zero (the shader's unsigned
 * bounds test in_y < IN_H && in_x < IN_W, direct_conv.comp:209-212,304-311),
 * bias added before the activation and ReLU = max(x, 0)
 * (direct_conv.comp:562-590).  Weights arrive in ONNX order KCRS
 * (common/src/denox/memory/tensor/FilterLayout.hpp:49-116, layout KCRS).
 *
 * in      : fp32 HWC activations [H][W][C] (callers widen binary16 exactly)
 * weights : fp32 KCRS [K][C][R][S]
 * bias    : fp32 [K] or NULL
 * act     : 0 none, 1 ReLU, 2 LeakyReLU(alpha)
 * out     : fp32 HWC [Ho][Wo][K], Ho = (H + 2*py - R)/sy + 1
 * round_f16: when non-zero every output is rounded to binary16 and widened
 *           again, i.e. what a layer boundary stored as fp16 holds.
 * Accumulation is fp32 in (r, s, c) order.                                   */
DNXO_API int dnxo_conv2d_hwc(const float *in, int64_t H, int64_t W, int64_t C,
                             const float *weights, const float *bias, int64_t K,
                             int64_t R, int64_t S, int64_t sy, int64_t sx,
                             int64_t py, int64_t px, int act, float alpha,
                             int round_f16, float *out) {
  if (H <= 0 || W <= 0 || C <= 0 || K <= 0 || R <= 0 || S <= 0 || sy <= 0 ||
      sx <= 0)
    return -1;
  const int64_t Ho = (H + 2 * py - R) / sy + 1;
  const int64_t Wo = (W + 2 * px - S) / sx + 1;
  if (Ho <= 0 || Wo <= 0)
    return -1;
  /* repack weights to [r][s][c][k] so the inner loop is unit stride in k */
  float *wt = (float *)__builtin_malloc(sizeof(float) * (size_t)(R * S * C * K));
  if (!wt)
    return -2;
  for (int64_t k = 0; k < K; ++k)
    for (int64_t c = 0; c < C; ++c)
      for (int64_t r = 0; r < R; ++r)
        for (int64_t s = 0; s < S; ++s)
          wt[((r * S + s) * C + c) * K + k] = weights[((k * C + c) * R + r) * S + s];

#pragma omp parallel for schedule(static)
  for (int64_t y = 0; y < Ho; ++y) {
    float acc[1024];
    float *accp = acc;
    float *heap = NULL;
    if (K > 1024) {
      heap = (float *)__builtin_malloc(sizeof(float) * (size_t)K);
      accp = heap;
    }
    for (int64_t x = 0; x < Wo; ++x) {
      for (int64_t k = 0; k < K; ++k)
        accp[k] = 0.0f;
      for (int64_t r = 0; r < R; ++r) {
        const int64_t iy = y * sy + r - py;
        if (iy < 0 || iy >= H)
          continue;
        for (int64_t s = 0; s < S; ++s) {
          const int64_t ix = x * sx + s - px;
          if (ix < 0 || ix >= W)
            continue;
          const float *ip = in + (iy * W + ix) * C;
          const float *wp = wt + (r * S + s) * C * K;
          for (int64_t c = 0; c < C; ++c) {
            const float v = ip[c];
            const float *wk = wp + c * K;
            for (int64_t k = 0; k < K; ++k)
              accp[k] += v * wk[k];
          }
        }
      }
      float *op = out + (y * Wo + x) * K;
      for (int64_t k = 0; k < K; ++k) {
        float v = accp[k] + (bias ? bias[k] : 0.0f);
        if (act == 1)
          v = v > 0.0f ? v : 0.0f;
        else if (act == 2)
          v = v > alpha * v ? v : alpha * v;
        if (round_f16)
          v = dnxo_f16_to_f32(dnxo_f32_to_f16(v));
        op[k] = v;
      }
    }
    if (heap)
      __builtin_free(heap);
  }
  __builtin_free(wt);
  return 0;
}

/* ------------------------------------------------------------------------- */
/* Max pool, kernel == stride, no padding.
 * compiler/.../shaders/pool/basic_pool.comp:27-230: output extent is
 * floor(H/k) x floor(W/k) (:41-42), accumulator starts at -inf 0xFC00 (:60),
 * out = max over the k x k window.  Compared as binary16 values; inputs are
 * finite so the result is one of the window's bit patterns (for +0 / -0 the
 * numerically-equal tie keeps the first seen, matching a max that only
 * replaces on strictly-greater).                                             */
static inline int f16_gt(uint16_t a, uint16_t b) { /* a > b for finite/inf values */
  int sa = a >> 15, sb = b >> 15;
  uint16_t ma = a & 0x7FFFu, mb = b & 0x7FFFu;
  if (ma == 0 && mb == 0)
    return 0; /* +-0 equal */
  if (sa != sb)
    return sb; /* a positive, b negative */
  return sa ? (ma < mb) : (ma > mb);
}

/* Average pool, kernel == stride, no padding.  The reference carries the
 * function in its model (common/src/denox/common/PoolFunction.hpp:7-10,
 * frontend/onnx/details/ops/average_pool.cpp:154) but has no shader for it
 * (BasicPoolShader.cpp:170), so the arithmetic is this build's own contract:
 * sum the window in binary32 in row-major order, multiply by the binary32
 * constant 1/(ky*kx), round once to binary16. */
DNXO_API int dnxo_avgpool_hwc_f16(const uint16_t *in, int64_t H, int64_t W,
                                  int64_t C, int64_t ky, int64_t kx,
                                  uint16_t *out) {
  if (ky <= 0 || kx <= 0)
    return -1;
  const int64_t Ho = H / ky, Wo = W / kx;
  const float inv = 1.0f / (float)(kx * ky);
#pragma omp parallel for schedule(static)
  for (int64_t oh = 0; oh < Ho; ++oh)
    for (int64_t ow = 0; ow < Wo; ++ow)
      for (int64_t c = 0; c < C; ++c) {
        float sum = 0.0f;
        for (int64_t r = 0; r < ky; ++r)
          for (int64_t s = 0; s < kx; ++s) {
            const float v = dnxo_f16_to_f32(in[((oh * ky + r) * W + (ow * kx + s)) * C + c]);
            sum = (r == 0 && s == 0) ? v : sum + v;
          }
        out[(oh * Wo + ow) * C + c] = dnxo_f32_to_f16(sum * inv);
      }
  return 0;
}

DNXO_API int dnxo_maxpool_hwc_f16(const uint16_t *in, int64_t H, int64_t W,
                                  int64_t C, int64_t ky, int64_t kx,
                                  uint16_t *out) {
  if (ky <= 0 || kx <= 0)
    return -1;
  const int64_t Ho = H / ky, Wo = W / kx;
#pragma omp parallel for schedule(static)
  for (int64_t oh = 0; oh < Ho; ++oh)
    for (int64_t ow = 0; ow < Wo; ++ow)
      for (int64_t c = 0; c < C; ++c) {
        uint16_t acc = 0xFC00u;
        for (int64_t r = 0; r < ky; ++r)
          for (int64_t s = 0; s < kx; ++s) {
            uint16_t v = in[((oh * ky + r) * W + (ow * kx + s)) * C + c];
            if (f16_gt(v, acc))
              acc = v;
          }
        out[(oh * Wo + ow) * C + c] = acc;
      }
  return 0;
}

/* Nearest-neighbour upsample by an integer factor.
 * compiler/.../shaders/upsample/basic_upsample.comp:49,56,95,103:
 *   out[h2, w2, c] = in[h2 / f, w2 / f, c]   (integer division).             */
DNXO_API int dnxo_upsample_nearest_hwc_f16(const uint16_t *in, int64_t H,
                                           int64_t W, int64_t C, int64_t f,
                                           uint16_t *out) {
  if (f <= 0)
    return -1;
  const int64_t Ho = H * f, Wo = W * f;
#pragma omp parallel for schedule(static)
  for (int64_t h = 0; h < Ho; ++h)
    for (int64_t w = 0; w < Wo; ++w)
      memcpy(out + (h * Wo + w) * C, in + ((h / f) * W + (w / f)) * C,
             (size_t)C * 2);
  return 0;
}

/* Strided channel copy, the building block of an explicit concat.
 * compiler/.../shaders/copy/copy_transform.comp:58-62,95-99:
 *   dst[h, w, dst_off + c] = src[h, w, src_off + c]   for c < count.         */
DNXO_API int dnxo_copy_channels_hwc_f16(const uint16_t *src, int64_t H,
                                        int64_t W, int64_t src_C,
                                        int64_t src_off, uint16_t *dst,
                                        int64_t dst_C, int64_t dst_off,
                                        int64_t count) {
  if (src_off + count > src_C || dst_off + count > dst_C)
    return -1;
  for (int64_t p = 0; p < H * W; ++p)
    memcpy(dst + p * dst_C + dst_off, src + p * src_C + src_off,
           (size_t)count * 2);
  return 0;
}

/* Channel concat = two channel copies
 * (compiler/.../shaders/copy/CopyTransformShader.cpp:437-537).               */
DNXO_API int dnxo_concat_hwc_f16(const uint16_t *a, int64_t Ca,
                                 const uint16_t *b, int64_t Cb, int64_t H,
                                 int64_t W, uint16_t *out) {
  int r = dnxo_copy_channels_hwc_f16(a, H, W, Ca, 0, out, Ca + Cb, 0, Ca);
  if (r)
    return r;
  return dnxo_copy_channels_hwc_f16(b, H, W, Cb, 0, out, Ca + Cb, Ca, Cb);
}

/* Replicate padding by clamped source index.
 * compiler/.../shaders/pad/memory_pad.comp:70-78:
 *   out[ho, wo, c] = in[clamp(ho - top, 0, H-1), clamp(wo - left, 0, W-1), c] */
DNXO_API int dnxo_pad_replicate_hwc_f16(const uint16_t *in, int64_t H,
                                        int64_t W, int64_t C, int64_t left,
                                        int64_t right, int64_t top,
                                        int64_t bottom, uint16_t *out) {
  if (left < 0 || right < 0 || top < 0 || bottom < 0)
    return -1;
  const int64_t Ho = H + top + bottom, Wo = W + left + right;
  for (int64_t ho = 0; ho < Ho; ++ho) {
    int64_t hi = ho - top;
    hi = hi < 0 ? 0 : (hi > H - 1 ? H - 1 : hi);
    for (int64_t wo = 0; wo < Wo; ++wo) {
      int64_t wi = wo - left;
      wi = wi < 0 ? 0 : (wi > W - 1 ? W - 1 : wi);
      memcpy(out + (ho * Wo + wo) * C, in + (hi * W + wi) * C, (size_t)C * 2);
    }
  }
  return 0;
}

/* Zero padding: the border is 0 (PaddingMode::Zero of the reference's model, common/src/denox/common/PaddingMode.hpp;
 * torch: F.pad(mode="constant", value=0)). */
DNXO_API int dnxo_pad_zero_hwc_f16(const uint16_t *in, int64_t H, int64_t W,
                                   int64_t C, int64_t left, int64_t right,
                                   int64_t top, int64_t bottom, uint16_t *out) {
  if (left < 0 || right < 0 || top < 0 || bottom < 0)
    return -1;
  const int64_t Ho = H + top + bottom, Wo = W + left + right;
  memset(out, 0, (size_t)(Ho * Wo * C) * 2);
  for (int64_t h = 0; h < H; ++h)
    memcpy(out + ((h + top) * Wo + left) * C, in + h * W * C, (size_t)(W * C) * 2);
  return 0;
}

/* Crop.  compiler/.../shaders/slice/memory_slice.comp:55-67:
 *   out[h, w, c] = in[h + top, w + left, c]  for h < out_h, w < out_w.       */
DNXO_API int dnxo_slice_hwc_f16(const uint16_t *in, int64_t H, int64_t W,
                                int64_t C, int64_t left, int64_t top,
                                int64_t out_h, int64_t out_w, uint16_t *out) {
  if (left < 0 || top < 0 || top + out_h > H || left + out_w > W)
    return -1;
  for (int64_t h = 0; h < out_h; ++h)
    memcpy(out + h * out_w * C, in + ((h + top) * W + left) * C,
           (size_t)(out_w * C) * 2);
  return 0;
}

/* Stand-alone activation evaluated in binary16.
 * compiler/.../shaders/activation/basic_activation.comp:26-34:
 *   ReLU      : max(v, 0)
 *   LeakyReLU : max(v, alpha * v), alpha converted to binary16, the product
 *               rounded to binary16.                                         */
DNXO_API int dnxo_activation_f16(const uint16_t *in, size_t n, int act,
                                 float alpha, uint16_t *out) {
  const float ah = dnxo_f16_to_f32(dnxo_f32_to_f16(alpha));
  for (size_t i = 0; i < n; ++i) {
    float v = dnxo_f16_to_f32(in[i]);
    if (act == 1) {
      out[i] = (v > 0.0f) ? in[i] : (uint16_t)0; /* max(v,0): -0 and negatives -> +0 */
    } else if (act == 2) {
      float av = dnxo_f16_to_f32(dnxo_f32_to_f16(ah * v));
      out[i] = dnxo_f32_to_f16(v > av ? v : av);
    } else {
      return -1;
    }
  }
  return 0;
}

/* ------------------------------------------------------------------------- */
/* SymIR: straight-line int64 program.
 * common/src/denox/symbolic/SymIR.cpp:5-95 (evaluation) and
 * runtime/src/denox/runtime/model.cpp:395-487 (wire opcode decode):
 *   wire opcode = base | LHSC(0x8000) | RHSC(0x4000); base ADD=1 SUB=2 MUL=3
 *   DIV=4 MOD=5 MIN=6 MAX=7 (dnx.fbs:121-138).  A constant operand is the
 *   literal value, a non-constant operand indexes the value table whose
 *   first var_count slots are the free variables.  DIV truncates like C++,
 *   MOD is made non-negative by adding the divisor.                          */
DNXO_API int dnxo_symir_eval(int64_t var_count, const int64_t *var_values,
                             int64_t n_ops, const uint16_t *opcodes,
                             const int64_t *lhs, const int64_t *rhs,
                             int64_t *dp /* var_count + n_ops */) {
  for (int64_t i = 0; i < var_count; ++i)
    dp[i] = var_values[i];
  for (int64_t pc = 0; pc < n_ops; ++pc) {
    const int lc = (opcodes[pc] & 0x8000u) != 0;
    const int rc = (opcodes[pc] & 0x4000u) != 0;
    const int base = opcodes[pc] & 0x3FFF;
    if (lc && rc)
      return -3; /* both operands constant is never emitted */
    if (!lc && (lhs[pc] < 0 || lhs[pc] >= var_count + pc))
      return -1;
    if (!rc && (rhs[pc] < 0 || rhs[pc] >= var_count + pc))
      return -1;
    const int64_t a = lc ? lhs[pc] : dp[lhs[pc]];
    const int64_t b = rc ? rhs[pc] : dp[rhs[pc]];
    int64_t v;
    switch (base) {
    case 1:
      v = a + b;
      break;
    case 2:
      v = a - b;
      break;
    case 3:
      v = a * b;
      break;
    case 4:
      if (b == 0)
        return -2;
      v = a / b;
      break;
    case 5:
      if (b == 0)
        return -2;
      v = a % b;
      if (v < 0)
        v += b;
      break;
    case 6:
      v = a < b ? a : b;
      break;
    case 7:
      v = a > b ? a : b;
      break;
    default:
      return -3;
    }
    dp[var_count + pc] = v;
  }
  return 0;
}

DNXO_API int dnxo_num_threads(void) {
#if defined(_OPENMP)
  return omp_get_max_threads();
#else
  return 1;
#endif
}
