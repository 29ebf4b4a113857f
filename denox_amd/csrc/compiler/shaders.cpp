// Kernel families.  Each one matches a pattern of layer operations, lists the
// configurations it can be compiled in and registers the dispatches.
//
// Counterparts in the reference (compiler/src/denox/compiler/implement/shaders/):
//   ConvMfmaShader        conv/DirectConvShader.cpp:26-575, conv/DirectConvShaderCM.cpp:40-695,
//                         conv/ConcatConvCMShader.cpp:39-965
//   BasicPoolShader       pool/BasicPoolShader.cpp:11-610
//   BasicUpsampleShader   upsample/BasicUpsampleShader.cpp:13-604
//   CopyTransformShader   copy/CopyTransformShader.cpp:155-541
//   BasicActivationShader activation/BasicActivationShader.cpp
//   MemoryPadShader       pad/MemoryPadShader.cpp
//   MemorySliceShader     slice/MemorySliceShader.cpp
// registry: shaders.cpp:16-50.
#include "implement.hpp"
#include "../common/f16.hpp"
#include <algorithm>
#include <cstring>
#include <sstream>

namespace denox::compiler {

namespace {

constexpr unsigned WG_BANDWIDTH = 256; // threads per workgroup of the bandwidth kernels

bool singleUse(const Model &m, TensorHandle t) {
  const TensorNode &n = m.tensors()[t];
  return n.consumers.size() == 1 && !n.isOutput;
}

Sym bytesOf(SymGraph &sym, const TensorNode &t) { return sym.mul(sym.mul(t.width, t.height), static_cast<int64_t>(t.channels) * 2); }

std::string fmtFloat(float v) {
  std::ostringstream o;
  o.precision(9);
  o << std::scientific << v << "f";
  return o.str();
}

// ------------------------------------------------------------------ conv
// Two kernel sources share one configuration table: conv3x3_mfma.hip streams the
// weight slice of every reduction step through LDS (any layer size), conv3x3_mfma_ws.hip
// keeps the whole slice resident and runs persistently (layers whose weights fit LDS).
// waves: computing waves; pw: extra staging-only waves (wave specialisation, resident kernel only)
// waves: computing waves; rpw: image rows per wave; ck: input channels per LDS step (0 = all, 1 = half);
// resident: weights stay in LDS (persistent launch); pw: extra staging-only waves; maxKT: cap on output channels
// per workgroup (0 = none); mf: matrix shape 32 (32x32x16) or 16 (16x16x32); xb: 16-pixel blocks per row (mf 16).
// pp: two-phase schedule of the persistent kernel (two wave groups alternate matrix work and everything else).
// fold: the 2x upsample of source A folded into the weights (conv3x3_upfold.hip, with pw: conv3x3_upfold_ws.hip; rpw counts low-resolution rows).
// ntStore: the result is stored with the non-temporal cache policy.
// ostage: the finished tile goes to memory through LDS, stored by the staging waves (OSTAGE in conv3x3_mfma_ws.hip).
// ksplit: computing waves share a tile's rows AND its output channels (KSP in conv3x3_upfold_ws.hip): wave w takes block
// w % ksplit of the 32-channel blocks and row group w / ksplit.
// hrot: the staged halo unpadded, its 16-byte slots rotated per pixel instead (HROT in conv_common.h: 32-channel steps fit where the
// padded form allowed 16).  swp: the matrix loop reads the next group's fragments while it issues the current group's (SWP).
struct ConvConfig { unsigned waves, rpw, ck; bool resident; unsigned pw; unsigned maxKT; unsigned mf, xb; const char *name; bool pp = false; bool fold = false; bool wideHalo = false; bool ntStore = false; bool ostage = false; unsigned ksplit = 1; bool hrot = false; bool swp = false; };
const ConvConfig kConvConfigs[] = {
    // weights streamed per step
    {4, 2, 16, false, 0, 0, 32, 1, "w4r2k16"}, {4, 2, 32, false, 0, 0, 32, 1, "w4r2k32"}, {4, 4, 16, false, 0, 0, 32, 1, "w4r4k16"}, {4, 4, 32, false, 0, 0, 32, 1, "w4r4k32"},
    {8, 2, 16, false, 0, 0, 32, 1, "w8r2k16"}, {8, 2, 32, false, 0, 0, 32, 1, "w8r2k32"}, {4, 2, 64, false, 0, 0, 32, 1, "w4r2k64"}, {8, 1, 16, false, 0, 0, 32, 1, "w8r1k16"},
    // small tiles / one 32-channel block per workgroup: more workgroups for low-resolution layers
    {4, 1, 16, false, 0, 0, 32, 1, "w4r1k16"}, {4, 1, 32, false, 0, 0, 32, 1, "w4r1k32"}, {4, 1, 32, false, 0, 32, 32, 1, "w4r1k32n"}, {4, 2, 32, false, 0, 32, 32, 1, "w4r2k32n"},
    {2, 2, 32, false, 0, 32, 32, 1, "w2r2k32n"}, {2, 2, 32, false, 0, 0, 32, 1, "w2r2k32"},
    // ck = 0: the whole reduction (or half of it, ck = 1) in one step -- a single round of global loads per workgroup,
    // for layers with so few tiles that load latency, not throughput, is what a workgroup waits for
    {4, 1, 0, false, 0, 32, 32, 1, "w4r1kfn"}, {4, 1, 1, false, 0, 32, 32, 1, "w4r1khn"}, {4, 2, 0, false, 0, 32, 32, 1, "w4r2kfn"}, {2, 2, 0, false, 0, 32, 32, 1, "w2r2kfn"},
    {4, 1, 0, false, 0, 64, 32, 1, "w4r1kfm"}, {4, 2, 1, false, 0, 32, 32, 1, "w4r2khn"},
    // weights resident, persistent launch
    {8, 1, 16, true, 0, 0, 32, 1, "p8r1k16"},  {8, 1, 32, true, 0, 0, 32, 1, "p8r1k32"},  {16, 1, 16, true, 0, 0, 32, 1, "p16r1k16"}, {16, 1, 32, true, 0, 0, 32, 1, "p16r1k32"},
    {8, 2, 16, true, 0, 0, 32, 1, "p8r2k16"},  {8, 2, 32, true, 0, 0, 32, 1, "p8r2k32"},  {16, 2, 16, true, 0, 0, 32, 1, "p16r2k16"}, {4, 2, 32, true, 0, 0, 32, 1, "p4r2k32"},
    {8, 4, 16, true, 0, 0, 32, 1, "p8r4k16"},  {4, 4, 16, true, 0, 0, 32, 1, "p4r4k16"},  {4, 4, 32, true, 0, 0, 32, 1, "p4r4k32"},   {4, 1, 32, true, 0, 0, 32, 1, "p4r1k32"},
    {4, 2, 32, true, 0, 32, 32, 1, "p4r2k32n"}, {4, 1, 32, true, 0, 32, 32, 1, "p4r1k32n"},
    // resident + staging-only waves
    {8, 2, 16, true, 4, 0, 32, 1, "s8r2k16"},  {12, 1, 16, true, 4, 0, 32, 1, "s12r1k16"},
    // resident + staging-only waves that also store the result (whole pixels per store instruction, through LDS)
    {4, 2, 16, true, 4, 0, 32, 1, "r4r2k16", false, false, false, false, true}, {4, 2, 16, true, 4, 0, 32, 1, "r4r2k16n", false, false, false, true, true},
    {8, 1, 16, true, 4, 0, 32, 1, "r8r1k16n", false, false, false, true, true}, {4, 2, 32, true, 4, 0, 32, 1, "r4r2k32n", false, false, false, true, true},
    {4, 1, 16, true, 4, 0, 32, 1, "r4r1k16n", false, false, false, true, true},
    // ... with the rotated halo layout and the pipelined matrix loop
    {4, 2, 32, true, 4, 0, 32, 1, "c4r2k32n", false, false, false, true, true, 1, true, true}, {4, 2, 16, true, 4, 0, 32, 1, "c4r2k16n", false, false, false, true, true, 1, true, true},
    {4, 2, 16, true, 4, 0, 32, 1, "c4r2k16m", false, false, false, true, true, 1, false, true},
    // the pipelined matrix loop (and, with 32-channel steps, the rotated layout) in the other kernel families
    {4, 2, 16, false, 0, 0, 32, 1, "w4r2k16s", false, false, false, false, false, 1, false, true}, {4, 2, 32, false, 0, 0, 32, 1, "w4r2k32s", false, false, false, false, false, 1, true, true},
    {8, 2, 16, true, 4, 0, 32, 1, "s8r2k16s", false, false, false, false, false, 1, false, true}, {8, 2, 32, true, 4, 0, 32, 1, "s8r2k32s", false, false, false, false, false, 1, true, true},
    {8, 2, 32, true, 0, 0, 32, 1, "p8r2k32s", false, false, false, false, false, 1, true, true},
    // 16x16x32 matrix shape: output channels in blocks of 16, tiles of 16 or 32 pixels width
    {4, 2, 32, false, 0, 0, 16, 2, "m4r2k32x2"}, {4, 2, 64, false, 0, 0, 16, 2, "m4r2k64x2"}, {4, 1, 32, false, 0, 0, 16, 2, "m4r1k32x2"}, {4, 2, 32, false, 0, 0, 16, 1, "m4r2k32x1"},
    {4, 4, 32, false, 0, 0, 16, 1, "m4r4k32x1"}, {8, 2, 32, false, 0, 0, 16, 2, "m8r2k32x2"}, {4, 2, 0, false, 0, 0, 16, 1, "m4r2kfx1"},  {4, 1, 0, false, 0, 0, 16, 2, "m4r1kfx2"},
    {4, 2, 32, false, 0, 32, 16, 2, "m4r2k32x2n"}, {4, 2, 0, false, 0, 32, 16, 1, "m4r2kfx1n"}, {4, 1, 0, false, 0, 48, 16, 1, "m4r1kfx1n"}, {4, 2, 32, false, 0, 48, 16, 1, "m4r2k32x1n"},
    {8, 2, 32, true, 0, 0, 16, 2, "q8r2k32x2"}, {8, 1, 32, true, 0, 0, 16, 2, "q8r1k32x2"}, {4, 2, 32, true, 0, 0, 16, 2, "q4r2k32x2"}, {8, 2, 32, true, 0, 0, 16, 1, "q8r2k32x1"},
    {4, 2, 32, true, 0, 48, 16, 1, "q4r2k32x1n"},
    // resident, two-phase schedule
    {16, 1, 16, true, 0, 0, 32, 1, "t16r1k16", true}, {16, 1, 32, true, 0, 0, 32, 1, "t16r1k32", true}, {16, 2, 16, true, 0, 0, 32, 1, "t16r2k16", true},
    {8, 2, 16, true, 0, 0, 32, 1, "t8r2k16", true},   {8, 2, 32, true, 0, 0, 32, 1, "t8r2k32", true},   {8, 4, 16, true, 0, 0, 32, 1, "t8r4k16", true},
    {8, 1, 16, true, 0, 0, 32, 1, "t8r1k16", true},   {8, 2, 32, true, 0, 0, 16, 2, "u8r2k32x2", true}, {16, 1, 32, true, 0, 0, 16, 2, "u16r1k32x2", true},
    // upsample folded into the weights (layers whose source A is upsampled; one parity class of output pixels per workgroup)
    {8, 1, 16, true, 0, 0, 32, 1, "f8r1", false, true},  {4, 2, 16, true, 0, 0, 32, 1, "f4r2", false, true}, {4, 1, 16, true, 0, 0, 32, 1, "f4r1", false, true},
    // staging-only waves and one row parity (both column parities) per workgroup (conv3x3_upfold_ws.hip; layers with a second source);
    // ck: channels of the upsampled source per step, 0 = all
    {4, 1, 0, true, 4, 0, 32, 1, "g4r1", false, true},   {4, 1, 32, true, 4, 0, 32, 1, "g4r1k32", false, true},
    // ... and non-temporal stores of the result (whole lines written once, never read by this kernel)
    {4, 1, 0, true, 4, 0, 32, 1, "g4r1n", false, true, false, true}, {4, 1, 32, true, 4, 0, 32, 1, "g4r1k32n", false, true, false, true},
    // ... and two rows of half the output channels per wave instead of one row of all of them (fewer LDS reads per matrix instruction)
    {4, 2, 0, true, 4, 0, 32, 1, "h4r2", false, true, false, false, false, 2}, {4, 2, 0, true, 4, 0, 32, 1, "h4r2n", false, true, false, true, false, 2},
    {4, 2, 32, true, 4, 0, 32, 1, "h4r2k32n", false, true, false, true, false, 2},
    // ... and the fragment reads of the matrix loops issued three weight sets ahead (SWP in conv3x3_upfold_ws.hip)
    {4, 2, 0, true, 4, 0, 32, 1, "h4r2p", false, true, false, true, false, 2, false, true}, {4, 1, 0, true, 4, 0, 32, 1, "g4r1p", false, true, false, true, false, 1, false, true},
    {4, 2, 32, true, 4, 0, 32, 1, "h4r2k32p", false, true, false, true, false, 2, false, true},
    // the smallest tiles, offered to strided layers only: a stride multiplies the halo of a tile, and a 7 x 7 filter with
    // stride 4 fits the LDS next to its weights with nothing larger
    {2, 1, 16, false, 0, 32, 32, 1, "w2r1k16n", false, false, true}, {2, 1, 32, false, 0, 16, 16, 1, "m2r1k32x1n", false, false, true},
    {2, 2, 16, false, 0, 32, 32, 1, "w2r2k16n", false, false, true},
};
constexpr unsigned kNumConvConfigs = sizeof(kConvConfigs) / sizeof(kConvConfigs[0]);

// Configurations that are also offered with channel-block-major (CHWC8) sources and / or result: one or two of each kernel
// family and matrix shape, so that the layout alternative adds half as many candidates again instead of three times as many.
bool offeredBlocked(const ConvConfig &cfg) {
  for (const char *n : {"w4r2k16", "w8r2k32", "w4r1kfn", "p16r2k16", "s8r2k16", "t8r2k32", "t16r1k32", "m4r2k32x1", "m8r2k32x2", "m4r2kfx1", "q8r2k32x2", "s12r1k16", "r4r2k16n", "c4r2k32n", "s8r2k32s"})
    if (std::strcmp(n, cfg.name) == 0) return true;
  return false;
}

// A tensor that can exist in the blocked layout: whole 8-channel groups, and not an interface tensor (those keep the layout
// the caller declared; the conversion from and to it is a dispatch of its own).
bool canBeBlocked(const Model &model, TensorHandle t) {
  const TensorNode &n = model.tensors()[t];
  return n.channels % 8 == 0 && !n.isInput && !n.isOutput;
}

enum ConvPatternBits : unsigned { PAT_CONCAT = 1, PAT_UPSAMPLE = 2, PAT_ACT = 4, PAT_POOL = 8, PAT_PADA = 16, PAT_PADB = 32, PAT_CROP = 64, PAT_ACT_FIRST = 128 };

struct ConvGeometry {
  unsigned CA, CB, C, CPAD, K, KOUTP, KT, slots;
  unsigned R = 3, S = 3;   // filter rows / columns (set before chooseKT)
  unsigned SY = 1, SX = 1; // stride (set before chooseKT)
  size_t ldsBytes;
};

// Output channels per workgroup: the largest divisor of KOUTP (in blocks of 32)
// whose weights fit LDS next to the halo(s) and whose accumulators fit the
// register file.
// channels per LDS step of a configuration for a layer with `cpad` padded input channels
unsigned stepChannels(const ConvConfig &cfg, unsigned cpad) {
  const unsigned kstep = cfg.mf == 32 ? 16 : 32;
  if (cfg.ck == 0) return cpad;                                              // everything at once
  if (cfg.ck == 1) return std::max(kstep, (cpad / 2 + kstep - 1) / kstep * kstep); // two steps
  return cfg.ck;
}

// Output channels per workgroup: the largest divisor of KOUTP (in blocks of mf channels)
// whose weights fit LDS next to the halo(s) and whose accumulators fit the register file.
bool chooseKT(const ConvConfig &cfgIn, unsigned CA, unsigned CB, unsigned K, const DeviceInfo &dev, ConvGeometry &g) {
  const unsigned blk = cfgIn.mf, kstep = cfgIn.mf == 32 ? 16 : 32;
  g.CA = CA; g.CB = CB; g.C = CA + CB; g.CPAD = (g.C + kstep - 1) / kstep * kstep; g.K = K; g.KOUTP = (K + blk - 1) / blk * blk;
  ConvConfig cfg = cfgIn;
  cfg.ck = stepChannels(cfgIn, g.CPAD);
  if (cfg.ck > 192 || cfg.ck % kstep) return false; // staging registers; whole matrix steps only
  const unsigned th = cfg.waves * cfg.rpw;
  const unsigned tw = cfg.mf == 32 ? 32 : 16 * cfg.xb;
  const unsigned haloPix = ((th - 1) * g.SY + g.R) * ((tw - 1) * g.SX + g.S), taps = g.R * g.S;
  const unsigned ckp = cfg.hrot ? cfg.ck : cfg.ck + 8; // halves per staged halo pixel
  if (cfg.hrot && (cfg.mf != 32 || g.SY != 1 || g.SX != 1 || (cfg.ck != 16 && cfg.ck != 32 && cfg.ck != 64))) return false;
  if (cfg.swp && (cfg.mf != 32 || g.SY != 1)) return false;
  const unsigned blocks = g.KOUTP / blk;
  // registers per lane: 512 shared by the waves of one SIMD; a workgroup of `waves` waves puts waves/4 on each
  const unsigned wavesPerSimd = (cfg.waves + cfg.pw + 3) / 4;
  const unsigned regBudget = std::min(256u, 512u / wavesPerSimd);
  for (unsigned kb = blocks; kb >= 1; --kb) {
    if (blocks % kb) continue;
    if (cfg.maxKT && kb * blk > cfg.maxKT) continue;
    const unsigned accRegs = cfg.mf == 32 ? kb * cfg.rpw * 16 : kb * cfg.rpw * cfg.xb * 4;
    if (accRegs + 64 + (cfg.mf == 16 ? kb * 4 : 0) > regBudget) continue;
    const size_t lds = (cfg.resident ? static_cast<size_t>(taps * kb * blk) * (g.CPAD + 8) * 2u + 2u * static_cast<size_t>(haloPix) * ckp * 2u
                                     : (static_cast<size_t>(haloPix) * ckp + static_cast<size_t>(taps * kb * blk) * (cfg.ck + 8)) * 2u) +
                       static_cast<size_t>(kb * blk) * 4u + // + the staged bias (fp32)
                       (cfg.ostage ? static_cast<size_t>(th * tw) * (kb * blk / 8 + 1) * 16u : 0u); // + the finished tile (one spare 16-byte slot per pixel)
    if (lds > dev.maxComputeSharedMemory) continue;
    {
      // a thread stages at most 64 halo vectors per step (the kernels' bookkeeping is one bit per vector)
      const unsigned stagers = (cfg.pw ? cfg.pw : cfg.waves) * 64;
      if ((haloPix * (cfg.ck / 8) + stagers - 1) / stagers > 64) continue;
    }
    if (taps > 9 || g.SY > 1 || g.SX > 1) { // larger filters / halos: the registers that stage one step's weights and halo share count as well
      const unsigned vppk = cfg.ck / 8, threads = cfg.waves * 64, stagers = (cfg.pw ? cfg.pw : cfg.waves) * 64;
      const unsigned stage = cfg.resident ? 2 * 4 * ((haloPix * vppk + stagers - 1) / stagers)
                                          : 4 * ((taps * kb * blk * vppk + threads - 1) / threads + (haloPix * vppk + threads - 1) / threads);
      if (accRegs + stage + 48 > regBudget) continue;
    }
    g.KT = kb * blk;
    g.ldsBytes = lds;
    const unsigned nkt = blocks / kb;
    g.slots = std::max(1u, dev.computeUnits / (dev.xcdCount * nkt));
    return true;
  }
  return false;
}

// Which output channel a weight row of a workgroup's KT rows computes (the inverse of the
// lane -> channel assignment of the kernels' epilogues).
unsigned rowChannel(unsigned mf, unsigned KT, unsigned row) {
  if (mf == 32) {
    const unsigned rho = row & 31;
    return (row & ~31u) + 16 * ((rho >> 2) & 1) + 4 * (rho >> 3) + (rho & 3);
  }
  const unsigned kb = row / 16, rho = row % 16, grp = rho / 4, jj = rho % 4, nblocks = KT / 16;
  const bool paired = 2 * (kb / 2) + 1 < nblocks;
  return paired ? 32 * (kb / 2) + 8 * grp + 4 * (kb % 2) + jj : 16 * kb + 4 * grp + jj;
}

// Weight layout the kernels read: [kt][chunk][tap r*S+s][KT rows][len(chunk)], rows
// permuted by rowChannel(); zero for c >= C or k >= K.
// (The resident kernel uses one chunk spanning the whole reduction.)
std::vector<uint8_t> packConvWeights(const Op &conv, const ConvGeometry &g, unsigned ck, unsigned mf) {
  const unsigned R = conv.R, S = conv.S;
  std::vector<uint16_t> out(static_cast<size_t>(g.KOUTP) * R * S * g.CPAD, 0);
  const unsigned nkt = g.KOUTP / g.KT;
  size_t pos = 0;
  for (unsigned kt = 0; kt < nkt; ++kt)
    for (unsigned c0 = 0; c0 < g.CPAD; c0 += ck) {
      const unsigned len = std::min(ck, g.CPAD - c0);
      for (unsigned tap = 0; tap < R * S; ++tap) {
        const unsigned r = tap / S, s = tap % S;
        for (unsigned row = 0; row < g.KT; ++row) {
          const unsigned k = kt * g.KT + rowChannel(mf, g.KT, row);
          for (unsigned e = 0; e < len; ++e, ++pos) {
            const unsigned c = c0 + e;
            if (k < g.K && c < g.C) out[pos] = conv.weights[((static_cast<size_t>(k) * g.C + c) * R + r) * S + s];
          }
        }
      }
    }
  std::vector<uint8_t> bytes(out.size() * 2);
  std::memcpy(bytes.data(), out.data(), bytes.size());
  return bytes;
}

// ---- upsample folded into the weights ------------------------------------------------------------------------
struct FoldGeometry {
  unsigned CA, CB, CAP, CBP, K, KOUTP, KT, slots, bpitch;
  unsigned cka; // channels of the upsampled source per step (staging-wave variant; CAP: one step)
  size_t ldsBytes;
};

bool chooseFold(const ConvConfig &cfg, unsigned CA, unsigned CB, unsigned K, const DeviceInfo &dev, FoldGeometry &g) {
  if (CA % 8 || (CB > 0 && CB < 8)) return false; // whole vectors of A; B's partial last vector is read ending at its last channel
  g.CA = CA; g.CB = CB; g.CAP = (CA + 15) / 16 * 16; g.CBP = CB ? (CB + 15) / 16 * 16 : 0; g.K = K; g.KOUTP = (K + 31) / 32 * 32;
  if (cfg.waves % cfg.ksplit) return false;
  const unsigned tlh = cfg.waves / cfg.ksplit * cfg.rpw, threads = (cfg.pw ? cfg.pw : cfg.waves) * 64; // threads that move halos
  const unsigned classes = cfg.pw ? 2 : 4; // kinds of workgroup: row parities, or row x column parities
  const unsigned aPix = (tlh + 1) * (cfg.pw ? 34 : 33), bPix = (2 * tlh + 1) * (cfg.pw ? 66 : 65), blocks = g.KOUTP / 32;
  const unsigned regBudget = std::min(256u, 512u / ((cfg.waves + cfg.pw + 3) / 4));
  const unsigned nva = (aPix * (g.CAP / 8) + threads - 1) / threads, nvb = CB ? (bPix * (g.CBP / 8) + threads - 1) / threads : 0;
  g.cka = g.CAP;
  if (cfg.pw) { // staging-wave variant: a second source of at most two matrix steps of channels (its weights live in registers), whole
                // 32- or 64-channel slices of the result; A in steps of cfg.ck channels
    if (!CB || g.CBP > 32 || K % 32) return false;
    if (cfg.ck) {
      if (cfg.ck >= g.CAP || g.CAP % cfg.ck) return false;
      g.cka = cfg.ck;
    }
  }
  const unsigned na = g.CAP / g.cka;
  for (unsigned kb = blocks; kb >= 1; --kb) {
    if (blocks % kb) continue;
    if (cfg.maxKT && kb * 32 > cfg.maxKT) continue;
    const unsigned kt = kb * 32;
    if (cfg.pw && kt > 64) continue;
    if (kb % cfg.ksplit) continue;
    const unsigned kbw = kb / cfg.ksplit; // blocks per computing wave
    // computing waves: accumulators, converted tile; waves that move halos: their registers and what locates them (3 per vector)
    if (cfg.pw && 9 * (g.CBP / 16) * kbw * 4 > 96) continue; // the second source's weights live in registers
    if (cfg.pw ? (std::max(2 * kbw * cfg.rpw * 24 + 9 * (g.CBP / 16) * kbw * 4 + 64, nva * 7 + nvb * 7 + 24) > regBudget) : (kb * cfg.rpw * 24 + (nva + nvb) * 4 + 64 > regBudget)) continue;
    for (unsigned pitchPad : {8u, 0u}) { // the B halo gives up its bank-conflict padding where LDS is short
      // the staging-wave variant keeps B's weights in registers and the finished tile (tlh rows of 64 pixels) in LDS
      const size_t lds = (static_cast<size_t>(16 / classes * kt) * (g.CAP + 8) + (cfg.pw ? static_cast<size_t>(tlh) * 64 * kt : CB ? static_cast<size_t>(9 * kt) * (g.CBP + 8) : 8) +
                          static_cast<size_t>(aPix) * (g.CAP + 8 * na) + (CB ? static_cast<size_t>(bPix) * (g.CBP + pitchPad) : 8) + 2 * kt) * 2u; // the last term: the staged bias, fp32
      if (lds > dev.maxComputeSharedMemory) continue;
      g.KT = kt; g.bpitch = g.CBP + pitchPad; g.ldsBytes = lds;
      g.slots = std::max(1u, dev.computeUnits / (dev.xcdCount * classes * (blocks / kb)));
      return true;
    }
  }
  return false;
}

// Folded weights: [class a*2+b][kt][A tap ty*2+tx][KT rows][CAP] [B tap r*3+s][KT rows][CBP].  Tap r of output row
// parity a reads low-resolution row y + a - 1 + ty with ty = (r + 1) / 2 for a = 0 and r / 2 for a = 1 (columns alike);
// coinciding taps are summed in fp32 and rounded to binary16 once.
std::vector<uint8_t> packFoldWeights(const Op &conv, const FoldGeometry &g) {
  const unsigned nkt = g.KOUTP / g.KT, C = g.CA + g.CB;
  std::vector<uint16_t> out(static_cast<size_t>(4) * g.KOUTP * (4 * g.CAP + 9 * g.CBP), 0);
  auto tmap = [](unsigned parity, unsigned tap) { return parity == 0 ? (tap + 1) / 2 : tap / 2; };
  size_t pos = 0;
  for (unsigned cls = 0; cls < 4; ++cls) {
    const unsigned a = cls >> 1, b = cls & 1;
    for (unsigned kt = 0; kt < nkt; ++kt) {
      for (unsigned ty = 0; ty < 2; ++ty)
        for (unsigned tx = 0; tx < 2; ++tx)
          for (unsigned row = 0; row < g.KT; ++row) {
            const unsigned k = kt * g.KT + rowChannel(32, g.KT, row);
            for (unsigned c = 0; c < g.CAP; ++c, ++pos) {
              if (k >= g.K || c >= g.CA) continue;
              float sum = 0.0f;
              for (unsigned r = 0; r < 3; ++r)
                for (unsigned s2 = 0; s2 < 3; ++s2)
                  if (tmap(a, r) == ty && tmap(b, s2) == tx) sum += f16_to_f32(conv.weights[((static_cast<size_t>(k) * C + c) * 3 + r) * 3 + s2]);
              out[pos] = f32_to_f16(sum);
            }
          }
      for (unsigned tap = 0; tap < 9; ++tap)
        for (unsigned row = 0; row < g.KT; ++row) {
          const unsigned k = kt * g.KT + rowChannel(32, g.KT, row);
          for (unsigned c = 0; c < g.CBP; ++c, ++pos)
            if (k < g.K && c < g.CB) out[pos] = conv.weights[((static_cast<size_t>(k) * C + g.CA + c) * 3 + tap / 3) * 3 + tap % 3];
        }
    }
  }
  std::vector<uint8_t> bytes(out.size() * 2);
  std::memcpy(bytes.data(), out.data(), bytes.size());
  return bytes;
}

bool isPairConfigName(const std::string &name); // a configuration of the conv -> conv shader below

class ConvMfmaShader final : public IShader {
public:
  explicit ConvMfmaShader(const hip::HipCompiler *c) : m_compiler(c) {}
  std::string name() const override { return "conv3x3_mfma"; }

  // A source of the conv after looking through one optional upsample or pad.
  struct Source { unsigned bits; std::vector<int> ops; int tensor; };
  static std::vector<Source> sourcesOf(const Model &model, TensorHandle t, bool allowUpsample, unsigned padBit, const CompileOptions &opt) {
    std::vector<Source> out;
    out.push_back(Source{0, {}, t});
    const int prod = model.tensors()[t].producer;
    if (prod >= 0) {
      const Op &p = model.ops()[prod];
      if (allowUpsample && p.kind == OpKind::Upsample && p.scale == 2 && opt.features.enableUpsampleFusion) out.push_back(Source{PAT_UPSAMPLE, {prod}, p.inputs[0]});
      // the conv loaders clamp coordinates, which is the replicate mode; a zero-mode pad stays a dispatch of its own
      if (p.kind == OpKind::Pad && p.padMode == PaddingMode::Replicate && opt.features.enablePadFusion) out.push_back(Source{padBit, {prod}, p.inputs[0]});
    }
    return out;
  }

  // What can be folded in front of a convolution (sources seen through an upsample, a replicate pad, a concat) and
  // behind it (activation, then a 2x2 max pool or a crop).  A fused-away tensor may have other consumers: whoever needs
  // it materialised gets it from another edge, and the selection weighs both.
  struct Pro { unsigned bits; std::vector<int> ops; std::vector<int> inputs; };
  struct Epi { unsigned bits; std::vector<int> ops; int output; };
  static bool convSupported(const Op &conv) {
    // filters up to 7 x 7, zero padding up to 15, strides up to 4, no dilation (the reference's conv shaders take
    // kernel size, STRIDE_* and PADDING_* as parameters as well and have no dilation either)
    return conv.kind == OpKind::Conv && !(conv.R < 1 || conv.S < 1 || conv.R > 7 || conv.S > 7 || conv.strideX < 1 || conv.strideY < 1 || conv.strideX > 4 ||
                                          conv.strideY > 4 || conv.padX > 15 || conv.padY > 15 || conv.dilX != 1 || conv.dilY != 1);
  }
  static std::vector<Pro> prologuesOf(const Model &model, const Op &conv, const CompileOptions &opt) {
    const auto &ops = model.ops();
    std::vector<Pro> pros;
    const TensorHandle in = conv.inputs[0];
    for (const Source &s : sourcesOf(model, in, true, PAT_PADA, opt)) pros.push_back(Pro{s.bits, s.ops, {s.tensor}});
    const int prod = model.tensors()[in].producer;
    if (prod >= 0 && ops[prod].kind == OpKind::Concat && opt.features.enableConcatConvFusion) {
      const Op &cat = ops[prod];
      for (const Source &a : sourcesOf(model, cat.inputs[0], true, PAT_PADA, opt))
        for (const Source &b : sourcesOf(model, cat.inputs[1], false, PAT_PADB, opt)) {
          if ((a.bits & PAT_PADA) && (b.bits & PAT_PADB)) continue; // one padded source per dispatch
          Pro p{PAT_CONCAT | a.bits | b.bits, a.ops, {a.tensor, b.tensor}};
          p.ops.insert(p.ops.end(), b.ops.begin(), b.ops.end());
          p.ops.push_back(prod);
          pros.push_back(std::move(p));
        }
    }
    return pros;
  }
  static std::vector<Epi> epiloguesOf(const Model &model, const Op &conv, const CompileOptions &opt) {
    const auto &ops = model.ops();
    std::vector<Epi> epis;
    epis.push_back(Epi{0, {}, conv.output});
    auto poolOk = [](const Op &q) { return q.kind == OpKind::Pool && q.poolFunc == PoolFunction::Max && q.kernelX == 2 && q.kernelY == 2 && q.poolStrideX == 2 && q.poolStrideY == 2 && q.poolPadX == 0 && q.poolPadY == 0; };
    auto tails = [&](TensorHandle t, unsigned bits, std::vector<int> chain) {
      if (!singleUse(model, t)) return;
      const int c = model.tensors()[t].consumers[0];
      if (poolOk(ops[c]) && opt.features.enablePoolFusion) { auto ch = chain; ch.push_back(c); epis.push_back(Epi{bits | PAT_POOL, ch, ops[c].output}); }
      if (ops[c].kind == OpKind::Slice && opt.features.enableSliceFusion) { auto ch = chain; ch.push_back(c); epis.push_back(Epi{bits | PAT_CROP, ch, ops[c].output}); }
    };
    tails(conv.output, 0, {});
    if (singleUse(model, conv.output)) {
      const int c1 = model.tensors()[conv.output].consumers[0];
      if (ops[c1].kind == OpKind::Activation && opt.features.enableConvReluFusion) {
        epis.push_back(Epi{PAT_ACT, {c1}, ops[c1].output});
        tails(ops[c1].output, PAT_ACT, {c1});
      }
    }
    return epis;
  }

  std::vector<Match> matchAll(const Model &model, const CompileOptions &opt) const override {
    std::vector<Match> out;
    const auto &ops = model.ops();
    for (size_t i = 0; i < ops.size(); ++i) {
      const Op &conv = ops[i];
      if (!convSupported(conv)) continue;
      const std::vector<Pro> pros = prologuesOf(model, conv, opt);
      const std::vector<Epi> epis = epiloguesOf(model, conv, opt);
      for (const auto &p : pros)
        for (const auto &e : epis) {
          Match m;
          m.pattern = p.bits | e.bits;
          m.ops = p.ops;
          m.ops.push_back(static_cast<int>(i));
          m.ops.insert(m.ops.end(), e.ops.begin(), e.ops.end());
          m.inputs = p.inputs;
          m.output = e.output;
          // the same dispatch writing straight into the channel range of the concat that consumes its output
          if (opt.features.enableImplicitConcat && concatViewOf(model, m.output).valid) {
            Match v = m;
            v.outputVariant = 1;
            out.push_back(std::move(v));
          }
          // the same dispatch with its sources and / or its result in the blocked layout
          if (opt.features.enableBlockedLayout) {
            const bool inOk = std::all_of(m.inputs.begin(), m.inputs.end(), [&](int t) { return canBeBlocked(model, t); });
            const bool outOk = canBeBlocked(model, m.output);
            for (int fin = 0; fin <= (inOk ? 1 : 0); ++fin)
              for (int fout = 0; fout <= (outOk ? 1 : 0); ++fout) {
                if (!fin && !fout) continue;
                Match v = m;
                v.inputFormats.assign(m.inputs.size(), fin);
                v.outputFormat = fout;
                out.push_back(std::move(v));
              }
          }
          out.push_back(std::move(m));
        }
    }
    return out;
  }

  const Op &opOf(const Model &model, const Match &m, OpKind kind) const {
    for (int o : m.ops) if (model.ops()[o].kind == kind) return model.ops()[o];
    fail(Status::Internal, "conv match lacks an expected operation");
  }

  std::vector<unsigned> acceptMatch(const Model &model, const Match &m, const CompileOptions &opt) const override {
    const Op &conv = opOf(model, m, OpKind::Conv);
    const unsigned CA = model.tensors()[m.inputs[0]].channels;
    const unsigned CB = m.inputs.size() > 1 ? model.tensors()[m.inputs[1]].channels : 0;
    std::vector<unsigned> out;
    // a forced configuration of the conv -> conv shader restricts that shader only: single convolutions keep their choice
    const std::string forced = isPairConfigName(opt.forceConvConfig) ? std::string() : opt.forceConvConfig;
    for (unsigned c = 0; c < kNumConvConfigs; ++c) {
      const ConvConfig &cfg = kConvConfigs[c];
      const unsigned kstep = cfg.mf == 32 ? 16 : 32;
      const unsigned cpad = (CA + CB + kstep - 1) / kstep * kstep;
      if (!forced.empty() && forced != cfg.name) continue;
      if (cfg.fold) {
        const unsigned others = PAT_POOL | PAT_CROP | PAT_PADA;
        FoldGeometry fg;
        if (!m.blocked() && (m.pattern & PAT_UPSAMPLE) && !(m.pattern & others) && conv.R == 3 && conv.S == 3 && conv.padX == 1 && conv.padY == 1 && conv.strideX == 1 && conv.strideY == 1 &&
            opt.features.enableUpsampleFold && chooseFold(cfg, CA, CB, conv.K, opt.deviceInfo, fg)) {
          if (cfg.pw && m.outputVariant) { // the staging-wave variant stores whole 16-byte slots
            const ConcatView v = concatViewOf(model, m.output);
            if (!v.valid || v.pitch % 8 || v.channelOffset % 8) continue;
          }
          out.push_back(c);
        }
        continue;
      }
      if (cfg.wideHalo && conv.strideX == 1 && conv.strideY == 1) continue;
      if (cfg.ostage) { // whole 16-byte slots of a pixel-major result, at least two steps per tile
        if ((m.pattern & (PAT_POOL | PAT_CROP)) || m.outputFormat || conv.K % 8 || (cpad + stepChannels(cfg, cpad) - 1) / stepChannels(cfg, cpad) < 2) continue; // (a shorter last step counts)
        if (m.outputVariant) {
          const ConcatView v = concatViewOf(model, m.output);
          if (!v.valid || v.pitch % 8 || v.channelOffset % 8) continue;
        }
      }
      if (m.blocked()) {
        if (!offeredBlocked(cfg)) continue;
        // block-major sources are read through the per-step buffer resource: every LDS step must lie in one source
        if (!m.inputFormats.empty() && m.inputFormats[0] && CB && CA % stepChannels(cfg, cpad)) continue;
      }
      if (cfg.ck > cpad && cfg.ck != kstep) continue; // a larger stage than the whole reduction adds nothing
      if (cfg.ck <= 1 && cpad <= 32) continue;     // "whole / half reduction" duplicates a fixed-size stage for narrow layers
      if ((m.pattern & PAT_POOL) && (cfg.rpw % 2)) continue;
      if ((cfg.waves + cfg.pw) * 64 > opt.deviceInfo.maxComputeWorkGroupInvocations) continue;
      ConvGeometry g;
      g.R = conv.R; g.S = conv.S; g.SY = conv.strideY; g.SX = conv.strideX;
      if (!chooseKT(cfg, CA, CB, conv.K, opt.deviceInfo, g)) continue;
      out.push_back(c);
    }
    bool forcedFold = false; // a forced upsample-folding configuration leaves matches without an upsample to nobody: not an error
    for (unsigned c = 0; c < kNumConvConfigs; ++c) forcedFold |= kConvConfigs[c].fold && forced == kConvConfigs[c].name;
    if (out.empty() && !forced.empty() && !m.blocked() && !(forcedFold && !(m.pattern & PAT_UPSAMPLE)))
      fail(Status::Unsupported, "conv configuration '" + forced + "' is not valid for this layer");
    return out;
  }

  size_t parameterMemorySize(const Model &model, const Match &m) const override {
    const Op &conv = opOf(model, m, OpKind::Conv);
    const unsigned C = conv.C, cpad = (C + 31) / 32 * 32, kp = (conv.K + 31) / 32 * 32; // upper bound over configurations
    return static_cast<size_t>(kp) * conv.R * conv.S * cpad * 2 + static_cast<size_t>(kp) * 2;
  }

  void implement(OpImpl &impl, const Model &model, const Match &m, unsigned config, SymGraph &sym, const CompileOptions &opt) const override {
    const ConvConfig &cfg = kConvConfigs[config];
    const Op &conv = opOf(model, m, OpKind::Conv);
    const TensorNode &convIn = model.tensors()[conv.inputs[0]];
    const TensorNode &tA = model.tensors()[m.inputs[0]];
    const unsigned CA = tA.channels;
    const unsigned CB = m.inputs.size() > 1 ? model.tensors()[m.inputs[1]].channels : 0;
    ConvGeometry g;
    g.R = conv.R; g.S = conv.S; g.SY = conv.strideY; g.SX = conv.strideX;
    FoldGeometry fg{};
    if (cfg.fold) {
      if (!chooseFold(cfg, CA, CB, conv.K, opt.deviceInfo, fg)) fail(Status::Internal, "conv config rejected at implement time");
      g.CA = CA; g.CB = CB; g.C = CA + CB; g.K = conv.K; g.KOUTP = fg.KOUTP; g.KT = fg.KT; g.slots = fg.slots; g.CPAD = fg.CAP + fg.CBP;
    } else if (!chooseKT(cfg, CA, CB, conv.K, opt.deviceInfo, g)) fail(Status::Internal, "conv config rejected at implement time");
    int act = 0;
    float alpha = 0.0f;
    if (m.pattern & PAT_ACT) {
      const Op &a = opOf(model, m, OpKind::Activation);
      act = a.func == ActivationFunction::ReLU ? 1 : 2;
      alpha = a.alpha;
    }
    const bool pool = (m.pattern & PAT_POOL) != 0, up = (m.pattern & PAT_UPSAMPLE) != 0, crop = (m.pattern & PAT_CROP) != 0;
    const bool padA = (m.pattern & PAT_PADA) != 0, padB = (m.pattern & PAT_PADB) != 0;

    hip::HipCompilerInstance k = m_compiler->read(cfg.fold ? (cfg.pw ? "conv3x3_upfold_ws.hip" : "conv3x3_upfold.hip") : cfg.resident ? "conv3x3_mfma_ws.hip" : "conv3x3_mfma.hip");
    if (cfg.fold) k.define("BPITCH", fg.bpitch ? fg.bpitch : 8);
    if (cfg.fold && cfg.pw) k.define("CKA", fg.cka);
    if (cfg.ksplit > 1) k.define("KSP", cfg.ksplit);
    if (cfg.ntStore) k.define("STORE_AUX", 2);
    if (cfg.ostage) k.define("OSTAGE", 1);
    if (cfg.hrot) k.define("HROT", 1);
    if (cfg.swp) k.define("SWP", 1);
    k.define("CA", CA); k.define("CB", CB); k.define("UPA", up ? 1 : 0);
    k.define("KOUT", conv.K); k.define("KT", g.KT);
    k.define("ACT", act);
    if (act == 2) k.define("ALPHA", fmtFloat(alpha));
    k.define("POOL", pool ? 1 : 0); k.define("HAS_BIAS", conv.hasBias ? 1 : 0);
    if (padA) k.define("PADA", 1);
    if (padB) k.define("PADB", 1);
    if (crop) k.define("CROP", 1);
    k.define("WAVES", cfg.waves); k.define("RPW", cfg.rpw); k.define("CK", cfg.fold ? 16u : stepChannels(cfg, g.CPAD));
    if (cfg.resident) { k.define("SLOTS", g.slots); k.define("NXCD", opt.deviceInfo.xcdCount); } // the grid below is xcdCount * nkt * slots workgroups
    if (cfg.pw) k.define("PW", cfg.pw);
    if (cfg.pp) k.define("PP", 1);
    if (conv.R != 3 || conv.S != 3) { k.define("KR", conv.R); k.define("KS", conv.S); }
    const bool samePad = conv.padY == (conv.R - 1) / 2 && conv.padX == (conv.S - 1) / 2, unitStride = conv.strideX == 1 && conv.strideY == 1;
    if (!samePad) { k.define("PY", conv.padY); k.define("PX", conv.padX); }
    if (!unitStride) { k.define("SY", conv.strideY); k.define("SX", conv.strideX); }
    if (cfg.mf != 32) { k.define("MF", cfg.mf); k.define("XB", cfg.xb); }
    const bool blockedIn = !m.inputFormats.empty() && m.inputFormats[0] != 0, blockedOut = m.outputFormat != 0;
    if (blockedIn) k.define("LAYIN", 1);
    if (blockedOut) k.define("LAYOUT_OUT", 1);
    const ConcatView view = m.outputVariant ? concatViewOf(model, m.output) : ConcatView{};
    if (m.outputVariant && !view.valid) fail(Status::Internal, "conv match writes into a concat that does not exist");
    const bool ovec = view.valid && view.pitch % 8 == 0 && view.channelOffset % 8 == 0;
    if (view.valid) { k.define("OPITCH", view.pitch); k.define("OVEC", ovec ? 1 : 0); }
    std::string entry = "conv" + std::to_string(conv.R) + "x" + std::to_string(conv.S) + (samePad ? "" : "p" + std::to_string(conv.padY) + "x" + std::to_string(conv.padX)) +
                        (unitStride ? "" : "s" + std::to_string(conv.strideY) + "x" + std::to_string(conv.strideX)) + "_c" + std::to_string(CA) + (up ? "u" : "") + (padA ? "e" : "") + (CB ? "p" + std::to_string(CB) + (padB ? "e" : "") : "") + "_k" +
                        std::to_string(conv.K) + (act == 1 ? "_relu" : act == 2 ? "_lrelu" : "") + (pool ? "_pool" : "") + (crop ? "_crop" : "") +
                        (view.valid ? "_into" + std::to_string(view.pitch) + (ovec ? "" : "e") : "") + (blockedIn ? "_bi" : "") + (blockedOut ? "_bo" : "") + "_" + cfg.name;
    k.define("KERNEL_NAME", entry);
    const Sym W = convIn.width, H = convIn.height;
    const TensorNode &convOut = model.tensors()[conv.output]; // the convolution's own result, whatever is fused behind it
    const Sym OW = convOut.width, OH = convOut.height;
    const unsigned th = cfg.waves * cfg.rpw;
    const unsigned nkt = g.KOUTP / g.KT;
    auto d = cfg.fold ? impl.registerDispatch(k, entry, Sym::Const(opt.deviceInfo.xcdCount * (cfg.pw ? 2 : 4) * nkt * g.slots), Sym::Const(1), Sym::Const(1), (cfg.waves + cfg.pw) * 64)
           : cfg.resident ? impl.registerDispatch(k, entry, Sym::Const(opt.deviceInfo.xcdCount * nkt * g.slots), Sym::Const(1), Sym::Const(1), (cfg.waves + cfg.pw) * 64)
                          : impl.registerDispatch(k, entry, sym.cdiv(OW, cfg.mf == 32 ? 32 : 16 * cfg.xb), sym.cdiv(OH, th), Sym::Const(nkt), cfg.waves * 64);
    d.addBinding(dnx::Access::ReadOnly, m.inputs[0]);
    if (CB) d.addBinding(dnx::Access::ReadOnly, m.inputs[1]);
    if (view.valid) {
      // from the range's first channel to the end of its last pixel: (pixels - 1) * pitch + K channels
      const TensorNode &o = model.tensors()[m.output];
      const Sym pixels = sym.mul(o.width, o.height);
      d.addBinding(dnx::Access::WriteOnly, m.output, sym.sub(sym.mul(pixels, static_cast<int64_t>(view.pitch) * 2), static_cast<int64_t>(view.pitch - conv.K) * 2));
    } else d.addBinding(dnx::Access::WriteOnly, m.output);
    const Op convCopy = conv; // the lazy packers outlive the model reference
    const unsigned ck = cfg.resident ? g.CPAD : stepChannels(cfg, g.CPAD);
    TensorId wt = cfg.fold ? impl.createParameter(static_cast<size_t>(4) * fg.KOUTP * (4 * fg.CAP + 9 * fg.CBP) * 2, dnx::ScalarType::F16,
                                                  [convCopy, fg]() { return packFoldWeights(convCopy, fg); })
                           : impl.createParameter(static_cast<size_t>(g.KOUTP) * conv.R * conv.S * g.CPAD * 2, dnx::ScalarType::F16,
                                                  [convCopy, g, ck, mf = cfg.mf]() { return packConvWeights(convCopy, g, ck, mf); });
    d.addParamBinding(wt);
    if (conv.hasBias) {
      const unsigned koutp = g.KOUTP;
      TensorId bt = impl.createParameter(static_cast<size_t>(koutp) * 2, dnx::ScalarType::F16, [convCopy, koutp]() {
        std::vector<uint8_t> b(static_cast<size_t>(koutp) * 2, 0);
        std::memcpy(b.data(), convCopy.bias.data(), convCopy.bias.size() * 2);
        return b;
      });
      d.addParamBinding(bt);
    }
    d.addPushConstant(W, dnx::ScalarType::U32);
    d.addPushConstant(H, dnx::ScalarType::U32);
    if (padA || padB) {
      const Op &pad = opOf(model, m, OpKind::Pad);
      const TensorNode &src = model.tensors()[pad.inputs[0]];
      d.addPushConstant(src.width); d.addPushConstant(src.height); d.addPushConstant(pad.left); d.addPushConstant(pad.top);
    }
    if (crop) {
      const Op &sl = opOf(model, m, OpKind::Slice);
      const TensorNode &o = model.tensors()[m.output];
      d.addPushConstant(o.width); d.addPushConstant(o.height); d.addPushConstant(sl.left); d.addPushConstant(sl.top);
    }
    d.addTraversalFlag();

    const std::string base = "conv" + std::to_string(conv.R) + "x" + std::to_string(conv.S);
    std::string nm = base;
    if (up) nm = "upsample+" + nm;
    if (padA || padB) nm = "pad+" + nm;
    if (m.pattern & PAT_CONCAT) nm = "concat+" + nm;
    if (act == 1) nm += "+relu"; else if (act == 2) nm += "+leaky_relu";
    if (pool) nm += "+maxpool";
    if (crop) nm += "+slice";
    if (view.valid) nm += "+concat";
    d.setName(nm);
    d.setOperation(nm);
    const std::string layouts = m.blocked() ? std::string("/") + (blockedIn ? "chwc8" : "hwc") + ">" + (blockedOut ? "chwc8" : "hwc") : std::string();
    d.setConfig(std::string(cfg.name) + "/kt" + std::to_string(g.KT) + layouts);
    impl.edge().config = cfg.name + layouts;
    // bytes that cross HBM: sources at their stored resolution, weights, bias; the (pooled / cropped) output
    Sym reads = bytesOf(sym, tA);
    if (CB) reads = sym.add(reads, bytesOf(sym, model.tensors()[m.inputs[1]]));
    reads = sym.add(reads, static_cast<int64_t>(conv.K) * conv.C * conv.R * conv.S * 2 + (conv.hasBias ? conv.K * 2 : 0));
    d.setMemoryReads(reads);
    d.setMemoryWrites(bytesOf(sym, model.tensors()[m.output]));
    d.setFlops(sym.mul(sym.mul(OW, OH), static_cast<int64_t>(2) * conv.R * conv.S * conv.C * conv.K));
  }

private:
  const hip::HipCompiler *m_compiler;
};

// ------------------------------------------------------------------ conv -> conv
// Two consecutive 3x3 convolutions (stride 1, extent-preserving) whose intermediate tensor has at most 32 channels and no
// other consumer, in one dispatch (conv3x3_pair.hip): the intermediate tensor stays in LDS.  Everything the
// single-convolution shader folds in front of a convolution is available in front of the first one, everything it folds
// behind a convolution behind the second one.  The reference fuses for the same purpose -- to keep a tensor from
// crossing memory -- in ConcatConvCMShader (conv/ConcatConvCMShader.cpp:760-965); a conv -> conv fusion it does not have.
// ck: input channels of the first convolution per LDS stage; pw: extra waves that only move halos (the others then only compute)
// w1reg: the first convolution's weights in registers of the computing waves (needs pw)
// c2stage: the second convolution, its epilogue and its stores on the staging waves (needs pw == waves)
// dlds: halos loaded from memory straight into LDS by the staging waves (DLDS in conv_common.h; needs pw, channel counts that
// are multiples of 8 and every LDS stage inside one source); nbuf: halo buffers (3: those loads are issued two stages ahead)
struct PairConfig { unsigned waves, rpw, ck; const char *name; unsigned pw = 0; bool w1reg = false; bool c2stage = false; bool dlds = false; unsigned nbuf = 2; };
const PairConfig kPairConfigs[] = {{8, 2, 16, "x8r2k16"}, {4, 2, 32, "x4r2k32"}, {4, 4, 16, "x4r4k16"}, {4, 2, 16, "x4r2k16"},
                                   {4, 2, 32, "y4r2k32", 4}, {4, 2, 64, "z4r2k64", 4, true},
                                   {4, 2, 64, "v4r2k64", 4, true, true}, {4, 2, 16, "v4r2k16", 4, true, true}, {4, 2, 32, "u4r2k32", 4, false, true},
                                   {4, 2, 64, "d4r2k64", 4, true, true, true},
                                   {4, 2, 32, "t4r2k32", 4, false, true, true, 3}};
constexpr unsigned kNumPairConfigs = sizeof(kPairConfigs) / sizeof(kPairConfigs[0]);

bool isPairConfigName(const std::string &name) {
  for (const PairConfig &c : kPairConfigs) if (name == c.name) return true;
  return false;
}

struct PairGeometry { unsigned CA, CB, C, CPAD, K1, K2, ck, slots; bool tapm; size_t ldsBytes; };

bool choosePair(const PairConfig &cfg, unsigned CA, unsigned CB, unsigned K1, unsigned K2, bool pool, const DeviceInfo &dev, PairGeometry &g) {
  g.CA = CA; g.CB = CB; g.C = CA + CB; g.CPAD = (g.C + 15) / 16 * 16; g.K1 = K1; g.K2 = K2;
  if (K1 > 32 || K2 > 32 || cfg.ck % 16 || cfg.ck > 64) return false;
  if (cfg.ck > g.CPAD && cfg.ck != 16) return false; // a larger stage than the whole reduction adds nothing
  g.ck = std::min(cfg.ck, g.CPAD);
  const unsigned ih = cfg.waves * cfg.rpw, haloPix = (ih + 2) * 34, ckp = g.ck + 8, threads = (cfg.pw ? cfg.pw : cfg.waves) * 64; // threads that move halos
  if ((haloPix * (g.ck / 8) + threads - 1) / threads > 64) return false;
  if (cfg.dlds && (!cfg.pw || CA % 8 || CB % 8 || (CB && CA % g.ck))) return false;
  const unsigned regBudget = std::min(256u, 512u / ((cfg.waves + cfg.pw + 3) / 4));
  // A second convolution with at most 5 output channels carries its three filter columns in the matrix rows (TAPM in
  // conv3x3_pair.hip): a third of the matrix instructions, weights of 3 instead of 9 taps in registers.
  g.tapm = 3 * K2 <= 15 && !pool;
  // the second convolution's weights (taps x 2 fragments of 4 registers), one accumulator set, fragments, the converted tile, halo registers
  if ((g.tapm ? 24 : 72) + cfg.rpw * 16 + 96 > regBudget) return false;
  if (cfg.c2stage) {
    // a staging wave then holds, besides its two sets of halo registers, what the second convolution needs
    const unsigned nv = cfg.dlds ? 0 : (haloPix * (g.ck / 8) + threads - 1) / threads; // (straight into LDS: no halo registers)
    if (cfg.pw != cfg.waves || 2 * nv * 4 + (g.tapm ? 24 : 72) + cfg.rpw * 16 + 2 * (cfg.rpw + 2) * 4 + 48 > regBudget) return false;
  }
  const unsigned nchunk = (g.CPAD + g.ck - 1) / g.ck;
  const unsigned ringRows = nchunk == 1 ? 2 * ih + 2 : ih + 2; // see conv3x3_pair.hip
  if (cfg.w1reg && 9 * (g.CPAD / 16) * 4 > 144) return false; // the first convolution's weights must fit the register file next to everything else
  // (straight into LDS: unpadded pixels, whole loads of all staging threads)
  const size_t haloBytes = cfg.dlds ? static_cast<size_t>((haloPix * (g.ck / 8) + threads - 1) / threads) * threads * 16 : static_cast<size_t>(haloPix) * ckp * 2;
  g.ldsBytes = (cfg.w1reg ? 0 : static_cast<size_t>(9 * 32) * (g.CPAD + 8) * 2) + cfg.nbuf * haloBytes + (static_cast<size_t>(ringRows) * 32 + 2) * 40 * 2 + 2 * 32 * 4;
  if (g.ldsBytes > dev.maxComputeSharedMemory) return false;
  g.slots = std::max(1u, dev.computeUnits / dev.xcdCount);
  return true;
}

// [tap][32 rows][cpad] with the rows permuted as the kernels' epilogue expects (rowChannel), zero beyond K and C
std::vector<uint8_t> packPairWeights(const Op &conv, unsigned cpad) {
  ConvGeometry g{};
  g.C = conv.C; g.CPAD = cpad; g.K = conv.K; g.KOUTP = 32; g.KT = 32;
  return packConvWeights(conv, g, cpad, 32);
}

// Second convolution with its filter columns in the matrix rows: [r][32 rows][32 channels]; the row that the epilogue
// reads as channel s * K + k holds W[k][c][r][s] (zero elsewhere).
std::vector<uint8_t> packPairWeightsTapM(const Op &conv) {
  std::vector<uint16_t> out(static_cast<size_t>(3) * 32 * 32, 0);
  for (unsigned r = 0; r < 3; ++r)
    for (unsigned row = 0; row < 32; ++row) {
      const unsigned lam = rowChannel(32, 32, row);
      if (lam >= 3 * conv.K) continue;
      const unsigned s = lam / conv.K, k = lam % conv.K;
      for (unsigned c = 0; c < conv.C; ++c) out[(static_cast<size_t>(r) * 32 + row) * 32 + c] = conv.weights[((static_cast<size_t>(k) * conv.C + c) * 3 + r) * 3 + s];
    }
  std::vector<uint8_t> bytes(out.size() * 2);
  std::memcpy(bytes.data(), out.data(), bytes.size());
  return bytes;
}

class ConvPairShader final : public IShader {
public:
  explicit ConvPairShader(const hip::HipCompiler *c) : m_compiler(c) {}
  std::string name() const override { return "conv3x3_pair"; }

  static bool plain3x3(const Op &c) {
    return ConvMfmaShader::convSupported(c) && c.R == 3 && c.S == 3 && c.strideX == 1 && c.strideY == 1 && c.padX == 1 && c.padY == 1 && c.K <= 32;
  }

  std::vector<Match> matchAll(const Model &model, const CompileOptions &opt) const override {
    std::vector<Match> out;
    if (!opt.features.enableConvConvFusion) return out;
    const auto &ops = model.ops();
    for (size_t i = 0; i < ops.size(); ++i) {
      const Op &first = ops[i];
      if (!plain3x3(first) || !singleUse(model, first.output)) continue;
      std::vector<int> mid{static_cast<int>(i)};
      unsigned midBits = 0;
      int next = model.tensors()[first.output].consumers[0];
      if (ops[next].kind == OpKind::Activation && opt.features.enableConvReluFusion && singleUse(model, ops[next].output)) {
        mid.push_back(next);
        midBits = PAT_ACT_FIRST;
        next = model.tensors()[ops[next].output].consumers[0];
      }
      const Op &second = ops[next];
      if (!plain3x3(second) || second.C != first.K) continue;
      mid.push_back(next);
      for (const auto &p : ConvMfmaShader::prologuesOf(model, first, opt))
        for (const auto &e : ConvMfmaShader::epiloguesOf(model, second, opt)) {
          Match m;
          m.pattern = p.bits | e.bits | midBits;
          m.ops = p.ops;
          m.ops.insert(m.ops.end(), mid.begin(), mid.end());
          m.ops.insert(m.ops.end(), e.ops.begin(), e.ops.end());
          m.inputs = p.inputs;
          m.output = e.output;
          // the same dispatch with its sources and / or its result in the blocked layout
          if (opt.features.enableBlockedLayout) {
            const bool inOk = std::all_of(m.inputs.begin(), m.inputs.end(), [&](int t) { return canBeBlocked(model, t); });
            const bool outOk = canBeBlocked(model, m.output);
            for (int fin = 0; fin <= (inOk ? 1 : 0); ++fin)
              for (int fout = 0; fout <= (outOk ? 1 : 0); ++fout) {
                if (!fin && !fout) continue;
                Match v = m;
                v.inputFormats.assign(m.inputs.size(), fin);
                v.outputFormat = fout;
                out.push_back(std::move(v));
              }
          }
          out.push_back(std::move(m));
        }
    }
    return out;
  }

  // the two convolutions of a match, in order
  static std::pair<const Op *, const Op *> convsOf(const Model &model, const Match &m) {
    const Op *a = nullptr, *b = nullptr;
    for (int o : m.ops)
      if (model.ops()[o].kind == OpKind::Conv) (a ? b : a) = &model.ops()[o];
    if (!a || !b) fail(Status::Internal, "conv pair match lacks a convolution");
    return {a, b};
  }

  std::vector<unsigned> acceptMatch(const Model &model, const Match &m, const CompileOptions &opt) const override {
    const auto [first, second] = convsOf(model, m);
    const unsigned CA = model.tensors()[m.inputs[0]].channels;
    const unsigned CB = m.inputs.size() > 1 ? model.tensors()[m.inputs[1]].channels : 0;
    std::vector<unsigned> out;
    for (unsigned c = 0; c < kNumPairConfigs; ++c) {
      const PairConfig &cfg = kPairConfigs[c];
      if (isPairConfigName(opt.forceConvConfig) && opt.forceConvConfig != cfg.name) continue;
      if ((m.pattern & PAT_POOL) && (cfg.rpw % 2)) continue;
      if ((cfg.waves + cfg.pw) * 64 > opt.deviceInfo.maxComputeWorkGroupInvocations) continue;
      PairGeometry g;
      if (!choosePair(cfg, CA, CB, first->K, second->K, (m.pattern & PAT_POOL) != 0, opt.deviceInfo, g)) continue;
      // block-major sources are read through the per-step buffer resource: every LDS step must lie in one source
      if (!m.inputFormats.empty() && m.inputFormats[0] && CB && CA % g.ck) continue;
      out.push_back(c);
    }
    return out;
  }

  size_t parameterMemorySize(const Model &model, const Match &m) const override {
    const auto [first, second] = convsOf(model, m);
    return static_cast<size_t>(9 * 32) * ((first->C + 15) / 16 * 16 + 32) * 2 + 4 * 32;
    (void)second;
  }

  void implement(OpImpl &impl, const Model &model, const Match &m, unsigned config, SymGraph &sym, const CompileOptions &opt) const override {
    const PairConfig &cfg = kPairConfigs[config];
    const auto [firstP, secondP] = convsOf(model, m);
    const Op &first = *firstP, &second = *secondP;
    const TensorNode &convIn = model.tensors()[first.inputs[0]];
    const TensorNode &tA = model.tensors()[m.inputs[0]];
    const unsigned CA = tA.channels, CB = m.inputs.size() > 1 ? model.tensors()[m.inputs[1]].channels : 0;
    PairGeometry g;
    if (!choosePair(cfg, CA, CB, first.K, second.K, (m.pattern & PAT_POOL) != 0, opt.deviceInfo, g)) fail(Status::Internal, "conv pair config rejected at implement time");
    // activations: the one between the convolutions is the first Activation op of the match when PAT_ACT_FIRST is set
    int act1 = 0, act2 = 0;
    float alpha1 = 0.0f, alpha2 = 0.0f;
    {
      bool seenSecond = false;
      for (int o : m.ops) {
        const Op &op = model.ops()[o];
        if (&op == &second) seenSecond = true;
        if (op.kind != OpKind::Activation) continue;
        const int a = op.func == ActivationFunction::ReLU ? 1 : 2;
        if (!seenSecond) { act1 = a; alpha1 = op.alpha; } else { act2 = a; alpha2 = op.alpha; }
      }
    }
    const bool pool = (m.pattern & PAT_POOL) != 0, up = (m.pattern & PAT_UPSAMPLE) != 0, crop = (m.pattern & PAT_CROP) != 0;
    const bool padA = (m.pattern & PAT_PADA) != 0, padB = (m.pattern & PAT_PADB) != 0;

    hip::HipCompilerInstance k = m_compiler->read("conv3x3_pair.hip");
    k.define("CA", CA); k.define("CB", CB); k.define("UPA", up ? 1 : 0);
    k.define("K1", first.K); k.define("ACT1", act1); k.define("HAS_BIAS1", first.hasBias ? 1 : 0);
    if (act1 == 2) k.define("ALPHA1", fmtFloat(alpha1));
    k.define("KOUT", second.K); k.define("KT", 32); k.define("ACT", act2); k.define("HAS_BIAS", second.hasBias ? 1 : 0);
    if (act2 == 2) k.define("ALPHA", fmtFloat(alpha2));
    k.define("POOL", pool ? 1 : 0);
    if (padA) k.define("PADA", 1);
    if (padB) k.define("PADB", 1);
    if (crop) k.define("CROP", 1);
    k.define("WAVES", cfg.waves); k.define("RPW", cfg.rpw); k.define("CK", g.ck);
    k.define("SLOTS", g.slots); k.define("NXCD", opt.deviceInfo.xcdCount);
    if (g.tapm) k.define("TAPM", 1);
    if (cfg.pw) k.define("PW", cfg.pw);
    if (cfg.w1reg) k.define("W1REG", 1);
    if (cfg.c2stage) k.define("C2STAGE", 1);
    if (cfg.dlds) k.define("DLDS", 1);
    if (cfg.nbuf != 2) k.define("NBUF", cfg.nbuf);
    const bool blockedIn = !m.inputFormats.empty() && m.inputFormats[0] != 0, blockedOut = m.outputFormat != 0;
    if (blockedIn) k.define("LAYIN", 1);
    if (blockedOut) k.define("LAYOUT_OUT", 1);
    auto actName = [](int a) { return a == 1 ? "_relu" : a == 2 ? "_lrelu" : ""; };
    const std::string entry = "convpair_c" + std::to_string(CA) + (up ? "u" : "") + (padA ? "e" : "") + (CB ? "p" + std::to_string(CB) + (padB ? "e" : "") : "") + "_k" +
                              std::to_string(first.K) + actName(act1) + "_k" + std::to_string(second.K) + actName(act2) + (pool ? "_pool" : "") + (crop ? "_crop" : "") + (blockedIn ? "_bi" : "") + (blockedOut ? "_bo" : "") + "_" + cfg.name;
    k.define("KERNEL_NAME", entry);
    auto d = impl.registerDispatch(k, entry, Sym::Const(opt.deviceInfo.xcdCount * g.slots), Sym::Const(1), Sym::Const(1), (cfg.waves + cfg.pw) * 64);
    d.addBinding(dnx::Access::ReadOnly, m.inputs[0]);
    if (CB) d.addBinding(dnx::Access::ReadOnly, m.inputs[1]);
    d.addBinding(dnx::Access::WriteOnly, m.output);
    const Op firstCopy = first, secondCopy = second; // the lazy packers outlive the model reference
    auto biasOf = [](const Op &conv) {
      std::vector<uint8_t> b(32 * 2, 0);
      std::memcpy(b.data(), conv.bias.data(), conv.bias.size() * 2);
      return b;
    };
    d.addParamBinding(impl.createParameter(static_cast<size_t>(9 * 32) * g.CPAD * 2, dnx::ScalarType::F16, [firstCopy, cpad = g.CPAD]() { return packPairWeights(firstCopy, cpad); }));
    if (first.hasBias) d.addParamBinding(impl.createParameter(32 * 2, dnx::ScalarType::F16, [firstCopy, biasOf]() { return biasOf(firstCopy); }));
    if (g.tapm) d.addParamBinding(impl.createParameter(static_cast<size_t>(3 * 32) * 32 * 2, dnx::ScalarType::F16, [secondCopy]() { return packPairWeightsTapM(secondCopy); }));
    else d.addParamBinding(impl.createParameter(static_cast<size_t>(9 * 32) * 32 * 2, dnx::ScalarType::F16, [secondCopy]() { return packPairWeights(secondCopy, 32); }));
    if (second.hasBias) d.addParamBinding(impl.createParameter(32 * 2, dnx::ScalarType::F16, [secondCopy, biasOf]() { return biasOf(secondCopy); }));
    d.addPushConstant(convIn.width, dnx::ScalarType::U32);
    d.addPushConstant(convIn.height, dnx::ScalarType::U32);
    if (padA || padB) {
      const Op *pad = nullptr;
      for (int o : m.ops) if (model.ops()[o].kind == OpKind::Pad) pad = &model.ops()[o];
      if (!pad) fail(Status::Internal, "conv pair match lacks its pad");
      const TensorNode &src = model.tensors()[pad->inputs[0]];
      d.addPushConstant(src.width); d.addPushConstant(src.height); d.addPushConstant(pad->left); d.addPushConstant(pad->top);
    }
    if (crop) {
      const Op *sl = nullptr;
      for (int o : m.ops) if (model.ops()[o].kind == OpKind::Slice) sl = &model.ops()[o];
      if (!sl) fail(Status::Internal, "conv pair match lacks its slice");
      const TensorNode &o = model.tensors()[m.output];
      d.addPushConstant(o.width); d.addPushConstant(o.height); d.addPushConstant(sl->left); d.addPushConstant(sl->top);
    }
    d.addTraversalFlag();

    std::string nm = "conv3x3";
    if (up) nm = "upsample+" + nm;
    if (padA || padB) nm = "pad+" + nm;
    if (m.pattern & PAT_CONCAT) nm = "concat+" + nm;
    if (act1 == 1) nm += "+relu"; else if (act1 == 2) nm += "+leaky_relu";
    nm += "+conv3x3";
    if (act2 == 1) nm += "+relu"; else if (act2 == 2) nm += "+leaky_relu";
    if (pool) nm += "+maxpool";
    if (crop) nm += "+slice";
    d.setName(nm);
    d.setOperation(nm);
    const std::string layouts = m.blocked() ? std::string("/") + (blockedIn ? "chwc8" : "hwc") + ">" + (blockedOut ? "chwc8" : "hwc") : std::string();
    d.setConfig(cfg.name + layouts);
    impl.edge().config = cfg.name + layouts;
    Sym reads = bytesOf(sym, tA);
    if (CB) reads = sym.add(reads, bytesOf(sym, model.tensors()[m.inputs[1]]));
    reads = sym.add(reads, static_cast<int64_t>(first.K) * first.C * 9 * 2 + (first.hasBias ? first.K * 2 : 0) + static_cast<int64_t>(second.K) * second.C * 9 * 2 + (second.hasBias ? second.K * 2 : 0));
    d.setMemoryReads(reads);
    d.setMemoryWrites(bytesOf(sym, model.tensors()[m.output]));
    d.setFlops(sym.mul(sym.mul(convIn.width, convIn.height), static_cast<int64_t>(2) * 9 * (static_cast<int64_t>(first.C) * first.K + static_cast<int64_t>(second.C) * second.K)));
  }

private:
  const hip::HipCompiler *m_compiler;
};

// ------------------------------------------------------------------ bandwidth kernels
// grid.x: workgroups covering one row of w * vectorsPerPixel vectors; grid.y: the rows
// threads per pixel of a bandwidth kernel: one per full chunk of 8 channels; with vec == 1 the thread of the last full
// chunk also moves the partial one behind it (DNX_CHUNKS of the kernels)
unsigned chunksPerPixel(unsigned channels, unsigned vec) { return vec == 8 || channels >= 8 ? channels / 8 : 1; }

// rows per thread of the two-source concat kernel (its RPT): several loads in flight help it on unaligned pixels
unsigned rowsPerThread(unsigned vec) { return vec == 8 ? 1 : 4; }
Sym rowBlocks(SymGraph &sym, Sym rows, unsigned rpt) { return rpt == 1 ? rows : sym.cdiv(rows, rpt); }

Sym rowGrid(SymGraph &sym, Sym w, unsigned vectorsPerPixel) {
  return sym.cdiv(sym.mul(w, static_cast<int64_t>(vectorsPerPixel)), WG_BANDWIDTH);
}
// FLAT mode of activation / pad / slice (kernels/common.h): a row is moved as w * channels / 8 + 1 aligned 16-byte vectors; the
// grid also covers the pixel-by-pixel path of the same kernel (pad with columns added)
Sym rowGridFlat(SymGraph &sym, Sym w, unsigned channels, unsigned vectorsPerPixel) {
  const Sym flat = sym.add(sym.cdiv(sym.mul(w, static_cast<int64_t>(channels)), 8), 1);
  const Sym general = sym.mul(w, static_cast<int64_t>(vectorsPerPixel));
  return sym.cdiv(sym.max(flat, general), WG_BANDWIDTH);
}

class SingleOpShader : public IShader {
public:
  SingleOpShader(const hip::HipCompiler *c, OpKind kind) : m_compiler(c), m_kind(kind) {}
  std::vector<Match> matchAll(const Model &model, const CompileOptions &opt) const override {
    std::vector<Match> out;
    for (size_t i = 0; i < model.ops().size(); ++i) {
      const Op &op = model.ops()[i];
      if (op.kind != m_kind || !supports(op)) continue;
      Match m;
      m.ops = {static_cast<int>(i)};
      m.inputs = op.inputs;
      m.output = op.output;
      // the same dispatch storing straight into the channel range of the concat that consumes its result
      if (m_kind != OpKind::Concat && opt.features.enableImplicitConcat && concatViewOf(model, m.output).valid) {
        Match v = m;
        v.outputVariant = 1;
        out.push_back(std::move(v));
      }
      // the same operation on a tensor stored channel-block-major, plane by plane (pool, upsample, activation: what the
      // reference's shaders take in CHWC8, BasicPoolShader.cpp:150-151; its pad and slice shaders have no such variant)
      if ((m_kind == OpKind::Pool || m_kind == OpKind::Upsample || m_kind == OpKind::Activation) && opt.features.enableBlockedLayout &&
          canBeBlocked(model, m.inputs[0]) && canBeBlocked(model, m.output)) {
        Match v = m;
        v.inputFormats = {1};
        v.outputFormat = 1;
        out.push_back(std::move(v));
      }
      out.push_back(std::move(m));
    }
    return out;
  }

  // Where a single-source dispatch stores: vector width (16-byte stores need an aligned channel range), the kernel
  // definition and name suffix, and the output binding with the bytes it may touch.
  // planes: 0 for a pixel-major tensor, else the number of 8-channel planes of a block-major one -- the kernel is then
  // compiled for 8 channels and launched once per plane (grid.z)
  struct Placement { ConcatView view; unsigned vec; std::string suffix; unsigned planes = 0; };
  static Placement placementOf(const Model &model, const Match &m, unsigned channels) {
    Placement p;
    p.view = m.outputVariant ? concatViewOf(model, m.output) : ConcatView{};
    if (m.outputVariant && !p.view.valid) fail(Status::Internal, "match writes into a concat that does not exist");
    const bool aligned = !p.view.valid || (p.view.pitch % 8 == 0 && p.view.channelOffset % 8 == 0);
    p.vec = channels % 8 == 0 && aligned ? 8 : 1;
    if (p.view.valid) p.suffix = "_into" + std::to_string(p.view.pitch);
    if (m.outputFormat) {
      p.planes = channels / 8;
      p.suffix = "_planar";
    }
    return p;
  }
  static void defineOutput(hip::HipCompilerInstance &k, const Placement &p) {
    if (p.view.valid) k.define("OPITCH", p.view.pitch);
    if (p.planes) { k.define("PLANAR", 1); k.define("CH", 8); } // (overrides the channel count defined before)
  }
  static unsigned kernelChannels(const Placement &p, unsigned channels) { return p.planes ? 8 : channels; }
  // rows moved as runs of halves (FLAT in kernels/common.h): any channel count that is not moved in aligned vectors anyway,
  // into a tensor of its own (inside a concat's wider tensor the rows are not contiguous)
  static bool isFlat(const Placement &p) { return p.vec == 1 && !p.view.valid && !p.planes; }
  static Sym gridZ(const Placement &p) { return Sym::Const(p.planes ? p.planes : 1); }
  static void bindOutput(ComputeDispatchBuilder &d, SymGraph &sym, const Model &model, const Match &m, const Placement &p) {
    if (!p.view.valid) { d.addBinding(dnx::Access::WriteOnly, m.output); return; }
    const TensorNode &o = model.tensors()[m.output];
    d.addBinding(dnx::Access::WriteOnly, m.output,
                 sym.sub(sym.mul(sym.mul(o.width, o.height), static_cast<int64_t>(p.view.pitch) * 2), static_cast<int64_t>(p.view.pitch - o.channels) * 2));
  }
  std::vector<unsigned> acceptMatch(const Model &, const Match &, const CompileOptions &) const override { return {0}; }
  virtual bool supports(const Op &) const { return true; }

protected:
  const hip::HipCompiler *m_compiler;
  OpKind m_kind;
};

class BasicPoolShader final : public SingleOpShader {
public:
  explicit BasicPoolShader(const hip::HipCompiler *c) : SingleOpShader(c, OpKind::Pool) {}
  std::string name() const override { return "basic_pool"; }
  // kernel == stride, no padding (the reference's restriction, BasicPoolShader.cpp:165-180).  The reference's shader
  // also refuses PoolFunction::Avg (BasicPoolShader.cpp:170), which its model and ONNX importer accept
  // (frontend/onnx/details/ops/average_pool.cpp:154); the kernel here has an averaging mode, so such models compile.
  bool supports(const Op &op) const override { return op.kernelX == op.poolStrideX && op.kernelY == op.poolStrideY && op.poolPadX == 0 && op.poolPadY == 0; }
  void implement(OpImpl &impl, const Model &model, const Match &m, unsigned, SymGraph &sym, const CompileOptions &) const override {
    const Op &op = model.ops()[m.ops[0]];
    const TensorNode &in = model.tensors()[m.inputs[0]], &out = model.tensors()[m.output];
    const Placement place = placementOf(model, m, in.channels);
    const unsigned vec = place.vec;
    auto k = m_compiler->read("pool.hip");
    const bool avg = op.poolFunc == PoolFunction::Avg;
    k.define("CH", in.channels); k.define("KX", op.kernelX); k.define("KY", op.kernelY); k.define("VEC", vec);
    if (avg) k.define("AVG", 1);
    defineOutput(k, place);
    const std::string entry = std::string(avg ? "pool_avg_c" : "pool_max_c") + std::to_string(in.channels) + "v" + std::to_string(vec) + place.suffix;
    k.define("KERNEL_NAME", entry);
    auto d = impl.registerDispatch(k, entry, rowGrid(sym, out.width, chunksPerPixel(kernelChannels(place, in.channels), vec)), out.height, gridZ(place), WG_BANDWIDTH);
    d.addBinding(dnx::Access::ReadOnly, m.inputs[0]);
    bindOutput(d, sym, model, m, place);
    d.addPushConstant(in.width); d.addPushConstant(in.height);
    d.setName(std::string(avg ? "avgpool" : "maxpool") + (place.view.valid ? "+concat" : "")); d.setOperation(avg ? "avgpool" : "maxpool"); d.setConfig("vec" + std::to_string(vec) + (place.planes ? "/chwc8" : ""));
    if (place.planes) impl.edge().config = "chwc8";
    d.setMemoryReads(bytesOf(sym, in)); d.setMemoryWrites(bytesOf(sym, out)); d.setFlops(Sym::Const(0));
  }
};

class BasicUpsampleShader final : public SingleOpShader {
public:
  explicit BasicUpsampleShader(const hip::HipCompiler *c) : SingleOpShader(c, OpKind::Upsample) {}
  std::string name() const override { return "basic_upsample"; }
  void implement(OpImpl &impl, const Model &model, const Match &m, unsigned, SymGraph &sym, const CompileOptions &) const override {
    const Op &op = model.ops()[m.ops[0]];
    const TensorNode &in = model.tensors()[m.inputs[0]], &out = model.tensors()[m.output];
    const Placement place = placementOf(model, m, in.channels);
    const unsigned vec = place.vec;
    auto k = m_compiler->read("upsample.hip");
    k.define("CH", in.channels); k.define("SCALE", op.scale); k.define("VEC", vec);
    defineOutput(k, place);
    // rows moved as runs of aligned vectors (kernels/upsample.hip): at most one pixel boundary per vector
    const bool flat = isFlat(place) && in.channels >= 8;
    if (flat) k.define("FLAT", 1);
    const std::string entry = "upsample_c" + std::to_string(in.channels) + "v" + std::to_string(vec) + (flat ? "f" : "") + place.suffix;
    k.define("KERNEL_NAME", entry);
    auto d = impl.registerDispatch(k, entry, flat ? rowGridFlat(sym, out.width, in.channels, 0) : rowGrid(sym, out.width, chunksPerPixel(kernelChannels(place, in.channels), vec)), in.height, gridZ(place), WG_BANDWIDTH);
    d.addBinding(dnx::Access::ReadOnly, m.inputs[0]);
    bindOutput(d, sym, model, m, place);
    d.addPushConstant(in.width); d.addPushConstant(in.height);
    d.setName(std::string("upsample") + (place.view.valid ? "+concat" : "")); d.setOperation("upsample"); d.setConfig("vec" + std::to_string(vec) + (flat ? "/rows" : "") + (place.planes ? "/chwc8" : ""));
    if (place.planes) impl.edge().config = "chwc8";
    d.setMemoryReads(bytesOf(sym, in)); d.setMemoryWrites(bytesOf(sym, out)); d.setFlops(Sym::Const(0));
  }
};

class CopyTransformShader final : public SingleOpShader {
public:
  explicit CopyTransformShader(const hip::HipCompiler *c) : SingleOpShader(c, OpKind::Concat) {}
  std::string name() const override { return "copy_transform"; }
  // Explicit concat: the reference issues one strided channel copy per source (CopyTransformShader.cpp:437-537); here
  // both copies are one launch that writes whole pixels, and the one-source copy serves the in-place mixes below.
  // Implicit concat: the reference aliases two channel-block-major (CHWC8) sources behind one another and needs no
  // dispatch (CopyTransformShader.cpp:198-237, OpImpl.cpp:43-65).  Activations here are pixel-major, where the
  // sources interleave per pixel; the same saving comes from the producer side instead: a source whose only
  // consumer is this concat may be written by its producer straight into its channel range of the output (variant 1
  // of the tensor, ConcatView), and the concat then copies only the sources that were not -- none, in the best case.
  std::vector<Match> matchAll(const Model &model, const CompileOptions &opt) const override {
    std::vector<Match> out;
    for (const Match &m : SingleOpShader::matchAll(model, opt)) {
      out.push_back(m);
      // Block-major sources: the concat is its first source's planes followed by its second source's.  When each source
      // is read by this concat only, the two are placed behind one another inside the result and no dispatch is needed
      // (the reference's implicit concat: placement/placement.cpp:232-255, CopyTransformShader.cpp:198-237).
      if (opt.features.enableImplicitConcat && opt.features.enableBlockedLayout && m.inputs[0] != m.inputs[1] && canBeBlocked(model, m.output) &&
          canBeBlocked(model, m.inputs[0]) && canBeBlocked(model, m.inputs[1]) && singleUse(model, m.inputs[0]) && singleUse(model, m.inputs[1])) {
        Match v = m;
        v.inputFormats = {1, 1};
        v.outputFormat = 1;
        out.push_back(std::move(v));
      }
      if (!opt.features.enableImplicitConcat) continue;
      const bool v0 = concatViewOf(model, m.inputs[0]).valid, v1 = concatViewOf(model, m.inputs[1]).valid;
      for (int a = 0; a <= (v0 ? 1 : 0); ++a)
        for (int b = 0; b <= (v1 ? 1 : 0); ++b) {
          if (!a && !b) continue;
          Match v = m;
          v.inputVariants = {a, b};
          out.push_back(std::move(v));
        }
    }
    return out;
  }
  void implement(OpImpl &impl, const Model &model, const Match &m, unsigned, SymGraph &sym, const CompileOptions &) const override {
    const TensorNode &out = model.tensors()[m.output];
    if (m.outputFormat) { // block-major: aliasing only, no dispatch
      impl.createImplicitConcatConstrain(m.inputs[0], m.inputs[1], m.output);
      impl.edge().config = "implicit/chwc8";
      return;
    }
    unsigned off = 0;
    impl.edge().config = m.inputVariants.empty() ? "copy" : std::string(m.inputVariants[0] ? "in-place" : "copy") + "/" + (m.inputVariants[1] ? "in-place" : "copy");
    if (m.inputVariants.empty()) { // both sources are copied: one launch that writes whole pixels
      const TensorNode &a = model.tensors()[m.inputs[0]], &b = model.tensors()[m.inputs[1]];
      const unsigned vec = (a.channels % 8 == 0 && b.channels % 8 == 0) ? 8 : 1;
      auto k = m_compiler->read("copy_transform.hip");
      k.define("COUNT", a.channels); k.define("COUNT1", b.channels); k.define("VEC", vec);
      // Pixels that are not whole 16-byte vectors are assembled in LDS from aligned loads (FLAT in copy_transform.hip): PQ
      // consecutive pixels per workgroup, a multiple of 8, at most 64 and as many as keep both staged source ranges within
      // 16 KB -- measured at 3840 x 2176: 73 + 73 channels 4.7 TB/s with 128 pixels (37 KB, four workgroups per CU), 5.6 with 64
      // or 32, 5.3 with 16; 64 + 9 channels 5.6 / 5.8 / 5.2 / 3.5 TB/s with 128 / 64 / 32 / 16.
      const unsigned total = a.channels + b.channels;
      const unsigned pq = vec == 1 ? std::min(64u, 16u * 1024u / (total * 2u) / 8u * 8u) : 0;
      const bool flat = pq >= 8;
      const unsigned rpt = flat ? 1 : rowsPerThread(vec);
      if (flat) { k.define("FLAT", 1); k.define("PQ", pq); }
      else if (rpt > 1) k.define("RPT", rpt);
      const std::string entry = "concat_c" + std::to_string(a.channels) + "_c" + std::to_string(b.channels) + "v" + std::to_string(vec) + (flat ? "f" : "");
      k.define("KERNEL_NAME", entry);
      auto d = flat ? impl.registerDispatch(k, entry, sym.cdiv(sym.mul(out.width, out.height), pq), Sym::Const(1), Sym::Const(1), WG_BANDWIDTH)
                    : impl.registerDispatch(k, entry, rowGrid(sym, out.width, chunksPerPixel(a.channels, vec) + chunksPerPixel(b.channels, vec)),
                                            rowBlocks(sym, out.height, rpt), Sym::Const(1), WG_BANDWIDTH);
      d.addBinding(dnx::Access::ReadOnly, m.inputs[0]);
      d.addBinding(dnx::Access::ReadOnly, m.inputs[1]);
      d.addBinding(dnx::Access::WriteOnly, m.output);
      d.addPushConstant(out.width); d.addPushConstant(out.height);
      d.setName("concat-copy"); d.setOperation("concat"); d.setConfig(std::string("vec") + std::to_string(vec) + (flat ? "/lds" : ""));
      d.setMemoryReads(bytesOf(sym, out)); d.setMemoryWrites(bytesOf(sym, out)); d.setFlops(Sym::Const(0));
      return;
    }
    for (int s = 0; s < 2; ++s) {
      const TensorNode &in = model.tensors()[m.inputs[s]];
      if (m.inputVariants[static_cast<size_t>(s)]) { // already where it belongs
        impl.createViewConstrain(m.inputs[s], m.output, static_cast<uint64_t>(off) * 2);
        off += in.channels;
        continue;
      }
      const unsigned vec = (in.channels % 8 == 0 && off % 8 == 0 && out.channels % 8 == 0) ? 8 : 1;
      auto k = m_compiler->read("copy_transform.hip");
      k.define("IN_CH", in.channels); k.define("IN_CH_OFFSET", 0); k.define("OUT_CH", out.channels); k.define("OUT_CH_OFFSET", off);
      k.define("COUNT", in.channels); k.define("VEC", vec);
      const std::string entry = "copy_c" + std::to_string(in.channels) + "_to_c" + std::to_string(out.channels) + "o" + std::to_string(off) + "v" + std::to_string(vec);
      k.define("KERNEL_NAME", entry);
      auto d = impl.registerDispatch(k, entry, rowGrid(sym, in.width, chunksPerPixel(in.channels, vec)), in.height, Sym::Const(1), WG_BANDWIDTH);
      d.addBinding(dnx::Access::ReadOnly, m.inputs[s]);
      d.addBinding(dnx::Access::WriteOnly, m.output);
      d.addPushConstant(in.width); d.addPushConstant(in.height);
      d.setName(s == 0 ? "concat-copy-src0" : "concat-copy-src1"); d.setOperation("concat"); d.setConfig("vec" + std::to_string(vec));
      d.setMemoryReads(bytesOf(sym, in)); d.setMemoryWrites(bytesOf(sym, in)); d.setFlops(Sym::Const(0));
      off += in.channels;
    }
  }
};

class BasicActivationShader final : public SingleOpShader {
public:
  explicit BasicActivationShader(const hip::HipCompiler *c) : SingleOpShader(c, OpKind::Activation) {}
  std::string name() const override { return "basic_activation"; }
  void implement(OpImpl &impl, const Model &model, const Match &m, unsigned, SymGraph &sym, const CompileOptions &) const override {
    const Op &op = model.ops()[m.ops[0]];
    const TensorNode &in = model.tensors()[m.inputs[0]];
    const Placement place = placementOf(model, m, in.channels);
    const unsigned vec = place.vec;
    auto k = m_compiler->read("activation.hip");
    k.define("CH", in.channels); k.define("VEC", vec); k.define("ACT", op.func == ActivationFunction::ReLU ? 1 : 2);
    if (op.func == ActivationFunction::LeakyReLU) k.define("ALPHA", fmtFloat(op.alpha));
    defineOutput(k, place);
    const bool flat = isFlat(place);
    if (flat) k.define("FLAT", 1);
    const std::string entry = std::string(op.func == ActivationFunction::ReLU ? "relu_c" : "leaky_relu_c") + std::to_string(in.channels) + "v" + std::to_string(vec) + (flat ? "f" : "") + place.suffix;
    k.define("KERNEL_NAME", entry);
    auto d = impl.registerDispatch(k, entry, flat ? rowGridFlat(sym, in.width, in.channels, 0) : rowGrid(sym, in.width, chunksPerPixel(kernelChannels(place, in.channels), vec)), in.height, gridZ(place), WG_BANDWIDTH);
    d.addBinding(dnx::Access::ReadOnly, m.inputs[0]);
    bindOutput(d, sym, model, m, place);
    d.addPushConstant(in.width); d.addPushConstant(in.height);
    const char *nm = op.func == ActivationFunction::ReLU ? "relu" : "leaky_relu";
    d.setName(std::string(nm) + (place.view.valid ? "+concat" : "")); d.setOperation(nm); d.setConfig("vec" + std::to_string(vec) + (flat ? "/rows" : "") + (place.planes ? "/chwc8" : ""));
    if (place.planes) impl.edge().config = "chwc8";
    d.setMemoryReads(bytesOf(sym, in)); d.setMemoryWrites(bytesOf(sym, in));
    d.setFlops(sym.mul(sym.mul(in.width, in.height), static_cast<int64_t>(in.channels))); // one FLOP per element, as the reference counts it
  }
};

class MemoryPadShader final : public SingleOpShader {
public:
  explicit MemoryPadShader(const hip::HipCompiler *c) : SingleOpShader(c, OpKind::Pad) {}
  std::string name() const override { return "memory_pad"; }
  void implement(OpImpl &impl, const Model &model, const Match &m, unsigned, SymGraph &sym, const CompileOptions &) const override {
    const Op &op = model.ops()[m.ops[0]];
    const TensorNode &in = model.tensors()[m.inputs[0]], &out = model.tensors()[m.output];
    const Placement place = placementOf(model, m, in.channels);
    const unsigned vec = place.vec;
    auto k = m_compiler->read("pad.hip");
    k.define("CH", in.channels); k.define("VEC", vec);
    const bool zeros = op.padMode == PaddingMode::Zero;
    if (zeros) k.define("ZERO", 1);
    defineOutput(k, place);
    const bool flat = isFlat(place);
    if (flat) k.define("FLAT", 1);
    const std::string entry = std::string(zeros ? "memory_pad_zero_c" : "memory_pad_c") + std::to_string(in.channels) + "v" + std::to_string(vec) + (flat ? "f" : "") + place.suffix;
    k.define("KERNEL_NAME", entry);
    auto d = impl.registerDispatch(k, entry, flat ? rowGridFlat(sym, out.width, in.channels, chunksPerPixel(in.channels, vec)) : rowGrid(sym, out.width, chunksPerPixel(in.channels, vec)), out.height, Sym::Const(1), WG_BANDWIDTH);
    d.addBinding(dnx::Access::ReadOnly, m.inputs[0]);
    bindOutput(d, sym, model, m, place);
    d.addPushConstant(out.width); d.addPushConstant(out.height);
    d.addPushConstant(op.left); d.addPushConstant(op.right); d.addPushConstant(op.top); d.addPushConstant(op.bottom);
    d.setName(std::string("pad") + (place.view.valid ? "+concat" : "")); d.setOperation("pad"); d.setConfig("vec" + std::to_string(vec) + (flat ? "/rows" : ""));
    d.setMemoryReads(bytesOf(sym, in)); d.setMemoryWrites(bytesOf(sym, out)); d.setFlops(Sym::Const(0));
  }
};

class MemorySliceShader final : public SingleOpShader {
public:
  explicit MemorySliceShader(const hip::HipCompiler *c) : SingleOpShader(c, OpKind::Slice) {}
  std::string name() const override { return "memory_slice"; }
  void implement(OpImpl &impl, const Model &model, const Match &m, unsigned, SymGraph &sym, const CompileOptions &) const override {
    const Op &op = model.ops()[m.ops[0]];
    const TensorNode &in = model.tensors()[m.inputs[0]], &out = model.tensors()[m.output];
    const Placement place = placementOf(model, m, in.channels);
    const unsigned vec = place.vec;
    auto k = m_compiler->read("slice.hip");
    k.define("CH", in.channels); k.define("VEC", vec);
    defineOutput(k, place);
    const bool flat = isFlat(place);
    if (flat) k.define("FLAT", 1);
    const std::string entry = "memory_slice_c" + std::to_string(in.channels) + "v" + std::to_string(vec) + (flat ? "f" : "") + place.suffix;
    k.define("KERNEL_NAME", entry);
    auto d = impl.registerDispatch(k, entry, flat ? rowGridFlat(sym, out.width, in.channels, 0) : rowGrid(sym, out.width, chunksPerPixel(in.channels, vec)), out.height, Sym::Const(1), WG_BANDWIDTH);
    d.addBinding(dnx::Access::ReadOnly, m.inputs[0]);
    bindOutput(d, sym, model, m, place);
    d.addPushConstant(op.top); d.addPushConstant(op.left);
    d.addPushConstant(in.width); d.addPushConstant(in.height);
    d.addPushConstant(out.width); d.addPushConstant(out.height);
    d.setName(std::string("slice") + (place.view.valid ? "+concat" : "")); d.setOperation("slice"); d.setConfig("vec" + std::to_string(vec) + (flat ? "/rows" : ""));
    d.setMemoryReads(bytesOf(sym, out)); d.setMemoryWrites(bytesOf(sym, out)); d.setFlops(Sym::Const(0));
  }
};

} // namespace

std::vector<std::string> conv_config_names() {
  std::vector<std::string> names;
  for (const ConvConfig &c : kConvConfigs) names.push_back(c.name);
  for (const PairConfig &c : kPairConfigs) names.push_back(c.name);
  return names;
}

std::vector<std::unique_ptr<IShader>> get_all_shaders(const hip::HipCompiler *c) {
  std::vector<std::unique_ptr<IShader>> s;
  s.push_back(std::make_unique<ConvMfmaShader>(c));
  s.push_back(std::make_unique<ConvPairShader>(c));
  s.push_back(std::make_unique<BasicPoolShader>(c));
  s.push_back(std::make_unique<BasicUpsampleShader>(c));
  s.push_back(std::make_unique<CopyTransformShader>(c));
  s.push_back(std::make_unique<BasicActivationShader>(c));
  s.push_back(std::make_unique<MemoryPadShader>(c));
  s.push_back(std::make_unique<MemorySliceShader>(c));
  return s;
}

} // namespace denox::compiler
