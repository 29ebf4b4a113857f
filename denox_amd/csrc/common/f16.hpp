// binary16 <-> binary32 on the host, round-to-nearest-even.
// (The reference's host conversion, common/src/denox/memory/dtype/f16.cpp:6-20,
// truncates and flushes subnormals; weights given as fp32 are rounded properly here.)
#pragma once
#include <cstdint>
#include <cstring>

namespace denox {

inline float f16_to_f32(uint16_t h) {
  const uint32_t sign = static_cast<uint32_t>(h & 0x8000u) << 16;
  uint32_t exp = (h >> 10) & 0x1Fu;
  uint32_t man = h & 0x3FFu;
  uint32_t bits;
  if (exp == 0) {
    if (man == 0) {
      bits = sign;
    } else {
      int shift = 0;
      while ((man & 0x400u) == 0) {
        man <<= 1;
        ++shift;
      }
      man &= 0x3FFu;
      bits = sign | (static_cast<uint32_t>(113 - shift) << 23) | (man << 13);
    }
  } else if (exp == 31) {
    bits = sign | 0x7F800000u | (man << 13);
  } else {
    bits = sign | ((exp + 112u) << 23) | (man << 13);
  }
  float f;
  std::memcpy(&f, &bits, 4);
  return f;
}

inline uint16_t f32_to_f16(float f) {
  uint32_t x;
  std::memcpy(&x, &f, 4);
  const uint16_t sign = static_cast<uint16_t>((x >> 16) & 0x8000u);
  x &= 0x7FFFFFFFu;
  if (x >= 0x7F800000u)
    return static_cast<uint16_t>(sign | (x > 0x7F800000u ? 0x7E00u : 0x7C00u));
  if (x >= 0x477FF000u)
    return static_cast<uint16_t>(sign | 0x7C00u);
  if (x < 0x38800000u) { // below the smallest normal half: build the subnormal by a float add
    float av;
    std::memcpy(&av, &x, 4);
    const float magic = 0.5f; // adding 0.5 aligns the 10 result bits at the bottom of the mantissa
    float r = av + magic;
    uint32_t rb;
    std::memcpy(&rb, &r, 4);
    return static_cast<uint16_t>(sign | ((rb - 0x3F000000u) & 0xFFFFu));
  }
  const uint32_t mant_odd = (x >> 13) & 1u;
  x += 0xC8000FFFu; // rebias exponent (127 -> 15) and add rounding bias minus one
  x += mant_odd;
  return static_cast<uint16_t>(sign | (x >> 13));
}

} // namespace denox
