// SHA-256 (FIPS 180-4) for content-addressed kernel code objects, the role of
// GlslCompilerInstance::fast_sha256 in the reference
// (spirv/src/denox/glsl/GlslCompilerInstance.hpp:18-81).
#pragma once
#include <array>
#include <cstdint>
#include <cstring>
#include <string>

namespace denox {

class Sha256 {
public:
  Sha256() { reset(); }
  void reset() {
    static const uint32_t init[8] = {0x6a09e667, 0xbb67ae85, 0x3c6ef372, 0xa54ff53a, 0x510e527f, 0x9b05688c, 0x1f83d9ab, 0x5be0cd19};
    std::memcpy(m_h, init, sizeof(init));
    m_len = 0; m_fill = 0;
  }
  void update(const void *data, size_t n) {
    const uint8_t *p = static_cast<const uint8_t *>(data);
    m_len += n;
    while (n > 0) {
      const size_t k = std::min<size_t>(n, 64 - m_fill);
      std::memcpy(m_buf + m_fill, p, k);
      m_fill += k; p += k; n -= k;
      if (m_fill == 64) { block(m_buf); m_fill = 0; }
    }
  }
  void update(const std::string &s) { update(s.data(), s.size()); }
  std::array<uint8_t, 32> digest() {
    const uint64_t bits = m_len * 8;
    const uint8_t pad = 0x80;
    update(&pad, 1);
    const uint8_t zero = 0;
    while (m_fill != 56) update(&zero, 1);
    uint8_t lenb[8];
    for (int i = 0; i < 8; ++i) lenb[i] = static_cast<uint8_t>(bits >> (56 - 8 * i));
    update(lenb, 8);
    std::array<uint8_t, 32> out;
    for (int i = 0; i < 8; ++i)
      for (int j = 0; j < 4; ++j) out[i * 4 + j] = static_cast<uint8_t>(m_h[i] >> (24 - 8 * j));
    return out;
  }
  static std::string hex(const std::array<uint8_t, 32> &d) {
    static const char *x = "0123456789abcdef";
    std::string s;
    for (uint8_t b : d) { s.push_back(x[b >> 4]); s.push_back(x[b & 15]); }
    return s;
  }

private:
  static uint32_t rotr(uint32_t v, int s) { return (v >> s) | (v << (32 - s)); }
  void block(const uint8_t *b) {
    static const uint32_t K[64] = {
        0x428a2f98, 0x71374491, 0xb5c0fbcf, 0xe9b5dba5, 0x3956c25b, 0x59f111f1, 0x923f82a4, 0xab1c5ed5, 0xd807aa98, 0x12835b01, 0x243185be, 0x550c7dc3, 0x72be5d74, 0x80deb1fe, 0x9bdc06a7, 0xc19bf174,
        0xe49b69c1, 0xefbe4786, 0x0fc19dc6, 0x240ca1cc, 0x2de92c6f, 0x4a7484aa, 0x5cb0a9dc, 0x76f988da, 0x983e5152, 0xa831c66d, 0xb00327c8, 0xbf597fc7, 0xc6e00bf3, 0xd5a79147, 0x06ca6351, 0x14292967,
        0x27b70a85, 0x2e1b2138, 0x4d2c6dfc, 0x53380d13, 0x650a7354, 0x766a0abb, 0x81c2c92e, 0x92722c85, 0xa2bfe8a1, 0xa81a664b, 0xc24b8b70, 0xc76c51a3, 0xd192e819, 0xd6990624, 0xf40e3585, 0x106aa070,
        0x19a4c116, 0x1e376c08, 0x2748774c, 0x34b0bcb5, 0x391c0cb3, 0x4ed8aa4a, 0x5b9cca4f, 0x682e6ff3, 0x748f82ee, 0x78a5636f, 0x84c87814, 0x8cc70208, 0x90befffa, 0xa4506ceb, 0xbef9a3f7, 0xc67178f2};
    uint32_t w[64];
    for (int i = 0; i < 16; ++i) w[i] = (uint32_t(b[i * 4]) << 24) | (uint32_t(b[i * 4 + 1]) << 16) | (uint32_t(b[i * 4 + 2]) << 8) | b[i * 4 + 3];
    for (int i = 16; i < 64; ++i) {
      const uint32_t s0 = rotr(w[i - 15], 7) ^ rotr(w[i - 15], 18) ^ (w[i - 15] >> 3);
      const uint32_t s1 = rotr(w[i - 2], 17) ^ rotr(w[i - 2], 19) ^ (w[i - 2] >> 10);
      w[i] = w[i - 16] + s0 + w[i - 7] + s1;
    }
    uint32_t a = m_h[0], bb = m_h[1], c = m_h[2], d = m_h[3], e = m_h[4], f = m_h[5], g = m_h[6], h = m_h[7];
    for (int i = 0; i < 64; ++i) {
      const uint32_t S1 = rotr(e, 6) ^ rotr(e, 11) ^ rotr(e, 25);
      const uint32_t ch = (e & f) ^ (~e & g);
      const uint32_t t1 = h + S1 + ch + K[i] + w[i];
      const uint32_t S0 = rotr(a, 2) ^ rotr(a, 13) ^ rotr(a, 22);
      const uint32_t mj = (a & bb) ^ (a & c) ^ (bb & c);
      const uint32_t t2 = S0 + mj;
      h = g; g = f; f = e; e = d + t1; d = c; c = bb; bb = a; a = t1 + t2;
    }
    m_h[0] += a; m_h[1] += bb; m_h[2] += c; m_h[3] += d; m_h[4] += e; m_h[5] += f; m_h[6] += g; m_h[7] += h;
  }
  uint32_t m_h[8];
  uint8_t m_buf[64];
  uint64_t m_len;
  size_t m_fill;
};

} // namespace denox
