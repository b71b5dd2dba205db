// SHA3-256 (FIPS 202), used as the kernel cache key the way the reference keys its
// kernels by a SHA3-256 digest of the term (Analysis/Hash.hs:107-111).  Plain
// Keccak-f[1600] on 64-bit lanes; checked against the FIPS known-answer vectors in tests.
#pragma once
#include <cstdint>
#include <cstring>
#include <string>

namespace acchip {

inline void keccakF1600(uint64_t st[25]) {
  static const uint64_t RC[24] = {
      0x0000000000000001ULL, 0x0000000000008082ULL, 0x800000000000808aULL, 0x8000000080008000ULL,
      0x000000000000808bULL, 0x0000000080000001ULL, 0x8000000080008081ULL, 0x8000000000008009ULL,
      0x000000000000008aULL, 0x0000000000000088ULL, 0x0000000080008009ULL, 0x000000008000000aULL,
      0x000000008000808bULL, 0x800000000000008bULL, 0x8000000000008089ULL, 0x8000000000008003ULL,
      0x8000000000008002ULL, 0x8000000000000080ULL, 0x000000000000800aULL, 0x800000008000000aULL,
      0x8000000080008081ULL, 0x8000000000008080ULL, 0x0000000080000001ULL, 0x8000000080008008ULL};
  static const int ROT[24] = {1, 3, 6, 10, 15, 21, 28, 36, 45, 55, 2, 14, 27, 41, 56, 8, 25, 43, 62, 18, 39, 61, 20, 44};
  static const int PIL[24] = {10, 7, 11, 17, 18, 3, 5, 16, 8, 21, 24, 4, 15, 23, 19, 13, 12, 2, 20, 14, 22, 9, 6, 1};
  for (int round = 0; round < 24; ++round) {
    uint64_t bc[5];
    for (int i = 0; i < 5; ++i) bc[i] = st[i] ^ st[i + 5] ^ st[i + 10] ^ st[i + 15] ^ st[i + 20];
    for (int i = 0; i < 5; ++i) {
      uint64_t t = bc[(i + 4) % 5] ^ ((bc[(i + 1) % 5] << 1) | (bc[(i + 1) % 5] >> 63));
      for (int j = 0; j < 25; j += 5) st[j + i] ^= t;
    }
    uint64_t t = st[1];
    for (int i = 0; i < 24; ++i) {
      int j = PIL[i];
      uint64_t b = st[j];
      st[j] = (t << ROT[i]) | (t >> (64 - ROT[i]));
      t = b;
    }
    for (int j = 0; j < 25; j += 5) {
      for (int i = 0; i < 5; ++i) bc[i] = st[j + i];
      for (int i = 0; i < 5; ++i) st[j + i] ^= (~bc[(i + 1) % 5]) & bc[(i + 2) % 5];
    }
    st[0] ^= RC[round];
  }
}

inline void sha3_256(const void* data, size_t len, uint8_t out[32]) {
  const size_t rate = 136;
  uint64_t st[25];
  std::memset(st, 0, sizeof st);
  const uint8_t* p = static_cast<const uint8_t*>(data);
  auto absorb = [&](const uint8_t* blk) {
    for (size_t i = 0; i < rate / 8; ++i) {
      uint64_t w = 0;
      for (int b = 0; b < 8; ++b) w |= (uint64_t)blk[8 * i + b] << (8 * b);
      st[i] ^= w;
    }
    keccakF1600(st);
  };
  while (len >= rate) {
    absorb(p);
    p += rate;
    len -= rate;
  }
  uint8_t last[136];
  std::memset(last, 0, sizeof last);
  std::memcpy(last, p, len);
  last[len] ^= 0x06;
  last[rate - 1] ^= 0x80;
  absorb(last);
  for (int i = 0; i < 32; ++i) out[i] = (uint8_t)(st[i / 8] >> (8 * (i % 8)));
}

inline std::string sha3_256_hex(const std::string& s) {
  uint8_t d[32];
  sha3_256(s.data(), s.size(), d);
  static const char* hx = "0123456789abcdef";
  std::string r;
  for (int i = 0; i < 32; ++i) {
    r += hx[d[i] >> 4];
    r += hx[d[i] & 15];
  }
  return r;
}

}  // namespace acchip
