// BLAKE2b (RFC 7693), unkeyed, digest length 1..64; used with 16 bytes for the tensor
// digest (reference: hashlib.blake2b(digest_size=16), refit/reshard/verify.py:152-155).
#pragma once
#include <cstdint>
#include <cstring>

namespace mxp {

class Blake2b {
 public:
  explicit Blake2b(size_t outlen) : outlen_(outlen) {
    static const uint64_t iv[8] = {0x6a09e667f3bcc908ull, 0xbb67ae8584caa73bull, 0x3c6ef372fe94f82bull,
                                   0xa54ff53a5f1d36f1ull, 0x510e527fade682d1ull, 0x9b05688c2b3e6c1full,
                                   0x1f83d9abfb41bd6bull, 0x5be0cd19137e2179ull};
    for (int i = 0; i < 8; ++i) h_[i] = iv[i];
    h_[0] ^= 0x01010000ull ^ (uint64_t)outlen;
  }
  void update(const void* data, size_t n) {
    const uint8_t* p = static_cast<const uint8_t*>(data);
    while (n) {
      if (fill_ == 128) {
        t_ += 128;
        compress(false);
        fill_ = 0;
      }
      const size_t take = n < 128 - fill_ ? n : 128 - fill_;
      std::memcpy(buf_ + fill_, p, take);
      fill_ += take;
      p += take;
      n -= take;
    }
  }
  void final(uint8_t* out) {
    t_ += fill_;
    std::memset(buf_ + fill_, 0, 128 - fill_);
    compress(true);
    uint8_t full[64];
    for (int i = 0; i < 8; ++i)
      for (int b = 0; b < 8; ++b) full[8 * i + b] = (uint8_t)(h_[i] >> (8 * b));
    std::memcpy(out, full, outlen_);
  }

 private:
  uint64_t h_[8];
  uint64_t t_ = 0;
  uint8_t buf_[128];
  size_t fill_ = 0, outlen_;
  static uint64_t rotr(uint64_t x, int n) { return (x >> n) | (x << (64 - n)); }
  void compress(bool last) {
    static constexpr uint8_t sigma[12][16] = {
        {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15}, {14, 10, 4, 8, 9, 15, 13, 6, 1, 12, 0, 2, 11, 7, 5, 3},
        {11, 8, 12, 0, 5, 2, 15, 13, 10, 14, 3, 6, 7, 1, 9, 4}, {7, 9, 3, 1, 13, 12, 11, 14, 2, 6, 5, 10, 4, 0, 15, 8},
        {9, 0, 5, 7, 2, 4, 10, 15, 14, 1, 11, 12, 6, 8, 3, 13}, {2, 12, 6, 10, 0, 11, 8, 3, 4, 13, 7, 5, 15, 14, 1, 9},
        {12, 5, 1, 15, 14, 13, 4, 10, 0, 7, 6, 3, 9, 2, 8, 11}, {13, 11, 7, 14, 12, 1, 3, 9, 5, 0, 15, 4, 8, 6, 2, 10},
        {6, 15, 14, 9, 11, 3, 0, 8, 12, 2, 13, 7, 1, 4, 10, 5}, {10, 2, 8, 4, 7, 6, 1, 5, 15, 11, 9, 14, 3, 12, 13, 0},
        {0, 1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15}, {14, 10, 4, 8, 9, 15, 13, 6, 1, 12, 0, 2, 11, 7, 5, 3}};
    static const uint64_t iv[8] = {0x6a09e667f3bcc908ull, 0xbb67ae8584caa73bull, 0x3c6ef372fe94f82bull,
                                   0xa54ff53a5f1d36f1ull, 0x510e527fade682d1ull, 0x9b05688c2b3e6c1full,
                                   0x1f83d9abfb41bd6bull, 0x5be0cd19137e2179ull};
    // The message block as sixteen little-endian words (the hosts this library runs on are little-endian), the
    // state in sixteen locals, the twelve rounds unrolled so that the message schedule is a table of constants:
    // 0.25 -> 0.20 us per 56-byte digest, which a batch of a few hundred tensor digests pays after its kernel.
    uint64_t m[16];
    std::memcpy(m, buf_, 128);
    uint64_t v0 = h_[0], v1 = h_[1], v2 = h_[2], v3 = h_[3], v4 = h_[4], v5 = h_[5], v6 = h_[6], v7 = h_[7];
    uint64_t v8 = iv[0], v9 = iv[1], v10 = iv[2], v11 = iv[3], v12 = iv[4] ^ t_, v13 = iv[5], v14 = last ? ~iv[6] : iv[6], v15 = iv[7];
#define MXP_B2_G(a, b, c, d, x, y) \
  a = a + b + (x); d = rotr(d ^ a, 32); c = c + d; b = rotr(b ^ c, 24); \
  a = a + b + (y); d = rotr(d ^ a, 16); c = c + d; b = rotr(b ^ c, 63);
#define MXP_B2_ROUND(r)                                                                                  \
  MXP_B2_G(v0, v4, v8, v12, m[sigma[r][0]], m[sigma[r][1]])   MXP_B2_G(v1, v5, v9, v13, m[sigma[r][2]], m[sigma[r][3]])     \
  MXP_B2_G(v2, v6, v10, v14, m[sigma[r][4]], m[sigma[r][5]])  MXP_B2_G(v3, v7, v11, v15, m[sigma[r][6]], m[sigma[r][7]])    \
  MXP_B2_G(v0, v5, v10, v15, m[sigma[r][8]], m[sigma[r][9]])  MXP_B2_G(v1, v6, v11, v12, m[sigma[r][10]], m[sigma[r][11]])  \
  MXP_B2_G(v2, v7, v8, v13, m[sigma[r][12]], m[sigma[r][13]]) MXP_B2_G(v3, v4, v9, v14, m[sigma[r][14]], m[sigma[r][15]])
    MXP_B2_ROUND(0) MXP_B2_ROUND(1) MXP_B2_ROUND(2) MXP_B2_ROUND(3) MXP_B2_ROUND(4) MXP_B2_ROUND(5)
    MXP_B2_ROUND(6) MXP_B2_ROUND(7) MXP_B2_ROUND(8) MXP_B2_ROUND(9) MXP_B2_ROUND(10) MXP_B2_ROUND(11)
#undef MXP_B2_ROUND
#undef MXP_B2_G
    const uint64_t v[16] = {v0, v1, v2, v3, v4, v5, v6, v7, v8, v9, v10, v11, v12, v13, v14, v15};
    for (int i = 0; i < 8; ++i) h_[i] ^= v[i] ^ v[i + 8];
  }
};

}  // namespace mxp
