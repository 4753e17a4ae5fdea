// CRC32C (Castagnoli, reflected polynomial 0x82F63B78) for artifact-manifest file and chunk
// checksums: the host-side counterpart of the reference's chunks_for_file / file_checksum
// (modelexpress_common/src/artifact_manifest.rs:260-324; vectors at :382-384:
// "xyz" -> 25236885, "abcd" -> 92c80a31, "ef" -> 6bb2dff5).  Uses the SSE4.2 crc32
// instruction when the host has it, a slicing-by-8 table otherwise.
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <cstring>
#include <memory>
#include <vector>

#include "mxp_internal.hpp"

namespace mxp {
namespace {

struct Tables {
  uint32_t t[8][256];
  Tables() {
    for (uint32_t i = 0; i < 256; ++i) {
      uint32_t c = i;
      for (int k = 0; k < 8; ++k) c = (c >> 1) ^ ((c & 1u) ? 0x82F63B78u : 0u);
      t[0][i] = c;
    }
    for (uint32_t i = 0; i < 256; ++i)
      for (int s = 1; s < 8; ++s) t[s][i] = (t[s - 1][i] >> 8) ^ t[0][t[s - 1][i] & 0xFFu];
  }
};

uint32_t crc_table(uint32_t crc, const uint8_t* p, size_t n) {
  static const Tables T;
  while (n && (reinterpret_cast<uintptr_t>(p) & 7u)) { crc = (crc >> 8) ^ T.t[0][(crc ^ *p++) & 0xFFu]; --n; }
  while (n >= 8) {
    uint64_t w;
    std::memcpy(&w, p, 8);
    w ^= crc;
    crc = T.t[7][w & 0xFF] ^ T.t[6][(w >> 8) & 0xFF] ^ T.t[5][(w >> 16) & 0xFF] ^ T.t[4][(w >> 24) & 0xFF] ^
          T.t[3][(w >> 32) & 0xFF] ^ T.t[2][(w >> 40) & 0xFF] ^ T.t[1][(w >> 48) & 0xFF] ^ T.t[0][(w >> 56) & 0xFF];
    p += 8;
    n -= 8;
  }
  while (n--) crc = (crc >> 8) ^ T.t[0][(crc ^ *p++) & 0xFFu];
  return crc;
}

#if defined(__x86_64__)
__attribute__((target("sse4.2"))) uint32_t crc_hw(uint32_t crc, const uint8_t* p, size_t n) {
  uint64_t c = crc;
  while (n && (reinterpret_cast<uintptr_t>(p) & 7u)) { c = __builtin_ia32_crc32qi((uint32_t)c, *p++); --n; }
  while (n >= 8) {
    uint64_t w;
    std::memcpy(&w, p, 8);
    c = __builtin_ia32_crc32di(c, w);
    p += 8;
    n -= 8;
  }
  while (n--) c = __builtin_ia32_crc32qi((uint32_t)c, *p++);
  return (uint32_t)c;
}
#endif

// crc32c_append semantics: `seed` is a finished CRC of the bytes so far (0 for none).
uint32_t crc32c_append(uint32_t seed, const uint8_t* p, size_t n) {
  uint32_t crc = ~seed;
#if defined(__x86_64__)
  static const bool hw = __builtin_cpu_supports("sse4.2");
  crc = hw ? crc_hw(crc, p, n) : crc_table(crc, p, n);
#else
  crc = crc_table(crc, p, n);
#endif
  return ~crc;
}

}  // namespace
}  // namespace mxp

using namespace mxp;

extern "C" {

uint32_t mxp_crc32c(uint32_t seed, const void* data, uint64_t nbytes) {
  if (!data || nbytes == 0) return seed;
  return crc32c_append(seed, static_cast<const uint8_t*>(data), (size_t)nbytes);
}

int mxp_file_crc32c(const char* path, uint64_t chunk_size, uint32_t* file_crc, uint32_t* chunk_crcs,
                    uint64_t max_chunks, uint64_t* n_chunks) {
  return guard([&] {
    if (!path || chunk_size == 0) throw Error(MXP_ERR_ARG, "mxp_file_crc32c: bad argument");
    const int fd = ::open(path, O_RDONLY);
    if (fd < 0) throw Error(MXP_ERR_IO, std::string("failed to open artifact file ") + path);
    struct Closer { int fd; ~Closer() { ::close(fd); } } closer{fd};
    std::vector<uint8_t> buf((size_t)std::min<uint64_t>(chunk_size, 4u << 20));
    uint32_t whole = 0;
    uint64_t count = 0, in_chunk = 0;
    uint32_t chunk = 0;
    for (;;) {
      const uint64_t want = std::min<uint64_t>(buf.size(), chunk_size - in_chunk);
      const ssize_t r = ::read(fd, buf.data(), (size_t)want);
      if (r < 0) throw Error(MXP_ERR_IO, std::string("failed to read artifact file ") + path);
      if (r == 0) break;
      whole = crc32c_append(whole, buf.data(), (size_t)r);
      chunk = crc32c_append(chunk, buf.data(), (size_t)r);
      in_chunk += (uint64_t)r;
      if (in_chunk == chunk_size) {
        if (chunk_crcs && count < max_chunks) chunk_crcs[count] = chunk;
        ++count;
        chunk = 0;
        in_chunk = 0;
      }
    }
    if (in_chunk) {
      if (chunk_crcs && count < max_chunks) chunk_crcs[count] = chunk;
      ++count;
    }
    if (file_crc) *file_crc = whole;
    if (n_chunks) *n_chunks = count;
    if (chunk_crcs && count > max_chunks) throw Error(MXP_ERR_ARG, "mxp_file_crc32c: more chunks than max_chunks");
  });
}

}  // extern "C"
