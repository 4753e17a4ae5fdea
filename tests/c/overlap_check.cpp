// Host-side check of the plan-time settlement of overlapping writes
// (modelexpress_amd/csrc/mxp_overlap.hpp): for random pairs of pitched boxes (an earlier write and a
// later one into the same buffer), the boxes clip_write leaves of the earlier write are replayed over a
// byte map and must cover exactly the earlier write's bytes that the later write does not cover, each
// once, paired with the source byte the earlier write paired them with (through the element-size ratio
// of a converting write); writes_may_overlap may only say "no" when the boxes share no byte.
// Usage: overlap_check <first seed> <number of seeds>.  Exit status 0 when every pair passes.
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "mxp_overlap.hpp"

using namespace mxp;

namespace {

struct Fail { std::string what; };
#define REQUIRE(cond, ...)                           \
  do {                                               \
    if (!(cond)) {                                   \
      char buf_[512];                                \
      std::snprintf(buf_, sizeof buf_, __VA_ARGS__); \
      throw Fail{std::string(#cond) + ": " + buf_};  \
    }                                                \
  } while (0)

uint64_t span_end(const WriteRec& w) { return w.dst_offset + (w.rows - 1) * w.dst_pitch + w.row_bytes; }

// destination byte -> source byte of the write (or -1)
void paint(const WriteRec& w, uint64_t se, uint64_t de, std::vector<int64_t>& map, std::vector<uint8_t>* hits) {
  for (uint64_t r = 0; r < w.rows; ++r)
    for (uint64_t c = 0; c < w.row_bytes; ++c) {
      const uint64_t at = w.dst_offset + r * w.dst_pitch + c;
      map[at] = (int64_t)(w.src_offset + r * w.src_pitch + c / de * se + (se == de ? c % de : 0));
      if (hits) {
        if ((*hits)[at]) throw Fail{"a destination byte is written twice"};
        (*hits)[at] = 1;
      }
    }
}

WriteRec random_box(std::mt19937_64& g, uint64_t se, uint64_t de, uint64_t buf_elems) {
  auto pick = [&](uint64_t lo, uint64_t hi) { return lo + g() % (hi - lo + 1); };
  WriteRec w;
  w.tensor = 0;
  w.param = 0;
  w.rows = g() % 3 == 0 ? 1 : pick(2, 24);
  const uint64_t row_elems = pick(1, w.rows == 1 ? 400 : 40);
  const uint64_t pitch_elems = row_elems + (g() % 3 == 0 ? 0 : pick(0, 30));
  const uint64_t need = (w.rows - 1) * pitch_elems + row_elems;
  const uint64_t off = pick(0, buf_elems - need);
  w.row_bytes = row_elems * de;
  w.dst_pitch = (w.rows == 1 ? row_elems : pitch_elems) * de;
  w.dst_offset = off * de;
  w.src_pitch = (w.rows == 1 ? row_elems : row_elems + pick(0, 9)) * se;
  w.src_offset = pick(0, 50) * se;
  return w;
}

void check_pair(std::mt19937_64& g) {
  static const uint64_t sizes[][2] = {{1, 1}, {2, 2}, {4, 4}, {4, 2}, {2, 4}, {1, 2}};
  const auto& sz = sizes[g() % 6];
  const uint64_t se = sz[0], de = sz[1], buf_elems = 2400;
  const WriteRec e = random_box(g, se, de, buf_elems);
  WriteRec k = random_box(g, se, de, buf_elems);
  if (g() % 4 == 0) {  // the later write shares the earlier one's pitch: column bands
    k.dst_pitch = e.rows > 1 ? e.dst_pitch : k.dst_pitch;
    if (k.rows > 1 && k.row_bytes > k.dst_pitch) k.row_bytes = k.dst_pitch;
    while (span_end(k) > buf_elems * de && k.rows > 1) --k.rows;
    if (span_end(k) > buf_elems * de) k.dst_offset = 0, k.rows = 1, k.row_bytes = std::min<uint64_t>(k.row_bytes, buf_elems * de);
    if (k.rows == 1) k.dst_pitch = k.row_bytes;
  }
  const uint64_t n = buf_elems * de;
  std::vector<int64_t> first(n, -1), later(n, -1), left(n, -1);
  std::vector<uint8_t> hits(n, 0);
  paint(e, se, de, first, nullptr);
  paint(k, se, de, later, nullptr);
  bool share = false;
  for (uint64_t i = 0; i < n; ++i) share = share || (first[i] >= 0 && later[i] >= 0);
  const bool may = writes_may_overlap(e, k);
  REQUIRE(may || !share, "writes_may_overlap said no for boxes that share a byte");
  const std::vector<WriteRec> pieces = clip_write(e, k, se, de, "p");
  for (const WriteRec& p : pieces) {
    REQUIRE(p.rows >= 1 && p.row_bytes >= 1 && p.row_bytes % de == 0, "piece of %" PRIu64 " rows x %" PRIu64 " bytes", p.rows, p.row_bytes);
    REQUIRE(span_end(p) <= n, "piece leaves the buffer");
    REQUIRE(p.tensor == e.tensor && p.param == e.param && p.cast == e.cast && p.kind == e.kind, "piece fields differ");
    paint(p, se, de, left, &hits);
  }
  for (uint64_t i = 0; i < n; ++i) {
    const int64_t want = later[i] >= 0 ? -1 : first[i];
    REQUIRE(left[i] == want, "byte %" PRIu64 ": source %" PRId64 ", expected %" PRId64, i, left[i], want);
  }
  if (!share) REQUIRE(pieces.size() == 1 && pieces[0].rows == e.rows && pieces[0].row_bytes == e.row_bytes, "an untouched write was cut");
}

}  // namespace

int main(int argc, char** argv) {
  const uint64_t first = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 0;
  const uint64_t count = argc > 2 ? std::strtoull(argv[2], nullptr, 10) : 1000;
  for (uint64_t seed = first; seed < first + count; ++seed) {
    std::mt19937_64 g(seed * 104729 + 7);
    try {
      check_pair(g);
    } catch (const Fail& f) {
      std::fprintf(stderr, "seed %" PRIu64 ": %s\n", seed, f.what.c_str());
      return 1;
    } catch (const std::exception& e) {
      std::fprintf(stderr, "seed %" PRIu64 ": threw: %s\n", seed, e.what());
      return 1;
    }
  }
  std::printf("%" PRIu64 " pairs clipped and replayed\n", count);
  return 0;
}
