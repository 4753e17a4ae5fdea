// Host-side check of the box lowering (modelexpress_amd/csrc/mxp_lower.hpp): random boxes are
// lowered to segments and work items, and the addressing place_kernel performs over those
// tables is replayed on the CPU.  Checked for every box:
//   * every destination byte of the box is written exactly once, from the source byte the box
//     pairs it with (through the conversion's size ratio), and nothing else is written;
//   * every store is whole and aligned to its unit, every load is element aligned;
//   * a contiguous run, and a pitched box whose destination pitch is a multiple of 16, move
//     all but fewer than 32 bytes per row through the widest path, whatever the offsets are;
//   * the reciprocal multiplication the kernel uses in place of a division is exact for every
//     unit of every tile, in-tile offsets fit 32 bits, and a tile of the wide paths is at most
//     one batch of the workgroup.
// Usage: lower_check <first seed> <number of seeds>.  Exit status 0 when every box passes.
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "mxp_lower.hpp"

using namespace mxp;

namespace {

struct Fail {
  std::string what;
};

#define REQUIRE(cond, ...)                            \
  do {                                                \
    if (!(cond)) {                                    \
      char buf_[512];                                 \
      std::snprintf(buf_, sizeof buf_, __VA_ARGS__);  \
      throw Fail{std::string(#cond) + ": " + buf_};   \
    }                                                 \
  } while (0)

uint32_t src_elem(uint32_t op) {
  if (op_narrows(op)) return 4;
  if (op_widens(op)) return op_dst_elem(op) / 2;
  if (op_recodes16(op)) return 2;
  return 1;
}
uint32_t dst_elem(uint32_t op) { return (op == kOpCopy || op == kOpChecksumOnly) ? 1 : op_dst_elem(op); }

void check_box(const BoxCopy& b, const LowerOptions& lo) {
  std::vector<Seg> segs;
  std::vector<WorkItem> work;
  lower_box(b, lo, segs, work);
  const uint64_t src_row = op_src_bytes(b.op, b.row_bytes);
  const uint64_t d_span = b.rows ? (b.rows - 1) * b.dst_pitch + b.row_bytes : 0;
  // destination byte -> source byte (relative to the box origins), or -1 where the box writes nothing
  std::vector<int64_t> want(d_span, -1), got(d_span, -1);
  std::vector<uint8_t> hits(d_span, 0);
  uint64_t wide_bytes = 0;
  const uint64_t ratio_n = op_narrows(b.op) ? 2 : 1, ratio_d = op_widens(b.op) ? 2 : 1;  // src = dst * n / d
  for (uint64_t r = 0; r < b.rows; ++r)
    for (uint64_t c = 0; c < b.row_bytes; ++c) {
      const uint64_t e = dst_elem(b.op);
      // byte c of a destination row comes from the element c / e of the source row
      want[r * b.dst_pitch + c] = (int64_t)(r * b.src_pitch + (c / e) * e * ratio_n / ratio_d);
    }
  for (const WorkItem& w : work) {
    REQUIRE(w.seg < segs.size(), "work item names segment %u of %zu", w.seg, segs.size());
    const Seg& s = segs[w.seg];
    const uint32_t unit = s.unit;
    const bool narrow = op_narrows(s.op), widen = op_widens(s.op);
    const uint32_t src_unit = narrow ? 2 * unit : widen ? unit / 2 : unit;
    REQUIRE(s.op == b.op && s.src_buf == b.src_buf && s.dst_buf == b.dst_buf, "segment fields differ from the box");
    REQUIRE(s.units_per_row * unit == s.row_bytes, "row of %u bytes is not a whole number of %u-byte units", s.row_bytes, unit);
    const uint64_t r0 = (uint64_t)w.tile * s.rows_per_tile;
    REQUIRE(r0 < s.rows, "tile %u starts past the segment's %u rows", w.tile, s.rows);
    const uint64_t nrows = std::min<uint64_t>(s.rows - r0, s.rows_per_tile);
    const uint64_t n_units = nrows * s.units_per_row;
    REQUIRE(n_units < (1ull << 32), "tile of %" PRIu64 " units", n_units);
    if (unit == 16 || (narrow && unit == 8))
      REQUIRE(n_units <= (uint64_t)kPlaceThreads * kPlaceBatch, "wide tile of %" PRIu64 " units exceeds one batch", n_units);
    const uint64_t tile_src = s.src_off + r0 * s.src_pitch, tile_dst = s.dst_off + r0 * s.dst_pitch;
    for (uint64_t v = 0; v < n_units; ++v) {
      const uint32_t row = s.units_per_row == 1 ? (uint32_t)v : (uint32_t)(((uint64_t)(uint32_t)v * s.div_magic) >> 32);
      REQUIRE(row == v / s.units_per_row, "reciprocal division: unit %" PRIu64 " of rows of %u", v, s.units_per_row);
      const uint32_t col = (uint32_t)v - row * s.units_per_row;
      const uint64_t so64 = (uint64_t)row * s.src_pitch + (uint64_t)col * src_unit, do64 = (uint64_t)row * s.dst_pitch + (uint64_t)col * unit;
      REQUIRE(so64 < (1ull << 32) && do64 < (1ull << 32), "in-tile offset beyond 32 bits");
      const uint64_t sa = tile_src + so64, da = tile_dst + do64;
      if (s.op != kOpChecksumOnly) REQUIRE(da % unit == 0, "store of %u bytes at destination offset %" PRIu64, unit, da);
      REQUIRE(sa % src_elem(s.op) == 0, "load at source offset %" PRIu64 " is not element aligned", sa);
      REQUIRE(da >= b.dst_off && da + unit <= b.dst_off + d_span, "store outside the box");
      if (unit == 16 || (narrow && unit == 8)) wide_bytes += unit;
      for (uint32_t k = 0; k < unit; ++k) {
        const uint64_t at = da - b.dst_off + k;
        REQUIRE(hits[at] == 0, "destination byte %" PRIu64 " written twice", at);
        hits[at] = 1;
        const uint64_t e = dst_elem(s.op);
        got[at] = (int64_t)(sa - b.src_off + (k / e) * e * ratio_n / ratio_d);
      }
    }
  }
  const bool abut = b.rows == 1 || (b.src_pitch == src_row && b.dst_pitch == b.row_bytes);
  if (b.op != kOpChecksumOnly && (abut || (b.dst_pitch % 16 == 0 && b.row_bytes >= 64))) {
    const uint64_t total = b.rows * b.row_bytes, slack = abut ? 32 : 32 * b.rows;
    REQUIRE(wide_bytes + slack > total, "only %" PRIu64 " of %" PRIu64 " bytes take the wide path", wide_bytes, total);
  }
  for (uint64_t i = 0; i < d_span; ++i)
    REQUIRE(got[i] == want[i], "destination byte %" PRIu64 ": source %" PRId64 ", expected %" PRId64, i, got[i], want[i]);
}

BoxCopy random_box(std::mt19937_64& g) {
  auto pick = [&](uint64_t lo, uint64_t hi) { return lo + g() % (hi - lo + 1); };
  static const uint32_t ops[] = {kOpCopy, kOpCopy, kOpCopy, kOpChecksumOnly, kOpCastF32Bf16, kOpCastBf16F32, kOpCastF16F32,
                                 kOpCastF32F16, kOpCastF8E4M3Bf16, kOpCastF16Bf16, kOpCastBf16F16};
  BoxCopy b;
  b.op = ops[g() % (sizeof ops / sizeof ops[0])];
  const uint64_t de = dst_elem(b.op), se = src_elem(b.op);
  const int shape = (int)(g() % 5);
  uint64_t row_elems;
  if (shape == 0) {  // a contiguous run, sometimes long
    b.rows = 1;
    row_elems = pick(1, g() % 4 ? 40000 : 1500000);
  } else if (shape == 1) {  // narrow rows, many of them
    b.rows = pick(2, 3000);
    row_elems = pick(1, 700);
  } else if (shape == 2) {  // wide rows (split by columns beyond 32 KiB)
    b.rows = pick(2, 40);
    row_elems = pick(1000, 60000);
  } else if (shape == 3) {  // aligned, power-of-two flavoured
    b.rows = pick(1, 512);
    row_elems = 8 * pick(1, 1024);
  } else {  // a column slice of a matrix whose row length is a multiple of 2 KiB, rows that fill whole batches
    const uint64_t unit_elems = (op_narrows(b.op) ? 8 : 16) / de;  // elements per lane access of the wide path
    row_elems = unit_elems << pick(0, 10);
    const uint64_t tile_rows = std::max<uint64_t>(1, 8192 * unit_elems / row_elems);
    b.rows = pick(tile_rows, 5 * tile_rows + 3);
    b.row_bytes = row_elems * de;
    const uint64_t src_row = op_src_bytes(b.op, b.row_bytes);
    b.src_pitch = (src_row + 2047) / 2048 * 2048 + 2048 * pick(0, 3);
    b.dst_pitch = g() % 2 ? b.row_bytes : (b.row_bytes + 2047) / 2048 * 2048 + 2048 * pick(0, 2);
    b.dst_off = 16 * pick(0, 40);
    b.src_off = 16 * pick(0, 40);
    return b;
  }
  b.row_bytes = row_elems * de;
  const uint64_t src_row = op_src_bytes(b.op, b.row_bytes);
  const bool tidy = g() % 2;
  b.dst_pitch = b.row_bytes + (tidy ? 16 * pick(0, 64) : de * pick(0, 100));
  b.src_pitch = src_row + (tidy ? 16 * pick(0, 64) : se * pick(0, 100));
  if (tidy && b.row_bytes % 16) b.dst_pitch = (b.dst_pitch + 15) / 16 * 16;
  if (g() % 5 == 0) {  // rows that abut on both sides
    b.dst_pitch = b.row_bytes;
    b.src_pitch = src_row;
  }
  b.dst_off = (tidy && g() % 2 ? 16 : de) * pick(0, 40);
  b.src_off = se * pick(0, 40);
  return b;
}

}  // namespace

int main(int argc, char** argv) {
  const uint64_t first = argc > 1 ? std::strtoull(argv[1], nullptr, 10) : 0;
  const uint64_t count = argc > 2 ? std::strtoull(argv[2], nullptr, 10) : 200;
  LowerOptions lo;
  uint64_t segs_total = 0;
  for (uint64_t seed = first; seed < first + count; ++seed) {
    std::mt19937_64 g(seed * 7919 + 13);
    const BoxCopy b = random_box(g);
    if (seed % 3 == 0) lo.tile_bytes = 1024u << (g() % 8);  // 1 KiB .. 128 KiB
    try {
      check_box(b, lo);
    } catch (const Fail& f) {
      std::fprintf(stderr,
                   "seed %" PRIu64 ": op %u rows %" PRIu64 " row_bytes %" PRIu64 " src_off %" PRIu64 " dst_off %" PRIu64
                   " src_pitch %" PRIu64 " dst_pitch %" PRIu64 " tile %u\n  %s\n",
                   seed, b.op, b.rows, b.row_bytes, b.src_off, b.dst_off, b.src_pitch, b.dst_pitch, lo.tile_bytes, f.what.c_str());
      return 1;
    } catch (const std::exception& e) {
      std::fprintf(stderr, "seed %" PRIu64 ": lowering threw: %s\n", seed, e.what());
      return 1;
    }
    ++segs_total;
  }
  std::printf("%" PRIu64 " boxes lowered and replayed\n", segs_total);
  return 0;
}
