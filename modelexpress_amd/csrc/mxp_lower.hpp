// Host-side lowering of logical pitched box copies into the device descriptor tables
// (segments + work items) that place_kernel executes.
#pragma once
#include <algorithm>
#include <cstdint>
#include <stdexcept>
#include <string>
#include <vector>

#include "mxp_device.h"

namespace mxp {

// One logical box of any size: `rows` rows of `row_bytes` DESTINATION bytes each.
// The source row is op_src_bytes(op, row_bytes) long (twice as long for a narrowing cast,
// half as long for a widening one).
struct BoxCopy {
  uint32_t src_buf = 0, dst_buf = 0;
  uint64_t src_off = 0, dst_off = 0;
  uint64_t src_pitch = 0, dst_pitch = 0;
  uint64_t rows = 1, row_bytes = 0;
  uint32_t op = kOpCopy;
  uint32_t csum_slot = 0xFFFFFFFFu;
  uint64_t csum_bias = 0;  // checksum position = destination offset + bias (mod 2^32)
};

struct LowerOptions {
  uint32_t tile_bytes = 128 * 1024;  // SOURCE bytes one workgroup handles (one batch of loads)
  uint32_t flat_row_bytes = 8192;   // virtual row width used to tile contiguous runs
  uint32_t max_row_bytes = 32768;   // wider pitched rows are split by columns
};

// `SegTable` / `WorkTable` are anything with push_back and size: std::vector, or a fixed-capacity
// view over memory the caller already owns.
template <class SegTable, class WorkTable>
inline void emit_seg(const BoxCopy& b, const LowerOptions& o, SegTable& segs, WorkTable& work) {
  if (b.rows == 0 || b.row_bytes == 0) return;
  if (b.rows > 0xFFFFFFFFull || b.row_bytes > o.max_row_bytes)
    throw std::logic_error("emit_seg: box not normalised");
  const uint64_t src_row = op_src_bytes(b.op, b.row_bytes);
  const bool pitched = b.rows > 1;
  auto all_mult = [&](uint64_t m_dst, uint64_t m_src) {
    if (b.dst_off % m_dst || b.row_bytes % m_dst) return false;
    if (b.src_off % m_src) return false;
    if (pitched && (b.dst_pitch % m_dst || b.src_pitch % m_src)) return false;
    return true;
  };
  // The unit is set by the destination side (whole, aligned stores); the source only has to be
  // element aligned, the device reads it with loads that carry no alignment promise.
  uint32_t unit;
  if (op_narrows(b.op)) {
    if (all_mult(8, 4)) unit = 8;
    else if (all_mult(2, 4)) unit = 2;
    else throw std::invalid_argument("cast box is not element aligned");
  } else if (op_widens(b.op)) {
    const uint64_t se = op_dst_elem(b.op) / 2;  // source element
    if (all_mult(16, se)) unit = 16;
    else if (all_mult(4, se)) unit = 4;
    else if (op_dst_elem(b.op) == 2 && all_mult(2, 1)) unit = 2;
    else throw std::invalid_argument("cast box is not element aligned");
  } else if (op_recodes16(b.op)) {
    if (all_mult(16, 2)) unit = 16;
    else if (all_mult(4, 2)) unit = 4;
    else if (all_mult(2, 2)) unit = 2;
    else throw std::invalid_argument("cast box is not element aligned");
  } else {
    unit = all_mult(16, 1) ? 16 : all_mult(4, 1) ? 4 : all_mult(2, 1) ? 2 : 1;
  }
  const uint64_t max_pitch = pitched ? std::max(b.src_pitch, b.dst_pitch) : std::max(b.row_bytes, src_row);
  if (max_pitch >= (1ull << 31)) throw std::invalid_argument("row pitch of 2 GiB or more is not supported");

  Seg s{};
  s.src_off = b.src_off;
  s.dst_off = b.dst_off;
  s.src_pitch = pitched ? b.src_pitch : src_row;
  s.dst_pitch = pitched ? b.dst_pitch : b.row_bytes;
  s.rows = (uint32_t)b.rows;
  s.row_bytes = (uint32_t)b.row_bytes;
  s.src_buf = b.src_buf;
  s.dst_buf = b.dst_buf;
  s.op = b.op;
  s.unit = unit;
  s.csum_slot = b.csum_slot;
  s.csum_bias = (uint32_t)b.csum_bias;
  s.units_per_row = s.row_bytes / unit;
  s.div_magic = s.units_per_row > 1 ? (uint32_t)((1ull << 32) / s.units_per_row) + 1u : 0u;
  uint64_t rpt = std::max<uint64_t>(1, o.tile_bytes / std::max(b.row_bytes, src_row));
  rpt = std::min<uint64_t>(rpt, b.rows);
  // In-tile byte offsets are 32-bit on the device, and the reciprocal division is exact
  // only while (units in tile) * (units per row) < 2^32.
  while (rpt > 1 && (rpt * max_pitch >= (1ull << 31) ||
                     rpt * s.units_per_row * (uint64_t)s.units_per_row >= (1ull << 32)))
    rpt = (rpt + 1) / 2;
  if ((uint64_t)s.units_per_row * s.units_per_row >= (1ull << 32))
    throw std::logic_error("emit_seg: row too wide for its unit");
  // The 16-byte (8-byte for narrowing casts) paths of place_kernel run one batch per tile.
  if ((unit == 16 || unit == 8) && rpt * s.units_per_row > (uint64_t)kPlaceThreads * kPlaceBatch)
    throw std::logic_error("emit_seg: tile larger than one batch");
  s.rows_per_tile = (uint32_t)rpt;
  const uint32_t seg_idx = (uint32_t)segs.size();
  segs.push_back(s);
  const uint64_t tiles = (b.rows + rpt - 1) / rpt;
  for (uint64_t t = 0; t < tiles; ++t) work.push_back(WorkItem{seg_idx, (uint32_t)t});
}

// Split one logical box into device segments.
template <class SegTable, class WorkTable>
inline void lower_box(const BoxCopy& in, const LowerOptions& o, SegTable& segs, WorkTable& work) {
  if (in.rows == 0 || in.row_bytes == 0) return;
  const uint32_t op = in.op;
  BoxCopy b = in;
  // Rows that abut in both layouts are one contiguous run.
  if (b.rows > 1 && b.src_pitch == op_src_bytes(op, b.row_bytes) && b.dst_pitch == b.row_bytes) {
    b.row_bytes *= b.rows;
    b.rows = 1;
  }
  if (b.rows == 1) {
    // Contiguous run: a head up to the destination's next 16-byte boundary (so that the rest
    // moves in whole aligned stores whatever the source's alignment), full virtual rows of
    // flat_row_bytes, then one short row.
    const uint64_t W = o.flat_row_bytes;
    uint64_t done = 0;
    if (b.dst_off % 16 && op != kOpChecksumOnly) {
      const uint64_t head = std::min<uint64_t>(16 - b.dst_off % 16, b.row_bytes);
      BoxCopy m = b;
      m.row_bytes = head;
      m.src_pitch = op_src_bytes(op, head);
      m.dst_pitch = head;
      emit_seg(m, o, segs, work);
      done = head;
    }
    uint64_t full = (b.row_bytes - done) / W;
    while (full) {
      const uint64_t n = std::min<uint64_t>(full, 0x80000000ull);
      BoxCopy m = b;
      m.src_off = b.src_off + op_src_bytes(op, done);
      m.dst_off = b.dst_off + done;
      m.rows = n;
      m.row_bytes = W;
      m.src_pitch = op_src_bytes(op, W);
      m.dst_pitch = W;
      emit_seg(m, o, segs, work);
      done += n * W;
      full -= n;
    }
    const uint64_t rem = b.row_bytes - done;
    if (rem) {
      // Keep the 16-byte path for as much of the remainder as possible.
      const uint64_t body = (rem / 16) * 16;
      BoxCopy m = b;
      m.rows = 1;
      if (body) {
        m.src_off = b.src_off + op_src_bytes(op, done);
        m.dst_off = b.dst_off + done;
        m.row_bytes = body;
        emit_seg(m, o, segs, work);
      }
      if (rem - body) {
        m.src_off = b.src_off + op_src_bytes(op, done + body);
        m.dst_off = b.dst_off + done + body;
        m.row_bytes = rem - body;
        emit_seg(m, o, segs, work);
      }
    }
    return;
  }
  // Pitched box whose rows all start at the same distance from a 16-byte boundary of the
  // destination, but not on one (or do not end on one): a column of head bytes, a body that is
  // stored whole and aligned, a column of tail bytes.
  if (op != kOpChecksumOnly && b.dst_pitch % 16 == 0 && (b.dst_off % 16 || b.row_bytes % 16) && b.row_bytes >= 64) {
    const uint64_t head = (16 - b.dst_off % 16) % 16;
    const uint64_t body = (b.row_bytes - head) / 16 * 16;
    const uint64_t cuts[4] = {0, head, head + body, b.row_bytes};
    for (int k = 0; k < 3; ++k) {
      if (cuts[k + 1] == cuts[k]) continue;
      BoxCopy m = b;
      m.src_off = b.src_off + op_src_bytes(op, cuts[k]);
      m.dst_off = b.dst_off + cuts[k];
      m.row_bytes = cuts[k + 1] - cuts[k];
      lower_box(m, o, segs, work);  // the body is aligned now, the edge columns are narrower than 64 bytes
    }
    return;
  }
  // Pitched box: split columns so a row fits max_row_bytes, rows so the count fits 32 bits.
  for (uint64_t c = 0; c < b.row_bytes; c += o.max_row_bytes) {
    const uint64_t cw = std::min<uint64_t>(o.max_row_bytes, b.row_bytes - c);
    for (uint64_t r = 0; r < b.rows; r += 0x80000000ull) {
      BoxCopy m = b;
      m.src_off = b.src_off + r * b.src_pitch + op_src_bytes(op, c);
      m.dst_off = b.dst_off + r * b.dst_pitch + c;
      m.rows = std::min<uint64_t>(0x80000000ull, b.rows - r);
      m.row_bytes = cw;
      emit_seg(m, o, segs, work);
    }
  }
}

}  // namespace mxp
