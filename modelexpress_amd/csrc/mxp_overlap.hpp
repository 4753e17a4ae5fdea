// Plan-time settlement of overlapping writes: what is left of an earlier write once a later
// write of the same parameter has taken its bytes ("later write wins", the outcome of the
// reference's serial destination.copy_ loop, engines/vllm/refit/installer.py:419-424, and of its
// ordered fallback for overlapping destinations, refit/reshard/receiver.py:939-955).
#pragma once
#include <algorithm>
#include <cstdint>
#include <string>
#include <utility>
#include <vector>

#include "mxp_internal.hpp"

namespace mxp {

// False only when the two boxes provably share no destination byte.
inline bool writes_may_overlap(const WriteRec& a, const WriteRec& b) {
  auto end = [](const WriteRec& w) { return w.dst_offset + (w.rows - 1) * w.dst_pitch + w.row_bytes; };
  if (a.rows == 0 || b.rows == 0 || a.row_bytes == 0 || b.row_bytes == 0) return false;
  if (a.dst_offset >= end(b) || b.dst_offset >= end(a)) return false;
  if (a.rows > 1 && b.rows > 1 && a.dst_pitch == b.dst_pitch) {
    // column bands of one pitch (the fused and strided slices): disjoint columns never meet
    const uint64_t pitch = a.dst_pitch, ca = a.dst_offset % pitch, cb = b.dst_offset % pitch;
    if (ca + a.row_bytes <= pitch && cb + b.row_bytes <= pitch && (ca + a.row_bytes <= cb || cb + b.row_bytes <= ca))
      return false;
  }
  return true;
}

// The bytes of `e` that `k` does not cover, as boxes with e's pitches (rows that lose the same
// columns stay together).  `src_elem` / `dst_elem`: element sizes on the two sides of e (they
// differ for a converting write); a cut inside an element is refused.
inline std::vector<WriteRec> clip_write(const WriteRec& e, const WriteRec& k, uint64_t src_elem, uint64_t dst_elem,
                                        const std::string& param_name) {
  using Cols = std::vector<std::pair<uint64_t, uint64_t>>;  // byte columns of a row that stay, relative to the row
  std::vector<WriteRec> out;
  Cols open;
  uint64_t open_from = 0;
  auto flush = [&](uint64_t upto) {
    for (const auto& c : open) {
      if (c.first % dst_elem || c.second % dst_elem)
        throw Error(MXP_ERR_UNSUPPORTED, "overlapping writes of '" + param_name + "' meet inside an element");
      WriteRec r = e;
      r.rows = upto - open_from;
      r.row_bytes = c.second - c.first;
      r.dst_offset = e.dst_offset + open_from * e.dst_pitch + c.first;
      r.src_offset = e.src_offset + open_from * e.src_pitch + c.first / dst_elem * src_elem;
      if (r.rows == 1) {
        r.dst_pitch = r.row_bytes;
        r.src_pitch = r.row_bytes / dst_elem * src_elem;
      }
      r.paired_runs = r.rows;
      out.push_back(r);
    }
  };
  for (uint64_t r = 0; r < e.rows; ++r) {
    const uint64_t lo = e.dst_offset + r * e.dst_pitch, hi = lo + e.row_bytes;
    Cols keep{{0, e.row_bytes}};
    uint64_t rb = 0;  // first row of k that can reach past lo
    if (k.rows > 1 && k.dst_pitch && lo >= k.dst_offset + k.row_bytes) rb = (lo - k.dst_offset - k.row_bytes) / k.dst_pitch + 1;
    for (; rb < k.rows; ++rb) {
      const uint64_t klo = k.dst_offset + rb * k.dst_pitch, khi = klo + k.row_bytes;
      if (klo >= hi) break;
      if (khi > lo) {
        const uint64_t c0 = klo > lo ? klo - lo : 0, c1 = std::min(khi, hi) - lo;
        Cols next;
        for (const auto& c : keep) {
          if (c1 <= c.first || c0 >= c.second) { next.push_back(c); continue; }
          if (c.first < c0) next.emplace_back(c.first, c0);
          if (c1 < c.second) next.emplace_back(c1, c.second);
        }
        keep.swap(next);
      }
      if (k.dst_pitch == 0) break;
    }
    if (keep != open) {
      flush(r);
      open = keep;
      open_from = r;
    }
  }
  flush(e.rows);
  return out;
}

}  // namespace mxp
