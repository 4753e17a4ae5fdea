// Placement planner: maps every checkpoint tensor to a box inside one of the rank's
// parameters, following the destination-map rules of the reference's direct loader
// (modelexpress/engines/vllm/refit/installer.py): classification order premerged ->
// direct -> expert -> fused member (:498-543), resolution order premerged -> fused ->
// expert -> direct (:341-387), everything resolved before the first byte moves
// (:389-391).  Views are tracked as (base, shape, stride) in elements so a write is a
// strided copy between two views of equal shape; it is then reduced to pitched 2-D
// byte boxes by merging dimensions that are contiguous in both layouts, which is the
// run decomposition of refit/reshard/slice_plan.py:259-294 with the innermost
// non-contiguous dimension kept as the row index instead of being enumerated.
#include <algorithm>
#include <cstring>
#include <memory>
#include <set>

#include "mxp_internal.hpp"
#include "mxp_overlap.hpp"

namespace mxp {
namespace {

using Shape = std::vector<int64_t>;

struct View {
  int64_t param = -1;  // destination parameter (unused for sources)
  int64_t base = 0;    // element offset
  Shape shape, stride;
};

Shape row_major(const Shape& s) {
  Shape st(s.size(), 1);
  for (int d = (int)s.size() - 2; d >= 0; --d) st[d] = st[d + 1] * s[d + 1];
  return st;
}
View full_view(const Shape& s, int64_t param = -1) {
  View v;
  v.param = param;
  v.shape = s;
  v.stride = row_major(s);
  return v;
}
View narrow(View v, int axis, int64_t start, int64_t size) {
  v.base += start * v.stride[axis];
  v.shape[axis] = size;
  return v;
}
View index0(View v, int64_t i) {
  v.base += i * v.stride[0];
  v.shape.erase(v.shape.begin());
  v.stride.erase(v.stride.begin());
  return v;
}
int64_t numel(const Shape& s) {
  int64_t n = 1;
  for (auto d : s) n *= d;
  return n;
}
std::string shape_str(const Shape& s) {
  std::string o = "(";
  for (size_t i = 0; i < s.size(); ++i) o += (i ? ", " : "") + std::to_string(s[i]);
  return o + ")";
}

bool contains(const std::string& hay, const std::string& needle) {
  return hay.find(needle) != std::string::npos;
}
bool ends_with(const std::string& s, const std::string& suf) {
  return s.size() >= suf.size() && s.compare(s.size() - suf.size(), suf.size(), suf) == 0;
}
// Python str.replace: every non-overlapping occurrence, left to right.
std::string replace_all(const std::string& s, const std::string& from, const std::string& to) {
  if (from.empty()) return s;
  std::string o;
  size_t pos = 0;
  for (;;) {
    const size_t hit = s.find(from, pos);
    if (hit == std::string::npos) break;
    o.append(s, pos, hit - pos);
    o += to;
    pos = hit + from.size();
  }
  o.append(s, pos, std::string::npos);
  return o;
}

// installer.py:440-449
bool is_scale_name(const std::string& n) {
  return ends_with(n, "weight_scale") || ends_with(n, "weight_scale_inv") ||
         ends_with(n, "input_scale") || ends_with(n, "activation_scale");
}
bool is_fp8(int dtype) { return dtype == MXP_DTYPE_F8_E4M3 || dtype == MXP_DTYPE_F8_E5M2; }

const char* kAliases[2][2] = {{"weight_scale_inv", "weight_scale"}, {"input_scale", "activation_scale"}};

struct Planner {
  mxp_plan& pl;
  const mxp_ckpt& ck;
  const int tp, rank;

  std::vector<StackedRec> groups_def;
  std::unordered_map<std::string, int64_t> direct;             // tensor name -> param
  std::unordered_map<std::string, View> fused, expert;         // tensor name -> dest view
  std::unordered_map<std::string, std::pair<int64_t, int>> premerged;  // -> (param, parts)
  std::set<int64_t> covered;

  explicit Planner(mxp_plan& p) : pl(p), ck(*p.ckpt), tp(p.tp_size), rank(p.tp_rank) {}

  // installer.py:451-468
  int64_t find_param(const std::string& name) const {
    std::vector<std::string> cands{name};
    for (const auto& a : kAliases) {
      if (contains(name, a[0])) cands.push_back(replace_all(name, a[0], a[1]));
      if (contains(name, a[1])) cands.push_back(replace_all(name, a[1], a[0]));
    }
    for (const auto& c : cands) {
      auto it = pl.param_by_name.find(c);
      if (it != pl.param_by_name.end()) return it->second;
    }
    return -1;
  }

  // installer.py:319-339
  bool tp_shape_compatible(const Shape& loaded, const Shape& expected) const {
    if (loaded == expected) return true;
    if (tp <= 1 || loaded.size() != expected.size()) return false;
    int mism = -1, n = 0;
    for (size_t d = 0; d < loaded.size(); ++d)
      if (loaded[d] != expected[d]) { mism = (int)d; ++n; }
    return n == 1 && loaded[mism] == expected[mism] * tp;
  }

  // installer.py:292-317: this rank's shard of a global tensor, as a view of the source.
  bool tp_local(const View& src, const Shape& expected, View& out) const {
    if (src.shape == expected) { out = src; return true; }
    if (tp <= 1 || src.shape.size() != expected.size()) return false;
    std::vector<int> cand;
    for (size_t a = 0; a < expected.size(); ++a) {
      if (src.shape[a] != expected[a] * tp) continue;
      bool rest = true;
      for (size_t d = 0; d < expected.size(); ++d)
        if (d != a && src.shape[d] != expected[d]) rest = false;
      if (rest) cand.push_back((int)a);
    }
    if (cand.size() != 1) return false;
    out = narrow(src, cand[0], (int64_t)rank * expected[cand[0]], expected[cand[0]]);
    return true;
  }

  // installer.py:773-797 / :72-78
  void stacked_groups() {
    groups_def = pl.stacked;
    if (groups_def.empty()) {
      groups_def = {{"qkv_proj", "q_proj", 0}, {"qkv_proj", "k_proj", 1}, {"qkv_proj", "v_proj", 2},
                    {"gate_up_proj", "gate_proj", 0}, {"gate_up_proj", "up_proj", 1}};
    }
  }

  // installer.py:629-668
  bool premerged_destination(const std::string& name, const Shape& src_shape,
                             const std::vector<std::string>& suffixes, int64_t& param) const {
    if (tp <= 1 || src_shape.empty()) return false;
    bool hit = false;
    for (const auto& suf : suffixes)
      if (ends_with(name, suf + ".weight") || contains(name, suf + ".")) hit = true;
    if (!hit) return false;
    const int64_t p = find_param(name);
    if (p < 0) return false;
    const Shape& ps = pl.params[p].shape;
    if (ps.empty() || ps.size() != src_shape.size()) return false;
    const int64_t dest0 = ps[0], src0 = src_shape[0];
    if (src0 != dest0 * tp) return false;
    if (dest0 % 2 != 0 || src0 % (2 * (int64_t)tp) != 0) return false;
    for (size_t d = 1; d < ps.size(); ++d)
      if (src_shape[d] != ps[d]) return false;
    param = p;
    return true;
  }

  // installer.py:695-754
  // Returns 1 mapped, 0 unmapped, 2 expert not local to this rank (skip).
  int resolve_expert(const std::string& name, const Shape& hf_shape, View& out) const {
    for (const auto& e : pl.experts) {
      if (!contains(name, e.weight_prefix)) continue;
      const int64_t p = find_param(replace_all(name, e.weight_prefix, e.param_prefix));
      if (p < 0) return 0;
      const ParamRec& fp = pl.params[p];
      if (fp.shape.empty()) return 0;
      if (e.local_id == -1) return (pl.flags & MXP_PLAN_NONLOCAL_EXPERTS_UNMAPPED) ? 0 : 2;
      if (e.local_id < 0 || e.local_id >= fp.shape[0]) return 0;
      const View slot = index0(full_view(fp.shape, p), e.local_id);
      if (e.shard == "w2") {
        if (tp_shape_compatible(hf_shape, slot.shape)) { out = slot; return 1; }
        return 0;
      }
      if (hf_shape.empty()) {
        const int64_t n = numel(slot.shape);
        if (n == 1 || n == 2) {
          View v;
          v.param = p;
          // A contiguous slot: element `index` of its flattening.
          v.base = slot.base + ((n == 2 && e.shard != "w1") ? 1 : 0);
          out = v;
          return 1;
        }
        return 0;
      }
      if (hf_shape.size() != slot.shape.size()) return 0;
      if ((e.shard == "w1" || e.shard == "w3") && slot.shape[0] % 2 == 0) {
        const int64_t half = slot.shape[0] / 2;
        const View dest = narrow(slot, 0, e.shard == "w1" ? 0 : half, half);
        if (tp_shape_compatible(hf_shape, dest.shape)) { out = dest; return 1; }
      }
      for (size_t axis = 0; axis < slot.shape.size(); ++axis) {
        bool rest = true;
        for (size_t d = 0; d < slot.shape.size(); ++d)
          if (d != axis && hf_shape[d] != slot.shape[d]) rest = false;
        if (!rest) continue;
        const int64_t source = hf_shape[axis], dest = slot.shape[axis];
        int64_t local_size;
        if (dest == source * 2) local_size = source;
        else if (tp > 1 && dest * tp == source * 2) local_size = dest / 2;
        else continue;
        out = narrow(slot, (int)axis, e.shard == "w1" ? 0 : local_size, local_size);
        return 1;
      }
      return 0;
    }
    return 0;
  }

  struct Member { int order; std::string name; Shape shape; };

  // installer.py:566-616
  bool fused_destinations(int64_t p, const std::vector<Member>& members) {
    const ParamRec& fp = pl.params[p];
    const View data = full_view(fp.shape, p);
    bool all_scalar = true;
    for (const auto& m : members) if (!m.shape.empty()) all_scalar = false;
    if (all_scalar) {
      const int64_t n = numel(fp.shape);
      if (n == 1 || n == (int64_t)members.size()) {
        for (size_t i = 0; i < members.size(); ++i) {
          View v;
          v.param = p;
          v.base = (n == 1) ? 0 : (int64_t)i;
          fused[members[i].name] = v;
        }
        return true;
      }
      return false;
    }
    if (members.empty()) return false;
    for (const auto& m : members) if (m.shape.size() != fp.shape.size()) return false;
    int axis = -1;
    int64_t divisor = 1;
    for (size_t a = 0; a < fp.shape.size() && axis < 0; ++a) {
      bool ok = true;
      for (const auto& m : members)
        for (size_t d = 0; d < fp.shape.size(); ++d)
          if (d != a && m.shape[d] != fp.shape[d]) ok = false;
      if (!ok) continue;
      int64_t total = 0;
      for (const auto& m : members) total += m.shape[a];
      if (total == fp.shape[a]) { axis = (int)a; divisor = 1; }
      else if (tp > 1 && total == fp.shape[a] * tp) {
        bool div = true;
        for (const auto& m : members) if (m.shape[a] % tp) div = false;
        if (div) { axis = (int)a; divisor = tp; }
      }
    }
    if (axis < 0) return false;
    int64_t offset = 0;
    for (const auto& m : members) {
      const int64_t size = m.shape[axis] / divisor;
      fused[m.name] = narrow(data, axis, offset, size);
      offset += size;
    }
    return true;
  }

  // Strided copy between equal-shape views -> pitched byte boxes.
  void emit_writes(int64_t tensor, int kind, const View& src, const View& dst) {
    const TensorRec& t = ck.tensors[tensor];
    ParamRec& p = pl.params[dst.param];
    int cast = 0;
    if (t.dtype != p.dtype) {
      if (pl.flags & MXP_PLAN_ALLOW_CAST) {
        if (t.dtype == MXP_DTYPE_F32 && p.dtype == MXP_DTYPE_BF16) cast = MXP_CAST_F32_BF16;
        else if (t.dtype == MXP_DTYPE_BF16 && p.dtype == MXP_DTYPE_F32) cast = MXP_CAST_BF16_F32;
        else if (t.dtype == MXP_DTYPE_F16 && p.dtype == MXP_DTYPE_F32) cast = MXP_CAST_F16_F32;
        else if (t.dtype == MXP_DTYPE_F32 && p.dtype == MXP_DTYPE_F16) cast = MXP_CAST_F32_F16;
        else if (t.dtype == MXP_DTYPE_F8_E4M3 && p.dtype == MXP_DTYPE_BF16) cast = MXP_CAST_F8E4M3_BF16;
        else if (t.dtype == MXP_DTYPE_F16 && p.dtype == MXP_DTYPE_BF16) cast = MXP_CAST_F16_BF16;
        else if (t.dtype == MXP_DTYPE_BF16 && p.dtype == MXP_DTYPE_F16) cast = MXP_CAST_BF16_F16;
      }
      if (!cast)
        throw Error(MXP_ERR_UNSUPPORTED, "tensor '" + t.name + "' is " + mxp_dtype_name(t.dtype) +
                                             " but parameter '" + p.name + "' is " +
                                             mxp_dtype_name(p.dtype) + "; no conversion is planned");
    }
    const uint64_t es = (uint64_t)dtype_size(t.dtype), ed = (uint64_t)dtype_size(p.dtype);
    // Drop unit dims, then merge trailing dims that are packed in both layouts.
    Shape sh, ss, ds;
    for (size_t d = 0; d < src.shape.size(); ++d) {
      if (src.shape[d] == 1) continue;
      sh.push_back(src.shape[d]); ss.push_back(src.stride[d]); ds.push_back(dst.stride[d]);
    }
    if (numel(src.shape) == 0) return;
    int64_t run = 1;
    int pdim = (int)sh.size() - 1;
    while (pdim >= 0 && ss[pdim] == run && ds[pdim] == run) { run *= sh[pdim]; --pdim; }
    WriteRec w;
    w.tensor = tensor;
    w.param = dst.param;
    w.kind = kind;
    w.cast = cast;
    w.row_bytes = (uint64_t)run * ed;
    auto finish = [&](const WriteRec& r) {
      const uint64_t span = r.dst_offset + (r.rows - 1) * r.dst_pitch + r.row_bytes;
      const uint64_t sspan = r.src_offset + (r.rows - 1) * r.src_pitch + r.row_bytes / ed * es;
      if (span > p.nbytes || sspan > t.nbytes)
        throw Error(MXP_ERR_STATE, "internal: write for '" + t.name + "' leaves its buffers");
      p.bytes_written += r.rows * r.row_bytes;
      p.n_writes += 1;
      pl.writes.push_back(r);
    };
    if (pdim < 0) {
      w.rows = 1;
      w.src_offset = (uint64_t)src.base * es;
      w.dst_offset = (uint64_t)dst.base * ed;
      w.src_pitch = w.row_bytes / ed * es;
      w.dst_pitch = w.row_bytes;
      w.paired_runs = 1;
      finish(w);
      return;
    }
    // Row dimension = innermost unmerged dim, extended over outer dims that tile it.
    int64_t rows = sh[pdim];
    const int64_t sp = ss[pdim], dp = ds[pdim];
    int q = pdim - 1;
    while (q >= 0 && ss[q] == sp * rows && ds[q] == dp * rows) { rows *= sh[q]; --q; }
    int64_t outer = 1;
    for (int d = 0; d <= q; ++d) outer *= sh[d];
    if (outer > (1 << 20)) throw Error(MXP_ERR_UNSUPPORTED, "write for '" + t.name + "' needs too many boxes");
    w.rows = (uint64_t)rows;
    w.src_pitch = (uint64_t)sp * es;
    w.dst_pitch = (uint64_t)dp * ed;
    w.paired_runs = (uint64_t)rows;
    std::vector<int64_t> idx((size_t)(q + 1), 0);
    for (int64_t o = 0; o < outer; ++o) {
      int64_t so = src.base, d_o = dst.base;
      for (int d = 0; d <= q; ++d) { so += idx[d] * ss[d]; d_o += idx[d] * ds[d]; }
      WriteRec r = w;
      r.src_offset = (uint64_t)so * es;
      r.dst_offset = (uint64_t)d_o * ed;
      finish(r);
      for (int d = q; d >= 0; --d) { if (++idx[d] < sh[d]) break; idx[d] = 0; }
    }
  }

  // A write whose source is a virtual tensor: intersect the needed box with every shard
  // (refit/reshard/slice_plan.py:248-256,297-339) and emit one strided copy per overlap.
  void emit_virtual(const VirtualRec& v, int kind, const View& local, const View& dest) {
    const size_t nd = v.shape.size();
    const Shape vs = row_major(v.shape);
    Shape lo(nd), ext(nd);
    int64_t want = 1, got = 0;
    for (size_t d = 0; d < nd; ++d) {
      lo[d] = v.shape[d] ? (local.base / vs[d]) % v.shape[d] : 0;
      ext[d] = local.shape[d];
      want *= ext[d];
    }
    for (const auto& sh : v.shards) {
      const TensorRec& t = ck.tensors[sh.tensor];
      const Shape ts = row_major(t.shape);
      View sv, dv = dest;
      sv.shape.resize(nd);
      sv.stride = ts;
      bool empty = false;
      int64_t vol = 1;
      for (size_t d = 0; d < nd; ++d) {
        const int64_t a = std::max(lo[d], sh.shard_offset[d]);
        const int64_t b = std::min(lo[d] + ext[d], sh.shard_offset[d] + sh.shape[d]);
        if (a >= b) { empty = true; break; }
        sv.base += (sh.src_offset[d] + a - sh.shard_offset[d]) * ts[d];
        sv.shape[d] = b - a;
        dv.base += (a - lo[d]) * dest.stride[d];
        dv.shape[d] = b - a;
        vol *= b - a;
      }
      if (empty) continue;
      got += vol;
      emit_writes(sh.tensor, kind, sv, dv);
    }
    // (shards that overlap count twice here and are refused with the gaps: the reference reads shards with
    // unordered transfers, so it defines no winner for them; transfer_plan.py:160-172 refuses them too)
    if (got != want)
      throw Error(MXP_ERR_COVERAGE, "virtual tensor '" + v.name + "': its shards cover " + std::to_string(got) +
                                        " of the " + std::to_string(want) + " elements this rank needs");
  }

  // The fp8 block rule made explicit: when a weight has a companion scale of shape
  // [ceil(N/128), ceil(K/128)], a slice of the weight must start and end on 128
  // boundaries so the same shape rule applied to the scale selects exactly its tiles.
  void check_fp8_blocks(const TensorRec& t, const View& local) const {
    if (pl.flags & MXP_PLAN_NO_FP8_BLOCK_CHECK) return;
    if (!is_fp8(t.dtype) || t.shape.size() != 2 || !ends_with(t.name, "weight")) return;
    int64_t sidx = -1;
    for (const char* suf : {"_scale_inv", "_scale"}) {
      auto it = ck.by_name.find(t.name + suf);
      if (it != ck.by_name.end()) { sidx = it->second; break; }
    }
    if (sidx < 0) return;
    const TensorRec& s = ck.tensors[sidx];
    if (s.shape.size() != 2) return;
    for (int a = 0; a < 2; ++a) {
      if (t.shape[a] < 128 || s.shape[a] != (t.shape[a] + 127) / 128) return;  // not 128-blocked
    }
    for (int a = 0; a < 2; ++a) {
      if (local.shape[a] == t.shape[a]) continue;
      const int64_t start = (local.base / local.stride[a]) % t.shape[a];
      if (local.shape[a] % 128 || start % 128)
        throw Error(MXP_ERR_UNSUPPORTED,
                    "fp8 weight '" + t.name + "' would be sliced at [" + std::to_string(start) + ", " +
                        std::to_string(start + local.shape[a]) + ") on axis " + std::to_string(a) +
                        ", which is not aligned to its 128x128 scale blocks");
    }
  }

  void run() {
    if (tp < 1 || rank < 0 || rank >= tp) throw Error(MXP_ERR_ARG, "tp_rank must be in [0, tp_size)");
    stacked_groups();
    std::vector<std::string> premerge_suffixes;
    {
      std::vector<std::pair<std::string, int>> counts;
      for (const auto& g : groups_def) {
        auto it = std::find_if(counts.begin(), counts.end(), [&](auto& c) { return c.first == g.fused; });
        if (it == counts.end()) counts.emplace_back(g.fused, 1); else it->second++;
      }
      for (const auto& c : counts) if (c.second == 2) premerge_suffixes.push_back(c.first);
    }

    // Items to place: every real tensor that no virtual tensor consumes, then the virtual ones.
    struct Item { const std::string* name; const Shape* shape; int64_t real, virt; };
    std::vector<Item> todo;
    std::set<int64_t> consumed;
    for (const auto& v : pl.virtuals) {
      if (v.shards.empty()) throw Error(MXP_ERR_ARG, "virtual tensor '" + v.name + "' has no shards");
      if (ck.by_name.count(v.name)) throw Error(MXP_ERR_ARG, "virtual tensor '" + v.name + "' shadows a checkpoint tensor");
      for (const auto& sh : v.shards) consumed.insert(sh.tensor);
    }
    auto skipped_by_prefix = [&](const std::string& n) {
      for (const auto& pre : pl.skip_prefixes)
        if (n.compare(0, pre.size(), pre) == 0) return true;
      return false;
    };
    for (int64_t i = 0; i < (int64_t)ck.tensors.size(); ++i) {
      if (consumed.count(i)) continue;
      if (skipped_by_prefix(ck.tensors[i].name)) pl.skipped.push_back(ck.tensors[i].name);
      else todo.push_back(Item{&ck.tensors[i].name, &ck.tensors[i].shape, i, -1});
    }
    for (int64_t i = 0; i < (int64_t)pl.virtuals.size(); ++i) {
      if (skipped_by_prefix(pl.virtuals[i].name)) pl.skipped.push_back(pl.virtuals[i].name);
      else todo.push_back(Item{&pl.virtuals[i].name, &pl.virtuals[i].shape, -1, i});
    }

    // ---- classification (installer.py:470-564) ----
    std::vector<std::pair<int64_t, std::vector<Member>>> groups;
    std::unordered_map<int64_t, size_t> group_index;
    std::set<const std::string*> skipped_experts;
    for (const Item& it : todo) {
      struct { const std::string& name; const Shape& shape; } t{*it.name, *it.shape};
      int64_t pm_param;
      if (premerged_destination(t.name, t.shape, premerge_suffixes, pm_param)) {
        premerged[t.name] = {pm_param, 2};
        covered.insert(pm_param);
        continue;
      }
      const int64_t dp = find_param(t.name);
      if (dp >= 0 && tp_shape_compatible(t.shape, pl.params[dp].shape)) {
        direct[t.name] = dp;
        covered.insert(dp);
        continue;
      }
      if (contains(t.name, ".experts.") && !pl.experts.empty()) {
        View dest;
        const int r = resolve_expert(t.name, t.shape, dest);
        if (r == 1) { expert[t.name] = dest; covered.insert(dest.param); continue; }
        if (r == 2) { skipped_experts.insert(it.name); continue; }
      }
      for (const auto& g : groups_def) {
        if (contains(t.name, g.member + ".") || ends_with(t.name, g.member + ".weight")) {
          const int64_t fp = find_param(replace_all(t.name, g.member, g.fused));
          if (fp < 0) continue;
          auto slot = group_index.find(fp);
          if (slot == group_index.end()) {
            slot = group_index.emplace(fp, groups.size()).first;
            groups.emplace_back(fp, std::vector<Member>());
          }
          groups[slot->second].second.push_back(Member{g.order, t.name, t.shape});
          break;
        }
      }
    }
    for (auto& g : groups) {
      std::stable_sort(g.second.begin(), g.second.end(),
                       [](const Member& a, const Member& b) { return a.order < b.order; });
      if (fused_destinations(g.first, g.second)) covered.insert(g.first);
    }

    // ---- resolution (installer.py:341-410): every write before any copy ----
    std::vector<std::string> unmapped;
    auto emit = [&](const Item& it, int kind, const View& sv, const View& dv) {
      if (it.real >= 0) {
        check_fp8_blocks(ck.tensors[it.real], sv);
        emit_writes(it.real, kind, sv, dv);
      } else {
        emit_virtual(pl.virtuals[it.virt], kind, sv, dv);
      }
    };
    for (const Item& it : todo) {
      struct { const std::string& name; const Shape& shape; } t{*it.name, *it.shape};
      if (skipped_experts.count(it.name)) { pl.skipped.push_back(t.name); continue; }
      const View src = full_view(t.shape);
      auto pm = premerged.find(t.name);
      if (pm != premerged.end()) {
        // installer.py:670-693
        const ParamRec& dp = pl.params[pm->second.first];
        const int parts = pm->second.second;
        const int64_t src0 = t.shape[0], dst0 = dp.shape[0];
        if (src0 % parts || dst0 % parts || src0 / parts != (dst0 / parts) * tp) {
          unmapped.push_back(t.name);
          continue;
        }
        const int64_t part_src = src0 / parts, part_dst = dst0 / parts;
        const View dfull = full_view(dp.shape, pm->second.first);
        for (int part = 0; part < parts; ++part) {
          const View sv = narrow(src, 0, part * part_src + (int64_t)rank * part_dst, part_dst);
          const View dv = narrow(dfull, 0, part * part_dst, part_dst);
          emit(it, MXP_WRITE_PREMERGED, sv, dv);
        }
        continue;
      }
      int kind = -1;
      View dest;
      auto f = fused.find(t.name);
      if (f != fused.end()) { kind = MXP_WRITE_FUSED; dest = f->second; }
      else {
        auto e = expert.find(t.name);
        if (e != expert.end()) { kind = MXP_WRITE_EXPERT; dest = e->second; }
        else {
          auto d = direct.find(t.name);
          if (d != direct.end()) { kind = MXP_WRITE_DIRECT; dest = full_view(pl.params[d->second].shape, d->second); }
        }
      }
      View local;
      if (kind < 0 || !tp_local(src, dest.shape, local)) {
        unmapped.push_back(t.name);
        continue;
      }
      emit(it, kind, local, dest);
    }

    resolve_overlaps();

    // ---- coverage (installer.py:219-251), extended to every parameter ----
    if (!unmapped.empty() && !(pl.flags & MXP_PLAN_ALLOW_UNMAPPED)) {
      std::string m = "placement coverage incomplete; refusing a partially-written model. unmapped checkpoint tensors=[";
      for (size_t i = 0; i < unmapped.size() && i < 10; ++i) m += (i ? ", " : "") + unmapped[i];
      if (unmapped.size() > 10) m += " ...";
      throw Error(MXP_ERR_COVERAGE, m + "]");
    }
    for (const auto& u : unmapped) pl.skipped.push_back(u);
    std::vector<std::string> uncovered;
    for (size_t p = 0; p < pl.params.size(); ++p) {
      const ParamRec& pr = pl.params[p];
      const bool required = !(pl.flags & MXP_PLAN_ALLOW_UNCOVERED) || is_fp8(pr.dtype) || is_scale_name(pr.name);
      if (!required) continue;
      const bool strict = !(pl.flags & MXP_PLAN_ALLOW_UNCOVERED);
      if (!covered.count((int64_t)p) || (strict && pr.bytes_written != pr.nbytes)) uncovered.push_back(pr.name);
    }
    if (!uncovered.empty()) {
      std::string m = "placement coverage incomplete; refusing a partially-written model. uncovered local parameters=[";
      for (size_t i = 0; i < uncovered.size() && i < 10; ++i) m += (i ? ", " : "") + uncovered[i];
      if (uncovered.size() > 10) m += " ...";
      throw Error(MXP_ERR_COVERAGE, m + "]");
    }
  }

  // Later write wins.  The reference installs tensor after tensor on one stream, so where two
  // writes of a parameter overlap the later one's bytes stay (installer.py:419-424; the staged
  // re-slice keeps the captured order for overlapping destinations, receiver.py:939-955).  Here
  // chunks run on several streams and a launch gives no order between its workgroups, so the
  // order is settled at plan time instead: an earlier write gives up the bytes a later write of
  // the same parameter covers, and what is left of it is re-expressed as pitched boxes.  Every
  // destination byte then has exactly one writer, the fused checksums see the bytes that stay,
  // and `bytes_written` is the exact size of the union.
  void resolve_overlaps() {
    std::vector<std::vector<size_t>> per(pl.params.size());
    for (size_t i = 0; i < pl.writes.size(); ++i) per[pl.writes[i].param].push_back(i);
    std::vector<char> touched(pl.params.size(), 0);
    bool any = false;
    for (size_t p = 0; p < per.size() && !any; ++p) {
      // candidates by sorted spans, as cheap as the plain disjointness check
      auto v = per[p];
      std::sort(v.begin(), v.end(), [&](size_t a, size_t b) { return pl.writes[a].dst_offset < pl.writes[b].dst_offset; });
      auto end = [&](size_t i) { const WriteRec& w = pl.writes[i]; return w.dst_offset + (w.rows - 1) * w.dst_pitch + w.row_bytes; };
      for (size_t i = 0; i < v.size() && !any; ++i)
        for (size_t j = i + 1; j < v.size() && pl.writes[v[j]].dst_offset < end(v[i]); ++j)
          if (writes_may_overlap(pl.writes[v[i]], pl.writes[v[j]])) { any = true; break; }
    }
    if (!any) return;
    // plan order = the order the reference would install in
    std::vector<std::vector<WriteRec>> pieces(pl.writes.size());
    for (size_t i = 0; i < pl.writes.size(); ++i) pieces[i].push_back(pl.writes[i]);
    for (size_t p = 0; p < per.size(); ++p) {
      const auto& idx = per[p];
      for (size_t b = 1; b < idx.size(); ++b) {
        const WriteRec& later = pl.writes[idx[b]];
        for (size_t a = 0; a < b; ++a) {
          std::vector<WriteRec> next;
          bool changed = false;
          for (const WriteRec& e : pieces[idx[a]]) {
            if (!writes_may_overlap(e, later)) { next.push_back(e); continue; }
            std::vector<WriteRec> left =
                clip_write(e, later, dtype_size(ck.tensors[e.tensor].dtype), dtype_size(pl.params[e.param].dtype), pl.params[p].name);
            changed = changed || left.size() != 1 || left[0].rows != e.rows || left[0].row_bytes != e.row_bytes;
            next.insert(next.end(), left.begin(), left.end());
            if (next.size() > (1u << 20)) throw Error(MXP_ERR_UNSUPPORTED, "overlapping writes of '" + pl.params[p].name + "' need too many boxes");
          }
          if (changed) {
            pieces[idx[a]].swap(next);
            touched[p] = 1;
          }
        }
      }
    }
    std::vector<WriteRec> all;
    for (auto& v : pieces) all.insert(all.end(), v.begin(), v.end());
    pl.writes.swap(all);
    for (size_t p = 0; p < pl.params.size(); ++p) {
      if (!touched[p]) continue;
      pl.params[p].bytes_written = 0;
      pl.params[p].n_writes = 0;
    }
    for (const auto& w : pl.writes) {
      if (!touched[w.param]) continue;
      pl.params[w.param].bytes_written += w.rows * w.row_bytes;
      pl.params[w.param].n_writes += 1;
    }
  }
};

}  // namespace
}  // namespace mxp

using namespace mxp;

extern "C" {

int mxp_plan_create(const mxp_ckpt* ckpt, int32_t tp_size, int32_t tp_rank, uint32_t flags,
                    mxp_plan** out) {
  return guard([&] {
    if (!ckpt || !out) throw Error(MXP_ERR_ARG, "mxp_plan_create: null argument");
    *out = nullptr;
    if (tp_size < 1 || tp_rank < 0 || tp_rank >= tp_size)
      throw Error(MXP_ERR_ARG, "mxp_plan_create: tp_rank must be in [0, tp_size)");
    auto p = std::make_unique<mxp_plan>();
    p->ckpt = ckpt;
    p->tp_size = tp_size;
    p->tp_rank = tp_rank;
    p->flags = flags;
    *out = p.release();
  });
}

void mxp_plan_destroy(mxp_plan* plan) { delete plan; }

int64_t mxp_plan_add_param(mxp_plan* plan, const char* name, int32_t dtype, int32_t ndim,
                           const int64_t* shape) {
  int64_t idx = -1;
  const int rc = guard([&] {
    if (!plan || !name || ndim < 0 || ndim > MXP_MAX_DIMS || (ndim && !shape))
      throw Error(MXP_ERR_ARG, "mxp_plan_add_param: bad argument");
    if (plan->built) throw Error(MXP_ERR_STATE, "plan is already built");
    if (!dtype_size(dtype)) throw Error(MXP_ERR_UNSUPPORTED, "unknown dtype code");
    if (plan->param_by_name.count(name)) throw Error(MXP_ERR_ARG, std::string("duplicate parameter ") + name);
    ParamRec p;
    p.name = name;
    p.dtype = dtype;
    uint64_t n = 1;
    for (int d = 0; d < ndim; ++d) {
      if (shape[d] < 0) throw Error(MXP_ERR_ARG, "negative dimension");
      p.shape.push_back(shape[d]);
      if (__builtin_mul_overflow(n, (uint64_t)shape[d], &n)) throw Error(MXP_ERR_ARG, std::string("the shape of parameter ") + name + " overflows 64 bits");
    }
    // below 2^62 bytes every product of a subset of the extents with the element size fits a signed 64-bit value too
    if (__builtin_mul_overflow(n, (uint64_t)dtype_size(dtype), &p.nbytes) || p.nbytes >= (1ull << 62))
      throw Error(MXP_ERR_ARG, std::string("the size of parameter ") + name + " overflows");
    idx = (int64_t)plan->params.size();
    plan->param_by_name.emplace(p.name, idx);
    plan->params.push_back(std::move(p));
  });
  return rc == MXP_OK ? idx : rc;
}

int mxp_plan_add_stacked(mxp_plan* plan, const char* fused_suffix, const char* member_suffix) {
  return guard([&] {
    if (!plan || !fused_suffix || !member_suffix) throw Error(MXP_ERR_ARG, "mxp_plan_add_stacked: null argument");
    if (plan->built) throw Error(MXP_ERR_STATE, "plan is already built");
    // installer.py:784-796: strip leading dots, ignore empty or self-mapping entries,
    // pack order = encounter index per fused name.
    std::string f = fused_suffix, m = member_suffix;
    while (!f.empty() && f[0] == '.') f.erase(0, 1);
    while (!m.empty() && m[0] == '.') m.erase(0, 1);
    if (f.empty() || m.empty() || f == m) return;
    int order = 0;
    for (const auto& s : plan->stacked) if (s.fused == f) ++order;
    plan->stacked.push_back(StackedRec{f, m, order});
  });
}

int mxp_plan_add_expert(mxp_plan* plan, const char* param_prefix, const char* weight_prefix,
                        int32_t expert_id, const char* shard, int32_t local_expert_id) {
  return guard([&] {
    if (!plan || !param_prefix || !weight_prefix || !shard) throw Error(MXP_ERR_ARG, "mxp_plan_add_expert: null argument");
    if (plan->built) throw Error(MXP_ERR_STATE, "plan is already built");
    const std::string s = shard;
    if (s != "w1" && s != "w2" && s != "w3") throw Error(MXP_ERR_ARG, "expert shard must be w1, w2 or w3");
    // A dict keyed by weight prefix: a repeated key keeps its first position, last value
    // (installer.py:489-492).
    for (auto& e : plan->experts)
      if (e.weight_prefix == weight_prefix) {
        e = ExpertRec{param_prefix, weight_prefix, expert_id, s, local_expert_id};
        return;
      }
    plan->experts.push_back(ExpertRec{param_prefix, weight_prefix, expert_id, s, local_expert_id});
  });
}

int mxp_plan_add_skip_prefix(mxp_plan* plan, const char* prefix) {
  return guard([&] {
    if (!plan || !prefix) throw Error(MXP_ERR_ARG, "mxp_plan_add_skip_prefix: null argument");
    if (plan->built) throw Error(MXP_ERR_STATE, "plan is already built");
    plan->skip_prefixes.push_back(prefix);
  });
}

int64_t mxp_plan_add_virtual(mxp_plan* plan, const char* name, int32_t ndim, const int64_t* full_shape) {
  int64_t idx = -1;
  const int rc = guard([&] {
    if (!plan || !name || ndim < 0 || ndim > MXP_MAX_DIMS || (ndim && !full_shape))
      throw Error(MXP_ERR_ARG, "mxp_plan_add_virtual: bad argument");
    if (plan->built) throw Error(MXP_ERR_STATE, "plan is already built");
    for (const auto& v : plan->virtuals)
      if (v.name == name) throw Error(MXP_ERR_ARG, std::string("duplicate virtual tensor ") + name);
    VirtualRec v;
    v.name = name;
    for (int d = 0; d < ndim; ++d) {
      if (full_shape[d] < 0) throw Error(MXP_ERR_ARG, "negative dimension");
      v.shape.push_back(full_shape[d]);
    }
    idx = (int64_t)plan->virtuals.size();
    plan->virtuals.push_back(std::move(v));
  });
  return rc == MXP_OK ? idx : rc;
}

int mxp_plan_add_virtual_shard(mxp_plan* plan, int64_t virtual_index, const char* source_tensor,
                               const int64_t* source_offset, const int64_t* shard_offset, const int64_t* shape) {
  return guard([&] {
    if (!plan || !source_tensor || virtual_index < 0 || virtual_index >= (int64_t)plan->virtuals.size())
      throw Error(MXP_ERR_ARG, "mxp_plan_add_virtual_shard: bad argument");
    if (plan->built) throw Error(MXP_ERR_STATE, "plan is already built");
    VirtualRec& v = plan->virtuals[virtual_index];
    auto it = plan->ckpt->by_name.find(source_tensor);
    if (it == plan->ckpt->by_name.end())
      throw Error(MXP_ERR_ARG, std::string("virtual shard source '") + source_tensor + "' is not in the checkpoint");
    const TensorRec& t = plan->ckpt->tensors[it->second];
    const size_t nd = v.shape.size();
    if (t.shape.size() != nd) throw Error(MXP_ERR_ARG, "virtual shard: rank mismatch with '" + t.name + "'");
    if (nd && (!source_offset || !shard_offset || !shape)) throw Error(MXP_ERR_ARG, "virtual shard: null box");
    if (v.dtype >= 0 && v.dtype != t.dtype) throw Error(MXP_ERR_ARG, "virtual tensor '" + v.name + "' mixes dtypes");
    VirtualShard sh;
    sh.tensor = it->second;
    for (size_t d = 0; d < nd; ++d) {
      if (shape[d] < 0 || source_offset[d] < 0 || shard_offset[d] < 0 || source_offset[d] + shape[d] > t.shape[d] ||
          shard_offset[d] + shape[d] > v.shape[d])
        throw Error(MXP_ERR_ARG, "virtual shard of '" + v.name + "' leaves its source or the virtual tensor");
      sh.src_offset.push_back(source_offset[d]);
      sh.shard_offset.push_back(shard_offset[d]);
      sh.shape.push_back(shape[d]);
    }
    v.dtype = t.dtype;
    v.shards.push_back(std::move(sh));
  });
}

int mxp_plan_build(mxp_plan* plan) {
  return guard([&] {
    if (!plan) throw Error(MXP_ERR_ARG, "mxp_plan_build: null plan");
    if (plan->built) throw Error(MXP_ERR_STATE, "plan is already built");
    try {
      Planner(*plan).run();
    } catch (...) {
      plan->writes.clear();
      plan->skipped.clear();
      for (auto& p : plan->params) { p.bytes_written = 0; p.n_writes = 0; }
      throw;
    }
    plan->built = true;
  });
}

int64_t mxp_plan_param_count(const mxp_plan* p) { return p ? (int64_t)p->params.size() : 0; }
int64_t mxp_plan_write_count(const mxp_plan* p) { return p ? (int64_t)p->writes.size() : 0; }

int mxp_plan_param_info(const mxp_plan* plan, int64_t i, mxp_param_info* out) {
  return guard([&] {
    if (!plan || !out || i < 0 || i >= (int64_t)plan->params.size())
      throw Error(MXP_ERR_ARG, "mxp_plan_param_info: bad index");
    const ParamRec& p = plan->params[i];
    std::memset(out, 0, sizeof *out);
    out->name = p.name.c_str();
    out->dtype = p.dtype;
    out->ndim = (int32_t)p.shape.size();
    for (size_t d = 0; d < p.shape.size(); ++d) out->shape[d] = p.shape[d];
    out->nbytes = p.nbytes;
    out->bytes_written = p.bytes_written;
    out->n_writes = p.n_writes;
  });
}

int mxp_plan_write_info(const mxp_plan* plan, int64_t i, mxp_write_info* out) {
  return guard([&] {
    if (!plan || !out || i < 0 || i >= (int64_t)plan->writes.size())
      throw Error(MXP_ERR_ARG, "mxp_plan_write_info: bad index");
    const WriteRec& w = plan->writes[i];
    out->tensor_index = w.tensor;
    out->param_index = w.param;
    out->kind = w.kind;
    out->cast = w.cast;
    out->src_offset = w.src_offset;
    out->src_pitch = w.src_pitch;
    out->dst_offset = w.dst_offset;
    out->dst_pitch = w.dst_pitch;
    out->rows = w.rows;
    out->row_bytes = w.row_bytes;
    out->paired_runs = w.paired_runs;
  });
}

}  // extern "C"
