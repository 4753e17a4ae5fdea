// Drives the host engine (modelexpress_amd/csrc/mxp_engine.cpp: pinned ring, reader threads, stream and event
// ordering, error path) on the CPU, built against the HIP stand-in under tests/c/cpu_hip with
// -fsanitize=thread or -fsanitize=address,undefined (tests/test_host_sanitizers.py builds and runs both).
//
// A small Llama-shaped checkpoint (two shard files, bf16 or fp32) is written, one tensor-parallel rank's share is
// planned through the C ABI and ingested with every combination the engine has a code path for - rows packed by
// the readers / whole bands staged, page cache / direct I/O, final-address copies on / off / for tiny pieces,
// more readers than slots, one stream, a delay in front of every copy - several times each on one engine; the
// bytes that arrive and their checksums are compared with what the driver computes from the tensors itself.
// Then: a caller stream with work pending on the destinations, the resident path, the stand-alone checksum,
// a shard file truncated between plan and execute (the ingest must fail cleanly and work again afterwards); last,
// 96 random strided views (storage orders, paddings, element sizes, two conversions) as single recorded copies,
// as batched calls back to back on two streams and as view plans run repeatedly, and the small stand-alone operators.
//
// usage: engine_hosttest <empty working directory>      prints "ok" and exits 0 on success
#include <hip/hip_runtime.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <chrono>
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <map>
#include <random>
#include <string>
#include <thread>
#include <vector>

#include "mxp.h"
#include "mxp_bench.h"

namespace {

[[noreturn]] void die(const std::string& what) {
  std::fprintf(stderr, "engine_hosttest: %s (last error: %s)\n", what.c_str(), mxp_last_error());
  std::exit(1);
}
#define OK(call)                                                  \
  do {                                                            \
    const int rc_ = (call);                                       \
    if (rc_ != MXP_OK) die(std::string(#call) + " returned " + std::to_string(rc_)); \
  } while (0)

struct Tensor {
  std::string name;
  int64_t rows, cols;  // cols == 0: one-dimensional [rows]
  std::vector<uint8_t> data;  // in the checkpoint's element type
};

constexpr int64_t kHidden = 256, kKv = 128, kInter = 512, kVocab = 1000, kLayers = 4;
constexpr int kTp = 2, kRank = 1;

std::vector<Tensor> make_tensors(int elem, uint32_t seed) {
  std::mt19937 rng(seed);
  std::vector<Tensor> v;
  auto add = [&](const std::string& name, int64_t rows, int64_t cols) {
    Tensor t{name, rows, cols, {}};
    t.data.resize((size_t)(rows * (cols ? cols : 1) * elem));
    for (auto& b : t.data) b = (uint8_t)rng();
    if (elem == 4)  // keep fp32 patterns away from NaN so that the expected image does not depend on nan_bits
      for (size_t i = 3; i < t.data.size(); i += 4) t.data[i] &= 0x3F;
    v.push_back(std::move(t));
  };
  add("model.embed_tokens.weight", kVocab, kHidden);
  for (int64_t l = 0; l < kLayers; ++l) {
    const std::string p = "model.layers." + std::to_string(l) + ".";
    add(p + "input_layernorm.weight", kHidden, 0);
    add(p + "self_attn.q_proj.weight", kHidden, kHidden);
    add(p + "self_attn.k_proj.weight", kKv, kHidden);
    add(p + "self_attn.v_proj.weight", kKv, kHidden);
    add(p + "self_attn.o_proj.weight", kHidden, kHidden);
    add(p + "mlp.gate_proj.weight", kInter, kHidden);
    add(p + "mlp.up_proj.weight", kInter, kHidden);
    add(p + "mlp.down_proj.weight", kHidden, kInter);
  }
  add("model.norm.weight", kHidden, 0);
  add("lm_head.weight", kVocab, kHidden);
  return v;
}

// Two safetensors files: 8-byte little-endian header length, the JSON header padded with spaces, the data.
void write_checkpoint(const std::string& dir, const std::vector<Tensor>& tensors, const char* dtype) {
  for (int f = 0; f < 2; ++f) {
    std::string json = "{";
    std::vector<const Tensor*> mine;
    uint64_t at = 0;
    for (size_t i = 0; i < tensors.size(); ++i) {
      if ((int)(i * 2 / tensors.size()) != f) continue;
      const Tensor& t = tensors[i];
      if (!mine.empty()) json += ",";
      json += "\"" + t.name + "\":{\"dtype\":\"" + dtype + "\",\"shape\":[" + std::to_string(t.rows) +
              (t.cols ? "," + std::to_string(t.cols) : "") + "],\"data_offsets\":[" + std::to_string(at) + "," +
              std::to_string(at + t.data.size()) + "]}";
      at += t.data.size();
      mine.push_back(&t);
    }
    json += "}";
    while (json.size() % 8) json += " ";
    const std::string path = dir + "/model-0000" + std::to_string(f + 1) + "-of-00002.safetensors";
    FILE* fp = std::fopen(path.c_str(), "wb");
    if (!fp) die("cannot write " + path);
    const uint64_t n = json.size();
    std::fwrite(&n, 8, 1, fp);
    std::fwrite(json.data(), 1, json.size(), fp);
    for (const Tensor* t : mine) std::fwrite(t->data.data(), 1, t->data.size(), fp);
    std::fclose(fp);
  }
}

struct Param {
  std::string name;
  int64_t rows, cols;
  std::vector<uint8_t> want;  // in the parameter's element type
};

uint16_t f32_to_bf16(uint32_t u) { return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16); }

// Rows [r0, r0 + nr) x columns [c0, c0 + nc) of `t`, appended to `out` in the parameter's element type.
void take(const Tensor& t, int elem, bool cast, int64_t r0, int64_t nr, int64_t c0, int64_t nc, std::vector<uint8_t>& out) {
  const int64_t cols = t.cols ? t.cols : 1;
  for (int64_t r = r0; r < r0 + nr; ++r)
    for (int64_t c = c0; c < c0 + nc; ++c) {
      const uint8_t* p = t.data.data() + (size_t)((r * cols + c) * elem);
      if (cast) {
        uint32_t u;
        std::memcpy(&u, p, 4);
        const uint16_t h = f32_to_bf16(u);
        out.insert(out.end(), reinterpret_cast<const uint8_t*>(&h), reinterpret_cast<const uint8_t*>(&h) + 2);
      } else {
        out.insert(out.end(), p, p + elem);
      }
    }
}

std::vector<Param> expected_params(const std::vector<Tensor>& tensors, int elem, bool cast) {
  std::map<std::string, const Tensor*> by;
  for (const auto& t : tensors) by[t.name] = &t;
  std::vector<Param> ps;
  auto rows_of = [&](Param& p, const std::string& src) {  // this rank's block of rows
    const Tensor& t = *by.at(src);
    take(t, elem, cast, kRank * t.rows / kTp, t.rows / kTp, 0, t.cols, p.want);
  };
  auto cols_of = [&](Param& p, const std::string& src) {  // this rank's block of columns
    const Tensor& t = *by.at(src);
    take(t, elem, cast, 0, t.rows, kRank * t.cols / kTp, t.cols / kTp, p.want);
  };
  auto whole = [&](Param& p, const std::string& src) {
    const Tensor& t = *by.at(src);
    take(t, elem, cast, 0, t.rows, 0, t.cols ? t.cols : 1, p.want);
  };
  {
    Param p{"model.embed_tokens.weight", kVocab / kTp, kHidden, {}};
    rows_of(p, p.name);
    ps.push_back(std::move(p));
  }
  for (int64_t l = 0; l < kLayers; ++l) {
    const std::string b = "model.layers." + std::to_string(l) + ".";
    Param ln{b + "input_layernorm.weight", kHidden, 0, {}};
    whole(ln, ln.name);
    ps.push_back(std::move(ln));
    Param qkv{b + "self_attn.qkv_proj.weight", (kHidden + 2 * kKv) / kTp, kHidden, {}};
    rows_of(qkv, b + "self_attn.q_proj.weight");
    rows_of(qkv, b + "self_attn.k_proj.weight");
    rows_of(qkv, b + "self_attn.v_proj.weight");
    ps.push_back(std::move(qkv));
    Param o{b + "self_attn.o_proj.weight", kHidden, kHidden / kTp, {}};
    cols_of(o, o.name);
    ps.push_back(std::move(o));
    Param gu{b + "mlp.gate_up_proj.weight", 2 * kInter / kTp, kHidden, {}};
    rows_of(gu, b + "mlp.gate_proj.weight");
    rows_of(gu, b + "mlp.up_proj.weight");
    ps.push_back(std::move(gu));
    Param d{b + "mlp.down_proj.weight", kHidden, kInter / kTp, {}};
    cols_of(d, d.name);
    ps.push_back(std::move(d));
  }
  {
    Param n{"model.norm.weight", kHidden, 0, {}};
    whole(n, n.name);
    ps.push_back(std::move(n));
    Param h{"lm_head.weight", kVocab / kTp, kHidden, {}};
    rows_of(h, h.name);
    ps.push_back(std::move(h));
  }
  return ps;
}

uint32_t checksum(const std::vector<uint8_t>& b) {
  uint32_t s = 0;
  for (size_t i = 0; i < b.size(); ++i) s += b[i] * ((uint32_t)i * 2654435761u + 1u);
  return s;
}

struct Model {
  mxp_ckpt* ck = nullptr;
  mxp_plan* plan = nullptr;
  std::vector<Param> params;
  std::vector<void*> dst;
  std::vector<uint32_t> sums;
  std::string dir;
};

Model open_model(const std::string& dir, const std::vector<Tensor>& tensors, int elem, bool cast) {
  Model m;
  m.dir = dir;
  m.params = expected_params(tensors, elem, cast);
  OK(mxp_ckpt_open(dir.c_str(), &m.ck));
  OK(mxp_plan_create(m.ck, kTp, kRank, cast ? MXP_PLAN_ALLOW_CAST : 0u, &m.plan));
  const int dtype = (elem == 2 || cast) ? MXP_DTYPE_BF16 : MXP_DTYPE_F32;
  for (const auto& p : m.params) {
    const int64_t shape[2] = {p.rows, p.cols};
    if (mxp_plan_add_param(m.plan, p.name.c_str(), dtype, p.cols ? 2 : 1, shape) < 0) die("mxp_plan_add_param " + p.name);
  }
  OK(mxp_plan_build(m.plan));
  for (const auto& p : m.params) {
    void* d = nullptr;
    if (hipMalloc(&d, p.want.size()) != hipSuccess) die("hipMalloc");
    m.dst.push_back(d);
    m.sums.push_back(checksum(p.want));
  }
  return m;
}

void close_model(Model& m) {
  mxp_plan_destroy(m.plan);
  mxp_ckpt_close(m.ck);
  for (void* d : m.dst) (void)hipFree(d);
}

void scribble(Model& m, uint8_t v) {
  for (size_t i = 0; i < m.dst.size(); ++i) std::memset(m.dst[i], v, m.params[i].want.size());
}

void check(mxp_engine* eng, Model& m, const std::string& what) {
  std::vector<uint32_t> got(m.params.size());
  OK(mxp_plan_checksums(eng, m.plan, got.data(), (int64_t)got.size()));
  for (size_t i = 0; i < m.params.size(); ++i) {
    if (std::memcmp(m.dst[i], m.params[i].want.data(), m.params[i].want.size()) != 0) die(what + ": wrong bytes in " + m.params[i].name);
    if (got[i] != m.sums[i]) die(what + ": wrong checksum for " + m.params[i].name);
  }
}

mxp_engine* make_engine(int slots, uint64_t slot_bytes, int readers, int streams, int pack, int direct) {
  mxp_engine_options o{};
  o.ring_slots = slots;
  o.slot_bytes = slot_bytes;
  o.reader_threads = readers;
  o.streams = streams;
  o.pack_strided_on_host = (uint16_t)pack;
  o.use_o_direct = direct;
  mxp_engine* e = nullptr;
  OK(mxp_engine_create(&o, &e));
  return e;
}

// ---- recorded copies between strided views (mxp_copy_view, mxp_copy_views, mxp_view_plan_*) ----
struct View {
  std::vector<int64_t> shape, ss, ds;  // strides in elements
  int es = 1, eo = 1, cast = MXP_CAST_NONE;
  std::vector<uint8_t> src, want;       // host images of the whole source / destination buffers
  uint8_t* dsrc = nullptr;              // "device" copies
  uint8_t* ddst = nullptr;
  size_t src_off = 0;                   // elements the view starts into its source buffer
  uint32_t csum = 0;                    // checksum of the written bytes, positions counted from ddst
};

// Strides of a view of `shape` inside a buffer whose dimensions are stored in a random order, sometimes padded.
int64_t random_layout(std::mt19937& rng, const std::vector<int64_t>& shape, std::vector<int64_t>& strides) {
  std::vector<size_t> order(shape.size());
  for (size_t i = 0; i < order.size(); ++i) order[i] = i;
  std::shuffle(order.begin(), order.end(), rng);
  strides.assign(shape.size(), 0);
  int64_t run = 1;
  for (size_t k = order.size(); k-- > 0;) {
    strides[order[k]] = run;
    run *= shape[order[k]] + (rng() % 3 == 0 ? (int64_t)(rng() % 3) : 0);
  }
  return run;
}

View make_view(std::mt19937& rng, int index) {
  View v;
  const int pick = index % 6;
  if (pick == 4) { v.es = 4; v.eo = 2; v.cast = MXP_CAST_F32_BF16; }
  else if (pick == 5) { v.es = 2; v.eo = 4; v.cast = MXP_CAST_BF16_F32; }
  else v.es = v.eo = 1 << (pick % 4);
  const int ndim = 1 + (int)(rng() % 4);
  int64_t elems = 1;
  static const int64_t sizes[] = {1, 2, 3, 5, 8, 16, 31, 64, 70, 128, 256};
  do {
    v.shape.clear();
    for (int d = 0; d < ndim; ++d) v.shape.push_back(sizes[rng() % (ndim > 2 ? 8 : 11)]);
    if (index % 5 == 0 && ndim >= 2) {  // whole tiles, so that the staged-tile transposes are met as well
      v.shape[ndim - 1] = 128;
      v.shape[ndim - 2] = 256;
      for (int d = 0; d < ndim - 2; ++d) v.shape[d] = 1 + (int64_t)(rng() % 2);
    }
    elems = 1;
    for (int64_t e : v.shape) elems *= e;
  } while (elems > 140000);  // the whole run stays within seconds under ThreadSanitizer
  int64_t s_total, d_total;
  if (index % 5 == 0 && ndim >= 2) {
    // the shape of the MLA W_UK_T rewrite: destination row-major, source with its last two dimensions swapped
    v.ds.assign((size_t)ndim, 1);
    for (int d = ndim - 2; d >= 0; --d) v.ds[(size_t)d] = v.ds[(size_t)d + 1] * v.shape[(size_t)d + 1];
    v.ss = v.ds;
    v.ss[(size_t)ndim - 1] = v.shape[(size_t)ndim - 2];
    v.ss[(size_t)ndim - 2] = 1;
    s_total = d_total = v.ds[0] * v.shape[0];
  } else {
    s_total = random_layout(rng, v.shape, v.ss);
    d_total = random_layout(rng, v.shape, v.ds);
  }
  v.src_off = rng() % 4;
  v.src.resize((size_t)(s_total + (int64_t)v.src_off) * v.es);
  for (auto& b : v.src) b = (uint8_t)rng();
  if (v.cast == MXP_CAST_F32_BF16)
    for (size_t i = 3; i < v.src.size(); i += 4) v.src[i] &= 0x3F;  // no NaN
  v.want.assign((size_t)d_total * v.eo, 0xEE);
  std::vector<int64_t> idx(v.shape.size(), 0);
  int64_t n = 1;
  for (int64_t e : v.shape) n *= e;
  for (int64_t k = 0; k < n; ++k) {
    int64_t so = (int64_t)v.src_off, d_o = 0;
    for (size_t d = 0; d < idx.size(); ++d) { so += idx[d] * v.ss[d]; d_o += idx[d] * v.ds[d]; }
    const uint8_t* sp = v.src.data() + so * v.es;
    uint8_t* dp = v.want.data() + d_o * v.eo;
    if (v.cast == MXP_CAST_F32_BF16) {
      uint32_t u;
      std::memcpy(&u, sp, 4);
      const uint16_t h = f32_to_bf16(u);
      std::memcpy(dp, &h, 2);
    } else if (v.cast == MXP_CAST_BF16_F32) {
      uint16_t h;
      std::memcpy(&h, sp, 2);
      const uint32_t u = (uint32_t)h << 16;
      std::memcpy(dp, &u, 4);
    } else {
      std::memcpy(dp, sp, (size_t)v.es);
    }
    for (int e = 0; e < v.eo; ++e) v.csum += dp[e] * ((uint32_t)(d_o * v.eo + e) * 2654435761u + 1u);
    for (size_t d = idx.size(); d-- > 0;) {
      if (++idx[d] < v.shape[d]) break;
      idx[d] = 0;
    }
  }
  if (hipMalloc(reinterpret_cast<void**>(&v.dsrc), v.src.size()) != hipSuccess || hipMalloc(reinterpret_cast<void**>(&v.ddst), v.want.size()) != hipSuccess)
    die("hipMalloc");
  std::memcpy(v.dsrc, v.src.data(), v.src.size());
  return v;
}

mxp_view_copy as_abi(const View& v) {
  mxp_view_copy c{};
  c.src = v.dsrc + v.src_off * (size_t)v.es;
  c.dst = v.ddst;
  c.ndim = (int32_t)v.shape.size();
  c.elem_size = v.eo;
  c.cast = v.cast;
  for (size_t d = 0; d < v.shape.size(); ++d) { c.shape[d] = v.shape[d]; c.src_strides[d] = v.ss[d]; c.dst_strides[d] = v.ds[d]; }
  return c;
}

void check_views(std::vector<View>& views, const std::string& what) {
  if (hipDeviceSynchronize() != hipSuccess) die("sync");
  for (size_t k = 0; k < views.size(); ++k)
    if (std::memcmp(views[k].ddst, views[k].want.data(), views[k].want.size()) != 0) die(what + ": wrong bytes in view " + std::to_string(k));
}
void scribble_views(std::vector<View>& views) {
  for (auto& v : views) std::memset(v.ddst, 0xEE, v.want.size());
}

long exercise_views(mxp_engine* eng) {
  std::mt19937 rng(77);
  long checked = 0;
  hipStream_t side;
  if (hipStreamCreateWithFlags(&side, hipStreamNonBlocking) != hipSuccess) die("stream");
  std::vector<std::vector<View>> groups(4);
  int index = 0;
  for (auto& g : groups)
    for (int k = 0; k < 24; ++k) g.push_back(make_view(rng, index++));
  int kinds[3] = {0, 0, 0};
  for (auto& g : groups) {
    std::vector<mxp_view_copy> abi;
    for (const auto& v : g) abi.push_back(as_abi(v));
    std::vector<int32_t> kind(abi.size());
    OK(mxp_describe_views(eng, abi.data(), (int64_t)abi.size(), kind.data(), nullptr, nullptr));
    for (int32_t k : kind) ++kinds[k];
  }
  if (!kinds[0] || !kinds[1] || !kinds[2])
    die("the random views do not cover the three ways a view can run: " + std::to_string(kinds[0]) + " / " + std::to_string(kinds[1]) + " / " + std::to_string(kinds[2]));
  // one view at a time, with its checksum
  for (auto& g : groups) {
    scribble_views(g);
    for (auto& v : g) {
      const mxp_view_copy c = as_abi(v);
      uint32_t got = 0;
      OK(mxp_copy_view(eng, c.src, c.dst, c.ndim, c.shape, c.src_strides, c.dst_strides, c.elem_size, c.cast, &got, nullptr));
      if (got != v.csum) die("copy_view checksum");
    }
    check_views(g, "mxp_copy_view");
    checked += (long)g.size();
  }
  // batched calls back to back on two streams, nothing waited for in between: the descriptor arenas are taken in turn
  for (int rep = 0; rep < 2; ++rep) {
    for (auto& g : groups) scribble_views(g);
    for (size_t gi = 0; gi < groups.size(); ++gi) {
      std::vector<mxp_view_copy> abi;
      for (const auto& v : groups[gi]) abi.push_back(as_abi(v));
      OK(mxp_copy_views(eng, abi.data(), (int64_t)abi.size(), gi % 2 ? side : nullptr));
    }
    for (auto& g : groups) { check_views(g, "mxp_copy_views"); checked += (long)g.size(); }
  }
  // lowered once, run many times
  for (size_t gi = 0; gi < groups.size(); ++gi) {
    auto& g = groups[gi];
    std::vector<mxp_view_copy> abi;
    for (const auto& v : g) abi.push_back(as_abi(v));
    mxp_view_plan* vp = nullptr;
    OK(mxp_view_plan_create(eng, abi.data(), (int64_t)abi.size(), &vp));
    uint64_t bytes = 0, want_bytes = 0;
    OK(mxp_view_plan_bytes(vp, &bytes));
    for (const auto& v : g) { int64_t n = v.eo; for (int64_t e : v.shape) n *= e; want_bytes += (uint64_t)n; }
    if (bytes != want_bytes) die("view plan byte count");
    for (int rep = 0; rep < 3; ++rep) {
      scribble_views(g);
      OK(mxp_view_plan_run(eng, vp, rep == 1 ? side : nullptr));
      check_views(g, "mxp_view_plan_run");
      checked += (long)g.size();
    }
    mxp_view_plan_destroy(vp);
  }
  // boxes, whole-buffer copies, a cast and a pitched gather with their checksums
  {
    const size_t n = 70000;
    std::vector<uint8_t> host(n * 4);
    for (auto& b : host) b = (uint8_t)rng();
    for (size_t i = 3; i < host.size(); i += 4) host[i] &= 0x3F;
    uint8_t *a = nullptr, *b = nullptr;
    if (hipMalloc(reinterpret_cast<void**>(&a), host.size()) != hipSuccess || hipMalloc(reinterpret_cast<void**>(&b), host.size()) != hipSuccess) die("hipMalloc");
    std::memcpy(a, host.data(), host.size());
    uint32_t got = 0;
    OK(mxp_cast(eng, a, b, n, MXP_CAST_F32_BF16, &got, nullptr));
    std::vector<uint8_t> want(n * 2);
    for (size_t i = 0; i < n; ++i) { uint32_t u; std::memcpy(&u, host.data() + 4 * i, 4); const uint16_t h = f32_to_bf16(u); std::memcpy(want.data() + 2 * i, &h, 2); }
    if (std::memcmp(b, want.data(), want.size()) != 0 || got != checksum(want)) die("mxp_cast");
    OK(mxp_gather2d(eng, a + 48, 1000, b, 304, 200, 300, &got, side));
    std::vector<uint8_t> rows;
    uint32_t want_sum = 0;
    for (size_t r = 0; r < 200; ++r)
      for (size_t c = 0; c < 300; ++c) {
        if (b[r * 304 + c] != host[48 + r * 1000 + c]) die("mxp_gather2d bytes");
        want_sum += b[r * 304 + c] * ((uint32_t)(r * 304 + c) * 2654435761u + 1u);
      }
    if (got != want_sum) die("mxp_gather2d checksum");
    const void* srcs[3] = {a, a + 4096, a + 100000};
    void* dsts[3] = {b, b + 8192, b + 120000};
    const uint64_t sizes[3] = {4000, 1, 65537};
    uint32_t sums[3];
    OK(mxp_copy_batch(eng, srcs, dsts, sizes, 3, sums, nullptr));
    for (int k = 0; k < 3; ++k) {
      const std::vector<uint8_t> piece(static_cast<const uint8_t*>(srcs[k]), static_cast<const uint8_t*>(srcs[k]) + sizes[k]);
      if (std::memcmp(dsts[k], piece.data(), piece.size()) != 0 || sums[k] != checksum(piece)) die("mxp_copy_batch");
    }
    (void)hipFree(a);
    (void)hipFree(b);
    checked += 5;
  }
  for (auto& g : groups)
    for (auto& v : g) { (void)hipFree(v.dsrc); (void)hipFree(v.ddst); }
  (void)hipStreamDestroy(side);
  return checked;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc != 2) {
    std::fprintf(stderr, "usage: engine_hosttest <empty working directory>\n");
    return 2;
  }
  const std::string root = argv[1];
  const std::string dir16 = root + "/bf16", dir32 = root + "/f32";
  ::mkdir(dir16.c_str(), 0700);
  ::mkdir(dir32.c_str(), 0700);
  const auto t16 = make_tensors(2, 1), t32 = make_tensors(4, 2);
  write_checkpoint(dir16, t16, "BF16");
  write_checkpoint(dir32, t32, "F32");
  Model m16 = open_model(dir16, t16, 2, false), m32 = open_model(dir32, t32, 4, true);

  long runs = 0;
  struct Mode { int slots; uint64_t slot; int readers, streams, pack, direct; int64_t direct_min; unsigned delay_us; };
  const Mode modes[] = {
      {3, 1 << 16, 4, 2, 1, 0, 0, 0},        // rows packed by the readers, page cache
      {3, 1 << 16, 4, 2, 2, 0, 0, 0},        // whole row bands staged
      {3, 1 << 16, 4, 2, 1, 1, 0, 0},        // direct I/O, packed (falls back to buffered reads where the file system refuses)
      {3, 1 << 16, 4, 2, 2, 1, 0, 0},        // direct I/O, bands
      {4, 1 << 17, 4, 3, 1, 0, -1, 0},       // every byte through the bounce slot
      {4, 1 << 17, 4, 3, 1, 0, 4096, 0},     // final-address copies for pieces of 4 KiB and more
      {2, 1 << 16, 8, 1, 1, 0, 0, 0},        // more readers than slots, one stream
      {2, 1 << 16, 6, 2, 2, 0, 4096, 150},   // every copy reads its source 150 us late
      {5, 1 << 18, 3, 4, 1, 0, 0, 40},
  };
  for (const Mode& md : modes) {
    mxp_engine* eng = make_engine(md.slots, md.slot, md.readers, md.streams, md.pack, md.direct);
    if (md.direct_min) OK(mxp_engine_set_direct_placement(eng, md.direct_min));
    cpu_hip::set_copy_delay_us(md.delay_us);
    for (Model* m : {&m16, &m32}) {
      for (int rep = 0; rep < 3; ++rep) {
        scribble(*m, (uint8_t)(0xA0 + rep));
        mxp_exec_stats st{};
        if (rep == 1) OK(mxp_prepare(eng, m->plan));
        OK(mxp_execute(eng, m->plan, m->dst.data(), rep == 2 ? nullptr : &st));
        check(eng, *m, "ingest");
        if (rep != 2 && (!st.mutated || st.n_chunks < 4 || st.placed_bytes == 0)) die("ingest statistics");
        ++runs;
      }
    }
    cpu_hip::set_copy_delay_us(0);
    mxp_engine_destroy(eng);
  }

  mxp_engine* eng = make_engine(3, 1 << 16, 4, 2, 1, 0);
  {
    // Work pending on the caller's stream when the ingest starts: it must land first.
    hipStream_t caller;
    if (hipStreamCreateWithFlags(&caller, hipStreamNonBlocking) != hipSuccess) die("stream");
    Model* m = &m16;
    cpu_hip::enqueue(caller, [m] {
      std::this_thread::sleep_for(std::chrono::milliseconds(20));
      for (size_t i = 0; i < m->dst.size(); ++i) std::memset(m->dst[i], 0x77, m->params[i].want.size());
    });
    OK(mxp_execute_after(eng, m16.plan, m16.dst.data(), caller, nullptr));
    check(eng, m16, "ingest behind a caller stream");
    (void)hipStreamDestroy(caller);
    ++runs;
  }
  {
    // The resident path: the shard files staged in "device" memory, one launch; twice, then on another stream.
    for (Model* m : {&m16, &m32}) {
      std::vector<void*> files;
      for (int64_t f = 0; f < mxp_ckpt_file_count(m->ck); ++f) {
        mxp_file_info fi;
        OK(mxp_ckpt_file_info(m->ck, f, &fi));
        void* d = nullptr;
        if (hipMalloc(&d, fi.file_size) != hipSuccess) die("hipMalloc");
        FILE* fp = std::fopen(fi.path, "rb");
        if (!fp || std::fread(d, 1, fi.file_size, fp) != fi.file_size) die("cannot read a shard file back");
        std::fclose(fp);
        files.push_back(d);
      }
      hipStream_t other;
      if (hipStreamCreateWithFlags(&other, hipStreamNonBlocking) != hipSuccess) die("stream");
      for (int rep = 0; rep < 3; ++rep) {
        scribble(*m, (uint8_t)(0x30 + rep));
        mxp_exec_stats st{};
        OK(mxp_execute_resident(eng, m->plan, files.data(), m->dst.data(), rep == 2 ? other : nullptr, rep == 0 ? &st : nullptr));
        check(eng, *m, "resident placement");
        ++runs;
      }
      // stand-alone checksums of the finished buffers
      std::vector<uint64_t> sizes;
      for (const auto& p : m->params) sizes.push_back(p.want.size());
      std::vector<uint32_t> got(m->params.size());
      OK(mxp_checksum32(eng, m->dst.data(), sizes.data(), (int64_t)sizes.size(), got.data(), nullptr));
      if (got != m->sums) die("stand-alone checksums");
      OK(mxp_checksum32_static(eng, m->dst.data(), sizes.data(), (int64_t)sizes.size(), got.data(), nullptr));
      if (got != m->sums) die("stand-alone checksums through the static scratch");
      mxp_plan_destroy(m->plan);  // before the stream it was last launched on goes away
      m->plan = nullptr;
      (void)hipStreamDestroy(other);
      for (void* d : files) (void)hipFree(d);
    }
  }
  mxp_engine_destroy(eng);

  {
    // A shard file that lost its tail between plan and execute: every reader must come home, the first
    // error is reported, and the same engine ingests again once the file is whole.
    Model m = open_model(dir16, t16, 2, false);
    mxp_engine* e2 = make_engine(3, 1 << 16, 6, 2, 1, 0);
    const std::string victim = dir16 + "/model-00002-of-00002.safetensors";
    struct stat sb;
    if (::stat(victim.c_str(), &sb) != 0) die("stat");
    std::vector<uint8_t> whole((size_t)sb.st_size);
    FILE* fp = std::fopen(victim.c_str(), "rb");
    if (!fp || std::fread(whole.data(), 1, whole.size(), fp) != whole.size()) die("read back");
    std::fclose(fp);
    if (::truncate(victim.c_str(), sb.st_size / 2) != 0) die("truncate");
    mxp_exec_stats st{};
    const int rc = mxp_execute(e2, m.plan, m.dst.data(), &st);
    if (rc == MXP_OK) die("an ingest from a truncated file succeeded");
    if (!std::strstr(mxp_last_error(), "model-00002")) die("the error does not name the file");
    fp = std::fopen(victim.c_str(), "wb");
    if (!fp || std::fwrite(whole.data(), 1, whole.size(), fp) != whole.size()) die("restore");
    std::fclose(fp);
    for (int rep = 0; rep < 2; ++rep) {
      scribble(m, 0x11);
      OK(mxp_execute(e2, m.plan, m.dst.data(), nullptr));
      check(e2, m, "ingest after a failed one");
      ++runs;
    }
    mxp_engine_destroy(e2);
    close_model(m);
  }
  m16.plan = nullptr;
  m32.plan = nullptr;
  close_model(m16);
  close_model(m32);
  mxp_engine* e3 = make_engine(3, 1 << 16, 2, 2, 1, 0);
  const long views = exercise_views(e3);
  mxp_engine_destroy(e3);
  std::printf("ok: %ld placements and %ld view copies checked, %" PRIu64 " stream operations run\n", runs, views, cpu_hip::operations_run());
  return 0;
}
