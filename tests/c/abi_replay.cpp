// Replays a trace of host-side C-ABI calls (tests/abi_trace.py wrote it while the parser, planner and
// CRC32C tests ran against the product library) against the same sources built for the CPU with
// -fsanitize=address,undefined: csrc/mxp_ckpt.cpp, csrc/mxp_plan.cpp, csrc/mxp_crc32c.cpp.
//
// Every call must return what the product build returned; after a successful open every tensor and
// file entry is read back and looked up by name, after a successful build every parameter and write
// record is read back, so the introspection paths run under the sanitizers as well.  Handles the
// trace never closed are closed at the end, so the leak check speaks about the library only.
//
// usage: abi_replay <trace file>      exit status 0 and "<n> calls replayed" on success
#include <cinttypes>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <fstream>
#include <map>
#include <sstream>
#include <string>
#include <vector>

#include "mxp.h"

namespace {

struct Str {
  bool null = true;
  std::string s;
  const char* c() const { return null ? nullptr : s.c_str(); }
};

Str unhex(const std::string& t) {
  Str r;
  if (t == "-" || t.empty() || t[0] != 'x') return r;
  r.null = false;
  for (size_t i = 1; i + 1 < t.size(); i += 2) r.s.push_back((char)std::stoi(t.substr(i, 2), nullptr, 16));
  return r;
}

std::vector<int64_t> ints(const std::string& t) {
  std::vector<int64_t> v;
  if (t == "-") return v;
  std::stringstream ss(t);
  std::string item;
  while (std::getline(ss, item, ',')) v.push_back(std::stoll(item));
  return v;
}

std::map<long, mxp_ckpt*> g_ckpts;
std::map<long, mxp_plan*> g_plans;

template <typename T>
T* handle(std::map<long, T*>& m, const std::string& id) {
  if (id == "-") return nullptr;
  auto it = m.find(std::stol(id));
  return it == m.end() ? nullptr : it->second;
}

long g_line = 0;
int g_bad = 0;
void expect(long long got, long long want, const std::string& what) {
  if (got == want) return;
  std::fprintf(stderr, "line %ld: %s returned %lld, the product build returned %lld (%s)\n", g_line, what.c_str(), got, want,
               mxp_last_error());
  ++g_bad;
}

void walk_ckpt(const mxp_ckpt* ck) {
  const int64_t n = mxp_ckpt_tensor_count(ck), nf = mxp_ckpt_file_count(ck);
  uint64_t total = 0;
  for (int64_t i = 0; i < n; ++i) {
    mxp_tensor_info ti;
    if (mxp_ckpt_tensor_info(ck, i, &ti) != MXP_OK) { ++g_bad; continue; }
    total += ti.nbytes + (uint64_t)std::strlen(ti.name);
    if (i < 64 || i % 97 == 0) {
      if (mxp_ckpt_find(ck, ti.name) < 0) { std::fprintf(stderr, "line %ld: tensor '%s' is listed but not found\n", g_line, ti.name); ++g_bad; }
    }
  }
  for (int64_t f = 0; f < nf; ++f) {
    mxp_file_info fi;
    if (mxp_ckpt_file_info(ck, f, &fi) != MXP_OK) { ++g_bad; continue; }
    total += fi.file_size + (uint64_t)std::strlen(fi.path);
  }
  mxp_tensor_info ti;
  if (mxp_ckpt_tensor_info(ck, n, &ti) == MXP_OK || mxp_ckpt_tensor_info(ck, -1, &ti) == MXP_OK) ++g_bad;  // out of range is refused
  (void)mxp_ckpt_find(ck, "no such tensor");
  (void)total;
}

void walk_plan(const mxp_plan* pl) {
  const int64_t np = mxp_plan_param_count(pl), nw = mxp_plan_write_count(pl);
  uint64_t total = 0;
  for (int64_t i = 0; i < np; ++i) {
    mxp_param_info pi;
    if (mxp_plan_param_info(pl, i, &pi) != MXP_OK) { ++g_bad; continue; }
    total += pi.nbytes + pi.bytes_written + (uint64_t)std::strlen(pi.name);
  }
  for (int64_t i = 0; i < nw; ++i) {
    mxp_write_info wi;
    if (mxp_plan_write_info(pl, i, &wi) != MXP_OK) { ++g_bad; continue; }
    total += wi.rows * wi.row_bytes + wi.paired_runs;
  }
  mxp_write_info wi;
  if (mxp_plan_write_info(pl, nw, &wi) == MXP_OK) ++g_bad;
  (void)total;
}

}  // namespace

int main(int argc, char** argv) {
  if (argc != 2) { std::fprintf(stderr, "usage: abi_replay <trace file>\n"); return 2; }
  std::ifstream in(argv[1]);
  if (!in) { std::fprintf(stderr, "cannot open %s\n", argv[1]); return 2; }
  std::string line;
  long calls = 0;
  while (std::getline(in, line)) {
    ++g_line;
    std::stringstream ss(line);
    std::vector<std::string> t;
    for (std::string tok; ss >> tok;) t.push_back(tok);
    if (t.size() < 2) continue;
    const std::string& f = t[0];
    const long long want = std::stoll(t[1]);
    auto need = [&](size_t n) { if (t.size() < n) { std::fprintf(stderr, "line %ld: short record\n", g_line); std::exit(2); } };
    ++calls;
    if (f == "ckpt_open") {
      need(4);
      mxp_ckpt* ck = nullptr;
      const Str path = unhex(t[3]);
      const int rc = mxp_ckpt_open(path.c(), &ck);
      expect(rc, want, "mxp_ckpt_open");
      if (rc == MXP_OK && ck) {
        walk_ckpt(ck);
        if (t[2] != "-") g_ckpts[std::stol(t[2])] = ck; else mxp_ckpt_close(ck);
      }
    } else if (f == "ckpt_close") {
      need(3);
      mxp_ckpt* ck = handle(g_ckpts, t[2]);
      if (ck) { mxp_ckpt_close(ck); g_ckpts.erase(std::stol(t[2])); }
    } else if (f == "plan_create") {
      need(7);
      mxp_plan* pl = nullptr;
      const int rc = mxp_plan_create(handle(g_ckpts, t[3]), std::stoi(t[4]), std::stoi(t[5]), (uint32_t)std::stoul(t[6]), &pl);
      expect(rc, want, "mxp_plan_create");
      if (rc == MXP_OK && pl) { if (t[2] != "-") g_plans[std::stol(t[2])] = pl; else mxp_plan_destroy(pl); }
    } else if (f == "plan_destroy") {
      need(3);
      mxp_plan* pl = handle(g_plans, t[2]);
      if (pl) { mxp_plan_destroy(pl); g_plans.erase(std::stol(t[2])); }
    } else if (f == "plan_add_param") {
      need(7);
      const Str name = unhex(t[3]);
      std::vector<int64_t> shape = ints(t[6]);
      shape.resize(std::max<size_t>(shape.size(), 1));
      expect(mxp_plan_add_param(handle(g_plans, t[2]), name.c(), std::stoi(t[4]), std::stoi(t[5]), shape.data()), want, "mxp_plan_add_param");
    } else if (f == "plan_add_stacked") {
      need(5);
      const Str a = unhex(t[3]), b = unhex(t[4]);
      expect(mxp_plan_add_stacked(handle(g_plans, t[2]), a.c(), b.c()), want, "mxp_plan_add_stacked");
    } else if (f == "plan_add_expert") {
      need(8);
      const Str a = unhex(t[3]), b = unhex(t[4]), shard = unhex(t[6]);
      expect(mxp_plan_add_expert(handle(g_plans, t[2]), a.c(), b.c(), std::stoi(t[5]), shard.c(), std::stoi(t[7])), want, "mxp_plan_add_expert");
    } else if (f == "plan_add_skip_prefix") {
      need(4);
      const Str a = unhex(t[3]);
      expect(mxp_plan_add_skip_prefix(handle(g_plans, t[2]), a.c()), want, "mxp_plan_add_skip_prefix");
    } else if (f == "plan_add_virtual") {
      need(6);
      const Str name = unhex(t[3]);
      std::vector<int64_t> shape = ints(t[5]);
      shape.resize(std::max<size_t>(shape.size(), 1));
      expect(mxp_plan_add_virtual(handle(g_plans, t[2]), name.c(), std::stoi(t[4]), shape.data()), want, "mxp_plan_add_virtual");
    } else if (f == "plan_add_virtual_shard") {
      need(9);
      const Str src = unhex(t[4]);
      std::vector<int64_t> a = ints(t[6]), b = ints(t[7]), c = ints(t[8]);
      const size_t n = std::max<size_t>(std::stoul(t[5]), 1);
      a.resize(std::max(a.size(), n)); b.resize(std::max(b.size(), n)); c.resize(std::max(c.size(), n));
      expect(mxp_plan_add_virtual_shard(handle(g_plans, t[2]), std::stoll(t[3]), src.c(), a.data(), b.data(), c.data()), want,
             "mxp_plan_add_virtual_shard");
    } else if (f == "plan_build") {
      need(3);
      mxp_plan* pl = handle(g_plans, t[2]);
      const int rc = mxp_plan_build(pl);
      expect(rc, want, "mxp_plan_build");
      if (pl && rc == MXP_OK) walk_plan(pl);
      if (pl) (void)(mxp_plan_param_count(pl) + mxp_plan_write_count(pl));  // a failed build leaves the handle usable
    } else if (f == "crc32c") {
      need(4);
      const Str data = unhex(t[3]);
      expect(mxp_crc32c((uint32_t)std::stoul(t[2]), data.null ? "" : data.s.data(), data.null ? 0 : data.s.size()), want, "mxp_crc32c");
    } else if (f == "file_crc32c") {
      need(7);
      const Str path = unhex(t[2]);
      const uint64_t max_chunks = std::stoull(t[4]);
      std::vector<uint32_t> crcs(std::max<uint64_t>(max_chunks, 1));
      uint32_t whole = 0;
      uint64_t n = 0;
      const int rc = mxp_file_crc32c(path.c(), std::stoull(t[3]), &whole, crcs.data(), max_chunks, &n);
      expect(rc, want, "mxp_file_crc32c");
      if (rc == MXP_OK) {
        expect(whole, std::stoll(t[5]), "mxp_file_crc32c (file checksum)");
        expect((long long)n, std::stoll(t[6]), "mxp_file_crc32c (chunk count)");
      }
    } else {
      std::fprintf(stderr, "line %ld: unknown record '%s'\n", g_line, f.c_str());
      return 2;
    }
  }
  for (auto& kv : g_plans) mxp_plan_destroy(kv.second);
  for (auto& kv : g_ckpts) mxp_ckpt_close(kv.second);
  // the small entry points, once
  if (mxp_abi_version() != MXP_ABI_VERSION) ++g_bad;
  for (int d = -2; d < 16; ++d) {
    const char* name = mxp_dtype_name(d);
    if (mxp_dtype_size(d) && (!name || mxp_dtype_from_name(name) != d)) ++g_bad;
  }
  if (mxp_dtype_from_name("") >= 0 || mxp_dtype_from_name("BF17") >= 0) ++g_bad;
  if (g_bad) { std::fprintf(stderr, "%d disagreement(s)\n", g_bad); return 1; }
  std::printf("%ld calls replayed\n", calls);
  return 0;
}
