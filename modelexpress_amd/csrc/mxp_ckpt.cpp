// Safetensors discovery and header parse.
//
// Byte format and resolution order follow the reference's own reader
// (modelexpress/gds_loader.py:189-282): u64 little-endian header length, JSON header,
// tensor data at 8 + header_len + data_offsets[0]; a sharded model is described by
// model.safetensors.index.json's weight_map, else model.safetensors, else every
// *.safetensors file in sorted order.
#include <dirent.h>
#include <fcntl.h>
#include <sys/stat.h>
#include <unistd.h>

#include <algorithm>
#include <cstdio>
#include <cstring>
#include <map>

#include "mxp_internal.hpp"
#include "mxp_json.hpp"

namespace mxp {

static thread_local std::string g_last_error;
void set_last_error(const std::string& msg) { g_last_error = msg; }

static const struct { const char* name; int code; int size; } kDtypes[] = {
    {"F64", MXP_DTYPE_F64, 8},         {"F32", MXP_DTYPE_F32, 4},   {"F16", MXP_DTYPE_F16, 2},
    {"BF16", MXP_DTYPE_BF16, 2},       {"F8_E4M3", MXP_DTYPE_F8_E4M3, 1},
    {"F8_E5M2", MXP_DTYPE_F8_E5M2, 1}, {"I64", MXP_DTYPE_I64, 8},   {"I32", MXP_DTYPE_I32, 4},
    {"I16", MXP_DTYPE_I16, 2},         {"I8", MXP_DTYPE_I8, 1},     {"U8", MXP_DTYPE_U8, 1},
    {"BOOL", MXP_DTYPE_BOOL, 1}};

int dtype_size(int dtype) {
  for (const auto& d : kDtypes)
    if (d.code == dtype) return d.size;
  return 0;
}

static std::string read_all(const std::string& path, uint64_t limit) {
  FILE* f = std::fopen(path.c_str(), "rb");
  if (!f) throw Error(MXP_ERR_IO, "cannot open " + path + ": " + std::strerror(errno));
  std::string out;
  char buf[1 << 16];
  size_t n;
  while ((n = std::fread(buf, 1, sizeof buf, f)) > 0) {
    out.append(buf, n);
    if (out.size() > limit) {
      std::fclose(f);
      throw Error(MXP_ERR_FORMAT, path + " is larger than expected");
    }
  }
  std::fclose(f);
  return out;
}

static bool exists(const std::string& p, bool* is_dir = nullptr) {
  struct stat st;
  if (::stat(p.c_str(), &st) != 0) return false;
  if (is_dir) *is_dir = S_ISDIR(st.st_mode);
  return true;
}

// Parses one file's header and appends its tensors (ascending file offset).
// `wanted` (may be null) restricts to the names the shard index assigns to this file.
static void parse_file(mxp_ckpt& ck, const std::string& path, const std::vector<std::string>* wanted) {
  const int fd = ::open(path.c_str(), O_RDONLY);
  if (fd < 0) throw Error(MXP_ERR_IO, "cannot open " + path + ": " + std::strerror(errno));
  struct stat st;
  if (::fstat(fd, &st) != 0) {
    ::close(fd);
    throw Error(MXP_ERR_IO, "cannot stat " + path);
  }
  const uint64_t file_size = (uint64_t)st.st_size;
  unsigned char lenb[8];
  if (::pread(fd, lenb, 8, 0) != 8) {
    ::close(fd);
    throw Error(MXP_ERR_FORMAT, "Invalid safetensors file: " + path);
  }
  uint64_t header_len = 0;
  for (int k = 7; k >= 0; --k) header_len = (header_len << 8) | lenb[k];
  if (header_len > 100ull * 1024 * 1024) {
    ::close(fd);
    throw Error(MXP_ERR_FORMAT, "Safetensors header too large (" + std::to_string(header_len) +
                                    " bytes): " + path);
  }
  if (8 + header_len > file_size) {
    ::close(fd);
    throw Error(MXP_ERR_FORMAT, "Safetensors header runs past the end of " + path);
  }
  std::string hdr(header_len, '\0');
  uint64_t got = 0;
  while (got < header_len) {
    const ssize_t n = ::pread(fd, &hdr[got], header_len - got, (off_t)(8 + got));
    if (n <= 0) {
      ::close(fd);
      throw Error(MXP_ERR_IO, "short read of header in " + path);
    }
    got += (uint64_t)n;
  }
  ::close(fd);

  Json root;
  try {
    root = JsonParser(hdr.data(), hdr.size()).parse();
  } catch (const std::exception& e) {
    throw Error(MXP_ERR_FORMAT, path + ": " + e.what());
  }
  if (root.type != Json::Object) throw Error(MXP_ERR_FORMAT, path + ": header is not an object");

  const uint64_t data_start = 8 + header_len;
  const int file_index = (int)ck.files.size();
  std::vector<TensorRec> recs;
  for (const auto& kv : root.obj) {
    if (kv.first == "__metadata__") continue;
    const Json& info = kv.second;
    const Json* jd = info.get("dtype");
    const Json* js = info.get("shape");
    const Json* jo = info.get("data_offsets");
    if (info.type != Json::Object || !jd || !js || !jo || jd->type != Json::String ||
        js->type != Json::Array || jo->type != Json::Array || jo->arr.size() != 2 ||
        jo->arr[0].type != Json::Int || jo->arr[1].type != Json::Int)
      throw Error(MXP_ERR_FORMAT, path + ": malformed entry for tensor '" + kv.first + "'");
    TensorRec t;
    t.name = kv.first;
    t.dtype = mxp_dtype_from_name(jd->s.c_str());
    if (t.dtype < 0)
      throw Error(MXP_ERR_UNSUPPORTED,
                  "Unsupported safetensors dtype '" + jd->s + "' for tensor '" + kv.first + "'");
    if (js->arr.size() > MXP_MAX_DIMS)
      throw Error(MXP_ERR_UNSUPPORTED, "tensor '" + kv.first + "' has more than 8 dims");
    uint64_t numel = 1;
    for (const auto& d : js->arr) {
      if (d.type != Json::Int || d.i < 0)
        throw Error(MXP_ERR_FORMAT, path + ": bad shape for tensor '" + kv.first + "'");
      t.shape.push_back(d.i);
      // a product that wraps must not pass for a small tensor
      if (__builtin_mul_overflow(numel, (uint64_t)d.i, &numel))
        throw Error(MXP_ERR_FORMAT, path + ": the shape of tensor '" + kv.first + "' overflows 64 bits");
    }
    const int64_t b = jo->arr[0].i, e = jo->arr[1].i;
    if (b < 0 || e < b) throw Error(MXP_ERR_FORMAT, path + ": bad data_offsets for '" + kv.first + "'");
    t.file_index = file_index;
    t.file_offset = data_start + (uint64_t)b;
    t.nbytes = (uint64_t)(e - b);
    uint64_t need_bytes = 0;
    if (__builtin_mul_overflow(numel, (uint64_t)dtype_size(t.dtype), &need_bytes))
      throw Error(MXP_ERR_FORMAT, path + ": the size of tensor '" + kv.first + "' overflows 64 bits");
    if (t.nbytes != need_bytes)
      throw Error(MXP_ERR_FORMAT, path + ": tensor '" + kv.first + "' has " + std::to_string(t.nbytes) +
                                      " bytes but its shape and dtype need " + std::to_string(need_bytes));
    if (t.file_offset + t.nbytes > file_size)
      throw Error(MXP_ERR_IO, path + ": tensor '" + kv.first + "' extends past the end of the file");
    recs.push_back(std::move(t));
  }
  std::stable_sort(recs.begin(), recs.end(),
                   [](const TensorRec& a, const TensorRec& b) { return a.file_offset < b.file_offset; });
  // Two tensors may not share bytes (the format lays them out back to back); empty ones have none.
  {
    const TensorRec* prev = nullptr;
    for (const auto& r : recs) {
      if (r.nbytes == 0) continue;
      if (prev && r.file_offset < prev->file_offset + prev->nbytes)
        throw Error(MXP_ERR_FORMAT, path + ": tensors '" + prev->name + "' and '" + r.name + "' overlap in the file");
      prev = &r;
    }
  }
  if (wanted) {
    // Every name the index assigns to this shard must be in its header: the reference's per-file
    // loop looks each one up and fails on a missing key (gds_loader.py:297-313).
    std::unordered_map<std::string, int> want;
    for (const auto& w : *wanted) want.emplace(w, 0);
    std::vector<TensorRec> keep;
    for (auto& r : recs) {
      auto it = want.find(r.name);
      if (it == want.end()) continue;
      it->second = 1;
      keep.push_back(std::move(r));
    }
    for (const auto& w : *wanted)
      if (!want[w]) throw Error(MXP_ERR_FORMAT, "tensor '" + w + "' is assigned to " + path + " by the index but is not in its header");
    recs.swap(keep);
  }
  FileRec fr;
  fr.path = path;
  fr.size = file_size;
  fr.data_start = data_start;
  fr.n_tensors = (int64_t)recs.size();
  ck.files.push_back(fr);
  for (auto& r : recs) {
    if (ck.by_name.count(r.name))
      throw Error(MXP_ERR_FORMAT, "tensor '" + r.name + "' appears in more than one file");
    ck.by_name.emplace(r.name, (int64_t)ck.tensors.size());
    ck.tensors.push_back(std::move(r));
  }
}

static void open_ckpt(mxp_ckpt& ck, const std::string& model_path) {
  bool is_dir = false;
  if (!exists(model_path, &is_dir)) throw Error(MXP_ERR_IO, "no such path: " + model_path);
  if (!is_dir) {
    parse_file(ck, model_path, nullptr);
    return;
  }
  const std::string dir = model_path.back() == '/' ? model_path : model_path + "/";
  const std::string index_path = dir + "model.safetensors.index.json";
  if (exists(index_path)) {
    const std::string text = read_all(index_path, 1ull << 30);
    Json root;
    try {
      root = JsonParser(text.data(), text.size()).parse();
    } catch (const std::exception& e) {
      throw Error(MXP_ERR_FORMAT, index_path + ": " + e.what());
    }
    const Json* wm = root.get("weight_map");
    if (!wm || wm->type != Json::Object || wm->obj.empty())
      throw Error(MXP_ERR_FORMAT, "Empty weight_map in " + index_path);
    // file -> tensor names, files in first-appearance order (a dict keyed by file).
    std::vector<std::string> order;
    std::unordered_map<std::string, std::vector<std::string>> per_file;
    for (const auto& kv : wm->obj) {
      if (kv.second.type != Json::String)
        throw Error(MXP_ERR_FORMAT, index_path + ": weight_map value is not a string");
      auto it = per_file.find(kv.second.s);
      if (it == per_file.end()) {
        order.push_back(kv.second.s);
        it = per_file.emplace(kv.second.s, std::vector<std::string>()).first;
      }
      it->second.push_back(kv.first);
    }
    for (const auto& f : order) parse_file(ck, dir + f, &per_file[f]);
    return;
  }
  const std::string single = dir + "model.safetensors";
  if (exists(single)) {
    parse_file(ck, single, nullptr);
    return;
  }
  std::vector<std::string> found;
  if (DIR* d = ::opendir(dir.c_str())) {
    while (dirent* e = ::readdir(d)) {
      const std::string n = e->d_name;
      const std::string suf = ".safetensors";
      if (n.size() > suf.size() && n.compare(n.size() - suf.size(), suf.size(), suf) == 0)
        found.push_back(n);
    }
    ::closedir(d);
  }
  if (found.empty()) throw Error(MXP_ERR_IO, "No .safetensors files found in " + model_path);
  std::sort(found.begin(), found.end());
  for (const auto& f : found) parse_file(ck, dir + f, nullptr);
}

}  // namespace mxp

using namespace mxp;

extern "C" {

const char* mxp_last_error(void) { return g_last_error.c_str(); }
int mxp_abi_version(void) { return MXP_ABI_VERSION; }

int mxp_dtype_size(int dtype) { return dtype_size(dtype); }
int mxp_dtype_from_name(const char* name) {
  if (!name) return -1;
  for (const auto& d : kDtypes)
    if (std::strcmp(d.name, name) == 0) return d.code;
  return -1;
}
const char* mxp_dtype_name(int dtype) {
  for (const auto& d : kDtypes)
    if (d.code == dtype) return d.name;
  return "";
}

int mxp_ckpt_open(const char* model_path, mxp_ckpt** out) {
  return guard([&] {
    if (!model_path || !out) throw Error(MXP_ERR_ARG, "mxp_ckpt_open: null argument");
    *out = nullptr;
    auto ck = std::make_unique<mxp_ckpt>();
    open_ckpt(*ck, model_path);
    *out = ck.release();
  });
}
void mxp_ckpt_close(mxp_ckpt* ckpt) { delete ckpt; }
int64_t mxp_ckpt_tensor_count(const mxp_ckpt* c) { return c ? (int64_t)c->tensors.size() : 0; }
int64_t mxp_ckpt_file_count(const mxp_ckpt* c) { return c ? (int64_t)c->files.size() : 0; }
int mxp_ckpt_tensor_info(const mxp_ckpt* c, int64_t i, mxp_tensor_info* out) {
  return guard([&] {
    if (!c || !out || i < 0 || i >= (int64_t)c->tensors.size())
      throw Error(MXP_ERR_ARG, "mxp_ckpt_tensor_info: bad index");
    const TensorRec& t = c->tensors[i];
    std::memset(out, 0, sizeof *out);
    out->name = t.name.c_str();
    out->dtype = t.dtype;
    out->ndim = (int32_t)t.shape.size();
    for (size_t d = 0; d < t.shape.size(); ++d) out->shape[d] = t.shape[d];
    out->file_index = t.file_index;
    out->file_offset = t.file_offset;
    out->nbytes = t.nbytes;
  });
}
int mxp_ckpt_file_info(const mxp_ckpt* c, int64_t i, mxp_file_info* out) {
  return guard([&] {
    if (!c || !out || i < 0 || i >= (int64_t)c->files.size())
      throw Error(MXP_ERR_ARG, "mxp_ckpt_file_info: bad index");
    const FileRec& f = c->files[i];
    out->path = f.path.c_str();
    out->file_size = f.size;
    out->data_start = f.data_start;
    out->n_tensors = f.n_tensors;
  });
}
int64_t mxp_ckpt_find(const mxp_ckpt* c, const char* name) {
  if (!c || !name) return -1;
  auto it = c->by_name.find(name);
  return it == c->by_name.end() ? -1 : it->second;
}

}  // extern "C"
