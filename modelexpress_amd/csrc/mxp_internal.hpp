// Host-side data model shared by the checkpoint reader, the planner and the engine.
#pragma once
#include <cstdint>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

#include "mxp.h"
#include "mxp_bench.h"
#include "mxp_device.h"

namespace mxp {

// Error carrying an MXP_ERR_* class; converted to a status code at the C boundary.
struct Error : std::runtime_error {
  int code;
  Error(int c, const std::string& m) : std::runtime_error(m), code(c) {}
};

void set_last_error(const std::string& msg);
int dtype_size(int dtype);

// Runs `fn`, mapping exceptions to status codes and recording the message.
template <typename F>
int guard(F&& fn) {
  try {
    set_last_error("");
    fn();
    return MXP_OK;
  } catch (const Error& e) {
    set_last_error(e.what());
    return e.code;
  } catch (const std::bad_alloc&) {
    set_last_error("out of host memory");
    return MXP_ERR_STATE;
  } catch (const std::exception& e) {
    set_last_error(e.what());
    return MXP_ERR_STATE;
  }
}

struct TensorRec {
  std::string name;
  int dtype = 0;
  std::vector<int64_t> shape;
  int file_index = 0;
  uint64_t file_offset = 0;
  uint64_t nbytes = 0;
};

struct FileRec {
  std::string path;
  uint64_t size = 0;
  uint64_t data_start = 0;
  int64_t n_tensors = 0;
};

struct ParamRec {
  std::string name;
  int dtype = 0;
  std::vector<int64_t> shape;
  uint64_t nbytes = 0;
  uint64_t bytes_written = 0;
  int n_writes = 0;
};

struct WriteRec {
  int64_t tensor = -1, param = -1;
  int kind = 0, cast = 0;
  uint64_t src_offset = 0, src_pitch = 0, dst_offset = 0, dst_pitch = 0, rows = 0, row_bytes = 0;
  uint64_t paired_runs = 0;
};

// A virtual checkpoint tensor assembled from boxes of real tensors: the published-tensor /
// shard model of the reference's reshard path (a full shape plus shards at offsets).
struct VirtualShard {
  int64_t tensor = -1;                 // real source tensor
  std::vector<int64_t> src_offset;     // box origin inside the source tensor
  std::vector<int64_t> shard_offset;   // box origin inside the virtual tensor
  std::vector<int64_t> shape;
};
struct VirtualRec {
  std::string name;
  std::vector<int64_t> shape;
  int dtype = -1;
  std::vector<VirtualShard> shards;
};

struct StackedRec { std::string fused, member; int order; };
struct ExpertRec { std::string param_prefix, weight_prefix; int expert_id; std::string shard; int local_id; };

// One slot-sized unit of ingest work: byte ranges packed into a staging slot and the
// device segments that consume them.
// `rows` pieces of `nbytes`, `file_pitch` apart in the file, packed back to back in the slot.
struct FileRange {
  int file;
  uint64_t file_off, nbytes, slot_off;
  uint64_t rows = 1, file_pitch = 0;
  uint64_t need = 0;  // bytes that must exist (a direct-I/O range is rounded up past them); 0 = all
};
// A contiguous, unconverted piece of a chunk that is copied from the pinned slot straight to its
// final place in a parameter buffer.
struct DirectCopy {
  uint64_t slot_off, dst_off, nbytes;
  uint32_t param;
};
struct Chunk {
  std::vector<FileRange> ranges;
  std::vector<DirectCopy> direct;                           // pinned slot -> parameter buffer
  std::vector<std::pair<uint64_t, uint64_t>> bounce_runs;   // (slot offset, bytes): pinned slot -> bounce slot
  uint64_t used_bytes = 0;   // bytes of the slot in use
  uint32_t seg_begin = 0, seg_count = 0;    // into the ingest segment table
  uint32_t work_begin = 0, work_count = 0;  // into the ingest work table
};

}  // namespace mxp

struct mxp_ckpt {
  std::vector<mxp::FileRec> files;
  std::vector<mxp::TensorRec> tensors;
  std::unordered_map<std::string, int64_t> by_name;
};

struct mxp_plan {
  const mxp_ckpt* ckpt = nullptr;
  int tp_size = 1, tp_rank = 0;
  uint32_t flags = 0;
  std::vector<mxp::ParamRec> params;
  std::unordered_map<std::string, int64_t> param_by_name;
  std::vector<mxp::StackedRec> stacked;
  std::vector<mxp::ExpertRec> experts;
  std::vector<std::string> skip_prefixes;
  std::vector<mxp::VirtualRec> virtuals;
  std::vector<mxp::WriteRec> writes;
  std::vector<std::string> skipped;  // tensors deliberately not placed
  bool built = false;

  // ---- lowered state, owned by the engine that first executes the plan ----
  struct Lowered;
  Lowered* lowered = nullptr;
  void (*lowered_free)(Lowered*) = nullptr;
  ~mxp_plan() {
    if (lowered && lowered_free) lowered_free(lowered);
  }
};
