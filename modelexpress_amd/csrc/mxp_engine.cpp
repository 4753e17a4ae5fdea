// Engine: lowers a built plan to device descriptor tables and executes it, either by
// ingesting the planned byte ranges from storage through a bounded ring of pinned host
// slots (pread -> hipMemcpyAsync -> placement kernel, one HIP stream per slot group), or
// from a checkpoint already staged in HBM (one launch for the whole plan).
//
// Ownership: the caller owns every destination buffer; the engine owns the pinned ring,
// the device bounce slots, streams, events and descriptor tables.  All HIP work issued
// by a call has completed when the call returns, unless documented otherwise.
#include <fcntl.h>
#include <sys/stat.h>
#include <hip/hip_runtime.h>
#include <unistd.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <thread>

#include "mxp_blake2b.hpp"
#include "mxp_internal.hpp"
#include "mxp_lower.hpp"

namespace mxp {
namespace {

#define HIP_OK(expr)                                                                          \
  do {                                                                                        \
    const hipError_t e_ = (expr);                                                             \
    if (e_ != hipSuccess)                                                                     \
      throw Error(MXP_ERR_DEVICE, std::string(#expr) + ": " + hipGetErrorString(e_));         \
  } while (0)

// Scratch of the entry point that allocates nothing (mxp_checksum32_static): descriptor tables,
// source pointers and checksum accumulators of one call.  One copy per GPU, held until the
// process ends; every call on a GPU shares it.  Host code never uses the array's name as an
// address: mxp_engine_create looks the device address up once per device (static_scratch_for)
// and everything else goes through that pointer.
constexpr size_t kStaticMaxBuffers = 1024;                       // buffers per call
constexpr size_t kStaticMaxSegs = 3 * kStaticMaxBuffers;         // a contiguous run lowers to at most 3 segments
constexpr size_t kStaticMaxWork = 96 * 1024;                     // workgroups per call (128 KiB each: 12 GiB)
constexpr size_t kStaticOffSegs = 0;
constexpr size_t kStaticOffWork = kStaticOffSegs + kStaticMaxSegs * sizeof(Seg);
constexpr size_t kStaticOffPtrs = kStaticOffWork + kStaticMaxWork * sizeof(WorkItem);
constexpr size_t kStaticOffSums = kStaticOffPtrs + kStaticMaxBuffers * sizeof(void*);
constexpr size_t kStaticScratchBytes = 1u << 20;
static_assert(kStaticOffSums + kStaticMaxBuffers * sizeof(uint32_t) <= kStaticScratchBytes, "scratch layout");
static_assert(kStaticOffWork % 256 == 0 && kStaticOffPtrs % 256 == 0 && kStaticOffSums % 256 == 0, "scratch layout");
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
unsigned char* g_scratch_ptr[kMaxDevices] = {};  // device address of `scratch` on each GPU

// Device address of this GPU's copy of `scratch`; `device` must be current.
unsigned char* static_scratch_for(int device) {
  if (device < 0 || device >= kMaxDevices) throw Error(MXP_ERR_ARG, "device ordinal out of range");
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[device]) {
    void* p = nullptr;
    const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p)
      throw Error(MXP_ERR_DEVICE, std::string("hipGetSymbolAddress(scratch): ") + hipGetErrorString(e));
    g_scratch_ptr[device] = static_cast<unsigned char*>(p);
  }
  return g_scratch_ptr[device];
}

// push_back / size over memory the caller owns; refuses to grow.
template <typename T>
struct FixedTable {
  T* p;
  size_t cap, n = 0;
  const char* what;
  FixedTable(void* mem, size_t capacity, const char* name) : p(static_cast<T*>(mem)), cap(capacity), what(name) {}
  void push_back(const T& v) {
    if (n == cap) throw Error(MXP_ERR_ARG, std::string(what));
    p[n++] = v;
  }
  size_t size() const { return n; }
};

double now_s() {
  return std::chrono::duration<double>(std::chrono::steady_clock::now().time_since_epoch()).count();
}
uint64_t align_up(uint64_t v, uint64_t a) { return (v + a - 1) / a * a; }

// Waits for `ev` by polling for up to two milliseconds before it blocks: a blocking wait wakes up
// tens of microseconds after the event, which a caller that waits for a 0.3 ms launch notices.
hipError_t wait_event_promptly(hipEvent_t ev) {
  const double t0 = now_s();
  for (;;) {
    const hipError_t r = hipEventQuery(ev);
    if (r != hipErrorNotReady) return r;
    if (now_s() - t0 > 2e-3) return hipEventSynchronize(ev);
  }
}

}  // namespace

// Pieces below this size take the bounce slot by default: a copy call of their own would cost more than it saves.
constexpr uint64_t kDirectMinBytes = 64 * 1024;

template <typename T>
struct DevBuf {
  T* p = nullptr;
  size_t cap = 0;
  void reserve(size_t n) {
    if (n <= cap) return;
    if (p) (void)hipFree(p);
    p = nullptr;
    cap = 0;
    HIP_OK(hipMalloc(reinterpret_cast<void**>(&p), n * sizeof(T)));
    cap = n;
  }
  void upload(const T* host, size_t n) {
    reserve(n ? n : 1);
    if (n) HIP_OK(hipMemcpy(p, host, n * sizeof(T), hipMemcpyHostToDevice));
  }
  ~DevBuf() {
    if (p) (void)hipFree(p);
  }
};

struct Slot {
  uint8_t* host = nullptr;  // pinned
  uint8_t* dev = nullptr;   // bounce
  hipEvent_t done = nullptr;
  std::mutex mu;
  std::condition_variable cv;
  uint64_t submitted = 0;  // number of chunks this slot has carried to the GPU
};

}  // namespace mxp

using namespace mxp;

struct mxp_plan::Lowered {
  uint64_t slot_bytes = 0;
  uint32_t tile_bytes = 0;
  bool host_pack = false;
  uint64_t direct_min = 0;
  int reader_threads = 0;  // the chunk-size ramp depends on it
  bool direct_io = false;
  // resident tables: source buffer index = shard file index
  DevBuf<Seg> res_segs;
  DevBuf<WorkItem> res_work;
  uint32_t res_n_work = 0, res_n_segs = 0;
  // ingest tables: source buffer index 0 = the chunk's bounce slot
  std::vector<Chunk> chunks;
  DevBuf<Seg> ing_segs;
  DevBuf<WorkItem> ing_work;
  uint32_t ing_n_segs = 0, ing_n_work = 0;
  // per execute
  DevBuf<void*> dst_bases;
  DevBuf<const void*> src_bases;
  // Accumulators, two sets: a launch adds to one set and clears the other one on its way, so the
  // next launch finds zeros without a clearing launch of its own.  One set = [checksum per parameter]
  // [five 64-bit digest sums per parameter], both fanned by `fan`.  `clean[s]` = the host knows set s
  // holds zeros; `digest_used[s]` = a launch has added digest sums to set s since it was last
  // cleared (otherwise only the checksums need clearing).
  DevBuf<uint32_t> acc;
  Fan fan;
  size_t acc_stride = 0, acc_digest_off = 0, acc_words = 0;  // in 32-bit words
  int cur = 0;
  bool clean[2] = {false, false};
  bool digest_used[2] = {false, false};
  size_t dirty_words(int set) const { return digest_used[set] ? acc_words : acc_digest_off; }
  bool single_set = false;  // a launch of this plan was captured into a graph: set 0 only from then on
  uint32_t* sums(int set) { return acc.p + (size_t)set * acc_stride; }
  unsigned long long* digest_sums(int set) { return reinterpret_cast<unsigned long long*>(acc.p + (size_t)set * acc_stride + acc_digest_off); }
  DevBuf<unsigned long long> dst_sizes;    // byte size of every parameter (fused digests)
  bool digests_valid = false;              // the last execute accumulated them
  std::vector<void*> dst_host;        // what dst_bases currently holds
  std::vector<const void*> src_host;  // what src_bases currently holds
  // The pointer tables are rewritten with stream-ordered copies out of this pinned block
  // ([destinations][sources]); `upload_done` guards the block.  A call on another stream than the
  // last launch's (`last_stream`) records `launch_done` on that stream and waits for it, so the
  // tables and accumulators are not touched under a launch that still reads them.
  void** tab_host = nullptr;
  size_t tab_cap = 0;
  hipEvent_t upload_done = nullptr, launch_done = nullptr;
  bool upload_rec = false, launch_rec = false;
  hipStream_t last_stream = nullptr;
  uint64_t file_bytes = 0, h2d_bytes = 0, placed_bytes = 0, algo_bytes = 0;
  ~Lowered() {
    if (tab_host) (void)hipHostFree(tab_host);
    if (upload_done) (void)hipEventDestroy(upload_done);
    if (launch_done) (void)hipEventDestroy(launch_done);
  }
};

struct mxp_engine {
  mxp_engine_options opt{};
  std::vector<std::unique_ptr<Slot>> slots;
  uint8_t* pinned_base = nullptr;
  uint8_t* bounce_base = nullptr;
  std::vector<hipStream_t> streams;
  DevBuf<const void*> slot_ptrs;  // device table: slot i -> bounce address
  // Descriptor staging for the stand-alone operators: a pinned block and its device twin, kept
  // twice and used in turn, so a call fills one while the device may still read what the call
  // before it uploaded into the other (back-to-back calls do not wait for each other's kernels).
  // `busy` is recorded after the last device use of an arena; whoever takes it next waits for it.
  struct Arena {
    uint8_t* host = nullptr;      // pinned
    uint8_t* host_dev = nullptr;  // the address kernels read `host` at
    size_t host_cap = 0;
    DevBuf<uint8_t> dev;
    hipEvent_t busy = nullptr;
    bool recorded = false;
    ~Arena() {
      if (busy) (void)hipEventDestroy(busy);
      if (host) (void)hipHostFree(host);
    }
  };
  Arena arenas[2];
  unsigned arena_turn = 0;
  hipEvent_t ev_a = nullptr, ev_b = nullptr;
  hipEvent_t caller_ev = nullptr;   // what the caller had queued when an ingest started
  bool fused_digests = false;       // placements also accumulate the tensor_digest sums (mxp_engine_set_fused_digests)
  uint64_t direct_min = kDirectMinBytes;  // ingest copies contiguous pieces of at least this size straight to their
                                          // final address; 0 = none (mxp_engine_set_direct_placement)
  // descriptor table of batched transposes: same protocol as the arenas, also kept twice
  struct ItemTable {
    TransposeItem* host = nullptr;      // pinned
    TransposeItem* host_dev = nullptr;  // the address kernels read `host` at
    size_t cap = 0;
    DevBuf<TransposeItem> dev;
    hipEvent_t busy = nullptr;
    bool recorded = false;
    ~ItemTable() {
      if (busy) (void)hipEventDestroy(busy);
      if (host) (void)hipHostFree(host);
    }
  };
  ItemTable item_tabs[2];
  unsigned items_turn = 0;
  // launch timing (mxp_engine_set_launch_timing): event pairs around the placement kernel of the
  // last kTimingRing resident launches, recorded without synchronising
  std::vector<std::pair<hipEvent_t, hipEvent_t>> timing_ring;
  bool timing_on = false;
  uint64_t timing_count = 0;
  // mxp_checksum32_static: this GPU's scratch array and a pinned mirror of it, both set up at create
  unsigned char* static_dev = nullptr;
  unsigned char* static_host = nullptr;  // pinned

  ~mxp_engine() {
    for (auto& pr : timing_ring) { (void)hipEventDestroy(pr.first); (void)hipEventDestroy(pr.second); }
    if (static_host) (void)hipHostFree(static_host);
    if (caller_ev) (void)hipEventDestroy(caller_ev);
    for (auto s : streams) (void)hipStreamDestroy(s);
    for (auto& s : slots)
      if (s->done) (void)hipEventDestroy(s->done);
    if (pinned_base) (void)hipHostFree(pinned_base);
    if (bounce_base) (void)hipFree(bounce_base);
    if (ev_a) (void)hipEventDestroy(ev_a);
    if (ev_b) (void)hipEventDestroy(ev_b);
  }
};

namespace mxp {
namespace {

void free_lowered(mxp_plan::Lowered* l) { delete l; }

// Direct I/O, rows packed by the readers: how many consecutive rows (`pitch` bytes apart, `row_bytes`
// long) one read request covers.  A request per row is a 4-8 KiB random read, and the device's request
// rate then bounds the ingest (262,144 of them for a Llama-3-8B rank's column slices: 1.3 GB/s on a disk
// that gives 5 GB/s to large requests).  Where the rows lie close enough that reading what is between
// them costs less than that - at most eight times the blocks the rows themselves touch - a request
// covers as many rows as the reader's block-aligned buffer holds, and the rows are copied out of it.
inline uint64_t direct_rows_per_read(uint64_t buf_bytes, uint64_t pitch, uint64_t row_bytes) {
  const uint64_t window = align_up(row_bytes + 4095, 4096);  // blocks one unaligned row can touch
  if (pitch > 8 * window || buf_bytes < 2 * 4096 + row_bytes) return 1;
  return std::max<uint64_t>(1, (buf_bytes - 2 * 4096 - row_bytes) / pitch + 1);
}
// Bytes the requests for `rows` such rows starting at file offset `off` read in all.
inline uint64_t direct_rows_file_bytes(uint64_t buf_bytes, uint64_t off, uint64_t rows, uint64_t pitch, uint64_t row_bytes) {
  const uint64_t per = direct_rows_per_read(buf_bytes, pitch, row_bytes);
  uint64_t total = 0;
  for (uint64_t r = 0; r < rows; r += per) {
    const uint64_t nr = std::min(per, rows - r), o0 = off + r * pitch;
    total += align_up(o0 + (nr - 1) * pitch + row_bytes, 4096) - o0 / 4096 * 4096;
  }
  return total;
}

// Splits every write into slot-sized pieces, packs their byte ranges into chunks in
// (file, offset) order, and lowers both the ingest and the resident descriptor tables.
void lower_plan(mxp_plan& pl, const mxp_engine& eng) {
  if (!pl.built) throw Error(MXP_ERR_STATE, "plan has not been built");
  const bool host_pack = eng.opt.pack_strided_on_host == 1;
  if (pl.lowered && pl.lowered->slot_bytes == eng.opt.slot_bytes && pl.lowered->tile_bytes == eng.opt.tile_bytes &&
      pl.lowered->host_pack == host_pack && pl.lowered->direct_io == (eng.opt.use_o_direct != 0) &&
      pl.lowered->direct_min == eng.direct_min &&
      pl.lowered->reader_threads == eng.opt.reader_threads)
    return;
  if (pl.lowered) { free_lowered(pl.lowered); pl.lowered = nullptr; }
  auto L = std::make_unique<mxp_plan::Lowered>();
  L->slot_bytes = eng.opt.slot_bytes;
  L->tile_bytes = eng.opt.tile_bytes;
  L->host_pack = host_pack;
  L->direct_min = eng.direct_min;
  L->direct_io = eng.opt.use_o_direct != 0;
  L->reader_threads = eng.opt.reader_threads;
  // Direct I/O reads whole 4 KiB blocks at 4 KiB offsets into 4 KiB aligned memory: every
  // range is widened to block boundaries and the box starts that many bytes into the slot.
  const uint64_t blk = L->direct_io ? 4096 : 1;
  LowerOptions lo;
  lo.tile_bytes = eng.opt.tile_bytes;
  const mxp_ckpt& ck = *pl.ckpt;

  // ---- resident: one box per write, source = staged shard file ----
  {
    std::vector<Seg> segs;
    std::vector<WorkItem> work;
    for (const auto& w : pl.writes) {
      const TensorRec& t = ck.tensors[w.tensor];
      BoxCopy b;
      b.src_buf = (uint32_t)t.file_index;
      b.dst_buf = (uint32_t)w.param;
      b.src_off = t.file_offset + w.src_offset;
      b.dst_off = w.dst_offset;
      b.src_pitch = w.src_pitch;
      b.dst_pitch = w.dst_pitch;
      b.rows = w.rows;
      b.row_bytes = w.row_bytes;
      b.op = seg_op_of_cast(w.cast);
      b.csum_slot = (uint32_t)w.param;
      lower_box(b, lo, segs, work);
      L->placed_bytes += w.rows * w.row_bytes;
      L->algo_bytes += w.rows * (w.row_bytes + op_src_bytes(b.op, w.row_bytes));
    }
    L->res_n_segs = (uint32_t)segs.size();
    L->res_n_work = (uint32_t)work.size();
    L->res_segs.upload(segs.data(), segs.size());
    L->res_work.upload(work.data(), work.size());
  }

  // ---- ingest: pieces in file order ----
  struct Piece {
    int file;
    uint64_t file_off, nbytes;  // byte range to read (one row of it when rows > 1)
    BoxCopy box;                // src_off relative to the start of the range
    uint64_t rows = 1, file_pitch = 0;  // rows > 1: strided in the file, packed in the slot
  };
  std::vector<Piece> pieces;
  // A strided row packed by a reader costs a read call of its own, about as much as copying a page:
  // towards a chunk's capacity it counts as at least 4 KiB, so a chunk of 1 KiB rows holds a quarter
  // of the rows it has room for and the readers share such tensors more evenly (the end-to-end rate
  // of the Llama rank rose from 94.7-96.6 % to 95.4-98.4 % of pinned H2D in same-box runs).
  constexpr uint64_t kPackedRowCost = 4096;
  const uint64_t slot = L->direct_io ? eng.opt.slot_bytes - 2 * blk : eng.opt.slot_bytes;
  for (const auto& w : pl.writes) {
    const TensorRec& t = ck.tensors[w.tensor];
    const uint32_t op = seg_op_of_cast(w.cast);
    const uint64_t row_src = op_src_bytes(op, w.row_bytes);
    BoxCopy b;
    b.src_buf = 0;
    b.dst_buf = (uint32_t)w.param;
    b.op = op;
    b.csum_slot = (uint32_t)w.param;
    const uint64_t t0 = t.file_offset + w.src_offset;
    if (w.rows == 1 || (w.src_pitch == row_src && w.dst_pitch == w.row_bytes)) {
      // contiguous run: split on 4 KiB multiples of destination bytes
      const uint64_t total = w.rows * w.row_bytes;
      const uint64_t max_dst = std::min(slot, op_dst_bytes(op, slot)) / 4096 * 4096;
      for (uint64_t done = 0; done < total; done += max_dst) {
        const uint64_t n = std::min(max_dst, total - done);
        Piece p{t.file_index, t0 + op_src_bytes(op, done), op_src_bytes(op, n), b};
        p.box.src_off = 0;
        p.box.dst_off = w.dst_offset + done;
        p.box.rows = 1;
        p.box.row_bytes = n;
        p.box.src_pitch = op_src_bytes(op, n);
        p.box.dst_pitch = n;
        pieces.push_back(p);
      }
    } else if (host_pack) {
      // strided source, packed by the readers: only the needed bytes cross PCIe and the
      // slot holds the rows back to back, so the device sees a plain copy
      if (row_src > slot) throw Error(MXP_ERR_UNSUPPORTED, "a source row of '" + t.name + "' does not fit a staging slot");
      uint64_t max_rows = slot / std::max<uint64_t>(row_src, kPackedRowCost);
      // Direct I/O reads the file span the rows lie in: a piece is what one request covers, so that a chunk costs
      // its reader one request like any other (a piece of 4096 rows of a 28 KiB pitch would be seven requests in
      // a row for one reader while the others run out of work).
      if (L->direct_io) {
        const uint64_t per = direct_rows_per_read(eng.opt.slot_bytes, w.src_pitch, row_src);
        if (per > 1) max_rows = std::min(max_rows, per);  // per == 1: rows far apart, read one by one
      }
      for (uint64_t r = 0; r < w.rows; r += max_rows) {
        const uint64_t nr = std::min(max_rows, w.rows - r);
        Piece p{t.file_index, t0 + r * w.src_pitch, row_src, b, nr, w.src_pitch};
        p.box.src_off = 0;
        p.box.dst_off = w.dst_offset + r * w.dst_pitch;
        p.box.rows = nr;
        p.box.row_bytes = w.row_bytes;
        p.box.src_pitch = row_src;
        p.box.dst_pitch = w.dst_pitch;
        pieces.push_back(p);
      }
    } else {
      // strided source: stage whole row bands and gather on the device
      if (w.src_pitch > slot || row_src > slot)
        throw Error(MXP_ERR_UNSUPPORTED, "a source row of '" + t.name + "' does not fit a staging slot");
      const uint64_t max_rows = (slot - row_src) / w.src_pitch + 1;
      for (uint64_t r = 0; r < w.rows; r += max_rows) {
        const uint64_t nr = std::min(max_rows, w.rows - r);
        Piece p{t.file_index, t0 + r * w.src_pitch, (nr - 1) * w.src_pitch + row_src, b};
        p.box.src_off = 0;
        p.box.dst_off = w.dst_offset + r * w.dst_pitch;
        p.box.rows = nr;
        p.box.row_bytes = w.row_bytes;
        p.box.src_pitch = w.src_pitch;
        p.box.dst_pitch = w.dst_pitch;
        pieces.push_back(p);
      }
    }
  }
  std::stable_sort(pieces.begin(), pieces.end(), [](const Piece& a, const Piece& b) {
    return a.file != b.file ? a.file < b.file : a.file_off < b.file_off;
  });
  {
    std::vector<Seg> segs;
    std::vector<WorkItem> work;
    Chunk cur;
    uint64_t cur_cost = 0;
    auto close = [&] {
      if (cur.ranges.empty()) return;
      cur.seg_count = (uint32_t)segs.size() - cur.seg_begin;
      cur.work_count = (uint32_t)work.size() - cur.work_begin;
      for (const auto& d : cur.direct) L->h2d_bytes += d.nbytes;
      for (const auto& r : cur.bounce_runs) L->h2d_bytes += r.second;
      L->chunks.push_back(cur);
      cur = Chunk();
      cur_cost = 0;
    };
    // Chunk capacity ramps up: every reader thread starts on a small chunk, so the first
    // host-to-device copy is issued after a 2 MiB read instead of a whole slot's, and the
    // copies already queued hide the longer reads that follow.
    const uint64_t threads = (uint64_t)std::max(1, eng.opt.reader_threads);
    // A small checkpoint is cut into at least four chunks per reader, so that the readers finish together and
    // the last copy is short: a quarter-GB checkpoint in 16 MiB chunks gives sixteen readers one chunk each and
    // the link idles while the last ones are read (GPT-2-small: 0.81 -> 0.88 of pinned H2D with 4 MiB chunks).
    uint64_t staged_total = 0;
    for (const auto& p : pieces) staged_total += p.nbytes * p.rows;
    const uint64_t small_cap = std::max<uint64_t>((uint64_t)(2u << 20), staged_total / (4 * threads) / 4096 * 4096);
    auto capacity = [&](size_t chunk_index) -> uint64_t {
      if (L->direct_io) return eng.opt.slot_bytes;
      const uint64_t step = chunk_index / threads;
      const uint64_t cap = std::min(small_cap, step >= 3 ? eng.opt.slot_bytes : (uint64_t)(2u << 20) << step);
      return std::min<uint64_t>(eng.opt.slot_bytes, std::max<uint64_t>(cap, 64 * 1024));
    };
    for (size_t pi = 0; pi < pieces.size(); ++pi) {
      Piece p = pieces[pi];
      for (;;) {
        const uint64_t cap = capacity(L->chunks.size());
        uint64_t at = align_up(cur.used_bytes, L->direct_io ? blk : 256);
        // A contiguous run that does not fit what is left of this chunk is cut at a 4 KiB
        // multiple of destination bytes; the remainder goes on into the next chunk.
        Piece rest;
        bool have_rest = false;
        if (!L->direct_io && p.rows == 1 && p.box.rows == 1 && at + p.nbytes > cap) {
          const uint64_t room_src = cap > at ? cap - at : 0;
          const uint64_t k = op_dst_bytes(p.box.op, room_src) / 4096 * 4096;  // destination bytes that fit
          if (k == 0 && !cur.ranges.empty()) {
            close();
            continue;
          }
          if (k > 0 && k < p.box.row_bytes) {
            rest = p;
            have_rest = true;
            const uint64_t ks = op_src_bytes(p.box.op, k);
            rest.file_off += ks;
            rest.nbytes -= ks;
            rest.box.dst_off += k;
            rest.box.row_bytes -= k;
            rest.box.src_pitch = rest.nbytes;
            rest.box.dst_pitch = rest.box.row_bytes;
            p.nbytes = ks;
            p.box.row_bytes = k;
            p.box.src_pitch = ks;
            p.box.dst_pitch = k;
          }
        }
        uint64_t lead = 0, need = 0;
        if (L->direct_io && p.rows > 1) {
          // packed rows: whole blocks are read into the reader's own buffer (several rows per request
          // where they lie close together) and only the rows' bytes are copied into the slot, so the
          // slot layout is that of buffered packing
          L->file_bytes += direct_rows_file_bytes(eng.opt.slot_bytes, p.file_off, p.rows, p.file_pitch, p.nbytes);
          L->file_bytes -= p.nbytes * p.rows;  // added back below with the slot bytes
        } else if (L->direct_io) {
          const uint64_t a0 = p.file_off / blk * blk, a1 = align_up(p.file_off + p.nbytes, blk);
          lead = p.file_off - a0;
          need = lead + p.nbytes;
          p.file_off = a0;
          p.nbytes = a1 - a0;
        }
        const uint64_t in_slot = p.nbytes * p.rows;
        const uint64_t piece_cost = p.rows > 1 ? (L->direct_io ? direct_rows_file_bytes(eng.opt.slot_bytes, p.file_off, p.rows, p.file_pitch, p.nbytes)
                                                              : p.rows * std::max<uint64_t>(p.nbytes, kPackedRowCost))
                                               : in_slot;
        if (!cur.ranges.empty() && (at + in_slot > cap || cur_cost + piece_cost > cap)) {
          close();
          at = 0;
        }
        cur_cost += piece_cost;
        if (at + in_slot > eng.opt.slot_bytes) throw Error(MXP_ERR_STATE, "internal: a piece does not fit a staging slot");
        if (cur.ranges.empty()) {
          cur.seg_begin = (uint32_t)segs.size();
          cur.work_begin = (uint32_t)work.size();
        }
        cur.ranges.push_back(FileRange{p.file, p.file_off, p.nbytes, at, p.rows, p.file_pitch, need});
        cur.used_bytes = at + in_slot;
        L->file_bytes += in_slot;
        p.box.src_off = at + lead;
        const size_t w0 = work.size();
        // A piece that is contiguous on both sides and not converted needs no kernel to move it: the
        // host-to-device copy lands it at its final address (as the reference's loader reads a tensor
        // straight into its own device buffer, gds_loader.py:284-331) and the kernel only reads it
        // back for the checksum.  Everything else goes through the bounce slot.
        const uint64_t piece_dst = p.box.rows * p.box.row_bytes;
        const bool abutting = p.box.rows == 1 || (p.box.src_pitch == op_src_bytes(p.box.op, p.box.row_bytes) &&
                                                  p.box.dst_pitch == p.box.row_bytes);
        if (L->direct_min && p.box.op == kOpCopy && abutting && piece_dst >= L->direct_min) {
          cur.direct.push_back(DirectCopy{at + lead, p.box.dst_off, piece_dst, p.box.dst_buf});
          BoxCopy c;
          c.src_buf = kSrcIsDestination;
          c.dst_buf = p.box.dst_buf;
          c.src_off = c.dst_off = p.box.dst_off;
          c.row_bytes = piece_dst;
          c.op = kOpChecksumOnly;
          c.csum_slot = p.box.csum_slot;
          lower_box(c, lo, segs, work);
        } else {
          const uint64_t lo_off = at, hi_off = at + in_slot;
          if (!cur.bounce_runs.empty() && lo_off - (cur.bounce_runs.back().first + cur.bounce_runs.back().second) < 4096)
            cur.bounce_runs.back().second = hi_off - cur.bounce_runs.back().first;  // a small gap is cheaper than another copy
          else
            cur.bounce_runs.emplace_back(lo_off, hi_off - lo_off);
          lower_box(p.box, lo, segs, work);
        }
        // work items index segments relative to the chunk's first segment
        for (size_t k = w0; k < work.size(); ++k) work[k].seg -= cur.seg_begin;
        if (!have_rest) break;
        p = rest;
      }
    }
    close();
    L->ing_n_segs = (uint32_t)segs.size();
    L->ing_n_work = (uint32_t)work.size();
    L->ing_segs.upload(segs.data(), segs.size());
    L->ing_work.upload(work.data(), work.size());
  }
  L->dst_bases.reserve(pl.params.size() ? pl.params.size() : 1);
  L->src_bases.reserve(ck.files.size() ? ck.files.size() : 1);
  {
    const size_t n = pl.params.size();
    L->fan = make_fan(n);
    L->acc_digest_off = align_up(fan_elems(L->fan), 2);  // the 64-bit sums sit on an 8-byte boundary
    L->acc_words = L->acc_digest_off + 2 * fan_elems(L->fan, 5);
    L->acc_stride = align_up(L->acc_words, 64);
    L->acc.reserve(2 * L->acc_stride);
    HIP_OK(hipMemset(L->acc.p, 0, 2 * L->acc_stride * sizeof(uint32_t)));
    L->clean[0] = L->clean[1] = true;
  }
  L->tab_cap = pl.params.size() + ck.files.size() + 1;
  HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&L->tab_host), L->tab_cap * sizeof(void*), hipHostMallocDefault));
  HIP_OK(hipEventCreateWithFlags(&L->upload_done, hipEventDisableTiming));
  HIP_OK(hipEventCreateWithFlags(&L->launch_done, hipEventDisableTiming));
  {
    std::vector<unsigned long long> sizes;
    for (const auto& p : pl.params) sizes.push_back(p.nbytes);
    L->dst_sizes.upload(sizes.data(), sizes.size());
  }
  pl.lowered = L.release();
  pl.lowered_free = free_lowered;
}

void check_dst(const mxp_plan& pl, void* const* dst_ptrs) {
  if (!dst_ptrs) throw Error(MXP_ERR_ARG, "dst_ptrs is null");
  for (size_t i = 0; i < pl.params.size(); ++i) {
    if (pl.params[i].n_writes == 0) continue;
    if (!dst_ptrs[i]) throw Error(MXP_ERR_ARG, "destination of parameter '" + pl.params[i].name + "' is null");
    if (reinterpret_cast<uintptr_t>(dst_ptrs[i]) & 15u)
      throw Error(MXP_ERR_ARG, "destination of parameter '" + pl.params[i].name + "' is not 16-byte aligned");
  }
}

// Brings the plan's device pointer tables up to date, ordered on `stream` (the stream the
// launch that reads them goes to).  The tables and the accumulators belong to the plan, so
// launches of one plan are serialised: a call on another stream than the last one first waits
// for that launch.  Tables are re-sent only when the caller's pointers changed, by copies that
// `stream` orders behind whatever it still runs; the pinned block they come from is reused
// only once the previous upload has left it.
// A stream under capture records neither the waits nor the events of this protocol (they would
// tie the plan's events to the graph): a captured launch is the caller's to order, and its
// tables must already be on the device.
bool is_capturing(hipStream_t stream) {
  hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
  if (hipStreamIsCapturing(stream, &st) != hipSuccess) {
    (void)hipGetLastError();
    return false;
  }
  return st != hipStreamCaptureStatusNone;
}

void upload_tables(mxp_plan::Lowered& L, const mxp_plan& pl, void* const* dst_ptrs, const void* const* file_ptrs,
                   size_t n_files, hipStream_t stream) {
  const bool capturing = is_capturing(stream);
  if (!capturing && L.launch_rec && L.last_stream != stream) {
    // The plan's last launch went to another stream: this one waits for what that stream holds now (the
    // launch and whatever followed it).  The event is recorded here, when it is needed, and not behind
    // every launch: an event between two back-to-back launches costs several microseconds of stream time.
    if (hipEventRecord(L.launch_done, L.last_stream) == hipSuccess) {
      HIP_OK(hipStreamWaitEvent(stream, L.launch_done, 0));
    } else {
      (void)hipGetLastError();  // that stream is gone; whatever it still runs is waited for the slow way
      HIP_OK(hipDeviceSynchronize());
    }
    L.launch_rec = false;
  }
  const size_t n = pl.params.size();
  const bool dst_changed = !(L.dst_host.size() == n && std::equal(L.dst_host.begin(), L.dst_host.end(), dst_ptrs));
  const bool src_changed =
      file_ptrs && !(L.src_host.size() == n_files && std::equal(L.src_host.begin(), L.src_host.end(), file_ptrs));
  if (!dst_changed && !src_changed) return;
  if (capturing)
    throw Error(MXP_ERR_STATE, "the plan's pointer tables would change under stream capture: run the plan once "
                               "outside the capture with these pointers first");
  if (L.upload_rec) HIP_OK(hipEventSynchronize(L.upload_done));
  if (dst_changed && n) {
    std::memcpy(L.tab_host, dst_ptrs, n * sizeof(void*));
    HIP_OK(hipMemcpyAsync(L.dst_bases.p, L.tab_host, n * sizeof(void*), hipMemcpyHostToDevice, stream));
  }
  if (src_changed && n_files) {
    std::memcpy(L.tab_host + n, file_ptrs, n_files * sizeof(void*));
    HIP_OK(hipMemcpyAsync(L.src_bases.p, L.tab_host + n, n_files * sizeof(void*), hipMemcpyHostToDevice, stream));
  }
  HIP_OK(hipEventRecord(L.upload_done, stream));
  L.upload_rec = true;
  if (dst_changed) L.dst_host.assign(dst_ptrs, dst_ptrs + n);
  if (src_changed) L.src_host.assign(file_ptrs, file_ptrs + n_files);
}
void mark_launch(mxp_plan::Lowered& L, hipStream_t stream) {
  if (is_capturing(stream)) return;
  L.launch_rec = true;
  L.last_stream = stream;
}

// Reads n bytes at off.  `need` (0 = n) is how many of them must exist: a range rounded up
// for direct I/O may run past the end of the file.
void pread_full(int fd, uint8_t* dst, uint64_t n, uint64_t off, const std::string& path, uint64_t need = 0) {
  const uint64_t total = n;
  if (need == 0) need = n;
  while (n) {
    const ssize_t r = ::pread(fd, dst, (size_t)std::min<uint64_t>(n, 1ull << 30), (off_t)off);
    if (r < 0) {
      if (errno == EINTR) continue;
      throw Error(MXP_ERR_IO, "read failed on " + path + ": " + std::strerror(errno));
    }
    if (r == 0) {
      if (total - n >= need) return;
      throw Error(MXP_ERR_IO, "unexpected end of file in " + path + " at offset " + std::to_string(off));
    }
    dst += r;
    off += (uint64_t)r;
    n -= (uint64_t)r;
  }
}

// Launch timing (mxp_engine_set_launch_timing): an event pair of the engine's ring around one
// kernel launch on `stream`; nothing is recorded while the stream is being captured.
struct LaunchTimer {
  mxp_engine& e;
  hipStream_t stream;
  bool on;
  hipEvent_t last = nullptr;
  LaunchTimer(mxp_engine& eng, hipStream_t s) : e(eng), stream(s), on(eng.timing_on && !eng.timing_ring.empty() && !is_capturing(s)) {
    if (!on) return;
    const auto& pr = e.timing_ring[e.timing_count % e.timing_ring.size()];
    last = pr.second;
    HIP_OK(hipEventRecord(pr.first, stream));
  }
  void done() {
    if (!on) return;
    HIP_OK(hipEventRecord(last, stream));
    ++e.timing_count;
    on = false;
  }
};

// The descriptor arenas (pinned staging + its device twin, two of them taken in turn) are shared
// by the stand-alone operators.  A call may only overwrite or reallocate an arena once its
// previous user's device work is done, whichever stream that ran on: users record the arena's
// `busy` event after their last arena-dependent operation (release_arena), and whoever takes the
// arena next waits for it - which, with two arenas, is the call before the previous one.
mxp_engine::Arena& acquire_arena(mxp_engine& e) {
  mxp_engine::Arena& a = e.arenas[e.arena_turn++ & 1u];
  if (a.recorded) HIP_OK(hipEventSynchronize(a.busy));
  return a;
}
void release_arena(mxp_engine::Arena& a, hipStream_t stream) {
  HIP_OK(hipEventRecord(a.busy, stream));
  a.recorded = true;
}

void ensure_desc(mxp_engine::Arena& a, size_t bytes) {
  if (bytes > a.host_cap) {
    if (a.host) (void)hipHostFree(a.host);
    a.host = nullptr;
    a.host_cap = 0;
    const size_t cap = align_up(bytes * 2, 1 << 16);
    HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&a.host), cap, hipHostMallocDefault));
    a.host_cap = cap;
    HIP_OK(hipHostGetDevicePointer(reinterpret_cast<void**>(&a.host_dev), a.host, 0));
  }
  a.dev.reserve(a.host_cap);
}

// Sends the first `bytes` of an arena's pinned block to its device twin, ordered on `stream`.
// Small tables go by a copy kernel that reads the pinned block over the bus: the launch that
// consumes them follows on the same queue, where a copy call costs a hand-over to a copy engine
// and back (some 15 us of stream time per operator call, measured).
constexpr size_t kTableByKernelMax = 1u << 20;
void upload_arena(mxp_engine::Arena& a, size_t bytes, hipStream_t stream) {
  bytes = align_up(bytes, 16);
  if (bytes <= kTableByKernelMax && bytes <= a.host_cap) HIP_OK(launch_copy_table(a.dev.p, a.host_dev, bytes, stream));
  else HIP_OK(hipMemcpyAsync(a.dev.p, a.host, bytes, hipMemcpyHostToDevice, stream));
}

// Runs a batch of boxes whose sources / destinations are raw device pointers.
// Layout of the descriptor arena: [segs][work][src ptrs][dst ptrs][checksums, fanned][checksums, folded].
void run_boxes(mxp_engine& e, const std::vector<BoxCopy>& boxes, const std::vector<const void*>& srcs,
               const std::vector<void*>& dsts, uint32_t n_sums, uint32_t* sums_out, hipStream_t stream) {
  LowerOptions lo;
  lo.tile_bytes = e.opt.tile_bytes;
  std::vector<Seg> segs;
  std::vector<WorkItem> work;
  for (const auto& b : boxes) lower_box(b, lo, segs, work);
  const size_t o_segs = 0;
  const size_t o_work = align_up(o_segs + segs.size() * sizeof(Seg), 256);
  const size_t o_src = align_up(o_work + work.size() * sizeof(WorkItem), 256);
  const size_t o_dst = align_up(o_src + srcs.size() * sizeof(void*), 256);
  const size_t o_sum = align_up(o_dst + dsts.size() * sizeof(void*), 256);
  // [checksums, fanned][checksums, folded] follow the uploaded tables; both are written on the device only
  const Fan fan = sums_out ? make_fan(n_sums) : Fan{};
  const size_t o_out = align_up(o_sum + (sums_out ? fan_elems(fan) * 4 : 0), 256);
  const size_t total = align_up(o_out + (size_t)n_sums * 4, 256);
  mxp_engine::Arena& ar = acquire_arena(e);
  ensure_desc(ar, total);
  if (!segs.empty()) std::memcpy(ar.host + o_segs, segs.data(), segs.size() * sizeof(Seg));
  if (!work.empty()) std::memcpy(ar.host + o_work, work.data(), work.size() * sizeof(WorkItem));
  if (!srcs.empty()) std::memcpy(ar.host + o_src, srcs.data(), srcs.size() * sizeof(void*));
  if (!dsts.empty()) std::memcpy(ar.host + o_dst, dsts.data(), dsts.size() * sizeof(void*));
  upload_arena(ar, o_sum, stream);
  uint8_t* d = ar.dev.p;
  uint32_t* const fanned = reinterpret_cast<uint32_t*>(d + o_sum);
  if (sums_out) HIP_OK(launch_fill_u32(fanned, fan_elems(fan), 0u, stream));
  bool checksum_only = !boxes.empty(), widening_only = !boxes.empty();
  for (const auto& b : boxes) {
    checksum_only = checksum_only && b.op == kOpChecksumOnly;
    widening_only = widening_only && op_widens(b.op);
  }
  LaunchTimer timer(e, stream);
  HIP_OK(launch_place(reinterpret_cast<const Seg*>(d + o_segs), reinterpret_cast<const WorkItem*>(d + o_work),
                      (uint32_t)work.size(), reinterpret_cast<const void* const*>(d + o_src),
                      reinterpret_cast<void* const*>(d + o_dst), fanned, fan, e.opt.nan_bits, stream, checksum_only, nullptr, 0,
                      widening_only));
  timer.done();
  if (sums_out && n_sums) {
    // the kernel that adds the copies up stores the totals straight into the pinned block: no copy back
    HIP_OK(launch_fold_fan(fanned, fan, 1, (uint64_t)n_sums, reinterpret_cast<uint32_t*>(ar.host_dev + o_out), false, stream));
    release_arena(ar, stream);
    HIP_OK(wait_event_promptly(ar.busy));
    std::memcpy(sums_out, ar.host + o_out, (size_t)n_sums * 4);
    return;
  }
  release_arena(ar, stream);
}

// Splits an arbitrary device pointer into a 16-byte aligned base and an offset, so the
// lowering can pick the widest access the true address allows.
inline void split_ptr(const void* p, const void*& base, uint64_t& off) {
  const uintptr_t v = reinterpret_cast<uintptr_t>(p);
  off = v & 15u;
  base = reinterpret_cast<const void*>(v - off);
}

}  // namespace
}  // namespace mxp

extern "C" {

int mxp_engine_create(const mxp_engine_options* opts, mxp_engine** out) {
  return guard([&] {
    if (!out) throw Error(MXP_ERR_ARG, "mxp_engine_create: null out");
    *out = nullptr;
    auto e = std::make_unique<mxp_engine>();
    if (opts) e->opt = *opts;
    auto& o = e->opt;
    if (o.ring_slots <= 0) o.ring_slots = 32;
    if (o.slot_bytes == 0) o.slot_bytes = 16ull << 20;
    if (o.reader_threads <= 0) {  // 12-16 readers keep the pinned ring ahead of PCIe (8: 51, 16: 55 GB/s measured)
      const unsigned hw = std::thread::hardware_concurrency();
      o.reader_threads = (int)std::min(16u, std::max(4u, hw ? hw : 8u));
    }
    if (o.streams <= 0) o.streams = 4;
    if (o.tile_bytes == 0) o.tile_bytes = kPlaceThreads * kPlaceBatch * 16;
    if (o.nan_bits == 0) o.nan_bits = 0x7FC0;
    // Packing strided rows on the host is the default in both modes.  From the page cache it is one read
    // call per row; under direct I/O the readers fetch the rows of a band with large requests into their
    // own buffers (direct_rows_per_read) and copy only the rows into the slot - the same bytes leave
    // storage as when whole bands are staged, a third of them cross PCIe (Llama-3-8B rank share) and
    // the reader spends less time copying between two requests (measured 6.1-6.6 against 5.6-6.3 GB/s
    // from a disk that gave a plain read 6.6-7.1 GB/s).
    if (o.pack_strided_on_host == 0) o.pack_strided_on_host = 1;
    if (o.pack_strided_on_host > 2) throw Error(MXP_ERR_ARG, "pack_strided_on_host must be 0, 1 or 2");
    if (o.slot_bytes < (1u << 16) || o.slot_bytes % 4096) throw Error(MXP_ERR_ARG, "slot_bytes must be a multiple of 4096, at least 64 KiB");
    if (o.tile_bytes < 1024 || o.tile_bytes > (uint32_t)(kPlaceThreads * kPlaceBatch * 16))
      throw Error(MXP_ERR_ARG, "tile_bytes must be in [1 KiB, 128 KiB]");
    if (o.ring_slots > 256 || o.reader_threads > 256 || o.streams > 64) throw Error(MXP_ERR_ARG, "ring, thread or stream count too large");
    int n_dev = 0;
    HIP_OK(hipGetDeviceCount(&n_dev));
    if (n_dev <= 0) throw Error(MXP_ERR_DEVICE, "no HIP device is visible");
    if (o.device < 0 || o.device >= n_dev) throw Error(MXP_ERR_ARG, "device ordinal out of range");
    HIP_OK(hipSetDevice(o.device));
    HIP_OK(configure_place_kernels());
    for (int s = 0; s < o.streams; ++s) {
      hipStream_t st;
      HIP_OK(hipStreamCreateWithFlags(&st, hipStreamNonBlocking));
      e->streams.push_back(st);
    }
    HIP_OK(hipEventCreate(&e->ev_a));
    HIP_OK(hipEventCreate(&e->ev_b));
    for (auto& a : e->arenas) HIP_OK(hipEventCreateWithFlags(&a.busy, hipEventDisableTiming));
    for (auto& t : e->item_tabs) HIP_OK(hipEventCreateWithFlags(&t.busy, hipEventDisableTiming));
    HIP_OK(hipEventCreateWithFlags(&e->caller_ev, hipEventDisableTiming));
    e->static_dev = static_scratch_for(o.device);
    HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&e->static_host), kStaticScratchBytes, hipHostMallocDefault));
    *out = e.release();
  });
}

void mxp_engine_destroy(mxp_engine* engine) {
  if (!engine) return;
  (void)hipSetDevice(engine->opt.device);
  (void)hipDeviceSynchronize();
  delete engine;
}

}  // extern "C"

namespace mxp {
namespace {

// The ring is allocated on first ingest so that engines used only for resident
// placement or the stand-alone operators hold no pinned memory.
void ensure_ring(mxp_engine& e) {
  if (!e.slots.empty()) return;
  const auto& o = e.opt;
  const size_t total = (size_t)o.ring_slots * o.slot_bytes;
  HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&e.pinned_base), total, hipHostMallocDefault));
  HIP_OK(hipMalloc(reinterpret_cast<void**>(&e.bounce_base), total));
  std::vector<const void*> ptrs;
  for (int s = 0; s < o.ring_slots; ++s) {
    auto sl = std::make_unique<Slot>();
    sl->host = e.pinned_base + (size_t)s * o.slot_bytes;
    sl->dev = e.bounce_base + (size_t)s * o.slot_bytes;
    HIP_OK(hipEventCreateWithFlags(&sl->done, hipEventDisableTiming));
    ptrs.push_back(sl->dev);
    e.slots.push_back(std::move(sl));
  }
  e.slot_ptrs.upload(ptrs.data(), ptrs.size());
}

void do_execute(mxp_engine& e, mxp_plan& pl, void* const* dst_ptrs, hipStream_t caller_stream, mxp_exec_stats* stats) {
  const double t_start = now_s();
  HIP_OK(hipSetDevice(e.opt.device));
  check_dst(pl, dst_ptrs);
  lower_plan(pl, e);
  ensure_ring(e);
  auto& L = *pl.lowered;
  const mxp_ckpt& ck = *pl.ckpt;
  if (stats) std::memset(stats, 0, sizeof *stats);

  std::vector<int> fds(ck.files.size(), -1);
  struct FdCloser {
    std::vector<int>& f;
    ~FdCloser() { for (int fd : f) if (fd >= 0) ::close(fd); }
  } closer{fds};
  for (size_t f = 0; f < ck.files.size(); ++f) {
    int flags = O_RDONLY;
#ifdef O_DIRECT
    if (e.opt.use_o_direct) flags |= O_DIRECT;
#endif
    fds[f] = ::open(ck.files[f].path.c_str(), flags);
    if (fds[f] < 0 && e.opt.use_o_direct) fds[f] = ::open(ck.files[f].path.c_str(), O_RDONLY);
    if (fds[f] < 0) throw Error(MXP_ERR_IO, "cannot open " + ck.files[f].path + ": " + std::strerror(errno));
  }

  // Everything below may change destination bytes.  The engine's streams are private and
  // non-blocking: they first wait for what the caller already queued on its own stream
  // (initialisation kernels on the parameters, reads of buffers the allocator has since
  // handed back), as destination.copy_(source) on that stream would.
  HIP_OK(hipEventRecord(e.caller_ev, caller_stream));
  for (auto st : e.streams) HIP_OK(hipStreamWaitEvent(st, e.caller_ev, 0));
  upload_tables(L, pl, dst_ptrs, nullptr, 0, e.streams[0]);
  const bool digests = e.fused_digests;
  L.digests_valid = false;
  if (!L.clean[L.cur]) HIP_OK(launch_fill_u32(L.sums(L.cur), L.dirty_words(L.cur), 0u, e.streams[0]));
  L.clean[L.cur] = false;
  L.digest_used[L.cur] = digests;
  uint32_t* const sums_dev = L.sums(L.cur);
  unsigned long long* const dsums_dev = L.digest_sums(L.cur);
  HIP_OK(hipStreamSynchronize(e.streams[0]));
  for (auto& s : e.slots) s->submitted = 0;
  // MXP_INGEST_TRACE (read by the library itself, once): one line per ingest on stderr with the times at which the
  // first chunk had been read, the last one, the readers were done and the streams idle.
  static const bool trace = std::getenv("MXP_INGEST_TRACE") != nullptr;
  const double t_tables = now_s();
  std::atomic<double> t_first_submit{0.0}, t_last_read{0.0};

  std::atomic<size_t> next{0};
  std::atomic<bool> abort{false};
  std::atomic<int> mutated{0};
  std::mutex err_mu;
  std::unique_ptr<Error> first_err;
  std::vector<double> read_s((size_t)e.opt.reader_threads, 0.0);
  const size_t n_chunks = L.chunks.size();
  const size_t n_slots = e.slots.size();

  auto worker = [&](int tid) {
    // The kernel refuses direct I/O into HIP pinned memory (EFAULT: the mapping cannot be
    // pinned again by the block layer), so direct reads land in an ordinary block-aligned
    // buffer and are copied into the slot.  `stage_buf` is that buffer: the chunk as the slot will
    // hold it; `direct_buf` is where several packed rows are read at once before they are gathered.
    void* direct_buf = nullptr;
    void* stage_buf = nullptr;
    struct Free { void*& p; ~Free() { std::free(p); } } free_direct{direct_buf}, free_stage{stage_buf};
    try {
      HIP_OK(hipSetDevice(e.opt.device));
      if (L.direct_io && (::posix_memalign(&direct_buf, 4096, e.opt.slot_bytes) != 0 ||
                          ::posix_memalign(&stage_buf, 4096, e.opt.slot_bytes) != 0))
        throw Error(MXP_ERR_STATE, "out of host memory for the direct I/O buffers");
      for (;;) {
        const size_t c = next.fetch_add(1);
        if (c >= n_chunks || abort.load()) break;
        const Chunk& ch = L.chunks[c];
        Slot& sl = *e.slots[c % n_slots];
        const uint64_t turn = c / n_slots;
        auto wait_for_slot = [&]() -> bool {
          {
            // Wait until the previous chunk carried by this slot has been submitted, then
            // until the GPU has finished with it.
            std::unique_lock<std::mutex> lk(sl.mu);
            sl.cv.wait(lk, [&] { return sl.submitted == turn || abort.load(); });
          }
          if (abort.load()) return false;
          if (turn > 0) HIP_OK(hipEventSynchronize(sl.done));
          return true;
        };
        // read_s: time spent reading and packing, not waiting for a slot
        double t0 = now_s();
        if (direct_buf) {
          // Direct I/O: the whole chunk is read into the reader's own block-aligned copy of the slot BEFORE
          // the slot is waited for, so the number of storage requests in flight is the number of readers,
          // whatever the ring holds; a slot is then only needed for one copy out of that buffer.
          uint8_t* const stage = static_cast<uint8_t*>(stage_buf);
          for (const auto& r : ch.ranges) {
            if (r.rows == 1) {  // slot offsets are block aligned in this mode: read in place
              pread_full(fds[r.file], stage + r.slot_off, r.nbytes, r.file_off, ck.files[r.file].path, r.need);
              continue;
            }
            // packed rows: several rows per request (direct_rows_per_read), gathered out of the request's buffer
            const uint64_t per = direct_rows_per_read(e.opt.slot_bytes, r.file_pitch, r.nbytes);
            for (uint64_t row = 0; row < r.rows; row += per) {
              const uint64_t nr = std::min(per, r.rows - row);
              const uint64_t o0 = r.file_off + row * r.file_pitch, a0 = o0 / 4096 * 4096;
              const uint64_t last = o0 + (nr - 1) * r.file_pitch + r.nbytes;
              pread_full(fds[r.file], static_cast<uint8_t*>(direct_buf), align_up(last, 4096) - a0, a0, ck.files[r.file].path,
                         last - a0);
              for (uint64_t k = 0; k < nr; ++k)
                std::memcpy(stage + r.slot_off + (row + k) * r.nbytes,
                            static_cast<uint8_t*>(direct_buf) + (o0 - a0) + k * r.file_pitch, r.nbytes);
            }
          }
          read_s[tid] += now_s() - t0;
          if (!wait_for_slot()) break;
          t0 = now_s();
          std::memcpy(sl.host, stage, ch.used_bytes);
        } else {
          if (!wait_for_slot()) break;
          t0 = now_s();
          for (const auto& r : ch.ranges)
            for (uint64_t row = 0; row < r.rows; ++row)
              pread_full(fds[r.file], sl.host + r.slot_off + row * r.nbytes, r.nbytes, r.file_off + row * r.file_pitch,
                         ck.files[r.file].path, r.need);
        }
        read_s[tid] += now_s() - t0;
        if (trace) {
          const double t = now_s();
          double seen = t_first_submit.load();
          while (seen == 0.0 && !t_first_submit.compare_exchange_weak(seen, t)) {}
          double last = t_last_read.load();
          while (last < t && !t_last_read.compare_exchange_weak(last, t)) {}
        }
        hipStream_t st = e.streams[(c % n_slots) % e.streams.size()];
        mutated.store(1);
        for (const auto& r : ch.bounce_runs)
          HIP_OK(hipMemcpyAsync(sl.dev + r.first, sl.host + r.first, r.second, hipMemcpyHostToDevice, st));
        for (const auto& d : ch.direct)
          HIP_OK(hipMemcpyAsync(static_cast<uint8_t*>(dst_ptrs[d.param]) + d.dst_off, sl.host + d.slot_off, d.nbytes,
                                hipMemcpyHostToDevice, st));
        if (digests)
          HIP_OK(launch_place_digest(L.ing_segs.p + ch.seg_begin, L.ing_work.p + ch.work_begin, ch.work_count,
                                     e.slot_ptrs.p + (c % n_slots), L.dst_bases.p, sums_dev, L.fan, L.dst_sizes.p, dsums_dev,
                                     e.opt.nan_bits, st));
        else
          HIP_OK(launch_place(L.ing_segs.p + ch.seg_begin, L.ing_work.p + ch.work_begin, ch.work_count,
                              e.slot_ptrs.p + (c % n_slots), L.dst_bases.p, sums_dev, L.fan, e.opt.nan_bits, st));
        HIP_OK(hipEventRecord(sl.done, st));
        {
          std::lock_guard<std::mutex> lk(sl.mu);
          sl.submitted = turn + 1;
        }
        sl.cv.notify_all();
      }
    } catch (const Error& er) {
      std::lock_guard<std::mutex> lk(err_mu);
      if (!first_err) first_err = std::make_unique<Error>(er);
      abort.store(true);
      for (auto& s : e.slots) { { std::lock_guard<std::mutex> g(s->mu); } s->cv.notify_all(); }
    } catch (const std::exception& ex) {
      std::lock_guard<std::mutex> lk(err_mu);
      if (!first_err) first_err = std::make_unique<Error>(MXP_ERR_STATE, ex.what());
      abort.store(true);
      for (auto& s : e.slots) { { std::lock_guard<std::mutex> g(s->mu); } s->cv.notify_all(); }
    }
  };
  {
    std::vector<std::thread> pool;
    const int n_thr = (int)std::min<size_t>((size_t)e.opt.reader_threads, n_chunks ? n_chunks : 1);
    for (int t = 0; t < n_thr; ++t) pool.emplace_back(worker, t);
    for (auto& t : pool) t.join();
  }
  const double t_join = now_s();
  hipError_t sync_err = hipSuccess;
  for (auto st : e.streams) {
    const hipError_t r = hipStreamSynchronize(st);
    if (r != hipSuccess) sync_err = r;
  }
  if (trace)
    std::fprintf(stderr, "[mxp ingest] set-up %.3f ms, first chunk read %.3f ms later, last chunk read at %.3f ms, readers joined at %.3f ms, streams idle at %.3f ms (%zu chunks)\n",
                 (t_tables - t_start) * 1e3, (t_first_submit.load() - t_tables) * 1e3, (t_last_read.load() - t_start) * 1e3,
                 (t_join - t_start) * 1e3, (now_s() - t_start) * 1e3, n_chunks);
  if (stats) {
    stats->wall_seconds = now_s() - t_start;
    for (double r : read_s) stats->read_seconds += r;
    stats->file_bytes = L.file_bytes;
    stats->h2d_bytes = L.h2d_bytes;
    stats->placed_bytes = L.placed_bytes;
    stats->n_chunks = n_chunks;
    stats->n_segments = L.ing_n_segs;
    stats->n_workgroups = L.ing_n_work;
    stats->n_launches = n_chunks;
    stats->mutated = mutated.load();
  }
  L.launch_rec = false;  // every stream is idle
  if (first_err) throw *first_err;
  if (sync_err != hipSuccess) throw Error(MXP_ERR_DEVICE, std::string("stream synchronize: ") + hipGetErrorString(sync_err));
  L.digests_valid = digests;
}

void do_execute_resident(mxp_engine& e, mxp_plan& pl, const void* const* file_dev_ptrs, void* const* dst_ptrs,
                         hipStream_t stream, mxp_exec_stats* stats) {
  HIP_OK(hipSetDevice(e.opt.device));
  check_dst(pl, dst_ptrs);
  if (!file_dev_ptrs) throw Error(MXP_ERR_ARG, "file_dev_ptrs is null");
  const mxp_ckpt& ck = *pl.ckpt;
  for (size_t f = 0; f < ck.files.size(); ++f)
    if (!file_dev_ptrs[f] || (reinterpret_cast<uintptr_t>(file_dev_ptrs[f]) & 7u))  // elements (at most 8 bytes) keep their alignment
      throw Error(MXP_ERR_ARG, "staged file pointer " + std::to_string(f) + " is null or not 8-byte aligned");
  lower_plan(pl, e);
  auto& L = *pl.lowered;
  if (stats) std::memset(stats, 0, sizeof *stats);
  upload_tables(L, pl, dst_ptrs, file_dev_ptrs, ck.files.size(), stream);
  L.digests_valid = e.fused_digests;
  // Accumulators: a launch adds to one set and clears the other for the launch after it; only a set
  // the host does not know to be zero gets a clearing launch first.  A captured launch is replayed
  // with fixed arguments at times the host does not see, so from the first capture on the plan keeps
  // to set 0 and every launch clears it itself: what mxp_plan_checksums reads is then always the
  // set the last launch or replay wrote.
  const bool capturing = is_capturing(stream);
  if (capturing) L.single_set = true;
  const bool alternate = !L.single_set && L.res_n_work != 0;
  const int set = alternate ? (L.cur ^ 1) : 0;
  // (a captured clearing launch runs before every replay: it covers what this launch adds to as well)
  if (!alternate || !L.clean[set])
    HIP_OK(launch_fill_u32(L.sums(set), L.digest_used[set] || e.fused_digests ? L.acc_words : L.acc_digest_off, 0u, stream));
  uint32_t* zero_ptr = nullptr;
  uint32_t zero_n = 0;
  if (alternate) {
    zero_ptr = L.sums(set ^ 1);
    zero_n = (uint32_t)L.dirty_words(set ^ 1);
    L.digest_used[set ^ 1] = false;
  }
  L.digest_used[set] = e.fused_digests;
  const bool ring_timed = e.timing_on && !stats && !capturing;
  const auto& pair = e.timing_ring.empty() ? std::pair<hipEvent_t, hipEvent_t>() : e.timing_ring[e.timing_count % e.timing_ring.size()];
  if (stats) HIP_OK(hipEventRecord(e.ev_a, stream));
  if (ring_timed) HIP_OK(hipEventRecord(pair.first, stream));
  if (e.fused_digests)
    HIP_OK(launch_place_digest(L.res_segs.p, L.res_work.p, L.res_n_work, L.src_bases.p, L.dst_bases.p, L.sums(set), L.fan,
                               L.dst_sizes.p, L.digest_sums(set), e.opt.nan_bits, stream, zero_ptr, zero_n));
  else
    HIP_OK(launch_place(L.res_segs.p, L.res_work.p, L.res_n_work, L.src_bases.p, L.dst_bases.p, L.sums(set), L.fan,
                        e.opt.nan_bits, stream, false, zero_ptr, zero_n));
  L.cur = set;
  L.clean[set] = false;
  L.clean[set ^ 1] = zero_n != 0;
  if (ring_timed) {
    HIP_OK(hipEventRecord(pair.second, stream));
    ++e.timing_count;
  }
  mark_launch(L, stream);
  if (stats) {
    HIP_OK(hipEventRecord(e.ev_b, stream));
    HIP_OK(hipEventSynchronize(e.ev_b));
    float ms = 0;
    HIP_OK(hipEventElapsedTime(&ms, e.ev_a, e.ev_b));
    stats->kernel_ms = ms;
    stats->wall_seconds = ms * 1e-3;
    stats->placed_bytes = L.placed_bytes;
    stats->n_segments = L.res_n_segs;
    stats->n_workgroups = L.res_n_work;
    stats->n_launches = 1;
    stats->mutated = 1;
  }
}

}  // namespace
}  // namespace mxp

extern "C" {

int mxp_execute(mxp_engine* engine, mxp_plan* plan, void* const* dst_ptrs, mxp_exec_stats* stats) {
  return guard([&] {
    if (!engine || !plan) throw Error(MXP_ERR_ARG, "mxp_execute: null handle");
    do_execute(*engine, *plan, dst_ptrs, nullptr, stats);
  });
}

int mxp_execute_after(mxp_engine* engine, mxp_plan* plan, void* const* dst_ptrs, void* caller_stream,
                      mxp_exec_stats* stats) {
  return guard([&] {
    if (!engine || !plan) throw Error(MXP_ERR_ARG, "mxp_execute_after: null handle");
    do_execute(*engine, *plan, dst_ptrs, static_cast<hipStream_t>(caller_stream), stats);
  });
}

int mxp_execute_resident(mxp_engine* engine, mxp_plan* plan, const void* const* file_dev_ptrs,
                         void* const* dst_ptrs, void* stream, mxp_exec_stats* stats) {
  return guard([&] {
    if (!engine || !plan) throw Error(MXP_ERR_ARG, "mxp_execute_resident: null handle");
    do_execute_resident(*engine, *plan, file_dev_ptrs, dst_ptrs, static_cast<hipStream_t>(stream), stats);
  });
}

int mxp_prepare(mxp_engine* engine, mxp_plan* plan) {
  return guard([&] {
    if (!engine || !plan) throw Error(MXP_ERR_ARG, "mxp_prepare: null handle");
    HIP_OK(hipSetDevice(engine->opt.device));
    lower_plan(*plan, *engine);
    ensure_ring(*engine);  // the pinned ring too: allocating it takes longer than ingesting a small checkpoint
  });
}

int mxp_plan_checksums(mxp_engine* engine, mxp_plan* plan, uint32_t* out, int64_t n) {
  return guard([&] {
    if (!engine || !plan || !out) throw Error(MXP_ERR_ARG, "mxp_plan_checksums: null argument");
    if (!plan->lowered) throw Error(MXP_ERR_STATE, "plan has not been executed");
    if (n != (int64_t)plan->params.size()) throw Error(MXP_ERR_ARG, "mxp_plan_checksums: n must equal the parameter count");
    HIP_OK(hipSetDevice(engine->opt.device));
    HIP_OK(hipDeviceSynchronize());
    auto& L = *plan->lowered;
    std::vector<uint32_t> fanned(fan_elems(L.fan));
    HIP_OK(hipMemcpy(fanned.data(), L.sums(L.cur), fanned.size() * 4, hipMemcpyDeviceToHost));
    fold_fan(fanned.data(), L.fan, 1, (uint64_t)n, out);
  });
}

int mxp_engine_set_fused_digests(mxp_engine* engine, int32_t on) {
  return guard([&] {
    if (!engine) throw Error(MXP_ERR_ARG, "mxp_engine_set_fused_digests: null engine");
    engine->fused_digests = on != 0;
  });
}

int mxp_engine_set_direct_placement(mxp_engine* engine, int64_t min_bytes) {
  return guard([&] {
    if (!engine) throw Error(MXP_ERR_ARG, "mxp_engine_set_direct_placement: null engine");
    // a plan is lowered again when it next runs on this engine
    engine->direct_min = min_bytes < 0 ? 0 : min_bytes == 0 ? kDirectMinBytes : (uint64_t)min_bytes;
  });
}

int mxp_engine_set_launch_timing(mxp_engine* engine, int32_t on) {
  return guard([&] {
    if (!engine) throw Error(MXP_ERR_ARG, "mxp_engine_set_launch_timing: null engine");
    constexpr size_t kTimingRing = 256;
    HIP_OK(hipSetDevice(engine->opt.device));
    if (on && engine->timing_ring.empty()) {
      engine->timing_ring.reserve(kTimingRing);
      for (size_t k = 0; k < kTimingRing; ++k) {
        hipEvent_t a = nullptr, b = nullptr;
        HIP_OK(hipEventCreate(&a));
        if (hipEventCreate(&b) != hipSuccess) { (void)hipEventDestroy(a); throw Error(MXP_ERR_DEVICE, "hipEventCreate failed"); }
        engine->timing_ring.emplace_back(a, b);
      }
    }
    engine->timing_on = on != 0;
    engine->timing_count = 0;
  });
}

int mxp_engine_launch_times(mxp_engine* engine, float* out_ms, int32_t capacity, int32_t* n_out) {
  return guard([&] {
    if (!engine || !n_out || capacity < 0 || (capacity && !out_ms)) throw Error(MXP_ERR_ARG, "mxp_engine_launch_times: bad argument");
    mxp_engine& e = *engine;
    HIP_OK(hipSetDevice(e.opt.device));
    const uint64_t have = std::min<uint64_t>(e.timing_count, e.timing_ring.size());
    const uint64_t n = std::min<uint64_t>(have, (uint64_t)capacity);
    for (uint64_t k = 0; k < n; ++k) {
      const auto& pr = e.timing_ring[(e.timing_count - n + k) % e.timing_ring.size()];
      HIP_OK(hipEventSynchronize(pr.second));
      HIP_OK(hipEventElapsedTime(&out_ms[k], pr.first, pr.second));
    }
    *n_out = (int32_t)n;
  });
}

int mxp_plan_digests(mxp_engine* engine, mxp_plan* plan, uint8_t* out16, int64_t n) {
  return guard([&] {
    if (!engine || !plan || !out16) throw Error(MXP_ERR_ARG, "mxp_plan_digests: null argument");
    if (!plan->lowered || !plan->lowered->digests_valid)
      throw Error(MXP_ERR_STATE, "the plan's last execute did not accumulate digests (mxp_engine_set_fused_digests)");
    if (n != (int64_t)plan->params.size()) throw Error(MXP_ERR_ARG, "mxp_plan_digests: n must equal the parameter count");
    HIP_OK(hipSetDevice(engine->opt.device));
    HIP_OK(hipDeviceSynchronize());
    auto& L = *plan->lowered;
    std::vector<unsigned long long> fanned(fan_elems(L.fan, 5)), sums(5 * (size_t)n + 1);
    HIP_OK(hipMemcpy(fanned.data(), L.digest_sums(L.cur), fanned.size() * 8, hipMemcpyDeviceToHost));
    fold_fan(fanned.data(), L.fan, 5, 5 * (uint64_t)n, sums.data());
    for (int64_t i = 0; i < n; ++i) {
      const auto& p = plan->params[(size_t)i];
      if (p.bytes_written != p.nbytes)
        throw Error(MXP_ERR_STATE, "parameter '" + p.name + "' is not fully written by the plan: its digest is undefined");
      const uint64_t scalars[7] = {p.nbytes, sums[5 * i], sums[5 * i + 1], sums[5 * i + 2], sums[5 * i + 3], sums[5 * i + 4],
                                   p.nbytes % 4};
      const int rc = mxp_digest_from_scalars(scalars, out16 + 16 * i);
      if (rc != MXP_OK) throw Error(rc, mxp_last_error());
    }
  });
}

int mxp_plan_totals(const mxp_plan* plan, uint64_t* file_bytes, uint64_t* h2d_bytes, uint64_t* placed_bytes,
                    uint64_t* kernel_algorithmic_bytes) {
  return guard([&] {
    if (!plan) throw Error(MXP_ERR_ARG, "mxp_plan_totals: null plan");
    if (!plan->built) throw Error(MXP_ERR_STATE, "plan has not been built");
    uint64_t placed = 0, algo = 0;
    for (const auto& w : plan->writes) {
      placed += w.rows * w.row_bytes;
      algo += w.rows * (w.row_bytes + op_src_bytes(seg_op_of_cast(w.cast), w.row_bytes));
    }
    if (placed_bytes) *placed_bytes = placed;
    if (kernel_algorithmic_bytes) *kernel_algorithmic_bytes = algo;
    if (file_bytes) *file_bytes = plan->lowered ? plan->lowered->file_bytes : 0;
    if (h2d_bytes) *h2d_bytes = plan->lowered ? plan->lowered->h2d_bytes : 0;
  });
}

int mxp_checksum32(mxp_engine* engine, const void* const* ptrs, const uint64_t* nbytes, int64_t n, uint32_t* out,
                   void* stream) {
  return guard([&] {
    if (!engine || !out || n < 0 || (n && (!ptrs || !nbytes))) throw Error(MXP_ERR_ARG, "mxp_checksum32: bad argument");
    if (n == 0) return;
    HIP_OK(hipSetDevice(engine->opt.device));
    std::vector<BoxCopy> boxes;
    std::vector<const void*> srcs;
    for (int64_t k = 0; k < n; ++k) {
      if (nbytes[k] && !ptrs[k]) throw Error(MXP_ERR_ARG, "mxp_checksum32: null pointer");
      const void* base;
      uint64_t off;
      split_ptr(ptrs[k], base, off);
      srcs.push_back(base);
      // A misaligned start only narrows the access width the lowering picks.
      BoxCopy b;
      b.src_buf = (uint32_t)k;
      b.src_off = off;
      b.row_bytes = nbytes[k];
      b.op = kOpChecksumOnly;
      b.csum_slot = (uint32_t)k;
      boxes.push_back(b);
    }
    run_boxes(*engine, boxes, srcs, {}, (uint32_t)n, out, static_cast<hipStream_t>(stream));
  });
}

int mxp_checksum32_static(mxp_engine* engine, const void* const* ptrs, const uint64_t* nbytes, int64_t n,
                          uint32_t* out, void* stream_v) {
  return guard([&] {
    if (!engine || !out || n < 0 || (n && (!ptrs || !nbytes))) throw Error(MXP_ERR_ARG, "mxp_checksum32_static: bad argument");
    if (n == 0) return;
    if ((uint64_t)n > kStaticMaxBuffers)
      throw Error(MXP_ERR_ARG, "mxp_checksum32_static: " + std::to_string(n) + " buffers in one call, the static scratch holds " +
                                   std::to_string(kStaticMaxBuffers));
    mxp_engine& e = *engine;
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    HIP_OK(hipSetDevice(e.opt.device));
    // The call ends with a wait for `stream` and hands its results back on the host: neither can be
    // recorded.  Refused before anything is queued, so the caller's capture stays valid.
    if (is_capturing(stream))
      throw Error(MXP_ERR_STATE, "mxp_checksum32_static: the stream is being captured; the call waits for the stream and "
                                 "returns host results, so it cannot be recorded into a graph");
    // Tables are lowered straight into the pinned mirror; the previous call synchronised
    // `stream` before it returned, so nothing still reads it.
    unsigned char* h = e.static_host;
    unsigned char* d = e.static_dev;
    FixedTable<Seg> segs(h + kStaticOffSegs, kStaticMaxSegs, "mxp_checksum32_static: too many segments for the static scratch");
    FixedTable<WorkItem> work(h + kStaticOffWork, kStaticMaxWork,
                              "mxp_checksum32_static: the buffers need more than 98304 workgroups (about 12 GiB in all), "
                              "the limit of the static scratch");
    const void** src_tab = reinterpret_cast<const void**>(h + kStaticOffPtrs);
    uint32_t* sums = reinterpret_cast<uint32_t*>(h + kStaticOffSums);
    LowerOptions lo;
    lo.tile_bytes = e.opt.tile_bytes;
    for (int64_t k = 0; k < n; ++k) {
      if (nbytes[k] && !ptrs[k]) throw Error(MXP_ERR_ARG, "mxp_checksum32_static: null pointer");
      uint64_t off;
      split_ptr(ptrs[k], src_tab[k], off);
      BoxCopy b;
      b.src_buf = (uint32_t)k;
      b.src_off = off;
      b.row_bytes = nbytes[k];
      b.op = kOpChecksumOnly;
      b.csum_slot = (uint32_t)k;
      lower_box(b, lo, segs, work);
      sums[k] = 0;  // the accumulators keep the last call's values: they are cleared by the upload below
    }
    if (segs.size()) HIP_OK(hipMemcpyAsync(d + kStaticOffSegs, h + kStaticOffSegs, segs.size() * sizeof(Seg), hipMemcpyHostToDevice, stream));
    if (work.size()) HIP_OK(hipMemcpyAsync(d + kStaticOffWork, h + kStaticOffWork, work.size() * sizeof(WorkItem), hipMemcpyHostToDevice, stream));
    // pointers and zeroed accumulators are neighbours: one copy up to the end of the used sums
    HIP_OK(hipMemcpyAsync(d + kStaticOffPtrs, h + kStaticOffPtrs, kStaticOffSums - kStaticOffPtrs + (size_t)n * 4, hipMemcpyHostToDevice, stream));
    HIP_OK(launch_place(reinterpret_cast<const Seg*>(d + kStaticOffSegs), reinterpret_cast<const WorkItem*>(d + kStaticOffWork),
                        (uint32_t)work.size(), reinterpret_cast<const void* const*>(d + kStaticOffPtrs), nullptr,
                        reinterpret_cast<uint32_t*>(d + kStaticOffSums), Fan{}, e.opt.nan_bits, stream, true));  // one copy: the scratch is full
    HIP_OK(hipMemcpyAsync(h + kStaticOffSums, d + kStaticOffSums, (size_t)n * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    std::memcpy(out, sums, (size_t)n * 4);
  });
}

int mxp_cast(mxp_engine* engine, const void* src, void* dst, uint64_t n_elems, int32_t cast, uint32_t* checksum,
             void* stream) {
  return guard([&] {
    if (!engine || (n_elems && (!src || !dst))) throw Error(MXP_ERR_ARG, "mxp_cast: bad argument");
    if (cast < MXP_CAST_F32_BF16 || cast > MXP_CAST_LAST) throw Error(MXP_ERR_ARG, "mxp_cast: unknown conversion code");
    if (checksum) *checksum = 0;
    if (n_elems == 0) return;
    HIP_OK(hipSetDevice(engine->opt.device));
    const uint32_t op = seg_op_of_cast(cast);
    const uint64_t dst_es = op_dst_elem(op), src_es = op_src_bytes(op, dst_es);
    if (reinterpret_cast<uintptr_t>(src) % src_es) throw Error(MXP_ERR_ARG, "mxp_cast: src must be element aligned");
    if (reinterpret_cast<uintptr_t>(dst) & 15u) throw Error(MXP_ERR_ARG, "mxp_cast: dst must be 16-byte aligned");
    const void* sb;
    uint64_t so;
    split_ptr(src, sb, so);
    BoxCopy b;
    b.src_off = so;
    b.row_bytes = n_elems * dst_es;
    b.op = op;
    b.csum_slot = 0;
    std::vector<BoxCopy> boxes{b};
    uint32_t sum = 0;
    run_boxes(*engine, boxes, {sb}, {dst}, 1, checksum ? &sum : nullptr,
              static_cast<hipStream_t>(stream));
    if (checksum) *checksum = sum;
  });
}

int mxp_cast_f32_bf16(mxp_engine* engine, const void* src, void* dst, uint64_t n_elems, uint32_t* checksum,
                      void* stream) {
  return mxp_cast(engine, src, dst, n_elems, MXP_CAST_F32_BF16, checksum, stream);
}

int mxp_gather2d(mxp_engine* engine, const void* src, uint64_t src_pitch, void* dst, uint64_t dst_pitch,
                 uint64_t rows, uint64_t row_bytes, uint32_t* checksum, void* stream) {
  return guard([&] {
    if (!engine || (rows && row_bytes && (!src || !dst))) throw Error(MXP_ERR_ARG, "mxp_gather2d: bad argument");
    if (checksum) *checksum = 0;
    if (rows == 0 || row_bytes == 0) return;
    if (rows > 1 && (src_pitch < row_bytes || dst_pitch < row_bytes))
      throw Error(MXP_ERR_ARG, "mxp_gather2d: pitch smaller than row_bytes");
    HIP_OK(hipSetDevice(engine->opt.device));
    if (reinterpret_cast<uintptr_t>(dst) & 15u) throw Error(MXP_ERR_ARG, "mxp_gather2d: dst must be 16-byte aligned");
    const void* sb;
    uint64_t so;
    split_ptr(src, sb, so);
    BoxCopy b;
    b.src_off = so;
    b.src_pitch = src_pitch;
    b.dst_pitch = dst_pitch;
    b.rows = rows;
    b.row_bytes = row_bytes;
    b.op = kOpCopy;
    b.csum_slot = 0;
    uint32_t sum = 0;
    run_boxes(*engine, {b}, {sb}, {dst}, 1, checksum ? &sum : nullptr, static_cast<hipStream_t>(stream));
    if (checksum) *checksum = sum;
  });
}

int mxp_place_boxes(mxp_engine* engine, const mxp_box* in, int64_t n, uint32_t n_groups, uint32_t* out_checksums,
                    void* stream) {
  return guard([&] {
    if (!engine || n < 0 || (n && !in) || (out_checksums && n_groups == 0))
      throw Error(MXP_ERR_ARG, "mxp_place_boxes: bad argument");
    if (n == 0) {
      for (uint32_t g = 0; out_checksums && g < n_groups; ++g) out_checksums[g] = 0;
      return;
    }
    HIP_OK(hipSetDevice(engine->opt.device));
    std::vector<BoxCopy> boxes;
    std::vector<const void*> sv;
    std::vector<void*> dv;
    for (int64_t k = 0; k < n; ++k) {
      const mxp_box& x = in[k];
      if (x.rows == 0 || x.row_bytes == 0) continue;
      if (!x.src || !x.dst) throw Error(MXP_ERR_ARG, "mxp_place_boxes: null pointer");
      if (x.csum_group >= (n_groups ? n_groups : 1)) throw Error(MXP_ERR_ARG, "mxp_place_boxes: csum_group out of range");
      if (x.cast > (uint32_t)MXP_CAST_LAST) throw Error(MXP_ERR_ARG, "mxp_place_boxes: unknown conversion code");
      const uint32_t op = seg_op_of_cast((int)x.cast);
      if (op != kOpCopy && x.row_bytes % op_dst_elem(op))
        throw Error(MXP_ERR_ARG, "mxp_place_boxes: row_bytes is not a whole number of elements");
      if (x.rows > 1 && (x.src_pitch < op_src_bytes(op, x.row_bytes) || x.dst_pitch < x.row_bytes))
        throw Error(MXP_ERR_ARG, "mxp_place_boxes: pitch smaller than the row");
      const void* sb;
      const void* db;
      uint64_t so, d_o;
      split_ptr(x.src, sb, so);
      split_ptr(x.dst, db, d_o);
      BoxCopy b;
      b.src_buf = (uint32_t)sv.size();
      b.dst_buf = (uint32_t)dv.size();
      sv.push_back(sb);
      dv.push_back(const_cast<void*>(db));
      b.src_off = so;
      b.dst_off = d_o;
      b.src_pitch = x.src_pitch;
      b.dst_pitch = x.dst_pitch;
      b.rows = x.rows;
      b.row_bytes = x.row_bytes;
      b.op = op;
      b.csum_slot = out_checksums ? x.csum_group : 0xFFFFFFFFu;
      b.csum_bias = x.csum_index - d_o;  // positions are relative to the caller's buffer, not the aligned base
      boxes.push_back(b);
    }
    std::vector<uint32_t> sums(n_groups ? n_groups : 1, 0);
    run_boxes(*engine, boxes, sv, dv, n_groups ? n_groups : 1, out_checksums ? sums.data() : nullptr,
              static_cast<hipStream_t>(stream));
    if (out_checksums) std::memcpy(out_checksums, sums.data(), (size_t)n_groups * 4);
  });
}

extern "C++" {
namespace {

// Measurement switch (mxp_set_transpose_form): 0 = the library picks the form of a transpose, 1 = always the
// wavefront-autonomous form.
std::atomic<int> g_transpose_form{0};

// dst_view[...] = src_view[...] for two strided views of one shape (strides in elements).
// Dimensions are put in destination order (largest destination stride first) and merged
// where both sides allow; then
//   * innermost dimension contiguous on both sides  -> pitched row boxes through place_kernel,
//   * contiguous in the destination only, with another dimension contiguous in the source
//                                                   -> transpose_kernel (other dims = batch),
//   * anything else                                 -> one element per box row (the run length
//     the reference's paired_runs finds for such a view: slice_plan.py:259-294).
// The checksum, when asked for, weights every written byte by its offset from `dst`.
struct TransposeJob {
  const void* src;
  void* dst;
  TransposeDesc td;
  int elem_size;  // source element
  uint32_t op;    // kOpCopy, or the conversion applied on the way
};

enum ViewKind {
  kViewEmpty,     // nothing to move
  kViewBoxes,     // row boxes appended to `boxes`
  kViewTranspose  // `tr` filled in: one launch of the transpose kernel, converting on the way if asked
};

// Lowers one view copy.  Boxes are appended to `boxes` with their base pointers in `srcs` / `dsts`.
// `call_bytes`: destination bytes of all the views of the call this view belongs to (0 = this view alone);
// a transpose sizes its workgroups by whether the whole call, not this view, fills the chip.
ViewKind lower_view(const void* src, void* dst, std::vector<uint64_t> size, std::vector<uint64_t> ss,
                    std::vector<uint64_t> ds, int elem_size, int cast, uint32_t csum_slot, std::vector<BoxCopy>& boxes,
                    std::vector<const void*>& srcs, std::vector<void*>& dsts, TransposeJob& tr, const char* what,
                    uint64_t call_bytes = 0) {
  const uint32_t op = seg_op_of_cast(cast);
  const uint64_t es = (uint64_t)elem_size;          // destination element
  const uint64_t es_s = op_src_bytes(op, es);       // source element
  auto fail = [&](int code, const std::string& msg) { throw Error(code, std::string(what) + ": " + msg); };
  uint64_t total = 1;
  for (auto n : size) total *= n;
  if (total == 0) return kViewEmpty;
  if (!src || !dst) fail(MXP_ERR_ARG, "null pointer");
  if (reinterpret_cast<uintptr_t>(src) % es_s || reinterpret_cast<uintptr_t>(dst) % es) fail(MXP_ERR_ARG, "pointer is not element aligned");
  {
    // drop unit dims, order by destination stride, refuse a self-overlapping destination, merge
    std::vector<size_t> order;
    for (size_t d = 0; d < size.size(); ++d)
      if (size[d] != 1) order.push_back(d);
    std::stable_sort(order.begin(), order.end(), [&](size_t x, size_t y) { return ds[x] > ds[y]; });
    std::vector<uint64_t> n2, s2, d2;
    for (size_t d : order) { n2.push_back(size[d]); s2.push_back(ss[d]); d2.push_back(ds[d]); }
    for (size_t d = 0; d + 1 < n2.size(); ++d)
      if (d2[d] < d2[d + 1] * n2[d + 1]) fail(MXP_ERR_UNSUPPORTED, "the destination view overlaps itself");
    if (!n2.empty() && d2.back() == 0) fail(MXP_ERR_UNSUPPORTED, "the destination view overlaps itself");
    size.clear(); ss.clear(); ds.clear();
    for (size_t d = 0; d < n2.size(); ++d) {
      if (!size.empty() && ss.back() == s2[d] * n2[d] && ds.back() == d2[d] * n2[d]) {
        size.back() *= n2[d];
        ss.back() = s2[d];
        ds.back() = d2[d];
      } else {
        size.push_back(n2[d]); ss.push_back(s2[d]); ds.push_back(d2[d]);
      }
    }
    if (size.empty()) { size.push_back(1); ss.push_back(1); ds.push_back(1); }
  }
  const size_t nd = size.size();
  int c = -1;  // a dimension other than the innermost that is contiguous in the source
  for (size_t d = 0; d + 1 < nd; ++d)
    if (ss[d] == 1) c = (int)d;
  const bool dst_inner = ds[nd - 1] == 1 || total == 1;
  const bool transposed = dst_inner && ss[nd - 1] != 1 && total != 1 && c >= 0 && nd - 2 <= (size_t)kMaxBatchDims;

  // Row boxes: whole innermost rows when both sides are contiguous there, else one element per row.
  auto emit_boxes = [&] {
    const void* sp = src;
    const bool rows_ok = dst_inner && (ss[nd - 1] == 1 || total == 1);
    std::vector<uint64_t> n = size, s = ss, d = ds;
    if (!rows_ok) { n.push_back(1); s.push_back(1); d.push_back(1); }  // a virtual innermost dimension of one element
    const size_t m = n.size();
    const void* sb;
    const void* db;
    uint64_t so, d_o;
    split_ptr(sp, sb, so);
    split_ptr(dst, db, d_o);
    BoxCopy b;
    b.src_buf = (uint32_t)srcs.size();
    b.dst_buf = (uint32_t)dsts.size();
    srcs.push_back(sb);
    dsts.push_back(const_cast<void*>(db));
    b.row_bytes = n[m - 1] * es;
    b.op = op;
    b.csum_slot = csum_slot;
    b.csum_bias = (uint64_t)0 - d_o;
    if (m == 1) {
      b.src_off = so;
      b.dst_off = d_o;
      boxes.push_back(b);
      return;
    }
    b.rows = n[m - 2];
    b.src_pitch = s[m - 2] * es_s;
    b.dst_pitch = d[m - 2] * es;
    uint64_t outer = 1;
    for (size_t q = 0; q + 2 < m; ++q) outer *= n[q];
    if (outer > (1u << 20)) fail(MXP_ERR_UNSUPPORTED, "too many row bands");
    std::vector<uint64_t> idx(m, 0);
    for (uint64_t o = 0; o < outer; ++o) {
      uint64_t s_el = 0, d_el = 0;
      for (size_t q = 0; q + 2 < m; ++q) { s_el += idx[q] * s[q]; d_el += idx[q] * d[q]; }
      BoxCopy x = b;
      x.src_off = so + s_el * es_s;
      x.dst_off = d_o + d_el * es;
      boxes.push_back(x);
      for (int q = (int)m - 3; q >= 0; --q) { if (++idx[q] < n[q]) break; idx[q] = 0; }
    }
  };

  // Transpose: i = destination innermost, j = the source's unit-stride dimension.  The tile
  // shape follows the source element (`eb`); destination alignment follows its own (`es`).
  auto make_transpose = [&] {
    void* dp = dst;
    const std::vector<uint64_t>& d_in = ds;
    const uint64_t eb = es_s;
    TransposeDesc td{};
    td.ni = size[nd - 1];
    td.si = ss[nd - 1];
    td.nj = size[c];
    td.dj = d_in[c];
    uint64_t batches = 1;
    for (int d = (int)nd - 2; d >= 0; --d)
      if (d != c) batches *= size[d];
    // Workgroup shape: as many wavefronts along i (long destination runs) as the extent can
    // use, the rest along j; fewer wavefronts per workgroup while the launch would leave
    // compute units without one.
    const uint64_t sub_i = transpose_sub_rows((int)es), sub_j = transpose_sub_cols((int)eb);
    for (uint32_t waves = (uint32_t)kTransposeWaves;; waves /= 2) {
      uint32_t waves_i = 1;
      while (waves_i < waves && (uint64_t)waves_i * sub_i < td.ni) waves_i *= 2;
      // Larger destination pitch than source pitch: short, wide workgroups visited in bands along j
      // (measured +15% on 65536 x 4096 and 32768 x 8192); otherwise long destination runs, plain order.
      td.group_j = 1;
      if (td.dj > td.si) {
        waves_i = std::min(waves_i, 2u);
        td.group_j = 8;
      }
      td.waves = waves;
      td.waves_i = waves_i;
      const uint64_t tile_i = waves_i * sub_i, tile_j = (waves / waves_i) * sub_j;
      td.tiles_i = (uint32_t)((td.ni + tile_i - 1) / tile_i);
      td.tiles_j = (uint32_t)((td.nj + tile_j - 1) / tile_j);
      if (waves == 1 || batches * td.tiles_i * td.tiles_j >= 2ull * kChipCus) break;
    }
    // Alignment of each side: the largest power of two (at most 16) dividing the base address and every byte stride.
    auto pow2 = [](uint64_t v) { return (v | 16u) & (~(v | 16u) + 1u); };
    uint64_t vs = pow2(reinterpret_cast<uintptr_t>(src) | (td.si * eb));
    uint64_t vd = pow2(reinterpret_cast<uintptr_t>(dp) | (td.dj * es));
    int k = kMaxBatchDims - 1;
    for (int q = 0; q < kMaxBatchDims; ++q) { td.batch_size[q] = 1; td.batch_sstride[q] = 0; td.batch_dstride[q] = 0; }
    for (int d = (int)nd - 2; d >= 0; --d) {
      if (d == c) continue;
      td.batch_size[k] = size[d];
      td.batch_sstride[k] = ss[d];
      td.batch_dstride[k] = d_in[d];
      if (size[d] > 1) {
        vs = std::min(vs, pow2(ss[d] * eb));
        vd = std::min(vd, pow2(d_in[d] * es));
      }
      --k;
    }
    td.align_src = (uint32_t)vs;
    td.align_dst = (uint32_t)vd;
    // Panel form (mxp_permute.hip) where it measured faster than the wavefront-autonomous one; it has no edge
    // handling, so only whole tiles with 16-byte accesses on both sides qualify.
    if (vs >= 16 && vd >= 16 && eb <= 4 && es <= 4 && g_transpose_form.load(std::memory_order_relaxed) != 1) {
      auto is_pow2 = [](uint64_t v) { return v && !(v & (v - 1)); };
      auto log2u = [](uint64_t v) { uint32_t l = 0; while ((1ull << l) < v) ++l; return l; };
      const uint64_t row_src = td.nj * eb;  // bytes of one source row of the view
      const uint64_t src_pitch = td.si * eb, dst_pitch = td.dj * es, v_rows = 16 / es;
      uint64_t rows = 0, row_bytes = 0;
      if (td.dj == td.ni && is_pow2(td.ni) && td.ni >= v_rows && td.ni <= 1024 && td.ni * es <= 1024) {
        // short destination rows that abut: all of i in one tile, whose output is then one contiguous block
        rows = td.ni;
        row_bytes = 128;
        while (row_bytes * 2 <= 4096 && rows * row_bytes * 2 <= kPanelMaxBytes && row_src % (row_bytes * 2) == 0) row_bytes *= 2;
        // smaller tiles while the call would leave compute units without a workgroup
        const uint64_t all_bytes = std::max<uint64_t>(call_bytes, batches * td.ni * td.nj * es);
        while (row_bytes > 128 && rows * row_bytes / 2 >= 8192 && all_bytes / (rows * row_bytes / eb * es) < 2ull * kChipCus) row_bytes /= 2;
      } else if (eb == 2 && es == 2 && src_pitch >= 32768 && dst_pitch >= 32768) {
        rows = 512;      // 2-byte matrices with long pitches on both sides: 1 KiB destination runs, 256-byte source runs
        row_bytes = 256;
      } else if (eb == 2 && es == 4 && src_pitch >= 16384 && dst_pitch >= 32768) {
        rows = 256;      // widening: 1 KiB destination runs out of 512-byte source runs
        row_bytes = 512;
      }
      if (rows && td.ni % rows == 0 && row_src % row_bytes == 0 && rows * row_bytes >= 8192) {
        TransposeDesc pd = td;
        pd.panel_rows_log2 = log2u(rows);
        pd.panel_chunks_log2 = log2u(row_bytes / 16);
        pd.waves = (uint32_t)(rows * row_bytes / 16 / kPanelLoads / 64);
        pd.waves_i = 1;
        pd.group_j = 1;
        pd.tiles_i = (uint32_t)(td.ni / rows);
        pd.tiles_j = (uint32_t)(row_src / row_bytes);
        pd.n_tiles = (uint64_t)pd.tiles_i * pd.tiles_j * batches;
        if (panel_desc_ok(pd, (uint32_t)eb, (uint32_t)es)) td = pd;
      }
    }
    td.n_tiles = (uint64_t)td.tiles_i * td.tiles_j;
    for (int q = 0; q < kMaxBatchDims; ++q) td.n_tiles *= td.batch_size[q];
    if (!transpose_desc_ok(td)) fail(MXP_ERR_UNSUPPORTED, "the transposed view needs more workgroups than one launch holds");
    tr = TransposeJob{src, dp, td, (int)eb, op};
  };

  if (!transposed) {
    emit_boxes();
    return kViewBoxes;
  }
  make_transpose();
  return kViewTranspose;
}

void run_transpose(mxp_engine& e, const TransposeJob& t, uint32_t* checksum, hipStream_t stream) {
  uint32_t* sum_dev = nullptr;
  const Fan fan = make_fan(1);
  mxp_engine::Arena* ar = nullptr;
  if (checksum) {
    ar = &acquire_arena(e);
    ensure_desc(*ar, fan_elems(fan) * 4);
    sum_dev = reinterpret_cast<uint32_t*>(ar->dev.p);
    HIP_OK(launch_fill_u32(sum_dev, fan_elems(fan), 0u, stream));
  }
  LaunchTimer timer(e, stream);
  HIP_OK(launch_transpose(t.src, t.dst, t.td, t.elem_size, t.op, e.opt.nan_bits, sum_dev, fan, stream));
  timer.done();
  if (checksum) {
    HIP_OK(hipMemcpyAsync(ar->host, sum_dev, fan_elems(fan) * 4, hipMemcpyDeviceToHost, stream));
    HIP_OK(hipStreamSynchronize(stream));
    fold_fan(reinterpret_cast<const uint32_t*>(ar->host), fan, 1, 1, checksum);
    release_arena(*ar, stream);
  }
}

void copy_view(mxp_engine& e, const void* src, void* dst, std::vector<uint64_t> size, std::vector<uint64_t> ss,
               std::vector<uint64_t> ds, int elem_size, int cast, uint32_t* checksum, hipStream_t stream,
               const char* what) {
  if (checksum) *checksum = 0;
  std::vector<BoxCopy> boxes;
  std::vector<const void*> srcs;
  std::vector<void*> dsts;
  TransposeJob tr{};
  const uint32_t slot = checksum ? 0u : 0xFFFFFFFFu;
  const ViewKind kind = lower_view(src, dst, size, ss, ds, elem_size, cast, slot, boxes, srcs, dsts, tr, what);
  if (kind == kViewEmpty) return;
  HIP_OK(hipSetDevice(e.opt.device));
  if (kind == kViewTranspose) {
    run_transpose(e, tr, checksum, stream);
    return;
  }
  uint32_t sum = 0;
  run_boxes(e, boxes, srcs, dsts, 1, checksum ? &sum : nullptr, stream);
  if (checksum) *checksum = sum;
}

// Transposes that share a kernel instance and workgroup size, laid out for one launch each.
struct TransposeGroup {
  size_t first, count;  // slice of the item table
  uint64_t tiles;
  uint32_t waves;
  int elem_size;
  uint32_t op;
  uint32_t panel;  // 0, or panel_rows_log2 << 8 | panel_chunks_log2 of every item
  uint32_t uniform_tiles;  // != 0: a panel group whose items all have the descriptor `common` and this many tiles
  TransposeDesc common;
};
inline uint32_t panel_code(const TransposeDesc& d) { return d.panel_rows_log2 ? (d.panel_rows_log2 << 8 | d.panel_chunks_log2) : 0u; }

// Sorts `jobs` into launch groups (`items` receives their descriptor table) and `singles`
// (a kind of its own: launched with the descriptor as a kernel argument).
void group_transposes(const std::vector<TransposeJob>& jobs, std::vector<TransposeItem>& items,
                      std::vector<TransposeGroup>& groups, std::vector<TransposeJob>& singles) {
  std::vector<size_t> order;
  for (size_t k = 0; k < jobs.size(); ++k) {
    if (jobs[k].td.n_tiles) order.push_back(k);  // descriptors were checked when the views were lowered
  }
  auto key = [&](size_t k) {
    return ((uint64_t)panel_code(jobs[k].td) << 32) | ((uint64_t)jobs[k].op << 16) | ((uint64_t)jobs[k].elem_size << 8) | jobs[k].td.waves;
  };
  std::stable_sort(order.begin(), order.end(), [&](size_t x, size_t y) { return key(x) < key(y); });
  for (size_t q = 0; q < order.size();) {
    size_t r = q;
    uint64_t tiles = 0;
    while (r < order.size() && key(order[r]) == key(order[q]) && tiles + jobs[order[r]].td.n_tiles <= 0x7FFFFFFFull)
      tiles += jobs[order[r++]].td.n_tiles;
    if (r - q == 1) {
      singles.push_back(jobs[order[q]]);
    } else {
      const TransposeJob& j0 = jobs[order[q]];
      bool uniform = j0.td.panel_rows_log2 != 0 && j0.td.n_tiles <= 0xFFFFFFFFull;
      uint64_t first = 0;
      for (size_t k = q; k < r; ++k) {
        const TransposeJob& j = jobs[order[k]];
        uniform = uniform && same_transpose_desc(j.td, j0.td);
        items.push_back(TransposeItem{static_cast<const uint8_t*>(j.src), static_cast<uint8_t*>(j.dst), first, 0, j.td});
        first += j.td.n_tiles;
      }
      groups.push_back(TransposeGroup{items.size() - (r - q), r - q, tiles, j0.td.waves, j0.elem_size, j0.op, panel_code(j0.td),
                                      uniform ? (uint32_t)j0.td.n_tiles : 0u, j0.td});
    }
    q = r;
  }
}

// Runs transposes that report no checksum: those that share a kernel instance and workgroup
// size go out as one launch, the rest one by one.
void run_transposes(mxp_engine& e, const std::vector<TransposeJob>& jobs, hipStream_t stream) {
  std::vector<TransposeItem> items;
  std::vector<TransposeGroup> groups;
  std::vector<TransposeJob> singles;
  group_transposes(jobs, items, groups, singles);
  for (const auto& j : singles) run_transpose(e, j, nullptr, stream);
  if (groups.empty()) return;
  mxp_engine::ItemTable& tab = e.item_tabs[e.items_turn++ & 1u];
  if (tab.recorded) HIP_OK(hipEventSynchronize(tab.busy));
  if (items.size() > tab.cap) {
    if (tab.host) (void)hipHostFree(tab.host);
    tab.host = nullptr;
    tab.cap = 0;
    const size_t cap = std::max<size_t>(64, items.size() * 2);
    HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&tab.host), cap * sizeof(TransposeItem), hipHostMallocDefault));
    tab.cap = cap;
    HIP_OK(hipHostGetDevicePointer(reinterpret_cast<void**>(&tab.host_dev), tab.host, 0));
  }
  tab.dev.reserve(tab.cap);
  std::memcpy(tab.host, items.data(), items.size() * sizeof(TransposeItem));
  static_assert(sizeof(TransposeItem) % 16 == 0, "the table copy kernel moves 16-byte units");
  if (items.size() * sizeof(TransposeItem) <= kTableByKernelMax)
    HIP_OK(launch_copy_table(tab.dev.p, tab.host_dev, items.size() * sizeof(TransposeItem), stream));
  else
    HIP_OK(hipMemcpyAsync(tab.dev.p, tab.host, items.size() * sizeof(TransposeItem), hipMemcpyHostToDevice, stream));
  for (const TransposeGroup& g : groups) {
    LaunchTimer timer(e, stream);
    HIP_OK(launch_transpose_batch(tab.dev.p + g.first, (uint32_t)g.count, g.tiles, g.waves, g.elem_size, g.op,
                                  e.opt.nan_bits, stream, g.panel, g.uniform_tiles, &g.common, items.data() + g.first));
    timer.done();
  }
  HIP_OK(hipEventRecord(tab.busy, stream));
  tab.recorded = true;
}

std::vector<uint64_t> strides_or_row_major(const int64_t* strides, const int64_t* shape, int32_t ndim, const char* what) {
  std::vector<uint64_t> out((size_t)ndim, 1);
  if (!strides) {
    for (int d = ndim - 2; d >= 0; --d) out[d] = out[d + 1] * (uint64_t)shape[d + 1];
    return out;
  }
  for (int d = 0; d < ndim; ++d) {
    if (strides[d] < 0) throw Error(MXP_ERR_UNSUPPORTED, std::string(what) + ": negative strides are not supported");
    out[d] = (uint64_t)strides[d];
  }
  return out;
}

void check_view_args(const mxp_engine* engine, int32_t ndim, const int64_t* shape, int32_t elem_size, const char* what) {
  if (!engine || ndim < 0 || ndim > MXP_MAX_DIMS || (ndim && !shape)) throw Error(MXP_ERR_ARG, std::string(what) + ": bad argument");
  if (elem_size != 1 && elem_size != 2 && elem_size != 4 && elem_size != 8)
    throw Error(MXP_ERR_ARG, std::string(what) + ": elem_size must be 1, 2, 4 or 8");
  for (int d = 0; d < ndim; ++d)
    if (shape[d] < 0) throw Error(MXP_ERR_ARG, std::string(what) + ": negative extent");
}

// Lowers n view copies into row / element boxes and transposes; nothing is launched.
void lower_views(const mxp_engine* engine, const mxp_view_copy* views, int64_t n, std::vector<BoxCopy>& boxes,
                 std::vector<const void*>& srcs, std::vector<void*>& dsts, std::vector<TransposeJob>& transposes,
                 const char* what) {
  uint64_t call_bytes = 0;  // what the whole call writes: sizes the transposes' workgroups
  for (int64_t k = 0; k < n; ++k) {
    if (views[k].ndim < 0 || views[k].ndim > MXP_MAX_DIMS || views[k].elem_size <= 0) continue;  // refused below
    uint64_t el = 1;
    for (int d = 0; d < views[k].ndim; ++d) el *= views[k].shape[d] > 0 ? (uint64_t)views[k].shape[d] : 0;
    call_bytes += el * (uint64_t)views[k].elem_size;
  }
  for (int64_t k = 0; k < n; ++k) {
    const mxp_view_copy& v = views[k];
    check_view_args(engine, v.ndim, v.shape, v.elem_size, what);
    if (v.cast < MXP_CAST_NONE || v.cast > MXP_CAST_LAST) throw Error(MXP_ERR_ARG, std::string(what) + ": unknown conversion code");
    if (v.cast != MXP_CAST_NONE && v.elem_size != (int32_t)op_dst_elem(seg_op_of_cast(v.cast)))
      throw Error(MXP_ERR_ARG, std::string(what) + ": elem_size is not the destination element size of the conversion");
    std::vector<uint64_t> size;
    for (int d = 0; d < v.ndim; ++d) size.push_back((uint64_t)v.shape[d]);
    TransposeJob tr{};
    const auto s_st = strides_or_row_major(v.contiguous_src ? nullptr : v.src_strides, v.shape, v.ndim, what);
    const auto d_st = strides_or_row_major(v.contiguous_dst ? nullptr : v.dst_strides, v.shape, v.ndim, what);
    const ViewKind kind = lower_view(v.src, v.dst, size, s_st, d_st, v.elem_size, v.cast, 0xFFFFFFFFu, boxes, srcs, dsts, tr, what,
                                     call_bytes);
    if (kind == kViewTranspose) transposes.push_back(tr);
  }
}

}  // namespace
}  // extern "C++"

// View copies lowered once (mxp_view_plan_create): descriptor tables resident on the device,
// nothing to build, upload or allocate when it runs.
struct mxp_view_plan {
  int device = 0;
  DevBuf<uint8_t> tables;  // [segments][work items][source pointers][destination pointers]
  size_t o_work = 0, o_src = 0, o_dst = 0;
  uint32_t n_work = 0;
  std::vector<TransposeJob> singles;
  std::vector<TransposeGroup> groups;
  DevBuf<TransposeItem> items;
  std::vector<TransposeItem> items_host;  // the same table: small uniform batches pass their pointers as kernel arguments
  uint64_t bytes = 0;  // destination bytes one run writes
};

// A fixed set of device buffers lowered once for repeated verification (mxp_verify_plan_create):
// descriptor tables, accumulators and a pinned result block of its own, so a run neither builds
// nor uploads anything.
struct mxp_verify_plan {
  int device = 0;
  int64_t n = 0;
  std::vector<uint64_t> nbytes;
  // [segments][work items][source pointers][checksums, fanned][digest jobs][digest sums, fanned]
  DevBuf<uint8_t> tables;
  Fan fan;
  size_t o_work = 0, o_src = 0, o_sums = 0, o_jobs = 0, o_dsums = 0;
  uint32_t n_work = 0, n_blocks = 0;
  // pinned: [checksums][digest sums]; the kernel that adds the fanned copies up stores its results
  // here directly (`host_dev` is the device's address of the block), so no copy follows it
  uint8_t* host = nullptr;
  uint8_t* host_dev = nullptr;
  hipEvent_t cleared = nullptr;  // the results are in `host` and the accumulators are zero again
  bool cleared_rec = false;
  ~mxp_verify_plan() {
    if (host) (void)hipHostFree(host);
    if (cleared) (void)hipEventDestroy(cleared);
  }
};

int mxp_verify_plan_create(mxp_engine* engine, const void* const* ptrs, const uint64_t* nbytes, int64_t n,
                           mxp_verify_plan** out) {
  return guard([&] {
    if (!out) throw Error(MXP_ERR_ARG, "mxp_verify_plan_create: null out");
    *out = nullptr;
    if (!engine || n < 0 || (n && (!ptrs || !nbytes))) throw Error(MXP_ERR_ARG, "mxp_verify_plan_create: bad argument");
    auto vp = std::make_unique<mxp_verify_plan>();
    vp->device = engine->opt.device;
    vp->n = n;
    HIP_OK(hipSetDevice(vp->device));
    LowerOptions lo;
    lo.tile_bytes = engine->opt.tile_bytes;
    std::vector<Seg> segs;
    std::vector<WorkItem> work;
    std::vector<const void*> srcs;
    std::vector<DigestJob> jobs((size_t)n);
    uint64_t blocks = 0;
    for (int64_t k = 0; k < n; ++k) {
      if (nbytes[k] && !ptrs[k]) throw Error(MXP_ERR_ARG, "mxp_verify_plan_create: null pointer");
      vp->nbytes.push_back(nbytes[k]);
      const void* base;
      uint64_t off;
      split_ptr(ptrs[k], base, off);
      srcs.push_back(base);
      BoxCopy b;
      b.src_buf = (uint32_t)k;
      b.src_off = off;
      b.row_bytes = nbytes[k];
      b.op = kOpChecksumOnly;
      b.csum_slot = (uint32_t)k;
      lower_box(b, lo, segs, work);
      jobs[k].ptr = static_cast<const uint8_t*>(ptrs[k]);
      jobs[k].nbytes = nbytes[k];
      jobs[k].out_slot = (uint64_t)k * 5;
      jobs[k].first_block = blocks;
      const uint64_t rows = (nbytes[k] / 4) / kDigestRowWords;
      blocks += rows ? (rows + kDigestRowsPerBlock - 1) / kDigestRowsPerBlock : 1;
    }
    if (work.size() > 0x7FFFFFFFull || blocks > 0x7FFFFFFFull) throw Error(MXP_ERR_ARG, "mxp_verify_plan_create: batch too large for one launch");
    vp->n_work = (uint32_t)work.size();
    vp->n_blocks = (uint32_t)blocks;
    vp->o_work = align_up(segs.size() * sizeof(Seg), 256);
    vp->o_src = align_up(vp->o_work + work.size() * sizeof(WorkItem), 256);
    vp->o_sums = align_up(vp->o_src + srcs.size() * sizeof(void*), 256);
    vp->fan = make_fan((uint64_t)n);
    vp->o_jobs = align_up(vp->o_sums + fan_elems(vp->fan) * 4, 256);
    vp->o_dsums = align_up(vp->o_jobs + jobs.size() * sizeof(DigestJob), 256);
    std::vector<uint8_t> host(align_up(vp->o_dsums + fan_elems(vp->fan, 5) * 8, 256), 0);  // accumulators start at zero
    if (!segs.empty()) std::memcpy(host.data(), segs.data(), segs.size() * sizeof(Seg));
    if (!work.empty()) std::memcpy(host.data() + vp->o_work, work.data(), work.size() * sizeof(WorkItem));
    if (!srcs.empty()) std::memcpy(host.data() + vp->o_src, srcs.data(), srcs.size() * sizeof(void*));
    if (!jobs.empty()) std::memcpy(host.data() + vp->o_jobs, jobs.data(), jobs.size() * sizeof(DigestJob));
    vp->tables.upload(host.data(), host.size());
    HIP_OK(hipHostMalloc(reinterpret_cast<void**>(&vp->host), (size_t)(n ? n : 1) * 44 + 16, hipHostMallocDefault));
    HIP_OK(hipHostGetDevicePointer(reinterpret_cast<void**>(&vp->host_dev), vp->host, 0));
    HIP_OK(hipEventCreateWithFlags(&vp->cleared, hipEventDisableTiming));
    *out = vp.release();
  });
}

int mxp_verify_plan_checksums(mxp_engine* engine, mxp_verify_plan* plan, uint32_t* out, void* stream_v) {
  return guard([&] {
    if (!engine || !plan || (plan->n && !out)) throw Error(MXP_ERR_ARG, "mxp_verify_plan_checksums: null argument");
    if (plan->device != engine->opt.device) throw Error(MXP_ERR_ARG, "mxp_verify_plan_checksums: the plan was built for another device");
    if (plan->n == 0) return;
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    HIP_OK(hipSetDevice(plan->device));
    uint8_t* d = plan->tables.p;
    uint32_t* sums = reinterpret_cast<uint32_t*>(d + plan->o_sums);
    if (plan->cleared_rec) HIP_OK(hipStreamWaitEvent(stream, plan->cleared, 0));  // a run on another stream than the last
    LaunchTimer timer(*engine, stream);
    HIP_OK(launch_place(reinterpret_cast<const Seg*>(d), reinterpret_cast<const WorkItem*>(d + plan->o_work), plan->n_work,
                        reinterpret_cast<const void* const*>(d + plan->o_src), nullptr, sums, plan->fan, engine->opt.nan_bits, stream,
                        true));
    timer.done();
    // the copies are added up on the device, which leaves them cleared for the next run
    HIP_OK(launch_fold_fan(sums, plan->fan, 1, (uint64_t)plan->n, reinterpret_cast<uint32_t*>(plan->host_dev), true, stream));
    HIP_OK(hipEventRecord(plan->cleared, stream));
    plan->cleared_rec = true;
    HIP_OK(wait_event_promptly(plan->cleared));
    std::memcpy(out, plan->host, (size_t)plan->n * 4);
  });
}

int mxp_verify_plan_digests(mxp_engine* engine, mxp_verify_plan* plan, uint8_t* out16, uint64_t* scalars, void* stream_v) {
  return guard([&] {
    if (!engine || !plan || (plan->n && !out16)) throw Error(MXP_ERR_ARG, "mxp_verify_plan_digests: null argument");
    if (plan->device != engine->opt.device) throw Error(MXP_ERR_ARG, "mxp_verify_plan_digests: the plan was built for another device");
    if (plan->n == 0) return;
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    HIP_OK(hipSetDevice(plan->device));
    uint8_t* d = plan->tables.p;
    unsigned long long* dsums = reinterpret_cast<unsigned long long*>(d + plan->o_dsums);
    if (plan->cleared_rec) HIP_OK(hipStreamWaitEvent(stream, plan->cleared, 0));
    LaunchTimer timer(*engine, stream);
    HIP_OK(launch_digest(reinterpret_cast<const DigestJob*>(d + plan->o_jobs), (uint32_t)plan->n, plan->n_blocks, dsums, plan->fan,
                         stream));
    timer.done();
    const size_t h_off = align_up((size_t)plan->n * 4, 8);  // the 64-bit sums follow the checksums
    const uint8_t* h = plan->host + h_off;
    HIP_OK(launch_fold_fan(dsums, plan->fan, 5, 5 * (uint64_t)plan->n, reinterpret_cast<unsigned long long*>(plan->host_dev + h_off), true,
                           stream));
    HIP_OK(hipEventRecord(plan->cleared, stream));
    plan->cleared_rec = true;
    HIP_OK(wait_event_promptly(plan->cleared));
    const uint64_t* sums = reinterpret_cast<const uint64_t*>(h);
    for (int64_t k = 0; k < plan->n; ++k) {
      const uint64_t nb = plan->nbytes[(size_t)k];
      const uint64_t sc[7] = {nb, sums[5 * k], sums[5 * k + 1], sums[5 * k + 2], sums[5 * k + 3], sums[5 * k + 4], nb % 4};
      if (scalars) std::memcpy(scalars + 7 * k, sc, sizeof sc);
      const int rc = mxp_digest_from_scalars(sc, out16 + 16 * k);
      if (rc != MXP_OK) throw Error(rc, mxp_last_error());
    }
  });
}

void mxp_verify_plan_destroy(mxp_verify_plan* plan) {
  if (!plan) return;
  (void)hipSetDevice(plan->device);
  (void)hipDeviceSynchronize();
  delete plan;
}

int mxp_permute_copy(mxp_engine* engine, const void* src, void* dst, int32_t ndim, const int64_t* shape,
                     const int64_t* src_strides, const int32_t* perm, int32_t elem_size, uint32_t* checksum,
                     void* stream_v) {
  return guard([&] {
    const char* what = "mxp_permute_copy";
    check_view_args(engine, ndim, shape, elem_size, what);
    if (ndim && !perm) throw Error(MXP_ERR_ARG, "mxp_permute_copy: bad argument");
    if (dst && (reinterpret_cast<uintptr_t>(dst) & 15u)) throw Error(MXP_ERR_ARG, "mxp_permute_copy: dst must be 16-byte aligned");
    const std::vector<uint64_t> st = strides_or_row_major(src_strides, shape, ndim, what);
    // Dimensions in destination order; the destination is contiguous.
    std::vector<uint64_t> size, ss;
    std::vector<bool> seen((size_t)ndim, false);
    for (int d = 0; d < ndim; ++d) {
      if (perm[d] < 0 || perm[d] >= ndim || seen[perm[d]]) throw Error(MXP_ERR_ARG, "mxp_permute_copy: perm is not a permutation");
      seen[perm[d]] = true;
      size.push_back((uint64_t)shape[perm[d]]);
      ss.push_back(st[perm[d]]);
    }
    std::vector<uint64_t> ds(size.size(), 1);
    for (int d = (int)size.size() - 2; d >= 0; --d) ds[d] = ds[d + 1] * size[d + 1];
    copy_view(*engine, src, dst, size, ss, ds, elem_size, MXP_CAST_NONE, checksum, static_cast<hipStream_t>(stream_v), what);
  });
}

int mxp_copy_view(mxp_engine* engine, const void* src, void* dst, int32_t ndim, const int64_t* shape,
                  const int64_t* src_strides, const int64_t* dst_strides, int32_t elem_size, int32_t cast,
                  uint32_t* checksum, void* stream_v) {
  return guard([&] {
    const char* what = "mxp_copy_view";
    check_view_args(engine, ndim, shape, elem_size, what);
    if (cast < MXP_CAST_NONE || cast > MXP_CAST_LAST) throw Error(MXP_ERR_ARG, "mxp_copy_view: unknown conversion code");
    if (cast != MXP_CAST_NONE && elem_size != (int32_t)op_dst_elem(seg_op_of_cast(cast)))
      throw Error(MXP_ERR_ARG, "mxp_copy_view: elem_size is not the destination element size of the conversion");
    std::vector<uint64_t> size;
    for (int d = 0; d < ndim; ++d) size.push_back((uint64_t)shape[d]);
    copy_view(*engine, src, dst, size, strides_or_row_major(src_strides, shape, ndim, what),
              strides_or_row_major(dst_strides, shape, ndim, what), elem_size, cast, checksum,
              static_cast<hipStream_t>(stream_v), what);
  });
}

int mxp_copy_views(mxp_engine* engine, const mxp_view_copy* views, int64_t n, void* stream_v) {
  return guard([&] {
    if (!engine || n < 0 || (n && !views)) throw Error(MXP_ERR_ARG, "mxp_copy_views: bad argument");
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    std::vector<BoxCopy> boxes;
    std::vector<const void*> srcs;
    std::vector<void*> dsts;
    std::vector<TransposeJob> transposes;
    lower_views(engine, views, n, boxes, srcs, dsts, transposes, "mxp_copy_views");  // before anything is launched
    HIP_OK(hipSetDevice(engine->opt.device));
    if (!boxes.empty()) run_boxes(*engine, boxes, srcs, dsts, 1, nullptr, stream);
    run_transposes(*engine, transposes, stream);
  });
}

int mxp_set_transpose_form(int32_t form) {
  return guard([&] {
    if (form != 0 && form != 1) throw Error(MXP_ERR_ARG, "mxp_set_transpose_form: 0 (the library picks) or 1 (wavefront-autonomous)");
    g_transpose_form.store(form, std::memory_order_relaxed);
  });
}

int mxp_describe_views(mxp_engine* engine, const mxp_view_copy* views, int64_t n, int32_t* kinds, int32_t* tile_rows,
                       int32_t* tile_row_bytes) {
  return guard([&] {
    if (!engine || n < 0 || (n && (!views || !kinds))) throw Error(MXP_ERR_ARG, "mxp_describe_views: bad argument");
    uint64_t call_bytes = 0;
    for (int64_t k = 0; k < n; ++k) {
      uint64_t el = 1;
      for (int d = 0; d < views[k].ndim && d < MXP_MAX_DIMS; ++d) el *= views[k].shape[d] > 0 ? (uint64_t)views[k].shape[d] : 0;
      call_bytes += el * (uint64_t)(views[k].elem_size > 0 ? views[k].elem_size : 0);
    }
    for (int64_t k = 0; k < n; ++k) {  // each view lowered as mxp_copy_views would lower it among the others
      std::vector<BoxCopy> boxes;
      std::vector<const void*> srcs;
      std::vector<void*> dsts;
      const mxp_view_copy& v = views[k];
      check_view_args(engine, v.ndim, v.shape, v.elem_size, "mxp_describe_views");
      std::vector<uint64_t> size;
      for (int d = 0; d < v.ndim; ++d) size.push_back((uint64_t)v.shape[d]);
      TransposeJob tr{};
      const auto s_st = strides_or_row_major(v.contiguous_src ? nullptr : v.src_strides, v.shape, v.ndim, "mxp_describe_views");
      const auto d_st = strides_or_row_major(v.contiguous_dst ? nullptr : v.dst_strides, v.shape, v.ndim, "mxp_describe_views");
      const ViewKind kind = lower_view(v.src, v.dst, size, s_st, d_st, v.elem_size, v.cast, 0xFFFFFFFFu, boxes, srcs, dsts, tr,
                                       "mxp_describe_views", call_bytes);
      const bool panel = kind == kViewTranspose && tr.td.panel_rows_log2 != 0;
      kinds[k] = kind == kViewTranspose ? (panel ? 2 : 1) : 0;
      if (tile_rows) tile_rows[k] = panel ? (int32_t)(1u << tr.td.panel_rows_log2) : 0;
      if (tile_row_bytes) tile_row_bytes[k] = panel ? (int32_t)(16u << tr.td.panel_chunks_log2) : 0;
    }
  });
}

int mxp_view_plan_create(mxp_engine* engine, const mxp_view_copy* views, int64_t n, mxp_view_plan** out) {
  return guard([&] {
    if (!out) throw Error(MXP_ERR_ARG, "mxp_view_plan_create: null out");
    *out = nullptr;
    if (!engine || n < 0 || (n && !views)) throw Error(MXP_ERR_ARG, "mxp_view_plan_create: bad argument");
    std::vector<BoxCopy> boxes;
    std::vector<const void*> srcs;
    std::vector<void*> dsts;
    std::vector<TransposeJob> transposes;
    lower_views(engine, views, n, boxes, srcs, dsts, transposes, "mxp_view_plan_create");
    auto vp = std::make_unique<mxp_view_plan>();
    vp->device = engine->opt.device;
    HIP_OK(hipSetDevice(vp->device));
    LowerOptions lo;
    lo.tile_bytes = engine->opt.tile_bytes;
    std::vector<Seg> segs;
    std::vector<WorkItem> work;
    for (const auto& b : boxes) {
      lower_box(b, lo, segs, work);
      vp->bytes += b.rows * b.row_bytes;
    }
    vp->n_work = (uint32_t)work.size();
    if (!work.empty()) {
      // one table: [segments][work items][source pointers][destination pointers]
      vp->o_work = align_up(segs.size() * sizeof(Seg), 256);
      vp->o_src = align_up(vp->o_work + work.size() * sizeof(WorkItem), 256);
      vp->o_dst = align_up(vp->o_src + srcs.size() * sizeof(void*), 256);
      std::vector<uint8_t> host(align_up(vp->o_dst + dsts.size() * sizeof(void*), 256), 0);
      std::memcpy(host.data(), segs.data(), segs.size() * sizeof(Seg));
      std::memcpy(host.data() + vp->o_work, work.data(), work.size() * sizeof(WorkItem));
      std::memcpy(host.data() + vp->o_src, srcs.data(), srcs.size() * sizeof(void*));
      std::memcpy(host.data() + vp->o_dst, dsts.data(), dsts.size() * sizeof(void*));
      vp->tables.upload(host.data(), host.size());
    }
    std::vector<TransposeItem> items;
    group_transposes(transposes, items, vp->groups, vp->singles);
    if (!items.empty()) vp->items.upload(items.data(), items.size());
    vp->items_host = items;
    for (const auto& t : transposes) {
      uint64_t elems = t.td.ni * t.td.nj;
      for (int q = 0; q < kMaxBatchDims; ++q) elems *= t.td.batch_size[q];
      vp->bytes += elems * (t.op == kOpCopy ? (uint64_t)t.elem_size : (uint64_t)op_dst_elem(t.op));
    }
    *out = vp.release();
  });
}

int mxp_view_plan_run(mxp_engine* engine, mxp_view_plan* plan, void* stream_v) {
  return guard([&] {
    if (!engine || !plan) throw Error(MXP_ERR_ARG, "mxp_view_plan_run: null handle");
    if (plan->device != engine->opt.device) throw Error(MXP_ERR_ARG, "mxp_view_plan_run: the plan was built for another device");
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    HIP_OK(hipSetDevice(plan->device));
    if (plan->n_work) {
      uint8_t* d = plan->tables.p;
      HIP_OK(launch_place(reinterpret_cast<const Seg*>(d), reinterpret_cast<const WorkItem*>(d + plan->o_work), plan->n_work,
                          reinterpret_cast<const void* const*>(d + plan->o_src), reinterpret_cast<void* const*>(d + plan->o_dst),
                          nullptr, Fan{}, engine->opt.nan_bits, stream));
    }
    for (const auto& t : plan->singles)
      HIP_OK(launch_transpose(t.src, t.dst, t.td, t.elem_size, t.op, engine->opt.nan_bits, nullptr, Fan{}, stream));
    for (const auto& g : plan->groups)
      HIP_OK(launch_transpose_batch(plan->items.p + g.first, (uint32_t)g.count, g.tiles, g.waves, g.elem_size, g.op,
                                    engine->opt.nan_bits, stream, g.panel, g.uniform_tiles, &g.common,
                                    plan->items_host.empty() ? nullptr : plan->items_host.data() + g.first));
  });
}

int mxp_view_plan_bytes(const mxp_view_plan* plan, uint64_t* out_bytes) {
  return guard([&] {
    if (!plan || !out_bytes) throw Error(MXP_ERR_ARG, "mxp_view_plan_bytes: null argument");
    *out_bytes = plan->bytes;
  });
}

void mxp_view_plan_destroy(mxp_view_plan* plan) {
  if (!plan) return;
  (void)hipSetDevice(plan->device);
  delete plan;
}

int mxp_copy_batch(mxp_engine* engine, const void* const* srcs, void* const* dsts, const uint64_t* nbytes, int64_t n,
                   uint32_t* out_checksums, void* stream) {
  return guard([&] {
    if (!engine || n < 0 || (n && (!srcs || !dsts || !nbytes))) throw Error(MXP_ERR_ARG, "mxp_copy_batch: bad argument");
    if (n == 0) return;
    HIP_OK(hipSetDevice(engine->opt.device));
    std::vector<BoxCopy> boxes;
    std::vector<const void*> sv;
    std::vector<void*> dv;
    std::vector<std::pair<uintptr_t, uintptr_t>> spans;
    for (int64_t k = 0; k < n; ++k) {
      if (nbytes[k] && (!srcs[k] || !dsts[k])) throw Error(MXP_ERR_ARG, "mxp_copy_batch: null pointer");
      if (reinterpret_cast<uintptr_t>(dsts[k]) & 15u) throw Error(MXP_ERR_ARG, "mxp_copy_batch: dst must be 16-byte aligned");
      const void* sb;
      uint64_t so;
      split_ptr(srcs[k], sb, so);
      sv.push_back(sb);
      dv.push_back(dsts[k]);
      BoxCopy b;
      b.src_buf = (uint32_t)k;
      b.dst_buf = (uint32_t)k;
      b.src_off = so;
      b.row_bytes = nbytes[k];
      b.op = kOpCopy;
      b.csum_slot = (uint32_t)k;
      boxes.push_back(b);
      if (nbytes[k]) spans.emplace_back(reinterpret_cast<uintptr_t>(dsts[k]), reinterpret_cast<uintptr_t>(dsts[k]) + nbytes[k]);
    }
    // One launch gives no ordering between copies: overlapping destinations are refused
    // (the reference serialises them in plan order instead, receiver.py:289-321).
    std::sort(spans.begin(), spans.end());
    for (size_t i = 1; i < spans.size(); ++i)
      if (spans[i].first < spans[i - 1].second) throw Error(MXP_ERR_ARG, "mxp_copy_batch: destinations overlap");
    std::vector<uint32_t> sums((size_t)n, 0);
    run_boxes(*engine, boxes, sv, dv, (uint32_t)n, out_checksums ? sums.data() : nullptr, static_cast<hipStream_t>(stream));
    if (out_checksums) std::memcpy(out_checksums, sums.data(), (size_t)n * 4);
  });
}

int mxp_digest_from_scalars(const uint64_t scalars[7], uint8_t out16[16]) {
  return guard([&] {
    if (!scalars || !out16) throw Error(MXP_ERR_ARG, "mxp_digest_from_scalars: null argument");
    const uint64_t n = scalars[0];
    const uint64_t body_words = n / 4, rows = body_words / kDigestRowWords;
    std::vector<uint64_t> list{n};
    if (rows) { list.push_back(scalars[1]); list.push_back(scalars[2]); }
    if (body_words - rows * kDigestRowWords) { list.push_back(scalars[3]); list.push_back(scalars[4]); }
    if (n % 4) { list.push_back(scalars[5]); list.push_back(n % 4); }
    Blake2b h(16);
    for (uint64_t v : list) {
      uint8_t le[8];
      for (int b = 0; b < 8; ++b) le[b] = (uint8_t)(v >> (8 * b));
      h.update(le, 8);
    }
    h.final(out16);
  });
}

int mxp_digest(mxp_engine* engine, const void* const* ptrs, const uint64_t* nbytes, int64_t n, uint8_t* out16,
               uint64_t* scalars, void* stream_v) {
  return guard([&] {
    if (!engine || !out16 || n < 0 || (n && (!ptrs || !nbytes))) throw Error(MXP_ERR_ARG, "mxp_digest: bad argument");
    if (n == 0) return;
    mxp_engine& e = *engine;
    HIP_OK(hipSetDevice(e.opt.device));
    hipStream_t stream = static_cast<hipStream_t>(stream_v);
    std::vector<DigestJob> jobs((size_t)n);
    uint64_t blocks = 0;
    for (int64_t k = 0; k < n; ++k) {
      if (nbytes[k] && !ptrs[k]) throw Error(MXP_ERR_ARG, "mxp_digest: null pointer");
      jobs[k].ptr = static_cast<const uint8_t*>(ptrs[k]);
      jobs[k].nbytes = nbytes[k];
      jobs[k].out_slot = (uint64_t)k * 5;
      jobs[k].first_block = blocks;
      const uint64_t rows = (nbytes[k] / 4) / kDigestRowWords;
      blocks += rows ? (rows + kDigestRowsPerBlock - 1) / kDigestRowsPerBlock : 1;
    }
    if (blocks > 0x7FFFFFFFull) throw Error(MXP_ERR_ARG, "mxp_digest: batch too large for one launch");
    const size_t o_jobs = 0;
    // [jobs][digest sums, fanned][digest sums, folded]: only the jobs are uploaded
    const Fan fan = make_fan((uint64_t)n);
    const size_t o_fan = align_up(jobs.size() * sizeof(DigestJob), 256);
    const size_t o_out = align_up(o_fan + fan_elems(fan, 5) * 8, 256);
    const size_t total = o_out + (size_t)n * 5 * 8;
    mxp_engine::Arena& ar = acquire_arena(e);
    ensure_desc(ar, total);
    std::memcpy(ar.host + o_jobs, jobs.data(), jobs.size() * sizeof(DigestJob));
    upload_arena(ar, jobs.size() * sizeof(DigestJob), stream);
    unsigned long long* const fanned = reinterpret_cast<unsigned long long*>(ar.dev.p + o_fan);
    HIP_OK(launch_fill_u32(reinterpret_cast<uint32_t*>(fanned), 2 * fan_elems(fan, 5), 0u, stream));
    HIP_OK(launch_digest(reinterpret_cast<const DigestJob*>(ar.dev.p + o_jobs), (uint32_t)n, (uint32_t)blocks, fanned, fan, stream));
    HIP_OK(launch_fold_fan(fanned, fan, 5, 5 * (uint64_t)n, reinterpret_cast<unsigned long long*>(ar.host_dev + o_out), false, stream));
    release_arena(ar, stream);
    HIP_OK(wait_event_promptly(ar.busy));
    const uint64_t* sums = reinterpret_cast<const uint64_t*>(ar.host + o_out);
    for (int64_t k = 0; k < n; ++k) {
      uint64_t sc[7] = {nbytes[k], sums[5 * k], sums[5 * k + 1], sums[5 * k + 2], sums[5 * k + 3], sums[5 * k + 4],
                        nbytes[k] % 4};
      if (scalars) std::memcpy(scalars + 7 * k, sc, sizeof sc);
      Blake2b h(16);
      const uint64_t body_words = nbytes[k] / 4, rows = body_words / kDigestRowWords;
      std::vector<uint64_t> list{sc[0]};
      if (rows) { list.push_back(sc[1]); list.push_back(sc[2]); }
      if (body_words - rows * kDigestRowWords) { list.push_back(sc[3]); list.push_back(sc[4]); }
      if (nbytes[k] % 4) { list.push_back(sc[5]); list.push_back(sc[6]); }
      for (uint64_t v : list) {
        uint8_t le[8];
        for (int b = 0; b < 8; ++b) le[b] = (uint8_t)(v >> (8 * b));
        h.update(le, 8);
      }
      h.final(out16 + 16 * k);
    }
  });
}

int mxp_measure_h2d(mxp_engine* engine, uint64_t bytes, int32_t repeats, double* bytes_per_second) {
  return guard([&] {
    if (!engine || !bytes_per_second || bytes == 0) throw Error(MXP_ERR_ARG, "mxp_measure_h2d: bad argument");
    mxp_engine& e = *engine;
    HIP_OK(hipSetDevice(e.opt.device));
    if (repeats < 1) repeats = 1;
    void* h = nullptr;
    void* d = nullptr;
    HIP_OK(hipHostMalloc(&h, bytes, hipHostMallocDefault));
    if (hipMalloc(&d, bytes) != hipSuccess) {
      (void)hipHostFree(h);
      throw Error(MXP_ERR_DEVICE, "mxp_measure_h2d: device allocation failed");
    }
    std::memset(h, 0x5a, bytes);
    float best = 1e30f;
    hipError_t err = hipSuccess;
    for (int r = 0; r < repeats + 1 && err == hipSuccess; ++r) {
      err = hipEventRecord(e.ev_a, e.streams[0]);
      if (err == hipSuccess) err = hipMemcpyAsync(d, h, bytes, hipMemcpyHostToDevice, e.streams[0]);
      if (err == hipSuccess) err = hipEventRecord(e.ev_b, e.streams[0]);
      if (err == hipSuccess) err = hipEventSynchronize(e.ev_b);
      float ms = 0;
      if (err == hipSuccess) err = hipEventElapsedTime(&ms, e.ev_a, e.ev_b);
      if (r > 0 && ms < best) best = ms;  // first pass warms the path
    }
    (void)hipFree(d);
    (void)hipHostFree(h);
    if (err != hipSuccess) throw Error(MXP_ERR_DEVICE, std::string("mxp_measure_h2d: ") + hipGetErrorString(err));
    *bytes_per_second = (double)bytes / ((double)best * 1e-3);
  });
}

int mxp_measure_read(const char* const* paths, int64_t n_paths, int32_t threads, uint64_t request_bytes, int32_t direct,
                     uint64_t* total_bytes, double* bytes_per_second) {
  return guard([&] {
    if (!paths || n_paths <= 0 || !bytes_per_second || threads < 1 || request_bytes == 0 || request_bytes % 4096)
      throw Error(MXP_ERR_ARG, "mxp_measure_read: bad argument");
    struct Req { int file; uint64_t off, n; };
    std::vector<int> fds((size_t)n_paths, -1);
    struct FdCloser {
      std::vector<int>& f;
      ~FdCloser() { for (int fd : f) if (fd >= 0) ::close(fd); }
    } closer{fds};
    std::vector<Req> reqs;
    uint64_t total = 0;
    for (int64_t f = 0; f < n_paths; ++f) {
      int flags = O_RDONLY;
#ifdef O_DIRECT
      if (direct) flags |= O_DIRECT;
#endif
      fds[(size_t)f] = ::open(paths[f], flags);
      if (fds[(size_t)f] < 0) throw Error(MXP_ERR_IO, std::string("cannot open ") + paths[f] + ": " + std::strerror(errno));
      struct stat st;
      if (::fstat(fds[(size_t)f], &st) != 0) throw Error(MXP_ERR_IO, std::string("cannot stat ") + paths[f]);
      for (uint64_t off = 0; off < (uint64_t)st.st_size; off += request_bytes)
        reqs.push_back(Req{(int)f, off, std::min<uint64_t>(request_bytes, (uint64_t)st.st_size - off)});
      total += (uint64_t)st.st_size;
    }
    std::atomic<size_t> next{0};
    std::atomic<bool> failed{false};
    std::mutex err_mu;
    std::string err;
    const double t0 = now_s();
    auto worker = [&] {
      void* buf = nullptr;
      if (::posix_memalign(&buf, 4096, request_bytes) != 0) { failed.store(true); return; }
      try {
        for (;;) {
          const size_t i = next.fetch_add(1);
          if (i >= reqs.size() || failed.load()) break;
          const Req& r = reqs[i];
          // whole blocks, as direct I/O wants them; the last request of a file may end short
          pread_full(fds[(size_t)r.file], static_cast<uint8_t*>(buf), align_up(r.n, 4096), r.off, paths[r.file], r.n);
        }
      } catch (const std::exception& ex) {
        std::lock_guard<std::mutex> lk(err_mu);
        if (err.empty()) err = ex.what();
        failed.store(true);
      }
      std::free(buf);
    };
    {
      std::vector<std::thread> pool;
      for (int t = 0; t < threads; ++t) pool.emplace_back(worker);
      for (auto& t : pool) t.join();
    }
    const double dt = now_s() - t0;
    if (failed.load()) throw Error(MXP_ERR_IO, "mxp_measure_read: " + (err.empty() ? std::string("out of host memory") : err));
    if (total_bytes) *total_bytes = total;
    *bytes_per_second = dt > 0 ? (double)total / dt : 0.0;
  });
}

int mxp_measure_gather(mxp_engine* engine, uint64_t rows, uint32_t row_bytes, uint64_t src_pitch, uint32_t col_offset,
                       int32_t cast, int32_t repeats, double* bytes_per_second) {
  return guard([&] {
    if (cast != MXP_CAST_NONE && cast != MXP_CAST_F32_BF16) throw Error(MXP_ERR_ARG, "mxp_measure_gather: cast must be none or fp32 -> bf16");
    const bool narrow = cast == MXP_CAST_F32_BF16;
    const uint64_t src_row = narrow ? 2ull * row_bytes : row_bytes;  // source bytes of a row
    const uint32_t out_unit = narrow ? 8u : 16u;                     // destination bytes per 16 source bytes
    if (!engine || !bytes_per_second || rows == 0 || row_bytes == 0 || row_bytes % out_unit || src_row > 32768 || src_pitch % 16 ||
        col_offset % 16 || (uint64_t)col_offset + src_row > src_pitch || src_pitch >= (1ull << 31))
      throw Error(MXP_ERR_ARG, "mxp_measure_gather: bad argument");
    mxp_engine& e = *engine;
    HIP_OK(hipSetDevice(e.opt.device));
    if (repeats < 1) repeats = 1;
    const uint32_t upr = (uint32_t)(src_row / 16);
    const uint32_t rpt = (uint32_t)std::min<uint64_t>(rows, (uint64_t)kPlaceThreads * kPlaceBatch / upr);
    const uint64_t n_tiles = rows / rpt;
    if (n_tiles == 0 || n_tiles > 0x7FFFFFFFull) throw Error(MXP_ERR_ARG, "mxp_measure_gather: bad argument");
    const uint64_t used_rows = n_tiles * rpt, src_bytes = used_rows * src_pitch, dst_bytes = used_rows * row_bytes;
    DevBuf<uint8_t> src, dst;
    src.reserve(src_bytes);
    dst.reserve(dst_bytes);
    // bf16 values ~N(0, 0.02): read as fp32, every pair of them is a finite number, so the narrowing probe meets no NaN
    HIP_OK(launch_synth(src.p, src_bytes / 2, MXP_DTYPE_BF16, 0u, 0x6a7468ull, e.streams[0]));
    float best = 1e30f;
    for (int r = 0; r < repeats + 1; ++r) {
      HIP_OK(hipEventRecord(e.ev_a, e.streams[0]));
      HIP_OK(launch_probe_gather(src.p + col_offset, dst.p, upr, (uint32_t)src_pitch, rpt, (uint32_t)n_tiles, narrow, e.streams[0]));
      HIP_OK(hipEventRecord(e.ev_b, e.streams[0]));
      HIP_OK(hipEventSynchronize(e.ev_b));
      float ms = 0;
      HIP_OK(hipEventElapsedTime(&ms, e.ev_a, e.ev_b));
      if (r > 0 && ms < best) best = ms;  // the first launch warms up
    }
    // The probe is only worth its figure if it moved the right bytes: the library's own gather of
    // the same rows (checksummed as it stores) must leave the checksum the probe's output has.
    {
      DevBuf<uint8_t> again;
      again.reserve(dst_bytes);
      BoxCopy g;
      g.src_off = col_offset;
      g.src_pitch = src_pitch;
      g.dst_pitch = row_bytes;
      g.rows = used_rows;
      g.row_bytes = row_bytes;
      g.op = narrow ? kOpCastF32Bf16 : kOpCopy;
      g.csum_slot = 0;
      uint32_t want = 0, got = 0;
      run_boxes(e, {g}, {src.p}, {again.p}, 1, &want, e.streams[0]);
      BoxCopy c;
      c.row_bytes = dst_bytes;
      c.op = kOpChecksumOnly;
      c.csum_slot = 0;
      run_boxes(e, {c}, {dst.p}, {}, 1, &got, e.streams[0]);
      if (want != got) throw Error(MXP_ERR_STATE, "mxp_measure_gather: the probe kernel and the placement kernel disagree");
    }
    *bytes_per_second = ((double)dst_bytes + (double)used_rows * (double)src_row) / ((double)best * 1e-3);
  });
}

int mxp_synth_host(void* dst, uint64_t n_elems, int32_t dtype, uint32_t kind, uint64_t seed, int32_t threads) {
  return guard([&] {
    if (n_elems && !dst) throw Error(MXP_ERR_ARG, "mxp_synth_host: null dst");
    if (!dtype_size(dtype)) throw Error(MXP_ERR_UNSUPPORTED, "unknown dtype code");
    synth_host(dst, n_elems, (uint32_t)dtype, kind, seed, threads);
  });
}

int mxp_synth_device(void* dst_dev, uint64_t n_elems, int32_t dtype, uint32_t kind, uint64_t seed, void* stream) {
  return guard([&] {
    if (n_elems && !dst_dev) throw Error(MXP_ERR_ARG, "mxp_synth_device: null dst");
    if (!dtype_size(dtype)) throw Error(MXP_ERR_UNSUPPORTED, "unknown dtype code");
    HIP_OK(launch_synth(dst_dev, n_elems, (uint32_t)dtype, kind, seed, static_cast<hipStream_t>(stream)));
  });
}

}  // extern "C"
