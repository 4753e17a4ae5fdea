// Internal (non-ABI) declarations shared by the HIP kernels and the host engine.
//
// Everything the device executes is driven by flat descriptor tables built on
// the host: a "segment" is one pitched 2-D byte box (rows x row_bytes) moving
// from a source buffer to a destination buffer, optionally through the
// dtype conversion, with the position-weighted checksum of the bytes it writes
// accumulated on the way.  A "work item" is one tile (a band of rows) of one
// segment; one workgroup executes one work item, so one launch covers an
// arbitrary mix of tensors with thousands of workgroups.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mxp {

enum SegOp : uint32_t {
  kOpCopy = 0,       // dst bytes = src bytes
  kOpCastF32Bf16 = 1,  // src is fp32, dst is bf16 (round to nearest even)
  kOpChecksumOnly = 2,  // read src, write nothing, accumulate checksum at dst_off indices
  kOpCastBf16F32 = 3,  // src is bf16, dst is fp32 (exact)
  kOpCastF16F32 = 4,   // src is fp16, dst is fp32 (exact; NaNs made quiet)
  kOpCastF32F16 = 5,   // src is fp32, dst is fp16 (round to nearest even)
  kOpCastF8E4M3Bf16 = 6,  // src is fp8 e4m3fn, dst is bf16 (exact; NaN -> 0x7FC0)
  kOpCastF16Bf16 = 7,  // src is fp16, dst is bf16 (through fp32, round to nearest even)
  kOpCastBf16F16 = 8   // src is bf16, dst is fp16 (through fp32, round to nearest even)
};
// Conversions between two 16-bit formats: same size on both sides, values change.
constexpr bool op_recodes16(uint32_t op) { return op == kOpCastF16Bf16 || op == kOpCastBf16F16; }
constexpr bool op_narrows(uint32_t op) { return op == kOpCastF32Bf16 || op == kOpCastF32F16; }
constexpr bool op_widens(uint32_t op) { return op == kOpCastBf16F32 || op == kOpCastF16F32 || op == kOpCastF8E4M3Bf16; }
// Destination element size of a converting op (2 for a copy: only used for alignment rules).
constexpr uint32_t op_dst_elem(uint32_t op) { return (op == kOpCastBf16F32 || op == kOpCastF16F32) ? 4u : 2u; }
// Source bytes that produce `dst_bytes` destination bytes.
constexpr uint64_t op_src_bytes(uint32_t op, uint64_t dst_bytes) {
  return op_narrows(op) ? dst_bytes * 2 : op_widens(op) ? dst_bytes / 2 : dst_bytes;
}
// Destination bytes produced from `src_bytes` source bytes.
constexpr uint64_t op_dst_bytes(uint32_t op, uint64_t src_bytes) {
  return op_narrows(op) ? src_bytes / 2 : op_widens(op) ? src_bytes * 2 : src_bytes;
}
// Public conversion code of a write record (0 none, 1 fp32->bf16, 2 bf16->fp32, 3 fp16->fp32,
// 4 fp32->fp16, 5 fp8-e4m3->bf16, 6 fp16->bf16, 7 bf16->fp16) -> segment operation.
constexpr uint32_t seg_op_of_cast(int cast) {
  return cast == 1 ? kOpCastF32Bf16 : cast == 2 ? kOpCastBf16F32 : cast == 3 ? kOpCastF16F32
       : cast == 4 ? kOpCastF32F16 : cast == 5 ? kOpCastF8E4M3Bf16 : cast == 6 ? kOpCastF16Bf16
       : cast == 7 ? kOpCastBf16F16 : kOpCopy;
}

// 80 bytes, 16-byte aligned; the index is workgroup-uniform, so the whole record
// arrives through scalar loads.
struct alignas(16) Seg {
  uint64_t src_off;    // byte offset of the box inside source buffer `src_buf`
  uint64_t dst_off;    // byte offset inside destination buffer `dst_buf`; also the
                       // checksum position of the first byte
  uint64_t src_pitch;  // bytes between consecutive rows in the source
  uint64_t dst_pitch;  // bytes between consecutive rows in the destination
  uint32_t rows;
  uint32_t row_bytes;  // DESTINATION bytes per row (source bytes: op_src_bytes)
  uint32_t src_buf;    // index into the source base-pointer table
  uint32_t dst_buf;    // index into the destination base-pointer table
  uint32_t op;         // SegOp
  uint32_t unit;       // bytes per lane access on the destination side: 16, 8 (narrowing cast), 4, 2 or 1
  uint32_t rows_per_tile;
  uint32_t csum_slot;  // index into the checksum accumulator array, ~0u = none
  uint32_t units_per_row;  // row_bytes / unit
  uint32_t div_magic;  // floor(2^32 / units_per_row) + 1, exact for n*d < 2^32
  uint32_t csum_bias;  // added (mod 2^32) to the destination offset to get the checksum position
  uint32_t pad1;
};
static_assert(sizeof(Seg) == 80, "Seg layout is part of the host<->device contract");

// `src_buf` of a checksum-only segment that reads the destination buffer `dst_buf` itself (bytes a
// host-to-device copy placed there) instead of a source buffer.
constexpr uint32_t kSrcIsDestination = 0xFFFFFFFFu;

struct WorkItem {
  uint32_t seg;
  uint32_t tile;
};

// One tensor to digest: `out` receives five u64 scalars
// {sum_rows, sum_rows_weighted, sum_tail, sum_tail_weighted, sum_ragged}.
struct alignas(16) DigestJob {
  const uint8_t* ptr;
  uint64_t nbytes;
  uint64_t out_slot;  // index of the first of 5 u64 in the output array
  uint64_t first_block;  // first workgroup index that belongs to this job
};

constexpr uint32_t kKnuth = 2654435761u;
constexpr int kPlaceThreads = 1024;  // lanes per placement workgroup (16 wavefronts)
constexpr int kPlaceBatch = 8;       // 16-byte units each lane keeps in flight
constexpr int kDigestThreads = 1024;
constexpr uint32_t kDigestRowWords = 1024;   // 4 KiB rows
constexpr uint32_t kDigestRowsPerBlock = 32; // 128 KiB per workgroup, two rows per wavefront

// Accumulator fan.  Every workgroup ends with one atomic add per accumulator it feeds, and adds to
// one address are applied one after the other by the memory side: a launch whose workgroups all
// feed one checksum measured a tenth slower than the same launch without the add.  So each
// accumulator array is kept in `lanes()` copies, `pitch` elements apart (a 32-bit checksum is one
// element, a tensor_digest slot is five 64-bit elements), workgroup b adds to copy b & mask, and
// whoever reads the results adds the copies up (fold_fan): sums mod 2^32 / 2^64 commute.
// mask == 0 is the plain layout, one copy.
constexpr uint32_t kFanLanes = 64;
struct Fan {
  uint32_t mask = 0, pitch = 0;
  uint32_t lanes() const { return mask + 1; }
};
// Fan for `n_slots` accumulators: copies a multiple of 256 bytes apart, so that the copies of one
// accumulator fall into different cache lines.  The fanned table is bounded by size, not by slot
// count: copies x pitch stays at or below 65,536 elements (64 copies up to 1,024 slots, halved
// for every doubling after that, one copy - the plain layout - above 16,384), so a plan's two sets
// of checksum and digest accumulators (44 bytes per slot and copy) never take more than 5.5 MiB
// and clearing one set is at most 2.75 MiB of stores.  The more slots a launch feeds, the fewer
// workgroups meet in any one of them, so the narrower fan loses nothing.
inline Fan make_fan(uint64_t n_slots) {
  Fan f;
  if (n_slots > 16384) {
    f.pitch = (uint32_t)n_slots;
    return f;
  }
  f.pitch = (uint32_t)((n_slots ? n_slots : 1) + 63) / 64 * 64;
  uint32_t lanes = kFanLanes;
  while (lanes > 1 && (uint64_t)lanes * f.pitch > 65536) lanes >>= 1;
  f.mask = lanes - 1;
  return f;
}
// Elements (of either kind) the fanned array of `per_slot`-element accumulators holds.
inline uint64_t fan_elems(const Fan& f, uint32_t per_slot = 1) { return (uint64_t)f.lanes() * f.pitch * per_slot; }
// out[k] = sum over the copies of element k, k < n (n <= pitch * per_slot).
template <typename T>
inline void fold_fan(const T* fanned, const Fan& f, uint32_t per_slot, uint64_t n, T* out) {
  for (uint64_t k = 0; k < n; ++k) out[k] = 0;
  for (uint32_t l = 0; l < f.lanes(); ++l) {
    const T* lane = fanned + (uint64_t)l * f.pitch * per_slot;
    for (uint64_t k = 0; k < n; ++k) out[k] += lane[k];
  }
}

// ---- launch wrappers (mxp_kernels.hip) -------------------------------------
// `sums_dev` is fanned by `fan`.  `zero_dev` / `zero_words`: 32-bit words the launch also clears
// (spread over its workgroups), e.g. the accumulators of the launch after it; they must not overlap
// anything this launch reads or adds to.
// `widening_only`: every segment is a conversion to a wider element (half as many bytes read as
// written); such a launch runs two workgroups per compute unit, which measured 3-4% faster for it.
hipError_t launch_place(const Seg* segs_dev, const WorkItem* work_dev, uint32_t n_work,
                        const void* const* src_bases_dev, void* const* dst_bases_dev,
                        uint32_t* sums_dev, Fan fan, uint16_t nan_bits, hipStream_t stream, bool checksum_only = false,
                        uint32_t* zero_dev = nullptr, uint32_t zero_words = 0, bool widening_only = false);
// launch_place that also accumulates the tensor_digest sums of the bytes it stores: five 64-bit
// words per destination buffer (whole-row sum, row-weighted sum, tail sum, tail-weighted sum,
// ragged-byte sum), added to `digest_sums_dev` (cleared by the caller, fanned by `fan` with five
// elements per slot); `dst_sizes_dev[b]` is the byte size of destination buffer b, segment offsets
// are offsets inside their buffer.
hipError_t launch_place_digest(const Seg* segs_dev, const WorkItem* work_dev, uint32_t n_work,
                               const void* const* src_bases_dev, void* const* dst_bases_dev, uint32_t* sums_dev, Fan fan,
                               const unsigned long long* dst_sizes_dev, unsigned long long* digest_sums_dev,
                               uint16_t nan_bits, hipStream_t stream, uint32_t* zero_dev = nullptr, uint32_t zero_words = 0);
// `out_dev` is fanned by `fan` with five 64-bit elements per slot (DigestJob::out_slot counts elements).
hipError_t launch_digest(const DigestJob* jobs_dev, uint32_t n_jobs, uint32_t n_blocks,
                         unsigned long long* out_dev, Fan fan, hipStream_t stream);
hipError_t launch_fill_u32(uint32_t* ptr, uint64_t n, uint32_t value, hipStream_t stream);
// Copies a small table (16-byte multiple, both sides 16-byte aligned) with a kernel; `src` may be
// pinned host memory the device can address.  Stays on the launch stream's own queue, where a
// copy call of this size costs a hand-over to a copy engine and back.
hipError_t launch_copy_table(void* dst, const void* src, size_t bytes, hipStream_t stream);
// Measurement support (mxp_synth.hip): a bare row gather with the placement kernel's workgroup shape.
hipError_t launch_probe_gather(const void* src, void* dst, uint32_t units_per_row, uint32_t src_pitch, uint32_t rows_per_tile,
                               uint32_t n_tiles, bool narrow, hipStream_t stream);
// Device-side fold_fan: out_dev[k] = sum over the copies of element k, k < n; with `clear` the
// elements read are left at zero.  T is uint32_t or unsigned long long.
template <typename T>
hipError_t launch_fold_fan(T* fanned_dev, Fan fan, uint32_t per_slot, uint64_t n, T* out_dev, bool clear, hipStream_t stream);

// Batched 2-D transpose (mxp_permute.hip).  "i" = the destination's innermost dimension,
// "j" = the source's innermost dimension; strides are in elements.
constexpr int kMaxBatchDims = 6;
// Transpose tiling.  One wavefront owns a sub-tile of 64 (128 for 1-byte destination elements)
// source rows (i) x 128 source bytes (j); a workgroup is `waves` <= kTransposeWaves wavefronts
// arranged waves_i x (waves / waves_i), chosen per call from the extents.
constexpr int kTransposeWaves = 8;
constexpr int kChipCus = 256;  // compute units of the one chip this library is written for
constexpr int transpose_sub_rows(int dst_elem_size) { return dst_elem_size == 1 ? 128 : 64; }
constexpr int transpose_sub_cols(int src_elem_size) { return 128 / src_elem_size; }
struct TransposeDesc {
  uint64_t ni, nj;   // extents
  uint64_t si;       // source stride of i (source stride of j is 1)
  uint64_t dj;       // destination stride of j (destination stride of i is 1)
  uint32_t tiles_i, tiles_j;
  uint64_t n_tiles;  // tiles_i * tiles_j * product of batch sizes
  uint64_t batch_size[kMaxBatchDims];     // unused entries are 1
  uint64_t batch_sstride[kMaxBatchDims];
  uint64_t batch_dstride[kMaxBatchDims];
  uint32_t align_src, align_dst;  // power of two <= 16 that divides every address a chunk access can have on that side
  uint32_t csum_bias;
  uint32_t waves_i;           // wavefronts of a workgroup along i (power of two, divides waves)
  uint32_t group_j;           // tiles along j that consecutive workgroups visit before stepping along i (>= 1)
  uint32_t waves;             // wavefronts of a workgroup (1, 2, 4 or 8; up to 16 for a panel)
  // Panel form (panel_rows_log2 != 0): the workgroup stages a whole tile of 2^panel_rows_log2 source rows
  // x 2^panel_chunks_log2 16-byte chunks in LDS, waits at a barrier and writes the transposed tile; the
  // extents are whole multiples of the tile, both sides 16-byte aligned, waves = rows * chunks / 512.
  uint32_t panel_rows_log2, panel_chunks_log2;
};
constexpr uint32_t kPanelLoads = 8;             // 16-byte loads per lane of a panel workgroup
constexpr uint32_t kPanelMaxBytes = 128 * 1024; // staged tile
// What the kernels assume of a descriptor (index arithmetic in 32 bits, workgroup shape).
inline bool transpose_desc_ok(const TransposeDesc& d) {
  if (d.panel_rows_log2) return d.n_tiles <= 0x7FFFFFFFull && (uint64_t)d.tiles_i * d.tiles_j <= 0x7FFFFFFFull;  // shape: panel_desc_ok
  return d.n_tiles <= 0x7FFFFFFFull && d.waves != 0 && d.waves <= (uint32_t)kTransposeWaves && (d.waves & (d.waves - 1)) == 0 &&
         d.waves_i != 0 && d.waves % d.waves_i == 0 && d.group_j != 0 && (uint64_t)d.tiles_i * d.tiles_j <= 0x7FFFFFFFull &&
         (uint64_t)d.tiles_i * d.group_j <= 0x7FFFFFFFull;
}
// What the panel kernels assume of a descriptor, for source / destination element sizes es / eo: they
// have no edge handling, so whole tiles and 16-byte accesses everywhere are checked here, on the host.
inline bool panel_desc_ok(const TransposeDesc& d, uint32_t es, uint32_t eo) {
  if (!d.panel_rows_log2 || d.panel_rows_log2 > 10 || d.panel_chunks_log2 < 3 || d.panel_chunks_log2 > 13) return false;
  if (es != 1 && es != 2 && es != 4) return false;
  if (eo != 1 && eo != 2 && eo != 4) return false;
  const uint64_t rows = 1ull << d.panel_rows_log2, chunks = 1ull << d.panel_chunks_log2, cols = chunks * 16 / es;
  const uint64_t threads = rows * chunks / kPanelLoads;
  return rows * chunks * 16 <= kPanelMaxBytes && threads >= 64 && threads <= 1024 && d.waves * 64ull == threads &&
         rows >= 16 / eo && d.align_src >= 16 && d.align_dst >= 16 && d.ni == (uint64_t)d.tiles_i * rows &&
         d.nj == (uint64_t)d.tiles_j * cols && d.n_tiles <= 0x7FFFFFFFull;
}
// One transpose of a batched launch: `first_tile` is the number of workgroups of the items
// before it (items sorted by it; every item has d.n_tiles >= 1 and the same d.waves).
struct alignas(16) TransposeItem {
  const uint8_t* src;
  uint8_t* dst;
  uint64_t first_tile;
  uint64_t pad;
  TransposeDesc d;
};
// Per-device set-up of the placement kernels (idempotent; also done lazily by launch_place).
hipError_t configure_place_kernels();
// `elem_size` is the source element; `op` is kOpCopy or a conversion whose source element it is
// (dj, batch_dstride and the checksum positions then count destination elements / bytes).
// `sum_out` (may be null) is one checksum accumulator fanned by `fan`.
hipError_t launch_transpose(const void* src, void* dst, const TransposeDesc& d, int elem_size, uint32_t op,
                            uint32_t nan_bits, uint32_t* sum_out, Fan fan, hipStream_t stream);
// `n_items` transposes of one (elem_size, op, waves) in a launch of `total_tiles` workgroups; the
// host checks each descriptor as launch_transpose would (transpose_desc_ok).
// `panel`: 0, or (panel_rows_log2 << 8 | panel_chunks_log2) shared by every item; `uniform_tiles`: 0, or - for
// a panel batch whose items all have the descriptor `*common` - the number of tiles of each
// (total_tiles == n_items * uniform_tiles); the kernel then takes the descriptor as an argument, and with
// `items_host` (the same items, on the host) their pointers as well, kPanelArgItems items to a launch.
hipError_t launch_transpose_batch(const TransposeItem* items_dev, uint32_t n_items, uint64_t total_tiles, uint32_t waves,
                                  int elem_size, uint32_t op, uint32_t nan_bits, hipStream_t stream, uint32_t panel = 0,
                                  uint32_t uniform_tiles = 0, const TransposeDesc* common = nullptr,
                                  const TransposeItem* items_host = nullptr);
// Items of a uniform panel batch whose pointers fit the kernel argument block of one launch (`items_host` given).
constexpr int kPanelArgItems = 96;
// Field by field (the struct may hold padding).
inline bool same_transpose_desc(const TransposeDesc& a, const TransposeDesc& b) {
  bool eq = a.ni == b.ni && a.nj == b.nj && a.si == b.si && a.dj == b.dj && a.tiles_i == b.tiles_i && a.tiles_j == b.tiles_j &&
            a.n_tiles == b.n_tiles && a.align_src == b.align_src && a.align_dst == b.align_dst && a.csum_bias == b.csum_bias &&
            a.waves_i == b.waves_i && a.group_j == b.group_j && a.waves == b.waves && a.panel_rows_log2 == b.panel_rows_log2 &&
            a.panel_chunks_log2 == b.panel_chunks_log2;
  for (int k = 0; k < kMaxBatchDims; ++k)
    eq = eq && a.batch_size[k] == b.batch_size[k] && a.batch_sstride[k] == b.batch_sstride[k] && a.batch_dstride[k] == b.batch_dstride[k];
  return eq;
}

// Synthetic-checkpoint generator (mxp_synth.hip), same arithmetic on host and device.
enum SynthKind : uint32_t {
  kSynthNormal = 0,   // ~N(0, 0.02): centred sum of four 16-bit uniforms times a constant
  kSynthOnes = 1,
  kSynthZeros = 2,
  kSynthNormalEdge = 3,  // kSynthNormal with denormal / +-inf / NaN injected at 1e-6 density each
  kSynthFp8Finite = 4,   // bytes uniform over the 254 finite e4m3 codes
  kSynthScale = 5        // fp32 uniform in [1e-4, 1e-2]
};
hipError_t launch_synth(void* dst, uint64_t n_elems, uint32_t dtype_code, uint32_t kind,
                        uint64_t seed, hipStream_t stream);
void synth_host(void* dst, uint64_t n_elems, uint32_t dtype_code, uint32_t kind, uint64_t seed,
                int threads);

}  // namespace mxp
