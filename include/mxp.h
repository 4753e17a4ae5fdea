/*
 * mxp.h - C ABI of the MI355X weight-placement engine (libmxplace.so).
 *
 * The library turns safetensors byte ranges on local storage into one serving rank's
 * parameter buffers in HBM: host-staged ingest through a bounded ring of pinned
 * buffers, then hand-written gfx950 kernels for tensor-parallel slicing, QKV / gate_up
 * fusing, MoE expert stacking, fp32->bf16 refit casts (and the receive-side widening ones), fp8 block-scale tile slicing and
 * per-tensor checksums.
 *
 * The boundary is plain C: opaque handles, pointers and sizes.  Device pointers are
 * ordinary HIP device addresses owned by the caller; a `stream` argument is a
 * `hipStream_t` passed as `void*` (NULL = the default stream).  Every function
 * returns MXP_OK (0) or a negative MXP_ERR_* class; the text of the last error on the
 * calling thread is available from mxp_last_error().  Handles are not re-entrant: use
 * one plan / engine from one thread at a time.
 *
 * The library is built for one part: MI355X (gfx950), 256 compute units in 8 XCDs; launch
 * shapes and the sizes of accumulator tables assume that count.  Entry points that exist
 * only for measurements and test inputs are declared in mxp_bench.h, not here.
 *
 * Each entry point names the piece of the reference (ai-dynamo/modelexpress,
 * modelexpress_client/python/modelexpress/...) whose behaviour it replaces.
 */
#ifndef MXP_H_
#define MXP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MXP_ABI_VERSION 1

/* ---- status codes -------------------------------------------------------- */
#define MXP_OK 0
#define MXP_ERR_IO (-1)          /* open / read failure, short file, offset past EOF     */
#define MXP_ERR_FORMAT (-2)      /* malformed safetensors header or index                */
#define MXP_ERR_UNSUPPORTED (-3) /* dtype outside the map, unsupported layout            */
#define MXP_ERR_COVERAGE (-4)    /* unmapped tensor / uncovered parameter (fail closed)  */
#define MXP_ERR_ARG (-5)         /* bad argument                                         */
#define MXP_ERR_DEVICE (-6)      /* HIP runtime error                                    */
#define MXP_ERR_STATE (-7)       /* call out of order                                    */
#define MXP_ERR_VERIFY (-8)      /* checksum / digest mismatch                           */

/* Text of the last error raised on the calling thread ("" if none). */
const char* mxp_last_error(void);
int mxp_abi_version(void);

/* ---- dtypes: the safetensors dtype map of gds_loader.py:36-49 ------------- */
#define MXP_DTYPE_F64 0
#define MXP_DTYPE_F32 1
#define MXP_DTYPE_F16 2
#define MXP_DTYPE_BF16 3
#define MXP_DTYPE_F8_E4M3 4
#define MXP_DTYPE_F8_E5M2 5
#define MXP_DTYPE_I64 6
#define MXP_DTYPE_I32 7
#define MXP_DTYPE_I16 8
#define MXP_DTYPE_I8 9
#define MXP_DTYPE_U8 10
#define MXP_DTYPE_BOOL 11
#define MXP_MAX_DIMS 8

/* Bytes per element, or 0 for an unknown code. */
int mxp_dtype_size(int dtype);
/* "BF16" -> MXP_DTYPE_BF16; -1 when the string is not in the map. */
int mxp_dtype_from_name(const char* safetensors_name);
const char* mxp_dtype_name(int dtype);

/* =========================================================================
 * 1. Checkpoint: safetensors discovery and header parse
 *    replaces MxGdsLoader._resolve_safetensors_files (gds_loader.py:189-243)
 *    and MxGdsLoader._parse_safetensors_header (gds_loader.py:245-282).
 * ========================================================================= */
typedef struct mxp_ckpt mxp_ckpt;

typedef struct mxp_tensor_info {
  const char* name;   /* owned by the checkpoint handle */
  int32_t dtype;      /* MXP_DTYPE_* */
  int32_t ndim;
  int64_t shape[MXP_MAX_DIMS];
  int32_t file_index; /* which shard file */
  int32_t reserved;
  uint64_t file_offset; /* absolute: 8 + header_len + data_offsets[0] */
  uint64_t nbytes;      /* data_offsets[1] - data_offsets[0] */
} mxp_tensor_info;

typedef struct mxp_file_info {
  const char* path;
  uint64_t file_size;
  uint64_t data_start; /* 8 + header_len */
  int64_t n_tensors;
} mxp_file_info;

/* `model_path` is a directory (model.safetensors.index.json, then model.safetensors,
 * then *.safetensors in sorted order) or a single .safetensors file.  Rejects files
 * shorter than 8 bytes, headers above 100 MiB, dtypes outside the map, data ranges
 * that run past the end of the file. */
int mxp_ckpt_open(const char* model_path, mxp_ckpt** out);
void mxp_ckpt_close(mxp_ckpt* ckpt);
int64_t mxp_ckpt_tensor_count(const mxp_ckpt* ckpt);
int64_t mxp_ckpt_file_count(const mxp_ckpt* ckpt);
/* Tensors are listed per file in ascending file offset (gds_loader.py:297-300). */
int mxp_ckpt_tensor_info(const mxp_ckpt* ckpt, int64_t index, mxp_tensor_info* out);
int mxp_ckpt_file_info(const mxp_ckpt* ckpt, int64_t index, mxp_file_info* out);
/* Index of the tensor called `name`, or -1. */
int64_t mxp_ckpt_find(const mxp_ckpt* ckpt, const char* name);

/* =========================================================================
 * 2. Placement plan: destination map for one rank
 *    replaces MdlLoader._extend_dest_map / _resolve_write / _warm_load resolution
 *    (engines/vllm/refit/installer.py:341-437,470-564), _tp_local_tensor (:292-317),
 *    _tp_shape_compatible (:319-339), _fused_destinations (:566-616),
 *    _premerged_destination / _premerged_writes (:629-693), _resolve_expert (:695-754),
 *    _assert_loaderless_coverage (:219-251), _check_moe_swizzle (:833-843), and the
 *    run decomposition of refit/reshard/slice_plan.py:259-294.
 *
 *    The caller describes the rank's parameters (what the serving engine allocated:
 *    name, dtype, local shape), the stacked-parameter groups and the expert mapping,
 *    exactly the three things MdlLoader reads off the model object.  mxp_plan_build
 *    resolves EVERY checkpoint tensor to its destination box before anything is
 *    written; any unmapped tensor or uncovered parameter fails the whole plan.
 * ========================================================================= */
typedef struct mxp_plan mxp_plan;

#define MXP_PLAN_ALLOW_CAST_F32_BF16 0x1u /* plan a dtype conversion where source and       */
#define MXP_PLAN_ALLOW_CAST MXP_PLAN_ALLOW_CAST_F32_BF16 /* parameter dtypes differ (MXP_CAST_*) */
#define MXP_PLAN_ALLOW_UNMAPPED 0x2u      /* skip checkpoint tensors with no destination  */
#define MXP_PLAN_ALLOW_UNCOVERED 0x4u     /* allow parameters no tensor writes            */
#define MXP_PLAN_NO_FP8_BLOCK_CHECK 0x8u  /* do not require 128-aligned fp8 scale slicing */
#define MXP_PLAN_NONLOCAL_EXPERTS_UNMAPPED 0x10u /* an expert that is not local to the rank counts as
                                           * unmapped, as in the reference's loaderless mode
                                           * (installer.py:708-710,219-251), instead of being skipped */

int mxp_plan_create(const mxp_ckpt* ckpt, int32_t tp_size, int32_t tp_rank, uint32_t flags,
                    mxp_plan** out);
void mxp_plan_destroy(mxp_plan* plan);
/* Returns the parameter index (>= 0) or a negative error. */
int64_t mxp_plan_add_param(mxp_plan* plan, const char* name, int32_t dtype, int32_t ndim,
                           const int64_t* shape);
/* One (fused_suffix, member_suffix) pair of the model's stacked_params_mapping, in pack
 * order.  With none added, the built-in groups apply: qkv_proj <- q_proj,k_proj,v_proj
 * and gate_up_proj <- gate_proj,up_proj (installer.py:72-78,773-797). */
int mxp_plan_add_stacked(mxp_plan* plan, const char* fused_suffix, const char* member_suffix);
/* One row of the model's get_expert_mapping(): shard is "w1", "w2" or "w3";
 * `local_expert_id` is the slot in the rank's stacked parameter, or -1 when the
 * expert is not local to this rank: such tensors are then skipped, not an error (a rank is
 * handed the whole checkpoint and there is no stock loader behind this one to hand them to),
 * unless the plan was created with MXP_PLAN_NONLOCAL_EXPERTS_UNMAPPED. */
int mxp_plan_add_expert(mxp_plan* plan, const char* param_prefix, const char* weight_prefix,
                        int32_t expert_id, const char* shard, int32_t local_expert_id);
/* Skip checkpoint tensors whose name starts with `prefix` (e.g. other pipeline stages). */
int mxp_plan_add_skip_prefix(mxp_plan* plan, const char* prefix);
/* A virtual checkpoint tensor: a full shape assembled from boxes ("shards") of real
 * checkpoint tensors, the published-tensor model of the reference's reshard path
 * (PublishedTensor.full_shape + shards[].shard_offset/shape; plan_pull intersects the
 * needed box with every shard box, refit/reshard/slice_plan.py:248-256,297-339).  The
 * virtual tensor is then placed like a checkpoint tensor of that name; the real tensors it
 * is made of are consumed.  This is how trainer-native layouts enter: Megatron's
 * by-KV-group interleaved linear_qkv becomes virtual q/k/v tensors made of row bands
 * (modelexpress_rl/train/engines/megatron/aliases.py:206-263,291-350), a fused gate/up
 * tensor two halves (aliases.py:116-168).  Shards must not overlap; the part of the virtual
 * tensor a rank needs must be covered (else MXP_ERR_COVERAGE from mxp_plan_build). */
int64_t mxp_plan_add_virtual(mxp_plan* plan, const char* name, int32_t ndim, const int64_t* full_shape);
int mxp_plan_add_virtual_shard(mxp_plan* plan, int64_t virtual_index, const char* source_tensor,
                               const int64_t* source_offset, const int64_t* shard_offset, const int64_t* shape);
int mxp_plan_build(mxp_plan* plan);

/* dtype conversions of dest.copy_(src): trainer fp32 -> wire bf16
 * (modelexpress_rl/train/engines/fsdp/adapter.py:203-206, publisher.py:44), served bf16 staging
 * -> fp32 receive buffer (refit/reshard/receiver.py:962-969), and their fp16 counterparts.
 * Narrowing rounds to nearest even; fp32 -> bf16 maps every NaN to mxp_engine_options.nan_bits;
 * the fp16 conversions keep a NaN's top payload bits and make it quiet. */
#define MXP_CAST_NONE 0
#define MXP_CAST_F32_BF16 1
#define MXP_CAST_BF16_F32 2
#define MXP_CAST_F16_F32 3
#define MXP_CAST_F32_F16 4
#define MXP_CAST_F8E4M3_BF16 5 /* exact; the .to(out_dtype) of engines/vllm/refit/receiver.py:258-261 */
#define MXP_CAST_F16_BF16 6 /* through fp32, as copy_ converts; NaN -> nan_bits */
#define MXP_CAST_BF16_F16 7
#define MXP_CAST_LAST MXP_CAST_BF16_F16

#define MXP_WRITE_DIRECT 0
#define MXP_WRITE_FUSED 1
#define MXP_WRITE_EXPERT 2
#define MXP_WRITE_PREMERGED 3

typedef struct mxp_write_info {
  int64_t tensor_index; /* source tensor in the checkpoint */
  int64_t param_index;  /* destination parameter */
  int32_t kind;         /* MXP_WRITE_* */
  int32_t cast;         /* MXP_CAST_* */
  /* The write as a pitched box, in bytes of the respective dtype. */
  uint64_t src_offset;  /* from the start of the source tensor's data */
  uint64_t src_pitch;
  uint64_t dst_offset;  /* from the start of the destination parameter */
  uint64_t dst_pitch;
  uint64_t rows;
  uint64_t row_bytes;   /* destination bytes per row */
  /* Number of maximal runs contiguous in both source and destination
   * (what slice_plan.paired_runs would enumerate). */
  uint64_t paired_runs;
} mxp_write_info;

typedef struct mxp_param_info {
  const char* name;
  int32_t dtype;
  int32_t ndim;
  int64_t shape[MXP_MAX_DIMS];
  uint64_t nbytes;
  uint64_t bytes_written; /* by the plan; == nbytes when fully covered */
  int32_t n_writes;
  int32_t reserved;
} mxp_param_info;

int64_t mxp_plan_param_count(const mxp_plan* plan);
int64_t mxp_plan_write_count(const mxp_plan* plan);
int mxp_plan_param_info(const mxp_plan* plan, int64_t index, mxp_param_info* out);
int mxp_plan_write_info(const mxp_plan* plan, int64_t index, mxp_write_info* out);
/* Bytes read from storage, bytes that cross PCIe and bytes placed, for one execute. */
int mxp_plan_totals(const mxp_plan* plan, uint64_t* file_bytes, uint64_t* h2d_bytes,
                    uint64_t* placed_bytes, uint64_t* kernel_algorithmic_bytes);

/* =========================================================================
 * 3. Engine: pinned ring, HIP streams, kernels
 *    replaces the host-staged ingest of the ModelStreamer path
 *    (VllmAdapter.build_model_streamer_weight_iter, engines/vllm/adapter.py:233-292 ->
 *    runai-model-streamer reader threads -> per-tensor copy_ inside model.load_weights,
 *    adapter.py:223-231) and the per-file batch load of gds_loader.py:284-331; the
 *    device side replaces destination.copy_(source) (installer.py:419-424), the
 *    narrow().contiguous() gather (installer.py:317), the staged re-slice and dtype
 *    conversion of refit/reshard/receiver.py:919-971.
 * ========================================================================= */
typedef struct mxp_engine mxp_engine;

typedef struct mxp_engine_options {
  int32_t device;          /* HIP device ordinal */
  int32_t ring_slots;      /* pinned host slots (each with a device bounce slot); 0 = default 32 */
  uint64_t slot_bytes;     /* bytes per slot; 0 = default 16 MiB */
  int32_t reader_threads;  /* pread workers; 0 = min(16, host cores) */
  int32_t streams;         /* HIP streams for H2D + kernels; 0 = default 4 */
  uint32_t tile_bytes;     /* source bytes per workgroup, 1 KiB .. 128 KiB; 0 = 128 KiB */
  uint16_t nan_bits;       /* bf16 image of every NaN in the cast; 0 = default 0x7FC0 */
  uint16_t pack_strided_on_host; /* strided slices: 1 = readers pack the needed rows into the
                                    slot (only placed bytes cross PCIe; with use_o_direct they
                                    read the rows of a band with large requests into their
                                    own buffers first), 2 = stage whole row bands and gather
                                    on the device, 0 = default (1) */
  int32_t use_o_direct;    /* 1 = open files with O_DIRECT (falls back if unsupported) */
} mxp_engine_options;

typedef struct mxp_exec_stats {
  double wall_seconds;     /* entry to last stream idle */
  double read_seconds;     /* reading and packing, summed over reader threads (waiting for a slot not included) */
  double kernel_ms;        /* HIP-event time of placement kernels (resident mode) */
  uint64_t file_bytes;     /* read from storage */
  uint64_t h2d_bytes;      /* copied host -> device */
  uint64_t placed_bytes;   /* written into parameter buffers */
  uint64_t n_chunks;
  uint64_t n_segments;
  uint64_t n_workgroups;
  uint64_t n_launches;
  int32_t mutated;         /* 1 once any destination byte may have been written */
  int32_t reserved;
} mxp_exec_stats;

int mxp_engine_create(const mxp_engine_options* opts, mxp_engine** out);
void mxp_engine_destroy(mxp_engine* engine);

/* Lowers `plan` to the engine's descriptor tables and chunk list and allocates the engine's pinned
 * ring without running anything (mxp_execute does both on first use); afterwards mxp_plan_totals
 * is complete and the first mxp_execute starts reading at once. */
int mxp_prepare(mxp_engine* engine, mxp_plan* plan);

/* Ingest from storage: reader threads pread each planned byte range into a pinned
 * slot, the slot is copied to its device bounce slot with hipMemcpyAsync on one of
 * the engine's streams, and the placement kernel for that slot runs on the same
 * stream.  `dst_ptrs[i]` is the device address of parameter i (16-byte aligned,
 * mxp_plan_param_info().nbytes long).  Blocks until every stream is idle.  Per
 * parameter checksums are left in the plan (mxp_plan_checksums).
 *
 * Ordering: the engine's streams are private.  Before the first byte moves they wait for the
 * work already queued on the caller's stream - the default (null) stream for mxp_execute,
 * `caller_stream` for mxp_execute_after - so kernels still pending on the destinations
 * (initialisation, reads of memory the caller's allocator has recycled into them) finish
 * first, as they would ahead of destination.copy_(source) on that stream
 * (installer.py:419-424).  Work the caller queues on other streams is the caller's to order.
 * On return everything has completed, so later work needs no further ordering. */
int mxp_execute(mxp_engine* engine, mxp_plan* plan, void* const* dst_ptrs, mxp_exec_stats* stats);
int mxp_execute_after(mxp_engine* engine, mxp_plan* plan, void* const* dst_ptrs, void* caller_stream,
                      mxp_exec_stats* stats);

/* Same placement with the checkpoint already staged in HBM: `file_dev_ptrs[f]` holds
 * the complete bytes of shard file f (8-byte aligned, so that elements keep their alignment).
 * Where the caller chooses the address, the best one puts the file's data section
 * (mxp_file_info.data_start) on a 256-byte boundary, i.e. the file's first byte
 * (256 - data_start % 256) % 256 bytes past one: tensors then start on cache-line boundaries and
 * the strided row gathers of column slices touch no line more than they need (worth 1.5 points of
 * HBM peak on a Llama-3-8B tensor-parallel rank share).  One kernel launch on `stream`
 * for the whole plan; asynchronous unless `stats` is non-NULL (then it synchronises and
 * reports the HIP-event time of the launch in stats->kernel_ms).  A plan's pointer tables and
 * accumulators are its own: launches of one plan are serialised (a call on another stream than
 * the previous one waits for that launch, through an event it records on the previous stream:
 * a stream a plan was launched on must stay alive until the plan's next launch or the plan's
 * destruction), and changed `dst_ptrs` / `file_dev_ptrs` reach the
 * device by copies ordered on `stream`, never under a launch that still runs. */
int mxp_execute_resident(mxp_engine* engine, mxp_plan* plan, const void* const* file_dev_ptrs,
                         void* const* dst_ptrs, void* stream, mxp_exec_stats* stats);

/* Final-address placement (on by default).  During mxp_execute a piece that is contiguous in the
 * file and in its parameter buffer and is not converted is copied by hipMemcpyAsync from the pinned
 * slot straight to its final address - the reference's own loader reads each tensor into its own
 * device buffer (gds_loader.py:284-331) - and the kernel only reads it back for the checksum (and
 * the digest sums); strided slices, conversions and pieces under `min_bytes` still go through the
 * bounce slot and the placement kernel.  min_bytes: 0 = the default (64 KiB), a negative value =
 * off (every byte takes the bounce slot).  Results are identical either way. */
int mxp_engine_set_direct_placement(mxp_engine* engine, int64_t min_bytes);

/* Checksums accumulated by the last execute, one per parameter (tensor_utils.py:27-44
 * over the parameter's row-major bytes).  Synchronises the engine first. */
int mxp_plan_checksums(mxp_engine* engine, mxp_plan* plan, uint32_t* out, int64_t n);
/* Fused verification: with this switched on, every placement (mxp_execute, mxp_execute_resident)
 * also accumulates, inside the same kernel, the sums tensor_digest is made of
 * (refit/reshard/verify.py:112-150) for every parameter buffer, so the digests of what was placed
 * cost no second pass over the buffers - in place of the reference's recompute-after-transfer
 * (modelexpress_rl/inference/nixl_staged_transfer.py:529-549).  mxp_plan_digests waits for the
 * device and writes 16 bytes per parameter (the blake2b-128 of the scalar list, as mxp_digest
 * gives for the finished buffer); it fails if the last execute ran with the switch off or if the
 * plan leaves part of a parameter unwritten.  The checksums are still produced. */
int mxp_engine_set_fused_digests(mxp_engine* engine, int32_t on);
int mxp_plan_digests(mxp_engine* engine, mxp_plan* plan, uint8_t* out16, int64_t n);

/* =========================================================================
 * 4. Stand-alone device operators (all batched: one launch for n tensors)
 * ========================================================================= */
/* safe_checksum (tensor_utils.py:27-44) of n device buffers:
 *   out[k] = sum_i byte_i * ((i * 2654435761 + 1) mod 2^32) mod 2^32. */
int mxp_checksum32(mxp_engine* engine, const void* const* ptrs, const uint64_t* nbytes, int64_t n,
                   uint32_t* out, void* stream);
/* mxp_checksum32 for callers that cannot allocate (tight serving loops, harnesses that forbid
 * hipMalloc).  No counterpart in the reference.  Same arguments and
 * results as mxp_checksum32; the descriptor tables and accumulators its kernel reads live in a
 * 1 MiB device array that is part of the library image (one copy per GPU, held until the process
 * ends) and in a pinned mirror allocated by mxp_engine_create, so the call itself allocates and
 * frees nothing on the host or the device.  Limits: n <= 1024 buffers and at most 98,304
 * workgroups of 128 KiB in all (about 12 GiB); beyond them the call fails with MXP_ERR_ARG and
 * launches nothing.  Every call on a GPU - from any engine - uses that GPU's one array: calls
 * that overlap in time on one GPU race and must be serialised by the caller.  Blocks until
 * `stream` is idle, like mxp_checksum32, and returns its results on the host: it cannot be
 * recorded into a HIP graph, and a `stream` that is being captured is refused with MXP_ERR_STATE
 * before anything is queued (the capture stays valid). */
int mxp_checksum32_static(mxp_engine* engine, const void* const* ptrs, const uint64_t* nbytes, int64_t n,
                          uint32_t* out, void* stream);
/* mxp_checksum32 / mxp_digest over a FIXED set of device buffers, lowered once: a refit loop
 * verifies the same buffers every step, and the reference keeps its descriptor lists for that
 * reason (refit/reshard/receiver.py:787-801; the verify loop is
 * modelexpress_rl/inference/nixl_staged_transfer.py:529-549).  _create lowers the buffers, uploads
 * the descriptor tables and allocates the pinned result block; a run is then one kernel launch
 * plus a small one that adds up the accumulator copies, clears them and stores the totals into
 * that block (no descriptor build, no upload, no allocation, no copy command), and waits for the
 * event behind it.
 * The addresses and sizes are the ones given at create; when a buffer moves, build a new plan.
 * One run of a plan at a time. */
typedef struct mxp_verify_plan mxp_verify_plan;
int mxp_verify_plan_create(mxp_engine* engine, const void* const* ptrs, const uint64_t* nbytes, int64_t n,
                           mxp_verify_plan** out);
int mxp_verify_plan_checksums(mxp_engine* engine, mxp_verify_plan* plan, uint32_t* out, void* stream);
/* `scalars` as for mxp_digest (7 u64 per buffer), or NULL. */
int mxp_verify_plan_digests(mxp_engine* engine, mxp_verify_plan* plan, uint8_t* out16, uint64_t* scalars, void* stream);
void mxp_verify_plan_destroy(mxp_verify_plan* plan);
/* tensor_digest (refit/reshard/verify.py:79-155) of n device buffers: 16 bytes each
 * (blake2b-128 over the little-endian u64 scalars).  `scalars`, if not NULL, receives
 * 7 u64 per tensor: n, sum_rows, sum_rows_weighted, sum_tail, sum_tail_weighted,
 * sum_ragged, n % 4. */
int mxp_digest(mxp_engine* engine, const void* const* ptrs, const uint64_t* nbytes, int64_t n,
               uint8_t* out16, uint64_t* scalars, void* stream);
/* fp32 -> bf16 round-to-nearest-even of `n_elems` contiguous elements (torch copy_ at
 * modelexpress_rl/train/engines/fsdp/adapter.py:203-206, receiver.py:964-971), with the
 * checksum of the bf16 bytes in *checksum when not NULL. */
int mxp_cast_f32_bf16(mxp_engine* engine, const void* src, void* dst, uint64_t n_elems,
                      uint32_t* checksum, void* stream);
/* Any MXP_CAST_* conversion of `n_elems` contiguous elements (same call sites), with the
 * checksum of the destination bytes in *checksum when not NULL. */
int mxp_cast(mxp_engine* engine, const void* src, void* dst, uint64_t n_elems, int32_t cast,
             uint32_t* checksum, void* stream);
/* Pitched 2-D byte gather, the device form of narrow(axis, r*n, n).contiguous()
 * (installer.py:317) and of the as_strided re-slice (receiver.py:919-960). */
int mxp_gather2d(mxp_engine* engine, const void* src, uint64_t src_pitch, void* dst,
                 uint64_t dst_pitch, uint64_t rows, uint64_t row_bytes, uint32_t* checksum,
                 void* stream);
/* One pitched box between two device addresses. */
typedef struct mxp_box {
  const void* src;
  void* dst;           /* 16-byte aligned unless rows == 1 and the box is byte-granular */
  uint64_t src_pitch;  /* bytes between rows in the source (ignored when rows == 1) */
  uint64_t dst_pitch;
  uint64_t rows;
  uint64_t row_bytes;  /* destination bytes per row */
  uint64_t csum_index; /* checksum position of the first destination byte */
  uint32_t csum_group; /* which output checksum this box adds to, 0 .. n_groups-1 */
  uint32_t cast;       /* MXP_CAST_*; row_bytes counts destination bytes */
} mxp_box;
/* n boxes in one launch: the batched form of the staged re-slice of
 * refit/reshard/receiver.py:919-960 (as_strided + copy_ per view) and of shard_region
 * (refit/reshard/verify.py:158-183).  out_checksums[g], when not NULL, receives the sum of
 * the position-weighted checksums of every box in group g (a whole buffer's checksum when
 * its boxes tile it and csum_index is the offset inside the buffer).  Boxes must not
 * overlap in the destination. */
int mxp_place_boxes(mxp_engine* engine, const mxp_box* boxes, int64_t n, uint32_t n_groups,
                    uint32_t* out_checksums, void* stream);
/* dst = src.permute(perm).contiguous() for an ndim-dimensional tensor (ndim <= 8) of
 * elem_size-byte elements (1, 2, 4 or 8).  `shape` is the source's shape, `src_strides`
 * its strides in elements (NULL = contiguous row-major; a narrowed view passes the parent's
 * strides), `perm[d]` the source dimension that becomes destination dimension d.
 * Replaces W_UV = w_uv.transpose(0,1) and W_UK_T = w_uk.permute(1,2,0)
 * (engines/vllm/refit/receiver.py:252-261) and the permuted views of
 * refit/reshard/slice_plan.py:166-220.  Permutations that keep the innermost dimension run
 * as a batched row gather; the others as an LDS-tiled transpose.  *checksum, when not
 * NULL, receives the checksum of the destination bytes. */
int mxp_permute_copy(mxp_engine* engine, const void* src, void* dst, int32_t ndim, const int64_t* shape,
                     const int64_t* src_strides, const int32_t* perm, int32_t elem_size, uint32_t* checksum,
                     void* stream);
/* dst_view[...] = src_view[...] for two strided views of one `shape` (ndim <= 8, strides in
 * elements, NULL = contiguous row-major): the device form of one RecordedCopy
 * (refit/reshard/types.py:57-71) once its op-chain has been replayed to a strided source view
 * (refit/reshard/slice_plan.py:136-164) - destination.as_strided(shape, dst_strides).copy_(
 * source.as_strided(shape, src_strides)).  Rows contiguous on both sides run as pitched boxes,
 * a transposed innermost dimension through the LDS transpose, anything else element by
 * element (the run length paired_runs would find).  A destination view that overlaps itself
 * is refused.  `cast` is an MXP_CAST_* code (then `elem_size` is the destination element's; a
 * transposed view converts inside the transpose, in one pass).  *checksum, when not NULL, receives
 * the position-weighted checksum of the written bytes, positions counted from `dst`. */
int mxp_copy_view(mxp_engine* engine, const void* src, void* dst, int32_t ndim, const int64_t* shape,
                  const int64_t* src_strides, const int64_t* dst_strides, int32_t elem_size,
                  int32_t cast, uint32_t* checksum, void* stream);
/* One entry of mxp_copy_views: the arguments of mxp_copy_view. */
typedef struct mxp_view_copy {
  const void* src;
  void* dst;
  int32_t ndim;
  int32_t elem_size;
  int32_t cast;            /* MXP_CAST_* */
  uint8_t contiguous_src;  /* 1: ignore src_strides, the source view is row-major contiguous */
  uint8_t contiguous_dst;  /* 1: ignore dst_strides */
  uint16_t reserved;
  int64_t shape[MXP_MAX_DIMS];
  int64_t src_strides[MXP_MAX_DIMS];
  int64_t dst_strides[MXP_MAX_DIMS];
} mxp_view_copy;
/* n recorded copies at once: every view is lowered first (an error moves nothing), then all
 * row / element boxes run in ONE launch and the transposed views in one launch per element
 * type and conversion - in place of the reference's launch per view ("thousands of
 * individual kernel launches", refit/reshard/receiver.py:920-923).  Destinations must not
 * overlap one another: the launches give no order between views. */
int mxp_copy_views(mxp_engine* engine, const mxp_view_copy* views, int64_t n, void* stream);
/* The same n copies lowered once and run many times - a refit loop re-slices the same views
 * every step (the reference caches its descriptor lists for that reason,
 * refit/reshard/receiver.py:787-801).  mxp_view_plan_create lowers the views, builds the descriptor
 * tables and uploads them; nothing moves.  mxp_view_plan_run only launches (one kernel for all
 * row / element boxes, one per kind of transposed view): it allocates nothing, copies nothing
 * from the host and does not synchronise, so it can be recorded into a HIP graph.  The source
 * and destination addresses are the ones given at create; when a buffer moves, build a new
 * plan.  Destinations must not overlap one another.  *out_bytes = destination bytes per run. */
typedef struct mxp_view_plan mxp_view_plan;
int mxp_view_plan_create(mxp_engine* engine, const mxp_view_copy* views, int64_t n, mxp_view_plan** out);
int mxp_view_plan_run(mxp_engine* engine, mxp_view_plan* plan, void* stream);
int mxp_view_plan_bytes(const mxp_view_plan* plan, uint64_t* out_bytes);
void mxp_view_plan_destroy(mxp_view_plan* plan);
/* n independent contiguous device copies in one launch, with the checksum of each
 * destination in out_checksums[k] when not NULL: the device form of the batched
 * torch._foreach_copy_ install (refit/reshard/receiver.py:939-955).  Destinations must
 * be 16-byte aligned and must not overlap each other. */
int mxp_copy_batch(mxp_engine* engine, const void* const* srcs, void* const* dsts, const uint64_t* nbytes,
                   int64_t n, uint32_t* out_checksums, void* stream);
/* ---- host-only helpers ---------------------------------------------------- */
/* blake2b-128 over the scalar list tensor_digest would hash (verify.py:152-155). */
int mxp_digest_from_scalars(const uint64_t scalars[7], uint8_t out16[16]);

/* CRC32C (Castagnoli) as the artifact manifest uses it: mxp_crc32c continues a finished
 * CRC (`seed` = 0 to start), like crc32c_append; mxp_file_crc32c gives the whole-file
 * checksum and one checksum per `chunk_size` piece (the last may be shorter; an empty file
 * has no chunks) -- file_checksum / chunks_for_file of
 * modelexpress_common/src/artifact_manifest.rs:260-324. */
uint32_t mxp_crc32c(uint32_t seed, const void* data, uint64_t nbytes);
int mxp_file_crc32c(const char* path, uint64_t chunk_size, uint32_t* file_crc, uint32_t* chunk_crcs,
                    uint64_t max_chunks, uint64_t* n_chunks);

#ifdef __cplusplus
}
#endif
#endif /* MXP_H_ */
