/*
 * mxp_bench.h - measurement and test-input entry points of libmxplace.so.
 *
 * These live in the same shared library as the product ABI (mxp.h) but are no part of the
 * drop-in boundary: none of them replaces an interface of the reference, and a binding that
 * plugs the engine into a loader chain does not need this file.  Their callers are the
 * benchmark and the tests: per-launch kernel durations, the pinned host-to-device rate an
 * ingest is compared with, a bare kernel of the placement kernel's shape, and the seeded
 * generator of synthetic checkpoints (same bytes on host and device).
 */
#ifndef MXP_BENCH_H_
#define MXP_BENCH_H_

#include "mxp.h"

#ifdef __cplusplus
extern "C" {
#endif

/* Launch timing for measurements.  Switched on, every asynchronous mxp_execute_resident (stats ==
 * NULL) records a HIP-event pair around its placement kernel on the launch stream and does NOT
 * synchronise, so a timed loop of K launches yields both its wall time and the K kernel
 * durations.  The stand-alone operators that launch through descriptor tables built per call
 * (mxp_cast, mxp_copy_view(s), mxp_permute_copy, mxp_place_boxes, mxp_copy_batch,
 * mxp_checksum32) and the runs of a verify plan (mxp_verify_plan_checksums / _digests) record a
 * pair around each of their placement / transpose launches in the same way.
 * mxp_engine_launch_times waits for the launches and writes the durations (ms) of the most recent
 * min(capacity, recorded, 256) of them, oldest first.  Switching on or off restarts the count. */
int mxp_engine_set_launch_timing(mxp_engine* engine, int32_t on);
int mxp_engine_launch_times(mxp_engine* engine, float* out_ms, int32_t capacity, int32_t* n_out);

/* Measured pinned host -> device bandwidth of this box in bytes per second
 * (hipMemcpyAsync of `bytes` from a pinned buffer, best of `repeats`). */
int mxp_measure_h2d(mxp_engine* engine, uint64_t bytes, int32_t repeats, double* bytes_per_second);
/* Plain read rate of a set of files, no GPU work: `threads` threads claim requests of `request_bytes`
 * (a multiple of 4096) in file order and read them into private block-aligned buffers, with O_DIRECT
 * when `direct` is non-zero (no page cache) - the way the ingest's readers read whole row bands.
 * What a cold ingest from the same files is compared with. */
int mxp_measure_read(const char* const* paths, int64_t n_paths, int32_t threads, uint64_t request_bytes, int32_t direct,
                     uint64_t* total_bytes, double* bytes_per_second);
/* What this box's memory system gives an access shape, measured with a bare kernel that has the
 * placement kernel's workgroup shape and nothing else (no descriptor tables, no checksum, no
 * conversion): `rows` rows of `row_bytes` bytes (a multiple of 16, at most 32 KiB), `src_pitch`
 * bytes apart (a multiple of 16; == row_bytes for a contiguous copy), `col_offset` bytes into each
 * pitch, gathered into a contiguous destination; the source buffer is filled with a seeded pattern.
 * `cast` is MXP_CAST_NONE or MXP_CAST_F32_BF16 (the rows are fp32, twice `row_bytes` long in the
 * source, and are stored as bf16).  Writes bytes moved (read + written) per second, best of
 * `repeats` launches.  Allocates and frees both buffers.  No counterpart in the reference: the
 * library's own kernels are compared with it. */
int mxp_measure_gather(mxp_engine* engine, uint64_t rows, uint32_t row_bytes, uint64_t src_pitch, uint32_t col_offset,
                       int32_t cast, int32_t repeats, double* bytes_per_second);

/* How mxp_copy_views would run each of `views` (nothing is launched): kinds[k] = 0 row or element
 * boxes through the placement kernel, 1 a transpose in which every wavefront moves its own sub-tile,
 * 2 a transpose in which a workgroup stages a whole tile of tile_rows[k] source rows x
 * tile_row_bytes[k] source bytes (both 0 otherwise).  For tests and measurements: the choice between
 * the two transpose forms is a heuristic of the library, not part of its contract. */
int mxp_describe_views(mxp_engine* engine, const mxp_view_copy* views, int64_t n, int32_t* kinds, int32_t* tile_rows,
                       int32_t* tile_row_bytes);

/* Process-wide measurement switch: 1 makes every transposed view run in the wavefront-autonomous form, 0
 * (the default) lets the library pick between that and the staged-tile form.  Results are identical. */
int mxp_set_transpose_form(int32_t form);

/* Seeded synthetic contents (test and benchmark inputs; same bytes on host and device).
 * kind: 0 ~N(0,0.02), 1 ones, 2 zeros, 3 normal with denormal/inf/NaN/tie edge cases at
 * 1e-6 density, 4 fp8 bytes over the finite e4m3 codes, 5 fp32 scales in [1e-4,1e-2],
 * 6 as 3 at 1/64 density. */
int mxp_synth_host(void* dst, uint64_t n_elems, int32_t dtype, uint32_t kind, uint64_t seed,
                   int32_t threads);
int mxp_synth_device(void* dst_dev, uint64_t n_elems, int32_t dtype, uint32_t kind, uint64_t seed,
                     void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MXP_BENCH_H_ */
