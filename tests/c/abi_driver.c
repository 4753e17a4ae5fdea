/*
 * A caller of libmxplace.so written in plain C: no Python, no torch.  It does what a
 * foreign-function binding (a Rust -sys crate, cgo, ctypes) would do through include/mxp.h:
 * open a checkpoint, declare one tensor-parallel rank's parameters, plan, allocate the
 * destinations itself with hipMalloc, ingest, and print one line per parameter:
 *     <name> <nbytes> <checksum %08x> <digest hex>
 * so that a test can compare it with the CPU oracle.
 *
 * usage: abi_driver <checkpoint dir> <tp_size> <tp_rank> <params file>
 * params file: one "<name> <dtype> <ndim> <d0> <d1> ..." per line, then optional
 *              "stacked <fused> <member>" lines.
 * Built by `python -m modelexpress_amd.build --abi-driver` (hipcc as a C compiler + linker).
 */
#include <hip/hip_runtime_api.h>
#include <stdint.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include "mxp.h"

#define CHECK(call)                                                          \
  do {                                                                       \
    int rc_ = (call);                                                        \
    if (rc_ < 0) {                                                           \
      fprintf(stderr, "%s -> %d: %s\n", #call, rc_, mxp_last_error());       \
      return 1;                                                              \
    }                                                                        \
  } while (0)

int main(int argc, char** argv) {
  if (argc != 5) {
    fprintf(stderr, "usage: %s <checkpoint dir> <tp_size> <tp_rank> <params file>\n", argv[0]);
    return 2;
  }
  if (mxp_abi_version() != MXP_ABI_VERSION) {
    fprintf(stderr, "header and library disagree on the ABI version\n");
    return 1;
  }
  mxp_ckpt* ck = NULL;
  mxp_plan* plan = NULL;
  mxp_engine* eng = NULL;
  CHECK(mxp_ckpt_open(argv[1], &ck));
  CHECK(mxp_plan_create(ck, atoi(argv[2]), atoi(argv[3]), 0, &plan));

  FILE* f = fopen(argv[4], "r");
  if (!f) { perror(argv[4]); return 1; }
  char a[512], b[512];
  while (fscanf(f, "%511s", a) == 1) {
    if (strcmp(a, "stacked") == 0) {
      if (fscanf(f, "%511s %511s", a, b) != 2) return 1;
      CHECK(mxp_plan_add_stacked(plan, a, b));
      continue;
    }
    int ndim = 0;
    int64_t shape[MXP_MAX_DIMS];
    if (fscanf(f, "%511s %d", b, &ndim) != 2 || ndim < 0 || ndim > MXP_MAX_DIMS) return 1;
    for (int d = 0; d < ndim; ++d) {
      long long v;
      if (fscanf(f, "%lld", &v) != 1) return 1;
      shape[d] = v;
    }
    const int dtype = mxp_dtype_from_name(b);
    if (dtype < 0) { fprintf(stderr, "unknown dtype %s\n", b); return 1; }
    if (mxp_plan_add_param(plan, a, dtype, ndim, shape) < 0) {
      fprintf(stderr, "add_param %s: %s\n", a, mxp_last_error());
      return 1;
    }
  }
  fclose(f);
  CHECK(mxp_plan_build(plan));

  mxp_engine_options opt;
  memset(&opt, 0, sizeof opt);
  opt.ring_slots = 4;
  opt.slot_bytes = 1u << 20;
  opt.reader_threads = 2;
  opt.streams = 2;
  CHECK(mxp_engine_create(&opt, &eng));

  const int64_t n = mxp_plan_param_count(plan);
  void** dst = (void**)calloc((size_t)n, sizeof(void*));
  uint64_t* sizes = (uint64_t*)calloc((size_t)n, sizeof(uint64_t));
  for (int64_t i = 0; i < n; ++i) {
    mxp_param_info pi;
    CHECK(mxp_plan_param_info(plan, i, &pi));
    sizes[i] = pi.nbytes;
    if (hipMalloc(&dst[i], pi.nbytes ? pi.nbytes : 16) != hipSuccess) { fprintf(stderr, "hipMalloc failed\n"); return 1; }
  }
  mxp_exec_stats st;
  CHECK(mxp_execute(eng, plan, dst, &st));
  uint32_t* sums = (uint32_t*)calloc((size_t)n, sizeof(uint32_t));
  uint8_t* dig = (uint8_t*)calloc((size_t)n, 16);
  CHECK(mxp_plan_checksums(eng, plan, sums, n));
  CHECK(mxp_digest(eng, (const void* const*)dst, sizes, n, dig, NULL, NULL));
  for (int64_t i = 0; i < n; ++i) {
    mxp_param_info pi;
    CHECK(mxp_plan_param_info(plan, i, &pi));
    printf("%s %llu %08x ", pi.name, (unsigned long long)pi.nbytes, sums[i]);
    for (int k = 0; k < 16; ++k) printf("%02x", dig[16 * i + k]);
    printf("\n");
  }
  fprintf(stderr, "placed %llu bytes in %llu chunks, %llu launches\n", (unsigned long long)st.placed_bytes,
          (unsigned long long)st.n_chunks, (unsigned long long)st.n_launches);
  for (int64_t i = 0; i < n; ++i) (void)hipFree(dst[i]);
  mxp_engine_destroy(eng);
  mxp_plan_destroy(plan);
  mxp_ckpt_close(ck);
  return 0;
}
