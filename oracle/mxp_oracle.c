/*
 * CPU oracle, C part.  TEST INFRASTRUCTURE ONLY: nothing in the product links or calls
 * this file; tests use it as the checker at sizes numpy is too slow for, and bench.py
 * times it as the CPU baseline.
 *
 * Each function restates one piece of the reference (ai-dynamo/modelexpress v0.5.0,
 * paths under modelexpress_client/python/):
 *   orc_checksum32        modelexpress/tensor_utils.py:27-44 (safe_checksum), one pass
 *   orc_digest_scalars    modelexpress/refit/reshard/verify.py:112-150 (tensor_digest)
 *   orc_cast_f32_bf16     torch copy_ at modelexpress_rl/train/engines/fsdp/adapter.py:203-206
 *                         and modelexpress/refit/reshard/receiver.py:964-971
 *   orc_copy2d            narrow(axis, r*n, n).contiguous() then dest.copy_(src)
 *                         (modelexpress/engines/vllm/refit/installer.py:317,419-424)
 *   orc_run_writes        the write loop of installer.py:419-424 over a resolved plan,
 *                         spread over host threads, with the checksum of each destination
 * It is pinned by tests/test_oracle_*.py against the numpy restatement, which in turn is
 * pinned against the reference's own test vectors, closed forms and brute force.
 */
#include <pthread.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define KNUTH 2654435761u

uint32_t orc_checksum32_at(const uint8_t* p, uint64_t n, uint64_t first_index) {
  uint32_t total = 0;
  uint32_t w = (uint32_t)first_index * KNUTH + 1u; /* weights advance by K per byte */
  for (uint64_t i = 0; i < n; ++i) {
    total += (uint32_t)p[i] * w;
    w += KNUTH;
  }
  return total;
}

uint32_t orc_checksum32(const uint8_t* p, uint64_t n) { return orc_checksum32_at(p, n, 0); }

/* out[7] = n, sum_rows, sum_rows_weighted, sum_tail, sum_tail_weighted, sum_ragged, n % 4 */
void orc_digest_scalars(const uint8_t* p, uint64_t n, uint64_t out[7]) {
  const uint64_t body_words = n / 4, rows = body_words / 1024;
  uint64_t a = 0, b = 0, at = 0, bt = 0, rg = 0;
  for (uint64_t r = 0; r < rows; ++r) {
    int64_t rs = 0;
    for (uint32_t j = 0; j < 1024; ++j) {
      int32_t w;
      memcpy(&w, p + 4 * (r * 1024 + j), 4);
      rs += w;
    }
    a += (uint64_t)rs;
    b += (uint64_t)rs * (r + 1);
  }
  const uint64_t tw = body_words - rows * 1024;
  for (uint64_t k = 0; k < tw; ++k) {
    int32_t w;
    memcpy(&w, p + 4 * (rows * 1024 + k), 4);
    at += (uint64_t)(int64_t)w;
    bt += (uint64_t)(int64_t)w * (k + 1);
  }
  for (uint64_t k = body_words * 4; k < n; ++k) rg += p[k];
  out[0] = n; out[1] = a; out[2] = b; out[3] = at; out[4] = bt; out[5] = rg; out[6] = n % 4;
}

static inline uint16_t bf16_bits(uint32_t u, uint16_t nan_bits) {
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return nan_bits;
  return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

void orc_cast_f32_bf16(const uint32_t* src, uint16_t* dst, uint64_t n, uint16_t nan_bits) {
  for (uint64_t i = 0; i < n; ++i) dst[i] = bf16_bits(src[i], nan_bits);
}

/* The other conversions of the same copy_ (receive side: refit/reshard/receiver.py:962-969).
 * Codes: 1 fp32->bf16, 2 bf16->fp32, 3 fp16->fp32, 4 fp32->fp16, 5 fp8-e4m3 -> bf16,
 * 6 fp16->bf16 and 7 bf16->fp16 (both through fp32). */
static inline uint16_t f8e4m3_to_bf16_bits(uint8_t c) {
  const uint16_t sign = (uint16_t)((c & 0x80u) << 8), e = (c >> 3) & 0xFu, m = c & 7u;
  if (e == 15u && m == 7u) return 0x7FC0u;
  if (e != 0u) return (uint16_t)(sign | ((e + 120u) << 7) | (m << 4));
  if (m == 0u) return sign;
  const uint16_t top = m >= 4u ? 2u : m >= 2u ? 1u : 0u;
  return (uint16_t)(sign | ((top + 118u) << 7) | ((m << (7u - top)) & 0x7Fu));
}

static inline uint32_t f16_to_f32_bits(uint16_t h) {
  const uint32_t sign = ((uint32_t)h & 0x8000u) << 16, e = (h >> 10) & 0x1Fu, m = h & 0x3FFu;
  if (e == 31u) return sign | 0x7F800000u | (m << 13) | (m ? 0x400000u : 0u);
  if (e != 0u) return sign | ((e + 112u) << 23) | (m << 13);
  if (m == 0u) return sign;
  uint32_t top = 9;
  while (!(m >> top)) --top;
  return sign | ((top + 103u) << 23) | ((m << (23u - top)) & 0x7FFFFFu);
}

static inline uint16_t f32_to_f16_bits(uint32_t u) {
  const uint32_t sign = (u >> 16) & 0x8000u, a = u & 0x7FFFFFFFu;
  if (a > 0x7F800000u) return (uint16_t)(sign | 0x7E00u | ((a >> 13) & 0x3FFu));
  if (a >= 0x38800000u) {
    const uint32_t r = a - 0x38000000u;
    uint32_t h = (r + 0xFFFu + ((r >> 13) & 1u)) >> 13;
    if (h > 0x7C00u) h = 0x7C00u;
    return (uint16_t)(sign | h);
  }
  const uint32_t e = a >> 23, m = (a & 0x7FFFFFu) | 0x800000u;
  uint32_t shift = 126u - e;
  if (shift > 25u) shift = 25u;
  const uint32_t q = m >> shift, rem = m & ((1u << shift) - 1u), half = 1u << (shift - 1u);
  return (uint16_t)(sign | (q + ((rem > half) || (rem == half && (q & 1u)))));
}

/* n elements; returns nothing, dst holds the converted elements */
void orc_cast(uint32_t code, const void* src, void* dst, uint64_t n, uint16_t nan_bits) {
  uint64_t i;
  switch (code) {
    case 1: orc_cast_f32_bf16((const uint32_t*)src, (uint16_t*)dst, n, nan_bits); break;
    case 2: for (i = 0; i < n; ++i) ((uint32_t*)dst)[i] = (uint32_t)((const uint16_t*)src)[i] << 16; break;
    case 3: for (i = 0; i < n; ++i) ((uint32_t*)dst)[i] = f16_to_f32_bits(((const uint16_t*)src)[i]); break;
    case 4: for (i = 0; i < n; ++i) ((uint16_t*)dst)[i] = f32_to_f16_bits(((const uint32_t*)src)[i]); break;
    case 5: for (i = 0; i < n; ++i) ((uint16_t*)dst)[i] = f8e4m3_to_bf16_bits(((const uint8_t*)src)[i]); break;
    case 6: for (i = 0; i < n; ++i) ((uint16_t*)dst)[i] = bf16_bits(f16_to_f32_bits(((const uint16_t*)src)[i]), nan_bits); break;
    case 7: for (i = 0; i < n; ++i) ((uint16_t*)dst)[i] = f32_to_f16_bits((uint32_t)((const uint16_t*)src)[i] << 16); break;
    default: break;
  }
}

void orc_copy2d(const uint8_t* src, uint64_t src_pitch, uint8_t* dst, uint64_t dst_pitch, uint64_t rows,
                uint64_t row_bytes) {
  for (uint64_t r = 0; r < rows; ++r) memcpy(dst + r * dst_pitch, src + r * src_pitch, row_bytes);
}

/* One resolved write: a pitched box from a source address to a destination parameter. */
typedef struct orc_write {
  const uint8_t* src;  /* first byte of the box in the (memory-mapped) checkpoint */
  uint8_t* dst;        /* first byte of the box in the destination parameter */
  uint64_t src_pitch, dst_pitch, rows, row_bytes; /* row_bytes in destination bytes */
  uint64_t dst_index;  /* byte offset of dst inside its parameter (checksum position) */
  uint32_t param;      /* which checksum accumulator */
  uint32_t cast;       /* 0 copy, else a conversion code of orc_cast */
} orc_write;

typedef struct {
  const orc_write* w;
  uint64_t n_writes;
  uint32_t* sums; /* per thread: n_params accumulators */
  uint64_t n_params;
  volatile uint64_t* next;
  uint16_t nan_bits;
} orc_job;

static void run_one(const orc_write* w, uint32_t* sums, uint16_t nan_bits) {
  for (uint64_t r = 0; r < w->rows; ++r) {
    const uint8_t* s = w->src + r * w->src_pitch;
    uint8_t* d = w->dst + r * w->dst_pitch;
    if (w->cast) orc_cast(w->cast, s, d, w->row_bytes / ((w->cast == 2 || w->cast == 3) ? 4 : 2), nan_bits);
    else memcpy(d, s, w->row_bytes);
    sums[w->param] += orc_checksum32_at(d, w->row_bytes, w->dst_index + r * w->dst_pitch);
  }
}

static void* worker(void* arg) {
  orc_job* j = (orc_job*)arg;
  for (;;) {
    const uint64_t k = __atomic_fetch_add(j->next, 1, __ATOMIC_RELAXED);
    if (k >= j->n_writes) break;
    run_one(&j->w[k], j->sums, j->nan_bits);
  }
  return NULL;
}

/* Executes `n_writes` writes on `threads` host threads; sums_out[p] receives the
 * checksum of everything written into parameter p (complete when the writes tile it). */
int orc_run_writes(const orc_write* w, uint64_t n_writes, uint64_t n_params, uint32_t* sums_out, int threads,
                   uint16_t nan_bits) {
  if (threads < 1) threads = 1;
  if (threads > 256) threads = 256;
  volatile uint64_t next = 0;
  pthread_t tid[256];
  orc_job jobs[256];
  uint32_t* all = (uint32_t*)calloc((size_t)threads * (n_params ? n_params : 1), sizeof(uint32_t));
  if (!all) return -1;
  for (int t = 0; t < threads; ++t) {
    jobs[t].w = w; jobs[t].n_writes = n_writes; jobs[t].sums = all + (size_t)t * n_params;
    jobs[t].n_params = n_params; jobs[t].next = &next; jobs[t].nan_bits = nan_bits;
    if (pthread_create(&tid[t], NULL, worker, &jobs[t]) != 0) { threads = t; break; }
  }
  for (int t = 0; t < threads; ++t) pthread_join(tid[t], NULL);
  for (uint64_t p = 0; p < n_params; ++p) {
    uint32_t s = 0;
    for (int t = 0; t < threads; ++t) s += all[(size_t)t * n_params + p];
    sums_out[p] = s;
  }
  free(all);
  return 0;
}
