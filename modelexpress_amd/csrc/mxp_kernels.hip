// CDNA4 (gfx950) kernels for the weight-placement path.
//
// All of them are HBM-bound byte movers or reducers; none is a contraction, so there
// is no MFMA here.  What matters is: 128-bit accesses that are contiguous across the
// 64 lanes of a wavefront, thousands of workgroups per launch (256 CUs in 8 XCDs),
// and one launch for a whole batch of tensors instead of one launch per tensor.
//
//  place_kernel   pitched box copy / fp32->bf16 cast with the position-weighted
//                 checksum of every byte written fused in (reads each output byte's
//                 source once, writes it once: 2 x output bytes of traffic for a
//                 copy, 6 bytes per element for the cast)
//  digest_kernel  int32-word row sums for the blake2b-hashed tensor digest
//                 (reads each byte once)
//  checksum_kernel the checksum alone over existing buffers (reads each byte once)
//  fold_fan_kernel adds up the copies the accumulators are kept in (mxp_device.h: Fan)
#include "mxp_device.h"
#include "mxp_checksum.h"
#include "mxp_convert.h"
#include <atomic>
#include <type_traits>

namespace mxp {

// Checksum plus the tensor_digest sums of the bytes being stored (reference:
// modelexpress/refit/reshard/verify.py:112-150), for launches that verify what they place
// without a second pass over the finished buffers.  The digest reads a buffer as little-endian
// signed 32-bit words: whole 1024-word rows contribute sum(w) and sum(w) * (row + 1), the
// words after the last whole row sum(w) and sum(w * (k + 1)), the 1..3 bytes after the last
// whole word their unsigned sum - every term is linear in the stored bytes, so each lane adds
// the share of the bytes it stores, weighted by where they land in the destination buffer,
// and the sums wrap mod 2^64 exactly as the reference's int64 arithmetic does.
struct DigestAcc {
  Csum cs;
  unsigned long long S = 0, SW = 0, T = 0, TW = 0, RG = 0;
  // Whole-row words of this tile, kept as 32-bit sums until the tile is done: low halves
  // (unsigned) and high halves (signed) of the words apart, plain and weighted by the row's
  // distance from the tile's first row.  A lane adds at most 64 units of at most 4 words at
  // distances below 64, so nothing wraps; rows further away take the 64-bit route.
  uint32_t a_lo = 0, b_lo = 0;
  int32_t a_hi = 0, b_hi = 0;
  uint64_t row0 = 0;        // row (4 KiB of the buffer) the tile starts in
  uint64_t base = 0;        // position of the tile's first destination byte inside its buffer
  uint32_t base32 = 0;      // the 32-bit checksum position the callers count from
  uint64_t tail_byte0 = 0;  // first byte after the last whole row
  uint64_t body_end = 0;    // first ragged byte
  __device__ __forceinline__ void init(uint64_t buffer_bytes, uint64_t tile_pos, uint32_t tile_pos32) {
    base = tile_pos;
    base32 = tile_pos32;
    row0 = tile_pos >> 12;
    body_end = buffer_bytes & ~3ull;
    tail_byte0 = buffer_bytes / (4ull * kDigestRowWords) * (4ull * kDigestRowWords);
  }
  static_assert(kDigestRowWords == 1024, "rows are 4 KiB: the row of byte p is p >> 12");
  typedef short s16x2 __attribute__((ext_vector_type(2)));
  typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));
  static __device__ __forceinline__ uint32_t lo_add(uint32_t w, uint32_t acc) {
    u16x2 v;
    __builtin_memcpy(&v, &w, 4);
    const u16x2 one_zero = {1, 0};
    return __builtin_amdgcn_udot2(v, one_zero, acc, false);
  }
  static __device__ __forceinline__ int32_t hi_add(uint32_t w, int32_t acc) {
    s16x2 v;
    __builtin_memcpy(&v, &w, 4);
    const s16x2 zero_one = {0, 1};
    return __builtin_amdgcn_sdot2(v, zero_one, acc, false);
  }
  // Words after the last whole row: `sum` of the words and `ramp` = sum of word k times k.
  __device__ __forceinline__ void tail_words(long long sum, long long ramp, uint64_t p) {
    T += (unsigned long long)sum;
    TW += (unsigned long long)sum * (unsigned long long)(((p - tail_byte0) >> 2) + 1) + (unsigned long long)ramp;
  }
  // Whole-row words far from the tile's first row (pitched boxes with a large pitch).
  __device__ __forceinline__ void far_words(long long sum, uint64_t p) {
    S += (unsigned long long)sum;
    SW += (unsigned long long)sum * (unsigned long long)((p >> 12) + 1);
  }
  __device__ __forceinline__ void add16(const uint4& x, uint32_t i) {
    cs.add16(x, i);
    const uint64_t p = base + (uint32_t)(i - base32);
    const uint64_t dr = (p >> 12) - row0;
    if (p < tail_byte0 && dr < 64) {
      const uint32_t lo = lo_add(x.w, lo_add(x.z, lo_add(x.y, lo_add(x.x, 0u))));
      const int32_t hi = hi_add(x.w, hi_add(x.z, hi_add(x.y, hi_add(x.x, 0))));
      a_lo += lo;
      a_hi += hi;
      b_lo += lo * (uint32_t)dr;
      b_hi += hi * (int32_t)dr;
    } else {
      const long long a = (int32_t)x.x, b = (int32_t)x.y, c = (int32_t)x.z, d = (int32_t)x.w;
      if (p < tail_byte0) far_words(a + b + c + d, p);
      else tail_words(a + b + c + d, b + 2 * c + 3 * d, p);
    }
  }
  __device__ __forceinline__ void add8(uint32_t lo_w, uint32_t hi_w, uint32_t i) {
    cs.add8(lo_w, hi_w, i);
    const uint64_t p = base + (uint32_t)(i - base32);
    const uint64_t dr = (p >> 12) - row0;
    if (p < tail_byte0 && dr < 64) {
      const uint32_t lo = lo_add(hi_w, lo_add(lo_w, 0u));
      const int32_t hi = hi_add(hi_w, hi_add(lo_w, 0));
      a_lo += lo;
      a_hi += hi;
      b_lo += lo * (uint32_t)dr;
      b_hi += hi * (int32_t)dr;
    } else {
      const long long a = (int32_t)lo_w, b = (int32_t)hi_w;
      if (p < tail_byte0) far_words(a + b, p);
      else tail_words(a + b, b, p);
    }
  }
  // Folds the tile's 32-bit sums into the 64-bit ones; call once, after the last add.
  __device__ __forceinline__ void flush() {
    const long long s = (long long)a_hi * 65536 + (long long)a_lo;
    const long long sw = (long long)b_hi * 65536 + (long long)b_lo;
    S += (unsigned long long)s;
    SW += (unsigned long long)sw + (unsigned long long)s * (unsigned long long)(row0 + 1);
  }
  template <int UNIT>
  __device__ __forceinline__ void addn(uint32_t x, uint32_t i) {
    cs.add4(x, i);
    const uint64_t p = base + (uint32_t)(i - base32);
    if constexpr (UNIT == 4) {
      const uint64_t dr = (p >> 12) - row0;
      if (p < tail_byte0 && dr < 64) {
        const uint32_t lo = lo_add(x, 0u);
        const int32_t hi = hi_add(x, 0);
        a_lo += lo;
        a_hi += hi;
        b_lo += lo * (uint32_t)dr;
        b_hi += hi * (int32_t)dr;
      } else if (p < tail_byte0) {
        far_words((long long)(int32_t)x, p);
      } else {
        tail_words((long long)(int32_t)x, 0, p);
      }
    } else {  // part of a word, or ragged bytes: byte by byte
#pragma unroll
      for (int e = 0; e < UNIT; ++e) {
        const uint32_t b = (x >> (8 * e)) & 0xFFu;
        const uint64_t q = p + e;
        if (q >= body_end) {
          RG += b;
          continue;
        }
        const uint32_t j = (uint32_t)q & 3u;
        const long long v = j == 3u ? (long long)(int32_t)(b << 24) : (long long)(b << (8u * j));
        if (q < tail_byte0) far_words(v, q);
        else tail_words(v, 0, q & ~3ull);
      }
    }
  }
};

// 128-bit non-temporal accesses: every byte is touched exactly once, so nothing is worth
// keeping in L2 / Infinity Cache (measured: +3..4% over plain accesses on this copy).
// Loads carry no alignment promise (the `_u` types): the source of a box only has to be element
// aligned - a tensor's offset in a safetensors file is - while stores are always whole and aligned.
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef u32x4 u32x4_u __attribute__((aligned(1)));
__device__ __forceinline__ uint4 ld16(const uint8_t* p) {
  const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4_u*>(p));
  return make_uint4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void st16(uint8_t* p, const uint4& v) {
  u32x4 t;
  t.x = v.x; t.y = v.y; t.z = v.z; t.w = v.w;
  __builtin_nontemporal_store(t, reinterpret_cast<u32x4*>(p));
}
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef u32x2 u32x2_u __attribute__((aligned(1)));
typedef uint32_t u32_u __attribute__((aligned(1)));
typedef uint16_t u16_u __attribute__((aligned(1)));
__device__ __forceinline__ uint2 ld8(const uint8_t* p) {
  const u32x2 t = __builtin_nontemporal_load(reinterpret_cast<const u32x2_u*>(p));
  return make_uint2(t.x, t.y);
}
__device__ __forceinline__ void st8(uint8_t* p, const uint2& v) {
  u32x2 t;
  t.x = v.x; t.y = v.y;
  __builtin_nontemporal_store(t, reinterpret_cast<u32x2*>(p));
}

// One tile of one segment.  UNIT = destination bytes handled per lane access.
// Lanes walk the tile in flattened (row, unit) order, so neighbouring lanes touch
// neighbouring 16-byte units of the same row: every wavefront access is a run of
// contiguous 1 KiB pieces in both the source and the destination.
template <int OP, int UNIT, class ACC>
__device__ __forceinline__ void run_tile(const Seg& s, const uint8_t* __restrict__ src,
                                         uint8_t* __restrict__ dst, uint32_t csum_base,
                                         uint32_t n_units, uint32_t nan_bits, ACC& cs) {
  constexpr bool NARROW = op_narrows(OP), WIDEN = op_widens(OP);
  constexpr int SRC_UNIT = NARROW ? 2 * UNIT : WIDEN ? UNIT / 2 : UNIT;
  const uint32_t upr = s.units_per_row;
  const uint32_t magic = s.div_magic;
  const uint32_t sp = (uint32_t)s.src_pitch, dp = (uint32_t)s.dst_pitch;
  // Within a tile the row offsets fit 32 bits (the planner bounds rows_per_tile * pitch).
  auto locate = [&](uint32_t v, uint32_t& so, uint32_t& d_o) {
    const uint32_t row = (upr == 1u) ? v : __umulhi(v, magic);
    const uint32_t col = v - row * upr;
    so = row * sp + col * (uint32_t)SRC_UNIT;
    d_o = row * dp + col * (uint32_t)UNIT;
  };

  constexpr bool BATCHED = (NARROW && UNIT == 8) || (!NARROW && UNIT == 16);
  if constexpr (BATCHED) {
    // The wide paths.  A lane moves kPlaceBatch units: 16 bytes in and out for a copy, 16 in /
    // 8 out for a narrowing cast, 8 in / 16 out for a widening one, so a wavefront access is
    // 1 KiB (512 B on the narrow side) of contiguous memory.  A tile is at most one batch (the
    // host bounds it): a single pass in four phases that the scheduler may not interleave -
    // all addresses, all loads, all stores, then the checksum arithmetic - so the workgroup
    // presents the memory system with one burst of reads over a contiguous region followed by
    // one burst of writes over another.  Measured on the Llama rank: 256 lanes x 4 loads
    // 5.16 TB/s, 1024 x 8 5.98 TB/s; sixteen loads per lane are slower.
    constexpr int U = kPlaceBatch;
    using In = typename std::conditional<WIDEN, uint2, uint4>::type;
    using Out = typename std::conditional<NARROW, uint2, uint4>::type;
    auto load = [&](uint32_t off) -> In {
      if constexpr (WIDEN) return ld8(src + off);
      else return ld16(src + off);
    };
    auto convert = [&](const In& a) -> Out {
      if constexpr (NARROW) return narrow4<OP>(a, nan_bits);
      else if constexpr (WIDEN) return widen4<OP>(a);
      else if constexpr (op_recodes16(OP))
        return make_uint4(recode2<OP>(a.x, nan_bits), recode2<OP>(a.y, nan_bits), recode2<OP>(a.z, nan_bits),
                          recode2<OP>(a.w, nan_bits));
      else return a;
    };
    auto store = [&](uint32_t off, const Out& x) {
      if constexpr (OP == kOpChecksumOnly) return;
      else if constexpr (NARROW) st8(dst + off, x);
      else st16(dst + off, x);
    };
    auto sum = [&](uint32_t off, const Out& x) {
      if constexpr (NARROW) cs.add8(x.x, x.y, csum_base + off);
      else cs.add16(x, csum_base + off);
    };
    // Which unit of the tile a lane handles k-th.  A copy interleaves the wavefronts (load k of
    // the whole workgroup covers 16 KiB in a row); a read-only pass gives every wavefront its
    // own contiguous 8 KiB instead - measured 3-4% faster when nothing is written, 2-5% slower
    // when the same tile is also stored.
    auto unit_of = [&](int k) -> uint32_t {
      if constexpr (OP == kOpChecksumOnly) return (threadIdx.x >> 6) * (64u * U) + (uint32_t)k * 64u + (threadIdx.x & 63u);
      else return threadIdx.x + (uint32_t)k * kPlaceThreads;
    };
    uint32_t so[U], d_o[U];
    In a[U];
    if (n_units == (uint32_t)U * kPlaceThreads) {  // full tile: nothing is predicated
#pragma unroll
      for (int k = 0; k < U; ++k) locate(unit_of(k), so[k], d_o[k]);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int k = 0; k < U; ++k) a[k] = load(so[k]);
      __builtin_amdgcn_sched_barrier(0);
      Out x[U];
#pragma unroll
      for (int k = 0; k < U; ++k) {
        x[k] = convert(a[k]);
        store(d_o[k], x[k]);
      }
      if constexpr (OP != kOpChecksumOnly) __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int k = 0; k < U; ++k) sum(d_o[k], x[k]);
    } else {
      bool ok[U];
#pragma unroll
      for (int k = 0; k < U; ++k) {
        const uint32_t v = unit_of(k);
        ok[k] = v < n_units;
        locate(ok[k] ? v : 0u, so[k], d_o[k]);
      }
#pragma unroll
      for (int k = 0; k < U; ++k)
        if (ok[k]) a[k] = load(so[k]);
#pragma unroll
      for (int k = 0; k < U; ++k) {
        if (ok[k]) {
          const Out x = convert(a[k]);
          store(d_o[k], x);
          sum(d_o[k], x);
        }
      }
    }
  } else {
    // The narrow paths (boxes the 16-byte grid does not fit): one unit of at most four bytes per
    // lane and step, eight steps at a time - all their loads first, then the stores - so a lane
    // keeps eight loads in flight here too.
    auto load_raw = [&](uint32_t so) -> uint32_t {
      if constexpr (NARROW) {
        static_assert(UNIT == 2, "the element-wise cast path moves one element per lane");
        return *reinterpret_cast<const uint32_t*>(src + so);
      } else if constexpr (op_recodes16(OP)) {
        static_assert(UNIT == 4 || UNIT == 2, "two elements or one per lane");
        if constexpr (UNIT == 4) return *reinterpret_cast<const u32_u*>(src + so);
        else return *reinterpret_cast<const uint16_t*>(src + so);
      } else if constexpr (OP == kOpCastF8E4M3Bf16) {
        static_assert(UNIT == 4 || UNIT == 2, "two elements or one per lane");
        if constexpr (UNIT == 4) return *reinterpret_cast<const u16_u*>(src + so);
        else return src[so];
      } else if constexpr (WIDEN) {
        static_assert(UNIT == 4, "the element-wise cast path moves one element per lane");
        return *reinterpret_cast<const uint16_t*>(src + so);
      } else if constexpr (UNIT == 4) {
        return *reinterpret_cast<const u32_u*>(src + so);
      } else if constexpr (UNIT == 2) {
        return *reinterpret_cast<const u16_u*>(src + so);
      } else {
        return src[so];
      }
    };
    auto finish = [&](uint32_t raw, uint32_t d_o) {
      uint32_t x;
      if constexpr (NARROW) x = narrow1<OP>(raw, nan_bits);
      else if constexpr (op_recodes16(OP)) x = UNIT == 4 ? recode2<OP>(raw, nan_bits) : recode1<OP>(raw, nan_bits);
      else if constexpr (OP == kOpCastF8E4M3Bf16)
        x = UNIT == 4 ? (f8e4m3_to_bf16_bits(raw & 0xFFu) | (f8e4m3_to_bf16_bits(raw >> 8) << 16)) : f8e4m3_to_bf16_bits(raw);
      else if constexpr (WIDEN) x = widen1<OP>(raw);
      else x = raw;
      if constexpr (OP != kOpChecksumOnly) {
        if constexpr (UNIT == 4) *reinterpret_cast<uint32_t*>(dst + d_o) = x;
        else if constexpr (UNIT == 2) *reinterpret_cast<uint16_t*>(dst + d_o) = (uint16_t)x;
        else dst[d_o] = (uint8_t)x;
      }
      cs.template addn<UNIT>(x, csum_base + d_o);
    };
    constexpr uint32_t G = 8;
    for (uint32_t v0 = threadIdx.x; v0 < n_units; v0 += G * kPlaceThreads) {
      uint32_t so[G], d_o[G], raw[G];
#pragma unroll
      for (uint32_t k = 0; k < G; ++k) {
        const uint32_t v = v0 + k * kPlaceThreads;
        locate(v < n_units ? v : v0, so[k], d_o[k]);  // a step past the end re-reads the lane's first unit and drops it
      }
#pragma unroll
      for (uint32_t k = 0; k < G; ++k) raw[k] = load_raw(so[k]);
#pragma unroll
      for (uint32_t k = 0; k < G; ++k)
        if (v0 + k * kPlaceThreads < n_units) finish(raw[k], d_o[k]);
    }
  }
}

template <bool CHECKSUM_ONLY, bool DIGEST = false>
__device__ __forceinline__ void place_body(
    const Seg* __restrict__ segs, const WorkItem* __restrict__ work,
    const void* const* __restrict__ src_bases, void* const* __restrict__ dst_bases,
    uint32_t* __restrict__ sums, Fan fan, uint32_t nan_bits, const unsigned long long* __restrict__ dst_sizes = nullptr,
    unsigned long long* __restrict__ digest_sums = nullptr, uint32_t* __restrict__ zero = nullptr, uint32_t zero_words = 0) {
  // Housekeeping for the launch after this one: its accumulators are cleared here, a slice per
  // workgroup, so it needs no clearing launch of its own.
  for (uint64_t i = (uint64_t)blockIdx.x * kPlaceThreads + threadIdx.x; i < zero_words; i += (uint64_t)gridDim.x * kPlaceThreads) zero[i] = 0u;
  // This workgroup's copy of the accumulators.
  const uint32_t lane_first = (blockIdx.x & fan.mask) * fan.pitch;
  const WorkItem w = work[blockIdx.x];
  const Seg s = segs[w.seg];
  const uint32_t r0 = w.tile * s.rows_per_tile;
  const uint32_t nrows = min(s.rows - r0, s.rows_per_tile);
  const uint32_t n_units = nrows * s.units_per_row;
  const void* src_base = s.src_buf == kSrcIsDestination ? dst_bases[s.dst_buf] : src_bases[s.src_buf];
  const uint8_t* src = static_cast<const uint8_t*>(src_base) + s.src_off + (uint64_t)r0 * s.src_pitch;
  uint8_t* dst = nullptr;
  if (s.op != kOpChecksumOnly)
    dst = static_cast<uint8_t*>(dst_bases[s.dst_buf]) + s.dst_off + (uint64_t)r0 * s.dst_pitch;
  // Checksum positions are taken mod 2^32, exactly as the weights are.
  const uint32_t csum_base = (uint32_t)(s.dst_off + (uint64_t)r0 * s.dst_pitch) + s.csum_bias;

  typename std::conditional<DIGEST, DigestAcc, Csum>::type cs;
  if constexpr (DIGEST) cs.init(dst_sizes[s.dst_buf], s.dst_off + (uint64_t)r0 * s.dst_pitch, csum_base);
  if constexpr (CHECKSUM_ONLY) {
    switch (s.unit) {
      case 16u: run_tile<kOpChecksumOnly, 16>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
      case 4u: run_tile<kOpChecksumOnly, 4>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
      case 2u: run_tile<kOpChecksumOnly, 2>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
      case 1u: run_tile<kOpChecksumOnly, 1>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
      default: break;
    }
  } else
  switch (s.op * 32u + s.unit) {
    case kOpCopy * 32u + 16u: run_tile<kOpCopy, 16>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCopy * 32u + 4u: run_tile<kOpCopy, 4>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCopy * 32u + 2u: run_tile<kOpCopy, 2>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCopy * 32u + 1u: run_tile<kOpCopy, 1>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastF32Bf16 * 32u + 8u: run_tile<kOpCastF32Bf16, 8>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastF32Bf16 * 32u + 2u: run_tile<kOpCastF32Bf16, 2>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastF32F16 * 32u + 8u: run_tile<kOpCastF32F16, 8>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastF32F16 * 32u + 2u: run_tile<kOpCastF32F16, 2>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastBf16F32 * 32u + 16u: run_tile<kOpCastBf16F32, 16>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastBf16F32 * 32u + 4u: run_tile<kOpCastBf16F32, 4>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastF16F32 * 32u + 16u: run_tile<kOpCastF16F32, 16>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastF16F32 * 32u + 4u: run_tile<kOpCastF16F32, 4>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastF8E4M3Bf16 * 32u + 16u: run_tile<kOpCastF8E4M3Bf16, 16>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastF8E4M3Bf16 * 32u + 4u: run_tile<kOpCastF8E4M3Bf16, 4>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastF8E4M3Bf16 * 32u + 2u: run_tile<kOpCastF8E4M3Bf16, 2>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastF16Bf16 * 32u + 16u: run_tile<kOpCastF16Bf16, 16>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastF16Bf16 * 32u + 4u: run_tile<kOpCastF16Bf16, 4>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastF16Bf16 * 32u + 2u: run_tile<kOpCastF16Bf16, 2>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastBf16F16 * 32u + 16u: run_tile<kOpCastBf16F16, 16>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastBf16F16 * 32u + 4u: run_tile<kOpCastBf16F16, 4>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpCastBf16F16 * 32u + 2u: run_tile<kOpCastBf16F16, 2>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpChecksumOnly * 32u + 16u: run_tile<kOpChecksumOnly, 16>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpChecksumOnly * 32u + 4u: run_tile<kOpChecksumOnly, 4>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpChecksumOnly * 32u + 2u: run_tile<kOpChecksumOnly, 2>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    case kOpChecksumOnly * 32u + 1u: run_tile<kOpChecksumOnly, 1>(s, src, dst, csum_base, n_units, nan_bits, cs); break;
    default: break;  // the host validates (op, unit) before upload
  }

  if constexpr (DIGEST) {
    // five 64-bit sums and the checksum per workgroup: wavefront reductions, then one lane adds them up
    __shared__ unsigned long long dpart[kPlaceThreads / 64][5];
    __shared__ uint32_t part[kPlaceThreads / 64];
    cs.flush();
    const unsigned long long v0 = wave_sum_u64(cs.S), v1 = wave_sum_u64(cs.SW), v2 = wave_sum_u64(cs.T),
                             v3 = wave_sum_u64(cs.TW), v4 = wave_sum_u64(cs.RG);
    const uint32_t wsum = wave_sum_u32(cs.cs.fold());
    if ((threadIdx.x & 63) == 0) {
      unsigned long long* row = dpart[threadIdx.x >> 6];
      row[0] = v0; row[1] = v1; row[2] = v2; row[3] = v3; row[4] = v4;
      part[threadIdx.x >> 6] = wsum;
    }
    __syncthreads();
    if (threadIdx.x < 5) {
      unsigned long long t = 0;
#pragma unroll
      for (int k = 0; k < kPlaceThreads / 64; ++k) t += dpart[k][threadIdx.x];
      if (t) atomicAdd(&digest_sums[5ull * (lane_first + s.dst_buf) + threadIdx.x], t);
    } else if (threadIdx.x == 64 && s.csum_slot != 0xFFFFFFFFu) {
      uint32_t t = 0;
#pragma unroll
      for (int k = 0; k < kPlaceThreads / 64; ++k) t += part[k];
      atomicAdd(&sums[lane_first + s.csum_slot], t);
    }
  } else if (s.csum_slot != 0xFFFFFFFFu) {
    __shared__ uint32_t part[kPlaceThreads / 64];
    const uint32_t wsum = wave_sum_u32(cs.fold());
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = wsum;
    __syncthreads();
    if (threadIdx.x == 0) {
      uint32_t t = 0;
#pragma unroll
      for (int k = 0; k < kPlaceThreads / 64; ++k) t += part[k];
      atomicAdd(&sums[lane_first + s.csum_slot], t);
    }
  }
}

// Writes parameter bytes (copy, cast) and accumulates their checksums.
__global__ __launch_bounds__(kPlaceThreads) void place_kernel(
    const Seg* __restrict__ segs, const WorkItem* __restrict__ work,
    const void* const* __restrict__ src_bases, void* const* __restrict__ dst_bases,
    uint32_t* __restrict__ sums, Fan fan, uint32_t nan_bits, uint32_t* __restrict__ zero, uint32_t zero_words) {
  place_body<false>(segs, work, src_bases, dst_bases, sums, fan, nan_bits, nullptr, nullptr, zero, zero_words);
}

// place_kernel that also accumulates the tensor_digest sums of every destination buffer
// (five 64-bit words per buffer in `digest_sums`; `dst_sizes` holds the buffers' byte sizes).
__global__ __launch_bounds__(kPlaceThreads) void place_digest_kernel(
    const Seg* __restrict__ segs, const WorkItem* __restrict__ work,
    const void* const* __restrict__ src_bases, void* const* __restrict__ dst_bases,
    uint32_t* __restrict__ sums, Fan fan, uint32_t nan_bits, const unsigned long long* __restrict__ dst_sizes,
    unsigned long long* __restrict__ digest_sums, uint32_t* __restrict__ zero, uint32_t zero_words) {
  place_body<false, true>(segs, work, src_bases, dst_bases, sums, fan, nan_bits, dst_sizes, digest_sums, zero, zero_words);
}

// Read-only variant for batches made of checksum-only segments.
__global__ __launch_bounds__(kPlaceThreads) void checksum_kernel(
    const Seg* __restrict__ segs, const WorkItem* __restrict__ work,
    const void* const* __restrict__ src_bases, uint32_t* __restrict__ sums, Fan fan) {
  place_body<true>(segs, work, src_bases, nullptr, sums, fan, 0u);
}

// One workgroup per compute unit: a unit then alternates between one 128 KiB read burst and
// one 128 KiB write burst instead of mixing the two.  Two resident workgroups measured 3-5%
// slower on every configuration.  The limit is imposed with an otherwise unused dynamic LDS
// allocation of more than half a unit's LDS, which needs the attribute below once per device.
// A launch that only reads (checksum_kernel) is the other way round: two resident workgroups, one
// loading while the other adds up, read a tenth faster than one.
constexpr uint32_t kOnePerCu = 96 * 1024;
constexpr uint32_t kTwoPerCu = 48 * 1024;

hipError_t configure_place_kernels() {
  static std::atomic<uint64_t> configured{0};  // bit per device
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (configured.load(std::memory_order_acquire) & bit) return hipSuccess;
  hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(place_kernel),
                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)kOnePerCu);
  if (e == hipSuccess)
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(checksum_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kOnePerCu);
  if (e == hipSuccess)
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(place_digest_kernel),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)kOnePerCu);
  if (e == hipSuccess) configured.fetch_or(bit, std::memory_order_release);
  return e;
}

hipError_t launch_place(const Seg* segs_dev, const WorkItem* work_dev, uint32_t n_work,
                        const void* const* src_bases_dev, void* const* dst_bases_dev,
                        uint32_t* sums_dev, Fan fan, uint16_t nan_bits, hipStream_t stream, bool checksum_only,
                        uint32_t* zero_dev, uint32_t zero_words, bool widening_only) {
  if (n_work == 0) return hipSuccess;
  if (hipError_t e = configure_place_kernels(); e != hipSuccess) return e;
  const uint32_t lds_place = widening_only ? kTwoPerCu : kOnePerCu, lds_csum = kTwoPerCu;
  if (checksum_only) {
    hipLaunchKernelGGL(checksum_kernel, dim3(n_work), dim3(kPlaceThreads), lds_csum, stream, segs_dev, work_dev,
                       src_bases_dev, sums_dev, fan);
    return hipGetLastError();
  }
  hipLaunchKernelGGL(place_kernel, dim3(n_work), dim3(kPlaceThreads), lds_place, stream, segs_dev,
                     work_dev, src_bases_dev, dst_bases_dev, sums_dev, fan, (uint32_t)nan_bits, zero_dev, zero_words);
  return hipGetLastError();
}

hipError_t launch_place_digest(const Seg* segs_dev, const WorkItem* work_dev, uint32_t n_work,
                               const void* const* src_bases_dev, void* const* dst_bases_dev, uint32_t* sums_dev, Fan fan,
                               const unsigned long long* dst_sizes_dev, unsigned long long* digest_sums_dev,
                               uint16_t nan_bits, hipStream_t stream, uint32_t* zero_dev, uint32_t zero_words) {
  if (n_work == 0) return hipSuccess;
  if (hipError_t e = configure_place_kernels(); e != hipSuccess) return e;
  hipLaunchKernelGGL(place_digest_kernel, dim3(n_work), dim3(kPlaceThreads), kOnePerCu, stream, segs_dev, work_dev,
                     src_bases_dev, dst_bases_dev, sums_dev, fan, (uint32_t)nan_bits, dst_sizes_dev, digest_sums_dev, zero_dev, zero_words);
  return hipGetLastError();
}

// ---------------------------------------------------------------------------
// tensor_digest row sums (reference: modelexpress/refit/reshard/verify.py:112-150).
// Bytes are read as little-endian signed int32 words; whole 1024-word rows give
// sum_r rs[r] and sum_r rs[r]*(r+1); the words after the last whole row give
// sum_k t[k] and sum_k t[k]*(k+1); the 1..3 bytes after the last whole word are summed
// unsigned.  All sums wrap mod 2^64.  The index weight is applied per lane before any
// reduction (sum_r (sum_lane p)*(r+1) == sum_lane sum_r p*(r+1)), so there is a single
// reduction per workgroup.
// ---------------------------------------------------------------------------
template <bool ALIGNED16>
__device__ __forceinline__ void digest_rows(const uint8_t* __restrict__ p, uint64_t row_begin,
                                            uint64_t row_end, unsigned long long& A,
                                            unsigned long long& B) {
  const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  constexpr uint32_t kWaves = kDigestThreads / 64;
  auto lane_sum = [](const uint4& x) {
    return (long long)(int32_t)x.x + (long long)(int32_t)x.y + (long long)(int32_t)x.z + (long long)(int32_t)x.w;
  };
  if constexpr (ALIGNED16) {
    // Two rows per wavefront at a time: eight 16-byte loads per lane in flight, a 128 KiB
    // read burst per workgroup, the shape that measured fastest for the copy kernel.
    for (uint64_t r = row_begin + 2u * wave; r < row_end; r += 2u * kWaves) {
      const bool two = r + 1 < row_end;
      const uint8_t* row0 = p + r * (uint64_t)(kDigestRowWords * 4);
      uint4 x[8];
#pragma unroll
      for (int k = 0; k < 4; ++k) x[k] = ld16(row0 + 16u * (lane + 64u * k));
      if (two) {
#pragma unroll
        for (int k = 0; k < 4; ++k) x[4 + k] = ld16(row0 + kDigestRowWords * 4 + 16u * (lane + 64u * k));
      }
      long long a0 = 0, a1 = 0;
#pragma unroll
      for (int k = 0; k < 4; ++k) a0 += lane_sum(x[k]);
      if (two) {
#pragma unroll
        for (int k = 0; k < 4; ++k) a1 += lane_sum(x[4 + k]);
      }
      A += (unsigned long long)a0 + (unsigned long long)a1;
      B += (unsigned long long)a0 * (unsigned long long)(r + 1) + (unsigned long long)a1 * (unsigned long long)(r + 2);
    }
  } else {
    for (uint64_t r = row_begin + wave; r < row_end; r += kWaves) {
      const uint8_t* row = p + r * (uint64_t)(kDigestRowWords * 4);
      long long acc = 0;
#pragma unroll
      for (int k = 0; k < 16; ++k) {
        const uint8_t* b = row + 4u * (lane + 64u * k);
        const uint32_t u = (uint32_t)b[0] | ((uint32_t)b[1] << 8) | ((uint32_t)b[2] << 16) |
                           ((uint32_t)b[3] << 24);
        acc += (long long)(int32_t)u;
      }
      A += (unsigned long long)acc;
      B += (unsigned long long)acc * (unsigned long long)(r + 1);
    }
  }
}

__global__ __launch_bounds__(kDigestThreads) void digest_kernel(
    const DigestJob* __restrict__ jobs, uint32_t n_jobs, unsigned long long* __restrict__ out, Fan fan) {
  // Workgroup-uniform binary search for the job that owns this workgroup.
  uint32_t lo = 0, hi = n_jobs;
  while (hi - lo > 1) {
    const uint32_t mid = (lo + hi) >> 1;
    if (jobs[mid].first_block <= blockIdx.x) lo = mid; else hi = mid;
  }
  const DigestJob j = jobs[lo];
  const uint64_t blk = blockIdx.x - j.first_block;
  const uint64_t body_words = j.nbytes >> 2;
  const uint64_t rows = body_words / kDigestRowWords;
  const uint64_t n_blocks = rows ? (rows + kDigestRowsPerBlock - 1) / kDigestRowsPerBlock : 1;
  const uint64_t row_begin = blk * kDigestRowsPerBlock;
  const uint64_t row_end = min(rows, row_begin + kDigestRowsPerBlock);

  unsigned long long A = 0, B = 0, At = 0, Bt = 0, Rg = 0;
  if (row_begin < row_end) {
    if ((reinterpret_cast<uintptr_t>(j.ptr) & 15u) == 0)
      digest_rows<true>(j.ptr, row_begin, row_end, A, B);
    else
      digest_rows<false>(j.ptr, row_begin, row_end, A, B);
  }
  if (blk == n_blocks - 1) {
    const uint8_t* tail = j.ptr + rows * (uint64_t)(kDigestRowWords * 4);
    const uint32_t tw = (uint32_t)(body_words - rows * kDigestRowWords);
    for (uint32_t k = threadIdx.x; k < tw; k += kDigestThreads) {
      const uint8_t* b = tail + 4u * k;
      const uint32_t u = (uint32_t)b[0] | ((uint32_t)b[1] << 8) | ((uint32_t)b[2] << 16) |
                         ((uint32_t)b[3] << 24);
      const long long w = (long long)(int32_t)u;
      At += (unsigned long long)w;
      Bt += (unsigned long long)w * (unsigned long long)(k + 1);
    }
    if (threadIdx.x == 0) {
      const uint32_t rag = (uint32_t)(j.nbytes & 3u);
      for (uint32_t k = 0; k < rag; ++k) Rg += j.ptr[body_words * 4 + k];
    }
  }

  __shared__ unsigned long long part[kDigestThreads / 64][5];
  unsigned long long v[5] = {A, B, At, Bt, Rg};
#pragma unroll
  for (int q = 0; q < 5; ++q) {
    const unsigned long long wsum = wave_sum_u64(v[q]);
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6][q] = wsum;
  }
  __syncthreads();
  if (threadIdx.x < 5) {
    unsigned long long t = 0;
#pragma unroll
    for (int k = 0; k < kDigestThreads / 64; ++k) t += part[k][threadIdx.x];
    if (t) atomicAdd(&out[5ull * ((blockIdx.x & fan.mask) * fan.pitch) + j.out_slot + threadIdx.x], t);
  }
}

hipError_t launch_digest(const DigestJob* jobs_dev, uint32_t n_jobs, uint32_t n_blocks,
                         unsigned long long* out_dev, Fan fan, hipStream_t stream) {
  if (n_jobs == 0 || n_blocks == 0) return hipSuccess;
  hipLaunchKernelGGL(digest_kernel, dim3(n_blocks), dim3(kDigestThreads), 0, stream, jobs_dev,
                     n_jobs, out_dev, fan);
  return hipGetLastError();
}

// out[k] = sum over the fan's copies of element k (k < n); with `clear`, the elements read are
// left at zero for the next launch that adds to them.  One wavefront per element: lane l reads
// copy l (a fan has at most 64 copies), so the loads of an element are all in flight at once.
__device__ __forceinline__ uint32_t wave_sum(uint32_t v) { return wave_sum_u32(v); }
__device__ __forceinline__ unsigned long long wave_sum(unsigned long long v) { return wave_sum_u64(v); }

template <typename T>
__global__ __launch_bounds__(256) void fold_fan_kernel(T* __restrict__ fanned, Fan fan, uint32_t per_slot, uint64_t n,
                                                       T* __restrict__ out, bool clear) {
  static_assert(kFanLanes <= 64, "one lane of a wavefront per copy");
  const uint64_t lane_elems = (uint64_t)fan.pitch * per_slot;
  const uint32_t lane = threadIdx.x & 63u;
  for (uint64_t k = blockIdx.x * 4ull + (threadIdx.x >> 6); k < n; k += (uint64_t)gridDim.x * 4ull) {
    T v = 0;
    if (lane <= fan.mask) {
      T* p = fanned + lane * lane_elems + k;
      v = *p;
      if (clear) *p = 0;
    }
    v = wave_sum(v);
    if (lane == 0) out[k] = v;
  }
}

template <typename T>
hipError_t launch_fold_fan(T* fanned, Fan fan, uint32_t per_slot, uint64_t n, T* out, bool clear, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  const uint64_t blocks = (n + 3) / 4;
  hipLaunchKernelGGL(fold_fan_kernel<T>, dim3((uint32_t)(blocks > 16384 ? 16384 : blocks)), dim3(256), 0, stream, fanned, fan,
                     per_slot, n, out, clear);
  return hipGetLastError();
}
template hipError_t launch_fold_fan<uint32_t>(uint32_t*, Fan, uint32_t, uint64_t, uint32_t*, bool, hipStream_t);
template hipError_t launch_fold_fan<unsigned long long>(unsigned long long*, Fan, uint32_t, uint64_t, unsigned long long*, bool,
                                                        hipStream_t);

// Plain vector-store fill; used instead of a memset node so callers may capture it.
__global__ __launch_bounds__(256) void fill_u32_kernel(uint32_t* __restrict__ p, uint64_t n,
                                                       uint32_t value) {
  for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < n; i += (uint64_t)gridDim.x * 256ull)
    p[i] = value;
}

hipError_t launch_fill_u32(uint32_t* ptr, uint64_t n, uint32_t value, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  const uint64_t blocks = (n + 255) / 256;
  hipLaunchKernelGGL(fill_u32_kernel, dim3((uint32_t)(blocks > 4096 ? 4096 : blocks)), dim3(256), 0,
                     stream, ptr, n, value);
  return hipGetLastError();
}

// Table copy by plain 16-byte loads and stores (no memcpy node: callers may capture it).
__global__ __launch_bounds__(256) void copy_table_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, uint64_t n16) {
  for (uint64_t i = blockIdx.x * 256ull + threadIdx.x; i < n16; i += (uint64_t)gridDim.x * 256ull) dst[i] = src[i];
}

hipError_t launch_copy_table(void* dst, const void* src, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return hipSuccess;
  if ((bytes & 15u) || (reinterpret_cast<uintptr_t>(dst) & 15u) || (reinterpret_cast<uintptr_t>(src) & 15u)) return hipErrorInvalidValue;
  const uint64_t n16 = bytes / 16, blocks = (n16 + 255) / 256;
  hipLaunchKernelGGL(copy_table_kernel, dim3((uint32_t)(blocks > 1024 ? 1024 : blocks)), dim3(256), 0, stream,
                     static_cast<uint4*>(dst), static_cast<const uint4*>(src), n16);
  return hipGetLastError();
}

}  // namespace mxp
