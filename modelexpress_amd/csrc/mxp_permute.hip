// Batched LDS transpose: dst = src.permute(...).contiguous() when the permutation moves the
// source's contiguous dimension away from the innermost position.
//
// Reference call sites: the MLA absorbed weights  W_UK_T = w_uk.permute(1, 2, 0)
// (modelexpress/engines/vllm/refit/receiver.py:252-261) and permuted box views
// (modelexpress/refit/reshard/slice_plan.py:166-220; tests/test_reshard_refit_slice_plan.py:155-197).
// Permutations that keep the innermost dimension (W_UV = w_uv.transpose(0, 1)) are row
// gathers and go through place_kernel instead.
//
// Naming: "i" is the destination's innermost dimension (strided in the source), "j" the
// source's innermost dimension (strided in the destination); every other dimension is a
// batch index.
//
// The element type may change on the way (OP: one of the conversions of mxp_convert.h), as in
// dest.copy_(src.t()) across dtypes (modelexpress/refit/reshard/receiver.py:962-969) or W_UK_T
// taken from an fp8 kv_b_proj: the conversion happens in registers between steps 3 and 4, so
// a converting transpose reads every source byte once and writes every destination byte once.
//
// Every wavefront moves its own sub-tile and never waits for another one (no workgroup
// barrier on the data path): 64 source rows (i; 128 for 1-byte destination elements) x 128
// source bytes (j).
//   1. global -> registers: lane = (row mod 8, 16-byte chunk); 8 (or 16) 128-bit loads per
//      lane, all issued before anything else; a wavefront load covers eight whole 128-byte lines.
//   2. registers -> LDS, row major, with the chunk index XOR-swizzled by the row group, one
//      ds_write_b128 per load, conflict free.
//   3. LDS -> registers: a lane owns a dword column (two bf16 / four fp8 columns) and reads it
//      down the V = 16 / (destination element size) rows that make one 16-byte destination
//      chunk; the swizzle makes the 32 lanes of an LDS cycle hit 32 different banks.  Bytes are
//      regrouped with v_perm_b32 and converted.
//   4. registers -> global: eight consecutive lanes write one whole 128-byte destination
//      line, so a wavefront store is eight full lines.  The checksum is taken from the
//      registers being stored.
// HBM traffic: every element read once and written once, in whole lines.
//
// A workgroup is up to eight such wavefronts, waves_i of them side by side along i (so the
// workgroup writes runs of up to 1 KiB per destination row) and the rest along j; the host
// picks both numbers from the extents (fewer wavefronts per workgroup when the launch is small).
// The workgroup only exists to share an LDS allocation and one checksum atomic.  Many
// transposes of one element type run as one launch (transpose_batch_kernel).  Measured on 2-byte elements: 16384 x 16384 5.4 TB/s, sixteen
// 4096 x 4096 matrices 6.2 TB/s (a plain copy of the same bytes through place_kernel: 5.7);
// the rate depends on the two pitches.  When the destination pitch is the larger one, the host
// asks for two wavefronts along i and bands of eight tiles along j (65536 x 4096: 5.3 against
// 4.6 TB/s in plain order; 32768 x 8192: 5.5 against 4.8); otherwise eight wavefronts along i
// and plain order are best (4096 x 65536: 5.8 TB/s).  Padding a power-of-two source pitch by
// 384 bytes lifts 16384 x 16384 to 6.0 TB/s: the loss is in how the strided source lines fall
// on the memory channels, which a caller controls and this kernel does not.
#include "mxp_device.h"
#include <atomic>
#include "mxp_checksum.h"
#include "mxp_convert.h"

namespace mxp {

namespace {

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ uint4 ld16_nt(const uint8_t* p) {
  const u32x4 t = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return make_uint4(t.x, t.y, t.z, t.w);
}
__device__ __forceinline__ void st16_nt(uint8_t* p, const uint4& v) {
  u32x4 t;
  t.x = v.x; t.y = v.y; t.z = v.z; t.w = v.w;
  __builtin_nontemporal_store(t, reinterpret_cast<u32x4*>(p));
}

constexpr int kWaves = kTransposeWaves;
constexpr int kThreads = kWaves * 64;

// Output element size of a transpose that converts on the way (OP = kOpCopy: none).
constexpr int out_elem(int es, int op) { return op == kOpCopy ? es : (int)op_dst_elem((uint32_t)op); }

template <int ES, int OP>
struct Sub {
  static constexpr int EO = out_elem(ES, OP);                 // destination element size
  static constexpr int RI = transpose_sub_rows(EO);          // rows (i) of a wavefront's sub-tile
  static constexpr int kLoads = RI / 8;                      // 16-byte loads per lane
  static constexpr int TJ = 128 / ES;                        // columns (j): 128 source bytes per row
  static constexpr int VJ = 16 / ES;                         // source elements in one 16-byte chunk of a row
  static constexpr int V = 16 / EO;                          // rows gathered into one 16-byte destination chunk
  static constexpr int G = ES == 8 ? 8 : 4;                  // bytes per LDS read
  static constexpr int DPC = 16 / G;                         // LDS reads across one 16-byte source chunk
  static constexpr int CPR = G / ES;                         // destination rows fed by one LDS column
  static constexpr int NW = V * G / 4;                       // dwords a lane gathers per iteration
  static constexpr int NCI = RI / V;                         // 16-byte chunks per destination row
  static constexpr int RESTN = 64 / (8 * DPC);               // (chunk column, row group) pairs per iteration
  static constexpr int kIters = NCI / RESTN;
  static constexpr int kLdsBytes = RI * 128;
  static_assert(NCI % 8 == 0 && kIters * RESTN == NCI, "sub-tile does not divide over the wavefront");
  static_assert(kWaves * kLdsBytes <= 160 * 1024, "workgroup exceeds the LDS of a compute unit");
};

// Byte e of a 16-byte register value, without indexing memory (a dynamically indexed local
// array would be placed in LDS and cost occupancy).
__device__ __forceinline__ uint32_t get_byte(const uint4& v, uint32_t e) {
  const uint64_t lo = (uint64_t)v.x | ((uint64_t)v.y << 32), hi = (uint64_t)v.z | ((uint64_t)v.w << 32);
  return (uint32_t)(((e < 8u) ? lo : hi) >> ((e & 7u) * 8u)) & 0xFFu;
}
__device__ __forceinline__ void or_byte(uint4& v, uint32_t e, uint32_t byte) {
  const uint32_t s = byte << ((e & 3u) * 8u);
  v.x |= (e < 4u) ? s : 0u;
  v.y |= (e >= 4u && e < 8u) ? s : 0u;
  v.z |= (e >= 8u && e < 12u) ? s : 0u;
  v.w |= (e >= 12u) ? s : 0u;
}

// Destination chunk p (0 <= p < CPR) out of the NW gathered dwords: element p of every row,
// converted where the transpose converts.  Sixteen destination bytes hold V rows; the gathered
// source bytes for them are 16 (same size), 8 (widening) or 32 (narrowing).
template <int ES, int OP, int P>
__device__ __forceinline__ uint4 make_chunk(const uint32_t (&w)[Sub<ES, OP>::NW], uint32_t nan_bits) {
  constexpr uint32_t kHalf = P == 0 ? 0x05040100u : 0x07060302u;                     // halfword P of two dwords
  constexpr uint32_t kByte = (uint32_t)P | ((uint32_t)(4 + P) << 8) | 0x0c0c0000u;   // byte P of two dwords, low half
  if constexpr (OP == kOpCopy && ES >= 4) {
    return make_uint4(w[0], w[1], w[2], w[3]);
  } else if constexpr ((OP == kOpCopy || op_recodes16(OP)) && ES == 2) {
    const uint4 g = make_uint4(__builtin_amdgcn_perm(w[1], w[0], kHalf), __builtin_amdgcn_perm(w[3], w[2], kHalf),
                               __builtin_amdgcn_perm(w[5], w[4], kHalf), __builtin_amdgcn_perm(w[7], w[6], kHalf));
    if constexpr (OP == kOpCopy) return g;
    else return recode8<OP>(g, nan_bits);
  } else if constexpr (OP == kOpCopy && ES == 1) {
    uint32_t o[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t a = __builtin_amdgcn_perm(w[4 * d + 1], w[4 * d], kByte);
      const uint32_t b = __builtin_amdgcn_perm(w[4 * d + 3], w[4 * d + 2], kByte);
      o[d] = a | (b << 16);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
  } else if constexpr (op_narrows(OP)) {  // eight fp32 rows -> eight 16-bit elements
    static_assert(ES == 4, "narrowing transposes read 4-byte elements");
    const uint2 lo = narrow4<OP>(make_uint4(w[0], w[1], w[2], w[3]), nan_bits);
    const uint2 hi = narrow4<OP>(make_uint4(w[4], w[5], w[6], w[7]), nan_bits);
    return make_uint4(lo.x, lo.y, hi.x, hi.y);
  } else if constexpr (OP == kOpCastF8E4M3Bf16) {  // eight fp8 rows -> eight bf16
    static_assert(ES == 1, "fp8 source");
    uint2 g;
    g.x = __builtin_amdgcn_perm(w[1], w[0], kByte) | (__builtin_amdgcn_perm(w[3], w[2], kByte) << 16);
    g.y = __builtin_amdgcn_perm(w[5], w[4], kByte) | (__builtin_amdgcn_perm(w[7], w[6], kByte) << 16);
    return widen4<OP>(g);
  } else {  // four 16-bit rows -> four fp32
    static_assert(op_widens(OP) && ES == 2, "widening transposes read 2-byte elements");
    uint2 g;
    g.x = __builtin_amdgcn_perm(w[1], w[0], kHalf);
    g.y = __builtin_amdgcn_perm(w[3], w[2], kHalf);
    return widen4<OP>(g);
  }
}

template <int ES, int OP, bool FULL>
__device__ __forceinline__ void store_chunk(const uint4& v, uint32_t jj, uint32_t ci, uint8_t* __restrict__ dp, uint32_t ni,
                                            uint32_t nj, uint64_t dj_bytes, uint32_t csum_base, uint32_t align_dst, Csum& cs) {
  using S = Sub<ES, OP>;
  const uint64_t off = (uint64_t)jj * dj_bytes + ci * 16u;
  const uint32_t pos = csum_base + (uint32_t)off;
  if constexpr (FULL) {
    st16_nt(dp + off, v);
    cs.add16(v, pos);
  } else {
    if (jj < nj && ci * S::V < ni) {
      const uint32_t n = min((uint32_t)S::V, ni - ci * S::V);
      if (n == (uint32_t)S::V && align_dst >= 2u) {
        // a whole chunk: the widest stores the destination's alignment allows
        uint8_t* q = dp + off;
        if (align_dst >= 16u) {
          st16_nt(q, v);
        } else if (align_dst >= 8u) {
          *reinterpret_cast<uint2*>(q) = make_uint2(v.x, v.y);
          *reinterpret_cast<uint2*>(q + 8) = make_uint2(v.z, v.w);
        } else if (align_dst >= 4u) {
          *reinterpret_cast<uint32_t*>(q) = v.x;
          *reinterpret_cast<uint32_t*>(q + 4) = v.y;
          *reinterpret_cast<uint32_t*>(q + 8) = v.z;
          *reinterpret_cast<uint32_t*>(q + 12) = v.w;
        } else {
          const uint32_t w[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
          for (int h = 0; h < 8; ++h) *reinterpret_cast<uint16_t*>(q + 2 * h) = (uint16_t)(w[h >> 1] >> (16 * (h & 1)));
        }
        cs.add16(v, pos);
      } else {
        for (uint32_t e = 0; e < n * S::EO; ++e) {
          const uint32_t byte = get_byte(v, e);
          dp[off + e] = (uint8_t)byte;
          cs.add_byte(byte, pos + e);
        }
      }
    }
  }
}

// Moves one sub-tile.  FULL: the sub-tile is complete and both sides allow 16-byte accesses,
// so nothing is predicated.  Otherwise rows / columns beyond (ni, nj) are skipped, whole chunks
// move in pieces as wide as the side's alignment allows (8, 4 or 2 bytes) and ragged chunks
// byte-wise.
template <int ES, int OP, bool FULL>
__device__ __forceinline__ void move_subtile(const uint8_t* __restrict__ sp, uint8_t* __restrict__ dp, uint32_t ni,
                                             uint32_t nj, uint64_t si_bytes, uint64_t dj_bytes, uint32_t csum_base,
                                             uint32_t align_src, uint32_t align_dst, uint32_t nan_bits, uint8_t* lds,
                                             Csum& cs) {
  using S = Sub<ES, OP>;
  const uint32_t lane = threadIdx.x & 63u;
  {
    const uint32_t lrow = lane >> 3, c = lane & 7u;
    uint4 x[S::kLoads];
#pragma unroll
    for (int k = 0; k < S::kLoads; ++k) {
      const uint32_t row = (uint32_t)k * 8u + lrow;
      const uint8_t* g = sp + (uint64_t)row * si_bytes + c * 16u;
      if constexpr (FULL) {
        x[k] = ld16_nt(g);
      } else {
        x[k] = make_uint4(0, 0, 0, 0);
        if (row < ni && c * S::VJ < nj) {
          if (c * S::VJ + S::VJ <= nj && align_src >= 2u) {
            // a whole chunk: the widest loads the source's alignment allows
            if (align_src >= 16u) {
              x[k] = ld16_nt(g);
            } else if (align_src >= 8u) {
              const uint2 lo = *reinterpret_cast<const uint2*>(g), hi = *reinterpret_cast<const uint2*>(g + 8);
              x[k] = make_uint4(lo.x, lo.y, hi.x, hi.y);
            } else if (align_src >= 4u) {
              x[k] = make_uint4(*reinterpret_cast<const uint32_t*>(g), *reinterpret_cast<const uint32_t*>(g + 4),
                                *reinterpret_cast<const uint32_t*>(g + 8), *reinterpret_cast<const uint32_t*>(g + 12));
            } else {
              uint32_t w[4];
#pragma unroll
              for (int q = 0; q < 4; ++q)
                w[q] = (uint32_t)*reinterpret_cast<const uint16_t*>(g + 4 * q) |
                       ((uint32_t)*reinterpret_cast<const uint16_t*>(g + 4 * q + 2) << 16);
              x[k] = make_uint4(w[0], w[1], w[2], w[3]);
            }
          } else {
            const uint32_t n = min((uint32_t)S::VJ, nj - c * S::VJ) * ES;
            for (uint32_t e = 0; e < n; ++e) or_byte(x[k], e, g[e]);
          }
        }
      }
    }
#pragma unroll
    for (int k = 0; k < S::kLoads; ++k) {
      const uint32_t row = (uint32_t)k * 8u + lrow;
      const uint32_t f = (row / S::V) & 7u;
      *reinterpret_cast<uint4*>(lds + row * 128u + ((c ^ f) << 4)) = x[k];
    }
  }
  // Only this wavefront touches its LDS region and its LDS operations complete in issue
  // order: no barrier, the fence just stops the compiler from moving reads above the writes.
  __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
  __builtin_amdgcn_wave_barrier();

  const uint32_t ci_lo = lane & 7u, dlo = (lane >> 3) % S::DPC, rest = lane / (8u * S::DPC);
#pragma unroll
  for (int it = 0; it < S::kIters; ++it) {
    const uint32_t m = (uint32_t)it * S::RESTN + rest;
    const uint32_t a = m & 7u, ci = (m >> 3) * 8u + ci_lo;
    const uint8_t* l = lds + (ci * S::V) * 128u + ((a ^ ci_lo) << 4) + dlo * S::G;
    uint32_t w[S::NW];
#pragma unroll
    for (int k = 0; k < S::V; ++k) {
      if constexpr (S::G == 8) {
        const uint2 t = *reinterpret_cast<const uint2*>(l + k * 128);
        w[2 * k] = t.x;
        w[2 * k + 1] = t.y;
      } else {
        w[k] = *reinterpret_cast<const uint32_t*>(l + k * 128);
      }
    }
    const uint32_t jj0 = a * (uint32_t)S::VJ + dlo * S::CPR;
    store_chunk<ES, OP, FULL>(make_chunk<ES, OP, 0>(w, nan_bits), jj0, ci, dp, ni, nj, dj_bytes, csum_base, align_dst, cs);
    if constexpr (S::CPR >= 2)
      store_chunk<ES, OP, FULL>(make_chunk<ES, OP, 1>(w, nan_bits), jj0 + 1, ci, dp, ni, nj, dj_bytes, csum_base, align_dst, cs);
    if constexpr (S::CPR == 4) {
      store_chunk<ES, OP, FULL>(make_chunk<ES, OP, 2>(w, nan_bits), jj0 + 2, ci, dp, ni, nj, dj_bytes, csum_base, align_dst, cs);
      store_chunk<ES, OP, FULL>(make_chunk<ES, OP, 3>(w, nan_bits), jj0 + 3, ci, dp, ni, nj, dj_bytes, csum_base, align_dst, cs);
    }
  }
}

// One workgroup's share of transpose `d`: tile number `tile` of its n_tiles.
template <int ES, int OP>
__device__ __forceinline__ void transpose_tile(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                               const TransposeDesc& d, uint64_t tile, uint32_t nan_bits, uint8_t* lds,
                                               uint32_t wave, Csum& cs) {
  using S = Sub<ES, OP>;
  // Linear tile index -> (batch, tile_j, tile_i), tile_i fastest.  Workgroup-uniform.
  const uint64_t per_batch = (uint64_t)d.tiles_i * d.tiles_j;
  uint64_t b = tile / per_batch;
  const uint32_t within = (uint32_t)(tile % per_batch);
  // Inside a batch, tiles are visited in bands of group_j tiles along j: with group_j > 1,
  // consecutive workgroups read neighbouring lines of the same source rows.
  const uint32_t gj = d.group_j;
  const uint32_t band = within / (gj * d.tiles_i), in_band = within % (gj * d.tiles_i);
  const uint32_t band_w = min(gj, d.tiles_j - band * gj);
  const uint32_t tj = band * gj + in_band % band_w;
  const uint32_t ti = in_band / band_w;
  uint64_t s_off = 0, d_off = 0;  // element offsets of the batch
#pragma unroll
  for (int k = kMaxBatchDims - 1; k >= 0; --k) {
    const uint64_t n = d.batch_size[k];
    const uint64_t idx = b % n;
    b /= n;
    s_off += idx * d.batch_sstride[k];
    d_off += idx * d.batch_dstride[k];
  }
  const uint32_t waves_j = d.waves / d.waves_i;
  const uint64_t i0 = ((uint64_t)ti * d.waves_i + wave % d.waves_i) * S::RI;
  const uint64_t j0 = ((uint64_t)tj * waves_j + wave / d.waves_i) * S::TJ;
  if (i0 < d.ni && j0 < d.nj) {
    const uint32_t ni = (uint32_t)min((uint64_t)S::RI, d.ni - i0), nj = (uint32_t)min((uint64_t)S::TJ, d.nj - j0);
    const uint64_t d_el = d_off + j0 * d.dj + i0;
    const uint8_t* sp = src + (s_off + i0 * d.si + j0) * ES;
    uint8_t* dp = dst + d_el * S::EO;
    const uint32_t csum_base = (uint32_t)(d_el * S::EO) + d.csum_bias;
    uint8_t* my_lds = lds + wave * S::kLdsBytes;
    if (d.align_src >= 16u && d.align_dst >= 16u && ni == (uint32_t)S::RI && nj == (uint32_t)S::TJ)
      move_subtile<ES, OP, true>(sp, dp, ni, nj, d.si * ES, d.dj * S::EO, csum_base, 16u, 16u, nan_bits, my_lds, cs);
    else
      move_subtile<ES, OP, false>(sp, dp, ni, nj, d.si * ES, d.dj * S::EO, csum_base, d.align_src, d.align_dst, nan_bits,
                                  my_lds, cs);
  }
}

template <int ES, int OP>
__global__ __launch_bounds__(kThreads) void transpose_kernel(const uint8_t* __restrict__ src,
                                                              uint8_t* __restrict__ dst,
                                                              const TransposeDesc d, uint32_t nan_bits,
                                                              uint32_t* __restrict__ sum_out, Fan fan) {
  using S = Sub<ES, OP>;
  extern __shared__ __align__(16) uint8_t lds[];  // S::kLdsBytes per wavefront of the workgroup
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  Csum cs;
  transpose_tile<ES, OP>(src, dst, d, blockIdx.x, nan_bits, lds, wave, cs);

  if (sum_out) {
    // Each wavefront leaves its partial sum in the first dword of its own LDS region (its
    // data-path accesses to that region are complete in issue order).
    const uint32_t w = wave_sum_u32(cs.fold());
    if ((threadIdx.x & 63) == 0) *reinterpret_cast<uint32_t*>(lds + wave * S::kLdsBytes) = w;
    __syncthreads();
    if (threadIdx.x == 0) {
      uint32_t t = 0;
#pragma unroll
      for (int k = 0; k < kWaves; ++k)
        if ((uint32_t)k < d.waves) t += *reinterpret_cast<const uint32_t*>(lds + k * S::kLdsBytes);
      atomicAdd(&sum_out[(blockIdx.x & fan.mask) * fan.pitch], t);
    }
  }
}

// Many transposes of one element type in one launch: `items` is sorted by first_tile, and a
// workgroup finds its transpose by bisection (workgroup-uniform, scalar loads).
template <int ES, int OP>
__global__ __launch_bounds__(kThreads) void transpose_batch_kernel(const TransposeItem* __restrict__ items,
                                                                    uint32_t n_items, uint32_t nan_bits) {
  extern __shared__ __align__(16) uint8_t lds[];  // Sub<ES, OP>::kLdsBytes per wavefront of the workgroup
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  uint32_t lo = 0, hi = n_items;  // the last item with first_tile <= blockIdx.x
  while (hi - lo > 1) {
    const uint32_t mid = (lo + hi) >> 1;
    if (items[mid].first_tile <= (uint64_t)blockIdx.x) lo = mid;
    else hi = mid;
  }
  const TransposeItem& it = items[lo];
  Csum cs;
  transpose_tile<ES, OP>(it.src, it.dst, it.d, (uint64_t)blockIdx.x - it.first_tile, nan_bits, lds, wave, cs);
}


// ---- panel form ------------------------------------------------------------------------------
// The whole workgroup stages one tile of A = 2^a source rows (i) x C = 2^c 16-byte chunks (j) in LDS
// in the source's format, waits at a barrier, and writes the transposed tile: every lane issues its
// eight 16-byte loads first (a wavefront load covers whole rows or whole 1 KiB pieces of a row), the
// tile lands in LDS with the chunk index XOR-swizzled by the row group, and after the barrier a lane
// gathers the V = 16 / (destination element) rows of one destination chunk as dwords down one LDS
// column - 4 / (source element) destination rows per gather - regroups bytes with v_perm_b32,
// converts, and stores; consecutive lanes take consecutive chunks along i, so a wavefront store is one
// contiguous KiB of a destination row (or of several abutting rows).  A compute unit alternates
// between a read burst and a write burst of up to 128 KiB, like the placement kernel.
//
// Where it pays (measured against the wavefront-autonomous form on the same box): destinations whose
// rows are short and abut, so that a tile's output is one contiguous block (the MLA W_UK_T batch out of
// bf16: 0.346 against 0.383 ms); 2-byte matrices with both pitches of 32 KiB or more (16384 x 16384:
// 0.178 against 0.198 ms); widening transposes, two thirds of whose traffic is stores (8192 x 8192
// bf16 -> fp32 x 4: 0.267 against 0.317 ms).  Tall, wide and small-pitch matrices stay with the
// wavefront-autonomous form, which reads their rows better.  The host picks (mxp_engine.cpp).
// No edge handling: whole tiles, 16-byte aligned on both sides (panel_desc_ok).
template <int ES, int OP>
__device__ __forceinline__ void panel_tile(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst, const TransposeDesc& d,
                                           uint64_t tile, uint32_t nan_bits, uint8_t* lds, Csum& cs) {
  constexpr int EO = out_elem(ES, OP);
  constexpr uint32_t V = 16 / EO;        // source rows in one 16-byte destination chunk
  constexpr uint32_t CPR = 4 / ES;       // destination rows fed by one LDS dword column
  constexpr int KT = 2 * EO;             // gathers per lane: (columns / CPR) * (rows / V) / lanes
  static_assert(ES == 1 || ES == 2 || ES == 4, "panel transposes read 1-, 2- or 4-byte elements");
  static_assert(Sub<ES, OP>::NW == (int)V && Sub<ES, OP>::CPR == (int)CPR, "one dword per gathered row");
  const uint32_t a = d.panel_rows_log2, c = d.panel_chunks_log2;
  const uint32_t C = 1u << c, row_bytes = C << 4, sw = 7u;  // C >= 8
  const uint32_t threads = blockDim.x, t = threadIdx.x;
  const uint32_t nic_log2 = a - (uint32_t)__builtin_ctz(V), nic_mask = (1u << nic_log2) - 1u;
  // tile -> (batch, tile_j, tile_i), tile_i fastest; workgroup-uniform
  const uint64_t per_batch = (uint64_t)d.tiles_i * d.tiles_j;
  uint64_t b = tile / per_batch;
  const uint32_t within = (uint32_t)(tile % per_batch);
  const uint32_t ti = within % d.tiles_i, tj = within / d.tiles_i;
  uint64_t s_off = 0, d_off = 0;
#pragma unroll
  for (int k = kMaxBatchDims - 1; k >= 0; --k) {
    const uint64_t n = d.batch_size[k];
    const uint64_t idx = b % n;
    b /= n;
    s_off += idx * d.batch_sstride[k];
    d_off += idx * d.batch_dstride[k];
  }
  const uint64_t i0 = (uint64_t)ti << a, j0 = (uint64_t)tj * (row_bytes / ES);
  const uint64_t d_el = d_off + j0 * d.dj + i0;
  const uint8_t* sp = src + (s_off + i0 * d.si + j0) * ES;
  uint8_t* dp = dst + d_el * EO;
  const uint64_t si_b = d.si * ES, dj_b = d.dj * EO;
  const uint32_t csum_base = (uint32_t)(d_el * EO) + d.csum_bias;
  {
    uint4 x[kPanelLoads];
#pragma unroll
    for (uint32_t k = 0; k < kPanelLoads; ++k) {
      const uint32_t q = k * threads + t, row = q >> c, cc = q & (C - 1u);
      x[k] = ld16_nt(sp + (uint64_t)row * si_b + (cc << 4));
    }
#pragma unroll
    for (uint32_t k = 0; k < kPanelLoads; ++k) {
      const uint32_t q = k * threads + t, row = q >> c, cc = q & (C - 1u);
      *reinterpret_cast<uint4*>(lds + row * row_bytes + ((cc ^ ((row / V) & sw)) << 4)) = x[k];
    }
  }
  __syncthreads();
#pragma unroll
  for (int k = 0; k < KT; ++k) {
    const uint32_t q = (uint32_t)k * threads + t, ic = q & nic_mask, jg = q >> nic_log2;
    const uint32_t bytecol = jg << 2;
    const uint8_t* l = lds + (ic * V) * row_bytes + (((bytecol >> 4) ^ (ic & sw)) << 4) + (bytecol & 15u);
    uint32_t w[V];
#pragma unroll
    for (uint32_t kk = 0; kk < V; ++kk) w[kk] = *reinterpret_cast<const uint32_t*>(l + kk * row_bytes);
    const uint64_t off = (uint64_t)(jg * CPR) * dj_b + (ic << 4);
    const uint32_t pos = csum_base + (uint32_t)off;
    {
      const uint4 v = make_chunk<ES, OP, 0>(w, nan_bits);
      st16_nt(dp + off, v);
      cs.add16(v, pos);
    }
    if constexpr (CPR >= 2) {
      const uint4 v = make_chunk<ES, OP, 1>(w, nan_bits);
      st16_nt(dp + off + dj_b, v);
      cs.add16(v, pos + (uint32_t)dj_b);
    }
    if constexpr (CPR == 4) {
      const uint4 v2 = make_chunk<ES, OP, 2>(w, nan_bits);
      st16_nt(dp + off + 2 * dj_b, v2);
      cs.add16(v2, pos + (uint32_t)(2 * dj_b));
      const uint4 v3 = make_chunk<ES, OP, 3>(w, nan_bits);
      st16_nt(dp + off + 3 * dj_b, v3);
      cs.add16(v3, pos + (uint32_t)(3 * dj_b));
    }
  }
}

template <int ES, int OP>
__global__ __launch_bounds__(1024) void panel_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                      const TransposeDesc d, uint32_t nan_bits, uint32_t* __restrict__ sum_out,
                                                      Fan fan) {
  extern __shared__ __align__(16) uint8_t lds[];  // the staged tile
  __shared__ uint32_t wave_sums[16];
  Csum cs;
  panel_tile<ES, OP>(src, dst, d, blockIdx.x, nan_bits, lds, cs);
  if (sum_out) {
    const uint32_t w = wave_sum_u32(cs.fold());
    if ((threadIdx.x & 63) == 0) wave_sums[threadIdx.x >> 6] = w;
    __syncthreads();
    if (threadIdx.x == 0) {
      uint32_t t = 0;
      for (uint32_t k = 0; k < (blockDim.x >> 6); ++k) t += wave_sums[k];
      atomicAdd(&sum_out[(blockIdx.x & fan.mask) * fan.pitch], t);
    }
  }
}

// `uniform_tiles` != 0: every item has that many tiles and the same descriptor (the usual batch: one transpose
// of one shape per layer), which then travels as the kernel argument `common`; the item is a division away
// and only its two pointers are loaded.  A panel workgroup has a compute unit to itself, so what it waits for
// before its first data load is not hidden by other workgroups: the bisection and the 224-byte descriptor load
// cost the 61-layer MLA batch 8 % (0.378 against 0.350 ms).
template <int ES, int OP>
__global__ __launch_bounds__(1024) void panel_batch_kernel(const TransposeItem* __restrict__ items, uint32_t n_items,
                                                            uint32_t nan_bits, uint32_t uniform_tiles, const TransposeDesc common) {
  extern __shared__ __align__(16) uint8_t lds[];
  uint32_t lo = 0;
  if (uniform_tiles) {
    lo = blockIdx.x / uniform_tiles;
    const TransposeItem& it = items[lo];
    Csum cs;
    panel_tile<ES, OP>(it.src, it.dst, common, (uint64_t)(blockIdx.x - lo * uniform_tiles), nan_bits, lds, cs);
    return;
  } else {
    uint32_t hi = n_items;  // the last item with first_tile <= blockIdx.x
    while (hi - lo > 1) {
      const uint32_t mid = (lo + hi) >> 1;
      if (items[mid].first_tile <= (uint64_t)blockIdx.x) lo = mid;
      else hi = mid;
    }
  }
  const TransposeItem& it = items[lo];
  Csum cs;
  panel_tile<ES, OP>(it.src, it.dst, it.d, (uint64_t)blockIdx.x - it.first_tile, nan_bits, lds, cs);
}

// The same for kPanelArgItems items of a uniform batch at a time, whose pointers travel in the kernel argument
// block as well: a workgroup's two pointers are then loaded together with the descriptor when the wavefront
// starts, instead of after it (a table in memory is addressed through a pointer that is itself an argument).
struct PanelPtrTable {
  const uint8_t* src[kPanelArgItems];
  uint8_t* dst[kPanelArgItems];
};
template <int ES, int OP>
__global__ __launch_bounds__(1024) void panel_batch_args_kernel(const PanelPtrTable ptrs, uint32_t nan_bits, uint32_t uniform_tiles,
                                                                 const TransposeDesc common) {
  extern __shared__ __align__(16) uint8_t lds[];
  const uint32_t item = blockIdx.x / uniform_tiles;
  Csum cs;
  panel_tile<ES, OP>(ptrs.src[item], ptrs.dst[item], common, (uint64_t)(blockIdx.x - item * uniform_tiles), nan_bits, lds, cs);
}

}  // namespace

namespace {

// Calls f.template operator()<ES, OP>() for the kernel instance of (elem_size, op); false if there is none.
template <typename F>
bool with_instance(int elem_size, uint32_t op, F&& f) {
  if (op != kOpCopy && (int)op_src_bytes(op, op_dst_elem(op)) != elem_size) return false;
  switch (op) {
    case kOpCopy:
      switch (elem_size) {
        case 1: f.template operator()<1, kOpCopy>(); return true;
        case 2: f.template operator()<2, kOpCopy>(); return true;
        case 4: f.template operator()<4, kOpCopy>(); return true;
        case 8: f.template operator()<8, kOpCopy>(); return true;
        default: return false;
      }
    case kOpCastF32Bf16: f.template operator()<4, kOpCastF32Bf16>(); return true;
    case kOpCastF32F16: f.template operator()<4, kOpCastF32F16>(); return true;
    case kOpCastBf16F32: f.template operator()<2, kOpCastBf16F32>(); return true;
    case kOpCastF16F32: f.template operator()<2, kOpCastF16F32>(); return true;
    case kOpCastF8E4M3Bf16: f.template operator()<1, kOpCastF8E4M3Bf16>(); return true;
    case kOpCastF16Bf16: f.template operator()<2, kOpCastF16Bf16>(); return true;
    case kOpCastBf16F16: f.template operator()<2, kOpCastBf16F16>(); return true;
    default: return false;
  }
}

// A workgroup's LDS is sized by the wavefronts it is launched with (a 2-wavefront workgroup that
// reserved room for 8 left a compute unit with four resident wavefronts).  Above 64 KiB the
// kernel needs the attribute once per device.  The flag is kept per kernel: `Kernel` is the
// function itself, so every instantiation of the transpose kernels has its own bit mask.
template <auto Kernel>
hipError_t allow_lds(uint32_t bytes) {
  static std::atomic<uint64_t> allowed{0};  // bit per device
  constexpr auto kernel = Kernel;
  if (bytes <= 64u * 1024u) return hipSuccess;
  int dev = 0;
  if (hipError_t e = hipGetDevice(&dev); e != hipSuccess) return e;
  const uint64_t bit = 1ull << (dev & 63);
  if (allowed.load(std::memory_order_acquire) & bit) return hipSuccess;
  const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kernel), hipFuncAttributeMaxDynamicSharedMemorySize,
                                           kWaves * 16 * 1024);
  if (e == hipSuccess) allowed.fetch_or(bit, std::memory_order_release);
  return e;
}

struct LaunchOne {
  dim3 grid, block;
  hipStream_t stream;
  const uint8_t* s;
  uint8_t* t;
  const TransposeDesc& d;
  uint32_t nan_bits;
  uint32_t* sum_out;
  Fan fan;
  mutable hipError_t err = hipSuccess;
  template <int ES, int OP>
  void operator()() const {
    if (d.panel_rows_log2) {
      if constexpr (ES <= 4) {
        if (!panel_desc_ok(d, ES, out_elem(ES, OP)) || block.x * (uint32_t)kPanelLoads != (1u << (d.panel_rows_log2 + d.panel_chunks_log2))) {
          err = hipErrorInvalidValue;
          return;
        }
        const uint32_t lds = 16u << (d.panel_rows_log2 + d.panel_chunks_log2);
        err = allow_lds<panel_kernel<ES, OP>>(lds);
        if (err != hipSuccess) return;
        hipLaunchKernelGGL((panel_kernel<ES, OP>), grid, block, lds, stream, s, t, d, nan_bits, sum_out, fan);
      } else {
        err = hipErrorInvalidValue;
      }
      return;
    }
    const uint32_t lds = (block.x / 64u) * Sub<ES, OP>::kLdsBytes;
    err = allow_lds<transpose_kernel<ES, OP>>(lds);
    if (err != hipSuccess) return;
    hipLaunchKernelGGL((transpose_kernel<ES, OP>), grid, block, lds, stream, s, t, d, nan_bits, sum_out, fan);
  }
};

struct LaunchBatch {
  dim3 grid, block;
  hipStream_t stream;
  const TransposeItem* items;
  uint32_t n_items, nan_bits;
  uint32_t panel;  // 0, or panel_rows_log2 << 8 | panel_chunks_log2 of every item
  uint32_t uniform_tiles;  // != 0: every item has this many tiles and the descriptor `common`
  const TransposeDesc* common;
  const TransposeItem* items_host;  // may be null
  mutable hipError_t err = hipSuccess;
  template <int ES, int OP>
  void operator()() const {
    if (panel) {
      if constexpr (ES <= 4) {
        const uint32_t bits = (panel >> 8) + (panel & 0xFFu);
        if (bits < 9 || (16ull << bits) > kPanelMaxBytes || block.x * (uint32_t)kPanelLoads != (1u << bits)) {
          err = hipErrorInvalidValue;
          return;
        }
        const uint32_t lds = 16u << bits;
        if (uniform_tiles && items_host) {
          // kPanelArgItems items to a launch: a few microseconds between launches cost less than a pointer table in memory
          err = allow_lds<panel_batch_args_kernel<ES, OP>>(lds);
          if (err != hipSuccess) return;
          for (uint32_t first = 0; first < n_items; first += (uint32_t)kPanelArgItems) {
            const uint32_t n = n_items - first < (uint32_t)kPanelArgItems ? n_items - first : (uint32_t)kPanelArgItems;
            PanelPtrTable ptrs{};
            for (uint32_t k = 0; k < n; ++k) {
              ptrs.src[k] = items_host[first + k].src;
              ptrs.dst[k] = items_host[first + k].dst;
            }
            hipLaunchKernelGGL((panel_batch_args_kernel<ES, OP>), dim3(n * uniform_tiles), block, lds, stream, ptrs, nan_bits,
                               uniform_tiles, *common);
          }
          return;
        }
        err = allow_lds<panel_batch_kernel<ES, OP>>(lds);
        if (err != hipSuccess) return;
        hipLaunchKernelGGL((panel_batch_kernel<ES, OP>), grid, block, lds, stream, items, n_items, nan_bits, uniform_tiles,
                           common ? *common : TransposeDesc{});
      } else {
        err = hipErrorInvalidValue;
      }
      return;
    }
    const uint32_t lds = (block.x / 64u) * Sub<ES, OP>::kLdsBytes;
    err = allow_lds<transpose_batch_kernel<ES, OP>>(lds);
    if (err != hipSuccess) return;
    hipLaunchKernelGGL((transpose_batch_kernel<ES, OP>), grid, block, lds, stream, items, n_items, nan_bits);
  }
};

}  // namespace

hipError_t launch_transpose(const void* src, void* dst, const TransposeDesc& d, int elem_size, uint32_t op,
                            uint32_t nan_bits, uint32_t* sum_out, Fan fan, hipStream_t stream) {
  if (d.n_tiles == 0) return hipSuccess;
  if (!transpose_desc_ok(d)) return hipErrorInvalidValue;
  const LaunchOne one{dim3((uint32_t)d.n_tiles), dim3(d.waves * 64u), stream, static_cast<const uint8_t*>(src),
                      static_cast<uint8_t*>(dst), d, nan_bits, sum_out, fan};
  if (!with_instance(elem_size, op, one)) return hipErrorInvalidValue;
  if (one.err != hipSuccess) return one.err;
  return hipGetLastError();
}

hipError_t launch_transpose_batch(const TransposeItem* items_dev, uint32_t n_items, uint64_t total_tiles, uint32_t waves,
                                  int elem_size, uint32_t op, uint32_t nan_bits, hipStream_t stream, uint32_t panel,
                                  uint32_t uniform_tiles, const TransposeDesc* common, const TransposeItem* items_host) {
  if (n_items == 0 || total_tiles == 0) return hipSuccess;
  if (total_tiles > 0x7FFFFFFFull || waves == 0 || waves > (panel ? 16u : (uint32_t)kWaves) || (waves & (waves - 1)))
    return hipErrorInvalidValue;
  if (uniform_tiles && ((uint64_t)uniform_tiles * n_items != total_tiles || !common || common->n_tiles != uniform_tiles ||
                        !panel || panel != (common->panel_rows_log2 << 8 | common->panel_chunks_log2)))
    return hipErrorInvalidValue;
  const LaunchBatch many{dim3((uint32_t)total_tiles), dim3(waves * 64u), stream, items_dev, n_items, nan_bits, panel, uniform_tiles,
                         common, items_host};
  if (!with_instance(elem_size, op, many)) return hipErrorInvalidValue;
  if (many.err != hipSuccess) return many.err;
  return hipGetLastError();
}

}  // namespace mxp
