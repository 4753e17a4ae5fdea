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
// Every wavefront moves its own sub-tile and never waits for another one (no workgroup
// barrier on the data path): 64 or 128 source rows (i) x 128 source bytes (j).
//   1. global -> registers: lane = (row mod 8, 16-byte chunk); 8 (16 for 1-byte elements)
//      128-bit loads per lane, all issued before anything else; a wavefront load covers eight
//      whole 128-byte lines.
//   2. registers -> LDS, row major, with the chunk index XOR-swizzled by the row group, one
//      ds_write_b128 per load, conflict free.
//   3. LDS -> registers: a lane owns a dword column (two bf16 / four fp8 columns) and reads it
//      down the V = 16 / elem_size rows that make one 16-byte destination chunk; the swizzle
//      makes the 32 lanes of an LDS cycle hit 32 different banks.  Bytes are regrouped with
//      v_perm_b32.
//   4. registers -> global: eight consecutive lanes write one whole 128-byte destination
//      line, so a wavefront store is eight full lines.  The checksum is taken from the
//      registers being stored.
// HBM traffic: every element read once and written once, in whole lines.
//
// A workgroup is eight such wavefronts, waves_i of them side by side along i (so the
// workgroup writes runs of up to 1 KiB per destination row) and the rest along j; the host
// picks waves_i from the extent of i.  The workgroup only exists to share an LDS allocation
// and one checksum atomic.  Measured on 2-byte elements: 16384 x 16384 5.4 TB/s, sixteen
// 4096 x 4096 matrices 6.2 TB/s (a plain copy of the same bytes through place_kernel: 5.7);
// the rate depends on the two pitches.  When the destination pitch is the larger one, the host
// asks for two wavefronts along i and bands of eight tiles along j (65536 x 4096: 5.3 against
// 4.6 TB/s in plain order; 32768 x 8192: 5.5 against 4.8); otherwise eight wavefronts along i
// and plain order are best (4096 x 65536: 5.8 TB/s).  Padding a power-of-two source pitch by
// 384 bytes lifts 16384 x 16384 to 6.0 TB/s: the loss is in how the strided source lines fall
// on the memory channels, which a caller controls and this kernel does not.
#include "mxp_device.h"

namespace mxp {

namespace {

__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o, 64);
  return v;
}

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

// Same checksum algebra as place_kernel (see mxp_kernels.hip).
struct Csum {
  uint32_t P = 0, Q = 0, R = 0;
  __device__ __forceinline__ void add16(const uint4& x, uint32_t i) {
    uint32_t s0 = __builtin_amdgcn_udot4(x.x, 0x01010101u, 0u, false);
    s0 = __builtin_amdgcn_udot4(x.y, 0x01010101u, s0, false);
    s0 = __builtin_amdgcn_udot4(x.z, 0x01010101u, s0, false);
    s0 = __builtin_amdgcn_udot4(x.w, 0x01010101u, s0, false);
    R = __builtin_amdgcn_udot4(x.x, 0x03020100u, R, false);
    R = __builtin_amdgcn_udot4(x.y, 0x07060504u, R, false);
    R = __builtin_amdgcn_udot4(x.z, 0x0b0a0908u, R, false);
    R = __builtin_amdgcn_udot4(x.w, 0x0f0e0d0cu, R, false);
    Q += s0;
    P += i * s0;
  }
  __device__ __forceinline__ void add_byte(uint32_t b, uint32_t i) {
    Q += b;
    P += i * b;
  }
  __device__ __forceinline__ uint32_t fold() const { return kKnuth * (P + R) + Q; }
};

constexpr int kWaves = kTransposeWaves;
constexpr int kThreads = kWaves * 64;

template <int ES>
struct Sub {
  static constexpr int kLoads = transpose_sub_rows(ES) / 8;  // 16-byte loads per lane
  static constexpr int RI = transpose_sub_rows(ES);          // rows (i) of a wavefront's sub-tile
  static constexpr int TJ = 128 / ES;                        // columns (j): 128 source bytes per row
  static constexpr int V = 16 / ES;                          // rows gathered into one 16-byte destination chunk
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

// Destination chunk p (0 <= p < CPR) out of the NW gathered dwords: element p of every row.
template <int ES, int P>
__device__ __forceinline__ uint4 regroup(const uint32_t (&w)[Sub<ES>::NW]) {
  if constexpr (ES >= 4) {
    return make_uint4(w[0], w[1], w[2], w[3]);
  } else if constexpr (ES == 2) {
    constexpr uint32_t sel = P == 0 ? 0x05040100u : 0x07060302u;
    return make_uint4(__builtin_amdgcn_perm(w[1], w[0], sel), __builtin_amdgcn_perm(w[3], w[2], sel),
                      __builtin_amdgcn_perm(w[5], w[4], sel), __builtin_amdgcn_perm(w[7], w[6], sel));
  } else {
    constexpr uint32_t sel = (uint32_t)P | ((uint32_t)(4 + P) << 8) | 0x0c0c0000u;  // byte P of both operands, low half
    uint32_t o[4];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t a = __builtin_amdgcn_perm(w[4 * d + 1], w[4 * d], sel);
      const uint32_t b = __builtin_amdgcn_perm(w[4 * d + 3], w[4 * d + 2], sel);
      o[d] = a | (b << 16);
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
  }
}

template <int ES, bool FULL>
__device__ __forceinline__ void store_chunk(const uint4& v, uint32_t jj, uint32_t ci, uint8_t* __restrict__ dp, uint32_t ni,
                                            uint32_t nj, uint64_t dj_bytes, uint32_t csum_base, bool vec_dst, Csum& cs) {
  using S = Sub<ES>;
  const uint64_t off = (uint64_t)jj * dj_bytes + ci * 16u;
  const uint32_t pos = csum_base + (uint32_t)off;
  if constexpr (FULL) {
    st16_nt(dp + off, v);
    cs.add16(v, pos);
  } else {
    if (jj < nj && ci * S::V < ni) {
      const uint32_t n = min((uint32_t)S::V, ni - ci * S::V);
      if (vec_dst && n == (uint32_t)S::V) {
        st16_nt(dp + off, v);
        cs.add16(v, pos);
      } else {
        for (uint32_t e = 0; e < n * ES; ++e) {
          const uint32_t byte = get_byte(v, e);
          dp[off + e] = (uint8_t)byte;
          cs.add_byte(byte, pos + e);
        }
      }
    }
  }
}

// Moves one sub-tile.  FULL: the sub-tile is complete and both sides allow 16-byte accesses,
// so nothing is predicated.  Otherwise rows / columns beyond (ni, nj) are skipped and chunks
// that cannot use a 16-byte access are moved byte-wise.
template <int ES, bool FULL>
__device__ __forceinline__ void move_subtile(const uint8_t* __restrict__ sp, uint8_t* __restrict__ dp, uint32_t ni,
                                             uint32_t nj, uint64_t si_bytes, uint64_t dj_bytes, uint32_t csum_base,
                                             bool vec_src, bool vec_dst, uint8_t* lds, Csum& cs) {
  using S = Sub<ES>;
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
        if (row < ni && c * S::V < nj) {
          if (vec_src && c * S::V + S::V <= nj) {
            x[k] = ld16_nt(g);
          } else {
            const uint32_t n = min((uint32_t)S::V, nj - c * S::V) * ES;
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
    const uint32_t jj0 = a * (16u / ES) + dlo * S::CPR;
    store_chunk<ES, FULL>(regroup<ES, 0>(w), jj0, ci, dp, ni, nj, dj_bytes, csum_base, vec_dst, cs);
    if constexpr (S::CPR >= 2) store_chunk<ES, FULL>(regroup<ES, 1>(w), jj0 + 1, ci, dp, ni, nj, dj_bytes, csum_base, vec_dst, cs);
    if constexpr (S::CPR == 4) {
      store_chunk<ES, FULL>(regroup<ES, 2>(w), jj0 + 2, ci, dp, ni, nj, dj_bytes, csum_base, vec_dst, cs);
      store_chunk<ES, FULL>(regroup<ES, 3>(w), jj0 + 3, ci, dp, ni, nj, dj_bytes, csum_base, vec_dst, cs);
    }
  }
}

template <int ES>
__global__ __launch_bounds__(kThreads) void transpose_kernel(const uint8_t* __restrict__ src,
                                                              uint8_t* __restrict__ dst,
                                                              const TransposeDesc d,
                                                              uint32_t* __restrict__ sum_out) {
  using S = Sub<ES>;
  __shared__ __align__(16) uint8_t lds[kWaves * S::kLdsBytes];
  const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  Csum cs;
  // Linear tile index -> (batch, tile_j, tile_i), tile_i fastest.  Workgroup-uniform.
  const uint64_t per_batch = (uint64_t)d.tiles_i * d.tiles_j;
  uint64_t b = blockIdx.x / per_batch;
  const uint32_t within = (uint32_t)(blockIdx.x % per_batch);
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
  const uint32_t waves_j = (uint32_t)kWaves / d.waves_i;
  const uint64_t i0 = ((uint64_t)ti * d.waves_i + wave % d.waves_i) * S::RI;
  const uint64_t j0 = ((uint64_t)tj * waves_j + wave / d.waves_i) * S::TJ;
  if (i0 < d.ni && j0 < d.nj) {
    const uint32_t ni = (uint32_t)min((uint64_t)S::RI, d.ni - i0), nj = (uint32_t)min((uint64_t)S::TJ, d.nj - j0);
    const uint64_t d_el = d_off + j0 * d.dj + i0;
    const uint8_t* sp = src + (s_off + i0 * d.si + j0) * ES;
    uint8_t* dp = dst + d_el * ES;
    const uint32_t csum_base = (uint32_t)(d_el * ES) + d.csum_bias;
    uint8_t* my_lds = lds + wave * S::kLdsBytes;
    if (d.vec_src && d.vec_dst && ni == (uint32_t)S::RI && nj == (uint32_t)S::TJ)
      move_subtile<ES, true>(sp, dp, ni, nj, d.si * ES, d.dj * ES, csum_base, true, true, my_lds, cs);
    else
      move_subtile<ES, false>(sp, dp, ni, nj, d.si * ES, d.dj * ES, csum_base, d.vec_src != 0, d.vec_dst != 0, my_lds, cs);
  }

  if (sum_out) {
    // Each wavefront leaves its partial sum in the first dword of its own LDS region (its
    // data-path accesses to that region are complete in issue order).
    const uint32_t w = wave_sum_u32(cs.fold());
    if ((threadIdx.x & 63) == 0) *reinterpret_cast<uint32_t*>(lds + wave * S::kLdsBytes) = w;
    __syncthreads();
    if (threadIdx.x == 0) {
      uint32_t t = 0;
#pragma unroll
      for (int k = 0; k < kWaves; ++k) t += *reinterpret_cast<const uint32_t*>(lds + k * S::kLdsBytes);
      atomicAdd(sum_out, t);
    }
  }
}

}  // namespace

hipError_t launch_transpose(const void* src, void* dst, const TransposeDesc& d, int elem_size,
                            uint32_t* sum_out, hipStream_t stream) {
  if (d.n_tiles == 0) return hipSuccess;
  if (d.n_tiles > 0x7FFFFFFFull || d.waves_i == 0 || kWaves % d.waves_i || d.group_j == 0 ||
      (uint64_t)d.tiles_i * d.tiles_j > 0x7FFFFFFFull || (uint64_t)d.tiles_i * d.group_j > 0x7FFFFFFFull)
    return hipErrorInvalidValue;
  const dim3 grid((uint32_t)d.n_tiles), block(kThreads);
  const uint8_t* s = static_cast<const uint8_t*>(src);
  uint8_t* t = static_cast<uint8_t*>(dst);
  switch (elem_size) {
    case 1: hipLaunchKernelGGL(transpose_kernel<1>, grid, block, 0, stream, s, t, d, sum_out); break;
    case 2: hipLaunchKernelGGL(transpose_kernel<2>, grid, block, 0, stream, s, t, d, sum_out); break;
    case 4: hipLaunchKernelGGL(transpose_kernel<4>, grid, block, 0, stream, s, t, d, sum_out); break;
    case 8: hipLaunchKernelGGL(transpose_kernel<8>, grid, block, 0, stream, s, t, d, sum_out); break;
    default: return hipErrorInvalidValue;
  }
  return hipGetLastError();
}

}  // namespace mxp
