// Batched LDS-tiled transpose: dst = src.permute(...).contiguous() when the permutation
// moves the source's contiguous dimension away from the innermost position.
//
// Reference call sites: the MLA absorbed weights  W_UK_T = w_uk.permute(1, 2, 0)
// (modelexpress/engines/vllm/refit/receiver.py:252-261) and permuted box views
// (modelexpress/refit/reshard/slice_plan.py:166-220; tests/test_reshard_refit_slice_plan.py:155-197).
// Permutations that keep the innermost dimension (W_UV = w_uv.transpose(0, 1)) are row
// gathers and go through place_kernel instead.
//
// Naming: "i" is the destination's innermost dimension (strided in the source), "j" the
// source's innermost dimension (strided in the destination); every other dimension is a
// batch index.  A workgroup moves one tile of 512 (i) x 128 bytes (j): source rows are read
// with 16-byte loads (eight per lane, all issued before the first LDS write) into LDS, and
// columns are read back out of LDS so that every store is 16 contiguous destination bytes.
// The transposition happens in LDS; the row pitch is a whole row plus one dword, and in the
// store phase one wavefront covers 16 neighbouring columns x 4 row groups so that its 64
// column reads spread over the banks.  HBM traffic: every element read once, written once.
#include "mxp_device.h"

namespace mxp {

namespace {

constexpr int kThreads = 512;
// Tile extents per element size: 66 KiB of LDS (two workgroups per CU), eight 16-byte loads
// per lane in flight.  Long destination runs matter most: 512 x 64 bf16 elements (1 KiB
// written per destination row) measured 4.56 TB/s on a 16384^2 transpose, 128 x 128 4.0 TB/s.
template <int ES> struct TileOf { static constexpr int I = 512, J = (ES == 1) ? 128 : (ES == 2) ? 64 : (ES == 4) ? 32 : 16; };

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

struct TileCtx {
  const uint8_t* sp;   // first source byte of the tile
  uint8_t* dp;         // first destination byte of the tile
  uint32_t ni, nj;     // valid extents inside the tile
  uint32_t csum_base;  // checksum position of dp
  bool valid;
};

// Linear tile index -> (batch, tile_j, tile_i), tile_i fastest.  Workgroup-uniform.
template <int ES>
__device__ __forceinline__ TileCtx locate_tile(const TransposeDesc& d, uint64_t tile, const uint8_t* src, uint8_t* dst) {
  constexpr int TI = TileOf<ES>::I, TJ = TileOf<ES>::J;
  TileCtx c{};
  c.valid = tile < d.n_tiles;
  if (!c.valid) return c;
  uint64_t b = tile;
  const uint32_t ti = (uint32_t)(b % d.tiles_i);
  b /= d.tiles_i;
  const uint32_t tj = (uint32_t)(b % d.tiles_j);
  b /= d.tiles_j;
  uint64_t s_off = 0, d_off = 0;  // element offsets of the batch
#pragma unroll
  for (int k = kMaxBatchDims - 1; k >= 0; --k) {
    const uint64_t n = d.batch_size[k];
    const uint64_t idx = b % n;
    b /= n;
    s_off += idx * d.batch_sstride[k];
    d_off += idx * d.batch_dstride[k];
  }
  const uint64_t i0 = (uint64_t)ti * TI, j0 = (uint64_t)tj * TJ;
  c.ni = (uint32_t)min((uint64_t)TI, d.ni - i0);
  c.nj = (uint32_t)min((uint64_t)TJ, d.nj - j0);
  c.sp = src + (s_off + i0 * d.si + j0) * ES;
  c.dp = dst + (d_off + j0 * d.dj + i0) * ES;
  c.csum_base = (uint32_t)((d_off + j0 * d.dj + i0) * ES) + d.csum_bias;
  return c;
}

template <int ES>
struct TileIO {
  static constexpr int V = 16 / ES;  // elements per 16-byte chunk
  static constexpr int TI = TileOf<ES>::I, TJ = TileOf<ES>::J;
  static constexpr int kPitch = TJ * ES + 4;  // LDS row pitch in bytes (dword aligned)
  static constexpr int kChunksJ = TJ / V, kChunksI = TI / V;
  static constexpr int kLoads = TI * kChunksJ / kThreads;  // 8 for every element size
  static_assert(kLoads * kThreads == TI * kChunksJ, "tile must divide evenly over the workgroup");

  // global -> registers: rows along j (contiguous in the source), 16 bytes per lane access.
  static __device__ __forceinline__ void issue_loads(const TileCtx& c, const TransposeDesc& d, uint4 (&x)[kLoads],
                                                     bool (&fast)[kLoads]) {
#pragma unroll
    for (int k = 0; k < kLoads; ++k) {
      const uint32_t q = threadIdx.x + (uint32_t)k * kThreads;
      const uint32_t ii = q / kChunksJ, cj = q % kChunksJ;
      fast[k] = d.vec_src && ii < c.ni && cj * V + V <= c.nj;
      if (fast[k]) x[k] = ld16_nt(c.sp + ((uint64_t)ii * d.si + cj * V) * ES);
    }
  }

  // registers -> LDS (chunks that could not use a 16-byte load are copied element-wise here).
  static __device__ __forceinline__ void to_lds(const TileCtx& c, const TransposeDesc& d, const uint4 (&x)[kLoads],
                                                const bool (&fast)[kLoads], uint8_t* lds) {
#pragma unroll
    for (int k = 0; k < kLoads; ++k) {
      const uint32_t q = threadIdx.x + (uint32_t)k * kThreads;
      const uint32_t ii = q / kChunksJ, cj = q % kChunksJ;
      uint8_t* l = lds + ii * kPitch + cj * 16;
      if (fast[k]) {
        uint32_t* lw = reinterpret_cast<uint32_t*>(l);
        lw[0] = x[k].x; lw[1] = x[k].y; lw[2] = x[k].z; lw[3] = x[k].w;
      } else if (ii < c.ni && cj * V < c.nj) {
        const uint8_t* g = c.sp + ((uint64_t)ii * d.si + cj * V) * ES;
        const uint32_t n = min((uint32_t)V, c.nj - cj * V) * ES;
        for (uint32_t e = 0; e < n; ++e) l[e] = g[e];
      }
    }
  }

  // LDS -> global: rows along i (contiguous in the destination), 16 bytes per lane access.
  // Work item q -> (column jj, row group ci): 16 neighbouring columns vary fastest, then 4
  // row groups, so one wavefront instruction reads 16 columns x 4 row groups from LDS.
  static __device__ __forceinline__ void to_global(const TileCtx& c, const TransposeDesc& d, const uint8_t* lds, Csum& cs) {
    for (uint32_t q = threadIdx.x; q < (uint32_t)(TJ * kChunksI); q += kThreads) {
      const uint32_t jj = (q & 15u) + 16u * (q / (16u * kChunksI));
      const uint32_t ci = (q >> 4) % kChunksI;
      if (jj >= c.nj || ci * V >= c.ni) continue;
      const uint32_t ii0 = ci * V;
      const uint32_t n = min((uint32_t)V, c.ni - ii0);
      union { uint4 v; uint8_t b[16]; } x;
      x.v = make_uint4(0, 0, 0, 0);
#pragma unroll
      for (int k = 0; k < V; ++k) {
        if ((uint32_t)k < n) {
          const uint8_t* l = lds + (ii0 + k) * kPitch + jj * ES;
          if constexpr (ES == 1) x.b[k] = l[0];
          else if constexpr (ES == 2) *reinterpret_cast<uint16_t*>(&x.b[2 * k]) = *reinterpret_cast<const uint16_t*>(l);
          else if constexpr (ES == 4) *reinterpret_cast<uint32_t*>(&x.b[4 * k]) = *reinterpret_cast<const uint32_t*>(l);
          else {
            *reinterpret_cast<uint32_t*>(&x.b[8 * k]) = *reinterpret_cast<const uint32_t*>(l);
            *reinterpret_cast<uint32_t*>(&x.b[8 * k + 4]) = *reinterpret_cast<const uint32_t*>(l + 4);
          }
        }
      }
      const uint64_t off = ((uint64_t)jj * d.dj + ii0) * ES;  // bytes from dp
      if (d.vec_dst && n == (uint32_t)V) {
        st16_nt(c.dp + off, x.v);
        cs.add16(x.v, c.csum_base + (uint32_t)off);
      } else {
        for (uint32_t k = 0; k < n * ES; ++k) {
          c.dp[off + k] = x.b[k];
          cs.add_byte(x.b[k], c.csum_base + (uint32_t)off + k);
        }
      }
    }
  }
};

// One workgroup walks kTilesPerGroup consecutive tiles (neighbours along i) and issues the
// next tile's global loads before the current tile goes LDS -> global.  With more than one
// tile per workgroup the wait before the next LDS fill also waits for the stores just
// issued (loads and stores share one in-order counter on this target), so the overlap does
// not materialise; one tile per workgroup, with two workgroups per CU alternating phases,
// measured faster and is the setting used.
template <int ES>
__global__ __launch_bounds__(kThreads) void transpose_kernel(const uint8_t* __restrict__ src,
                                                              uint8_t* __restrict__ dst,
                                                              const TransposeDesc d,
                                                              uint32_t* __restrict__ sum_out) {
  using IO = TileIO<ES>;
  __shared__ __align__(16) uint8_t lds[IO::TI * IO::kPitch];
  uint4 x[IO::kLoads];
  bool fast[IO::kLoads];
  Csum cs;
  const uint64_t first = (uint64_t)blockIdx.x * kTilesPerGroup;
  TileCtx cur = locate_tile<ES>(d, first, src, dst);
  if (cur.valid) IO::issue_loads(cur, d, x, fast);
  for (int t = 0; t < kTilesPerGroup && cur.valid; ++t) {
    IO::to_lds(cur, d, x, fast, lds);
    __syncthreads();
    const TileCtx next = (t + 1 < kTilesPerGroup) ? locate_tile<ES>(d, first + t + 1, src, dst) : TileCtx{};
    if (next.valid) IO::issue_loads(next, d, x, fast);
    IO::to_global(cur, d, lds, cs);
    __syncthreads();
    cur = next;
  }

  if (sum_out) {
    __shared__ uint32_t part[kThreads / 64];
    const uint32_t w = wave_sum_u32(cs.fold());
    if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = w;
    __syncthreads();
    if (threadIdx.x == 0) {
      uint32_t t = 0;
#pragma unroll
      for (int k = 0; k < kThreads / 64; ++k) t += part[k];
      atomicAdd(sum_out, t);
    }
  }
}

}  // namespace

hipError_t launch_transpose(const void* src, void* dst, const TransposeDesc& d, int elem_size,
                            uint32_t* sum_out, hipStream_t stream) {
  if (d.n_tiles == 0) return hipSuccess;
  const uint64_t blocks = (d.n_tiles + kTilesPerGroup - 1) / kTilesPerGroup;
  if (blocks > 0x7FFFFFFFull) return hipErrorInvalidValue;
  const dim3 grid((uint32_t)blocks), block(kThreads);
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
