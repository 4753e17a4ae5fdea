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

template <int ES>
__global__ __launch_bounds__(kThreads) void transpose_kernel(const uint8_t* __restrict__ src,
                                                              uint8_t* __restrict__ dst,
                                                              const TransposeDesc d,
                                                              uint32_t* __restrict__ sum_out) {
  constexpr int V = 16 / ES;                    // elements per 16-byte chunk
  constexpr int TI = TileOf<ES>::I, TJ = TileOf<ES>::J;
  constexpr int kPitch = TJ * ES + 4;           // LDS row pitch in bytes (dword aligned)
  __shared__ __align__(16) uint8_t lds[TI * kPitch];

  // blockIdx.x -> (batch, tile_j, tile_i), tile_i fastest.
  uint64_t b = blockIdx.x;
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
  const uint32_t ni = (uint32_t)min((uint64_t)TI, d.ni - i0);
  const uint32_t nj = (uint32_t)min((uint64_t)TJ, d.nj - j0);
  const uint8_t* sp = src + (s_off + i0 * d.si + j0) * ES;
  uint8_t* dp = dst + (d_off + j0 * d.dj + i0) * ES;

  // ---- load: rows along j (contiguous in the source) ----
  constexpr int kChunksJ = TJ / V;
  constexpr int kLoads = TI * kChunksJ / kThreads;  // 8 for every element size
  static_assert(kLoads * kThreads == TI * kChunksJ, "tile must divide evenly over the workgroup");
  {
    uint4 x[kLoads];
    bool fast[kLoads];
    // every 16-byte load of the tile is issued before the first LDS write
#pragma unroll
    for (int k = 0; k < kLoads; ++k) {
      const uint32_t q = threadIdx.x + (uint32_t)k * kThreads;
      const uint32_t ii = q / kChunksJ, cj = q % kChunksJ;
      fast[k] = d.vec_src && ii < ni && cj * V + V <= nj;
      if (fast[k]) x[k] = *reinterpret_cast<const uint4*>(sp + ((uint64_t)ii * d.si + cj * V) * ES);
    }
#pragma unroll
    for (int k = 0; k < kLoads; ++k) {
      const uint32_t q = threadIdx.x + (uint32_t)k * kThreads;
      const uint32_t ii = q / kChunksJ, cj = q % kChunksJ;
      uint8_t* l = lds + ii * kPitch + cj * 16;
      if (fast[k]) {
        uint32_t* lw = reinterpret_cast<uint32_t*>(l);
        lw[0] = x[k].x; lw[1] = x[k].y; lw[2] = x[k].z; lw[3] = x[k].w;
      } else if (ii < ni && cj * V < nj) {
        const uint8_t* g = sp + ((uint64_t)ii * d.si + cj * V) * ES;
        const uint32_t n = min((uint32_t)V, nj - cj * V) * ES;
        for (uint32_t e = 0; e < n; ++e) l[e] = g[e];
      }
    }
  }
  __syncthreads();

  // ---- store: rows along i (contiguous in the destination) ----
  Csum cs;
  const uint32_t csum_base = (uint32_t)((d_off + j0 * d.dj + i0) * ES) + d.csum_bias;
  constexpr int kChunksI = TI / V;
  // Work item q -> (column jj, row group ci): 16 neighbouring columns vary fastest, then 4
  // row groups, so one wavefront instruction reads 16 columns x 4 row groups from LDS.
  for (uint32_t q = threadIdx.x; q < (uint32_t)(TJ * kChunksI); q += kThreads) {
    const uint32_t jj = (q & 15u) + 16u * (q / (16u * kChunksI));
    const uint32_t ci = (q >> 4) % kChunksI;
    if (jj >= nj || ci * V >= ni) continue;
    const uint32_t ii0 = ci * V;
    const uint32_t n = min((uint32_t)V, ni - ii0);
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
      *reinterpret_cast<uint4*>(dp + off) = x.v;
      cs.add16(x.v, csum_base + (uint32_t)off);
    } else {
      for (uint32_t k = 0; k < n * ES; ++k) {
        dp[off + k] = x.b[k];
        cs.add_byte(x.b[k], csum_base + (uint32_t)off + k);
      }
    }
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
  uint64_t blocks = (uint64_t)d.tiles_i * d.tiles_j;
  for (int k = 0; k < kMaxBatchDims; ++k) blocks *= d.batch_size[k];
  if (blocks == 0) return hipSuccess;
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
