// Device-side checksum algebra and wavefront reductions shared by the placement kernels
// (mxp_kernels.hip) and the transpose kernels (mxp_permute.hip).  Device code only.
#pragma once
#include "mxp_device.h"

namespace mxp {

// ---------------------------------------------------------------------------
// Checksum algebra.  The per-tensor fingerprint is
//     sum_i  byte[i] * ((i * 2654435761 + 1) mod 2^32)   mod 2^32
// (reference: modelexpress/tensor_utils.py:27-44).  For a group of bytes starting at
// position i with local offsets j:
//     sum_j b_j * ((i + j) K + 1) = K * (i * S0 + S1) + S0,   S0 = sum b_j, S1 = sum j b_j
// so three wrapping 32-bit accumulators P = sum i*S0, R = sum S1, Q = sum S0 are kept
// per lane and folded once at the end as K * (P + R) + Q.  S0 and S1 come from the
// unsigned 8-bit dot-product instruction, four bytes at a time.
// ---------------------------------------------------------------------------
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
  __device__ __forceinline__ void add8(uint32_t lo, uint32_t hi, uint32_t i) {
    uint32_t s0 = __builtin_amdgcn_udot4(lo, 0x01010101u, 0u, false);
    s0 = __builtin_amdgcn_udot4(hi, 0x01010101u, s0, false);
    R = __builtin_amdgcn_udot4(lo, 0x03020100u, R, false);
    R = __builtin_amdgcn_udot4(hi, 0x07060504u, R, false);
    Q += s0;
    P += i * s0;
  }
  // Up to four bytes packed little-endian in x (missing bytes zero).
  __device__ __forceinline__ void add4(uint32_t x, uint32_t i) {
    uint32_t s0 = __builtin_amdgcn_udot4(x, 0x01010101u, 0u, false);
    R = __builtin_amdgcn_udot4(x, 0x03020100u, R, false);
    Q += s0;
    P += i * s0;
  }
  // One unit of UNIT <= 4 bytes (the narrow paths).
  template <int UNIT>
  __device__ __forceinline__ void addn(uint32_t x, uint32_t i) { add4(x, i); }
  // One byte at position i.
  __device__ __forceinline__ void add_byte(uint32_t b, uint32_t i) {
    Q += b;
    P += i * b;
  }
  __device__ __forceinline__ uint32_t fold() const { return kKnuth * (P + R) + Q; }
};

__device__ __forceinline__ uint32_t wave_sum_u32(uint32_t v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o, 64);
  return v;
}

__device__ __forceinline__ unsigned long long wave_sum_u64(unsigned long long v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_down(v, o, 64);
  return v;
}

}  // namespace mxp
