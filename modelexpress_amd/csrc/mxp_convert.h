// Element conversions of dest.copy_(src) on bit patterns (device side), shared by the placement
// kernel and the transpose kernel.  Every function works on raw bits so that the result is
// defined for every input pattern and can be pinned against torch's CPU conversions.
#pragma once
#include "mxp_device.h"

namespace mxp {

// fp32 bits -> bf16 bits, round to nearest even; every NaN becomes `nan_bits`.
// Reference arithmetic: torch `copy_` at modelexpress_rl/train/engines/fsdp/adapter.py:203-206
// and refit/reshard/receiver.py:964-971.
__device__ __forceinline__ uint32_t f32_to_bf16_bits(uint32_t u, uint32_t nan_bits) {
  const uint32_t r = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
  return ((u & 0x7FFFFFFFu) > 0x7F800000u) ? nan_bits : r;
}

// Two fp32 -> two bf16 (a in the low half), same result as f32_to_bf16_bits on each: the
// hardware's packed converter rounds to nearest even, and since rounding a finite value never
// gives a NaN, a NaN half of its result marks a NaN input; those halves become `nan_bits`.
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(uint32_t a, uint32_t b, uint32_t nan_bits) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  f32x2 f;
  f.x = __uint_as_float(a);
  f.y = __uint_as_float(b);
  const bf16x2 h = __builtin_convertvector(f, bf16x2);
  uint32_t p;
  __builtin_memcpy(&p, &h, 4);
  const uint32_t nan = (((p & 0x7FFF7FFFu) + 0x007F007Fu) & 0x80008000u) >> 15;  // bit 0 / bit 16 per NaN half
  const uint32_t mask = nan * 0xFFFFu;
  return (p & ~mask) | ((nan_bits * 0x00010001u) & mask);
}

// fp32 bits -> fp16 bits, round to nearest even (the wavefront's default rounding mode, with
// fp16 denormals enabled): overflow -> infinity, subnormal results rounded like any other.
// The hardware converter does the arithmetic in one instruction; the bit arithmetic it
// replaces kept this path VALU-bound (4.4 TB/s against 6.0 for fp32 -> bf16).  NaNs are set
// explicitly so the image does not depend on the converter: the top ten payload bits are kept
// and the NaN is made quiet (the rule of torch's CPU copy_).
__device__ __forceinline__ uint32_t f32_to_f16_bits(uint32_t u) {
  const uint32_t a = u & 0x7FFFFFFFu;
  const _Float16 h = (_Float16)__uint_as_float(u);
  uint16_t hb;
  __builtin_memcpy(&hb, &h, 2);
  return (a > 0x7F800000u) ? (((u >> 16) & 0x8000u) | 0x7E00u | ((a >> 13) & 0x3FFu)) : (uint32_t)hb;
}

// Two fp32 -> two fp16 (a in the low half), same result as f32_to_f16_bits on each, through the
// packed converter.  Rounding a finite value gives at most an infinity, so a NaN half of the
// converter's result marks a NaN input; only then (1e-6 of the elements at most in this path's
// workloads) are the halves rebuilt from the input bits by the rule above.
__device__ __forceinline__ uint32_t f32x2_to_f16x2(uint32_t a, uint32_t b) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
  f32x2 f;
  f.x = __uint_as_float(a);
  f.y = __uint_as_float(b);
  const f16x2 h = __builtin_convertvector(f, f16x2);
  uint32_t p;
  __builtin_memcpy(&p, &h, 4);
  if (((p & 0x7FFF7FFFu) + 0x03FF03FFu) & 0x80008000u)  // a half above 0x7C00: a NaN
    p = f32_to_f16_bits(a) | (f32_to_f16_bits(b) << 16);
  return p;
}

// fp16 bits -> fp32 bits, exact (subnormals renormalised by the converter); NaNs made quiet.
__device__ __forceinline__ uint32_t f16_to_f32_bits(uint32_t h) {
  const uint16_t hb = (uint16_t)h;
  _Float16 x;
  __builtin_memcpy(&x, &hb, 2);
  const uint32_t f = __float_as_uint((float)x);
  const uint32_t m = h & 0x3FFu;
  return ((h & 0x7C00u) == 0x7C00u && m) ? (((h & 0x8000u) << 16) | 0x7FC00000u | (m << 13)) : f;
}

// One 16-bit element of a conversion between the two 16-bit formats, through fp32 as torch's
// copy_ does: fp16 -> bf16 (NaN -> nan_bits) or bf16 -> fp16.
template <int OP>
__device__ __forceinline__ uint32_t recode1(uint32_t h, uint32_t nan_bits) {
  if constexpr (OP == kOpCastF16Bf16) return f32_to_bf16_bits(f16_to_f32_bits(h), nan_bits);
  else return f32_to_f16_bits(h << 16);
}
template <int OP>
__device__ __forceinline__ uint32_t recode2(uint32_t w, uint32_t nan_bits) {
  if constexpr (OP == kOpCastF16Bf16) {
    // exact widening by the converter (a NaN stays a NaN, whatever its payload), then the packed rounding
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    f16x2 h;
    __builtin_memcpy(&h, &w, 4);
    return f32x2_to_bf16x2(__float_as_uint((float)h.x), __float_as_uint((float)h.y), nan_bits);
  } else {
    return f32x2_to_f16x2(w << 16, w & 0xFFFF0000u);  // a bf16 is the upper half of its fp32
  }
}

template <int OP>
__device__ __forceinline__ uint32_t narrow1(uint32_t u, uint32_t nan_bits) {
  if constexpr (OP == kOpCastF32F16) return f32_to_f16_bits(u);
  else return f32_to_bf16_bits(u, nan_bits);
}
// fp8 e4m3fn bits -> bf16 bits, exact: bias 7 -> 127, subnormals (m * 2^-9) renormalised, the
// two NaN codes -> 0x7FC0 (torch's image).  Reference: .to(out_dtype) at
// engines/vllm/refit/receiver.py:258-261 when kv_b_proj is stored in fp8.
__device__ __forceinline__ uint32_t f8e4m3_to_bf16_bits(uint32_t c) {
  const uint32_t sign = (c & 0x80u) << 8, e = (c >> 3) & 0xFu, m = c & 7u;
  if ((c & 0x7Fu) == 0x7Fu) return 0x7FC0u;
  if (e != 0u) return sign | ((e + 120u) << 7) | (m << 4);
  if (m == 0u) return sign;
  const uint32_t top = 31u - (uint32_t)__clz((int)m);
  return sign | ((top + 118u) << 7) | ((m << (7u - top)) & 0x7Fu);
}

// Two fp8 e4m3fn elements (the low or the high half of `w`) -> two bf16, through the hardware
// fp8 -> fp32 converter (exact; gfx950 decodes the OCP e4m3fn format) and truncation, which is
// exact as well: every e4m3 value has a 3-bit mantissa.  e4m3fn has no infinities, so an
// all-ones bf16 exponent after conversion marks a NaN code; those become 0x7FC0 whatever
// pattern the converter produced.
template <bool HI>
__device__ __forceinline__ uint32_t f8e4m3x2_to_bf16x2(uint32_t w) {
  typedef float float2v __attribute__((ext_vector_type(2)));
  const float2v f = __builtin_amdgcn_cvt_pk_f32_fp8((int)w, HI);
  const uint32_t p = __builtin_amdgcn_perm(__float_as_uint(f.y), __float_as_uint(f.x), 0x07060302u);
  const uint32_t nan = (((p & 0x7F807F80u) + 0x00800080u) & 0x80008000u) >> 15;  // bit 0 / bit 16 set per NaN half
  const uint32_t mask = nan * 0xFFFFu;
  return (p & ~mask) | (0x7FC07FC0u & mask);
}

template <int OP>
__device__ __forceinline__ uint32_t widen1(uint32_t h) {
  if constexpr (OP == kOpCastF16F32) return f16_to_f32_bits(h);
  else return h << 16;
}
template <int OP>
__device__ __forceinline__ uint2 narrow4(const uint4& a, uint32_t nan_bits) {
  uint2 o;
  if constexpr (OP == kOpCastF32Bf16) {
    o.x = f32x2_to_bf16x2(a.x, a.y, nan_bits);
    o.y = f32x2_to_bf16x2(a.z, a.w, nan_bits);
  } else {
    static_assert(OP == kOpCastF32F16, "the narrowing conversions are fp32 -> bf16 and fp32 -> fp16");
    o.x = f32x2_to_f16x2(a.x, a.y);
    o.y = f32x2_to_f16x2(a.z, a.w);
  }
  return o;
}
template <int OP>
__device__ __forceinline__ uint4 widen4(const uint2& a) {
  if constexpr (OP == kOpCastF8E4M3Bf16) {  // eight one-byte elements in, eight bf16 out
    return make_uint4(f8e4m3x2_to_bf16x2<false>(a.x), f8e4m3x2_to_bf16x2<true>(a.x), f8e4m3x2_to_bf16x2<false>(a.y),
                      f8e4m3x2_to_bf16x2<true>(a.y));
  } else
  return make_uint4(widen1<OP>(a.x & 0xFFFFu), widen1<OP>(a.x >> 16), widen1<OP>(a.y & 0xFFFFu), widen1<OP>(a.y >> 16));
}

// Four elements at a time: `narrow4` packs four 32-bit inputs into four 16-bit outputs,
// `widen4` expands eight source bytes (four 16-bit or eight 8-bit elements) into 16 bytes,
// `recode8` converts eight 16-bit elements in place.
template <int OP>
__device__ __forceinline__ uint4 recode8(const uint4& a, uint32_t nan_bits) {
  return make_uint4(recode2<OP>(a.x, nan_bits), recode2<OP>(a.y, nan_bits), recode2<OP>(a.z, nan_bits),
                    recode2<OP>(a.w, nan_bits));
}

}  // namespace mxp
