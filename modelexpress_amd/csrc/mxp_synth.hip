// Seeded synthetic tensor contents, generated with identical integer arithmetic on the
// host (std::thread) and on the device, so a checkpoint file written on the CPU and a
// staged copy generated straight into HBM hold the same bytes.  Every value is a pure
// function of (seed, element index): any tensor, or any slice of one, can be
// regenerated alone.
//
// Floating-point values are produced with one int->float conversion and one multiply,
// both correctly rounded IEEE operations with no fused form, so host and device agree
// bit for bit; narrowing to bf16 / fp16 uses integer round-to-nearest-even.
#include <thread>
#include <vector>

#include "mxp_device.h"
#include "mxp.h"
#include "mxp_bench.h"

namespace mxp {

__host__ __device__ inline uint64_t mix64(uint64_t z) {
  z += 0x9E3779B97F4A7C15ull;
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

__host__ __device__ inline uint32_t f32_bits(float f) {
  union { float f; uint32_t u; } c;
  c.f = f;
  return c.u;
}

__host__ __device__ inline uint32_t synth_bf16_bits(uint32_t u) {
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return 0x7FC0u;
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

__host__ __device__ inline uint32_t synth_f16_bits(uint32_t u) {
  const uint32_t sign = (u >> 16) & 0x8000u;
  const uint32_t e = (u >> 23) & 0xFFu;
  uint32_t m = u & 0x7FFFFFu;
  if (e == 255u) return sign | 0x7C00u | (m ? 0x200u : 0u);
  const int E = (int)e - 127 + 15;
  if (E >= 31) return sign | 0x7C00u;
  if (E <= 0) {
    if (E < -10) return sign;
    m |= 0x800000u;
    const uint32_t shift = (uint32_t)(14 - E);
    uint32_t half = m >> shift;
    const uint32_t rem = m & ((1u << shift) - 1u);
    const uint32_t mid = 1u << (shift - 1u);
    if (rem > mid || (rem == mid && (half & 1u))) ++half;
    return sign | half;
  }
  uint32_t half = ((uint32_t)E << 10) | (m >> 13);
  const uint32_t rem = m & 0x1FFFu;
  if (rem > 0x1000u || (rem == 0x1000u && (half & 1u))) ++half;
  return sign | half;
}

// fp32 bit pattern of element k.
__host__ __device__ inline uint32_t synth_f32_bits(uint32_t kind, uint64_t seed, uint64_t k) {
  const uint64_t h = mix64(seed + k * 0x9E3779B97F4A7C15ull);
  if (kind == kSynthOnes) return 0x3F800000u;
  if (kind == kSynthZeros) return 0u;
  if (kind == kSynthScale) {
    // uniform in [1e-4, 1e-2]
    const int v = (int)(h & 0xFFFFFFu) + 169467;
    return f32_bits((float)v * 5.9008540e-10f);
  }
  const int s = (int)(h & 0xFFFFu) + (int)((h >> 16) & 0xFFFFu) + (int)((h >> 32) & 0xFFFFu) +
                (int)(h >> 48);
  uint32_t bits = f32_bits((float)(s - 131070) * 5.2857996e-07f);  // 0.02 / 37837.2
  if (kind == kSynthNormalEdge || kind == 6u) {
    const uint64_t h2 = mix64(h ^ 0xD1B54A32D192ED03ull);
    const uint64_t period = (kind == 6u) ? 64ull : 1000000ull;
    const uint64_t sel = h2 % (period * 8ull);
    if (sel < 8ull) {
      const uint32_t r = (uint32_t)(h2 >> 32);
      switch ((uint32_t)sel) {
        case 0: bits = (r & 0x807FFFFFu) | 1u; break;             // denormal
        case 1: bits = 0x7F800000u; break;                        // +inf
        case 2: bits = 0xFF800000u; break;                        // -inf
        case 3: bits = 0x7FC00000u | (r & 0x803FFFFFu); break;    // quiet NaN, any payload/sign
        case 4: bits = 0x7F800001u | (r & 0x803FFFFEu); break;    // signalling NaN
        case 5: bits = (bits & 0xFFFF0000u) | 0x8000u; break;     // exact tie
        case 6: bits = (r & 0x80000000u) | 0x7F7FFFFFu; break;    // largest finite: rounds to inf
        default: bits = (r & 0x80000000u) | (r & 0xFFFFu); break; // denormal below half a bf16 ulp
      }
    }
  }
  return bits;
}

template <typename F>
__host__ __device__ inline void synth_store(void* dst, uint64_t k, uint32_t dtype, uint32_t kind,
                                            uint64_t seed, F) {
  switch (dtype) {
    case MXP_DTYPE_F32:
      static_cast<uint32_t*>(dst)[k] = synth_f32_bits(kind, seed, k);
      break;
    case MXP_DTYPE_BF16:
      static_cast<uint16_t*>(dst)[k] = (uint16_t)synth_bf16_bits(synth_f32_bits(kind, seed, k));
      break;
    case MXP_DTYPE_F16:
      static_cast<uint16_t*>(dst)[k] = (uint16_t)synth_f16_bits(synth_f32_bits(kind, seed, k));
      break;
    case MXP_DTYPE_F64: {
      union { float f; uint32_t u; } c;
      c.u = synth_f32_bits(kind, seed, k);
      static_cast<double*>(dst)[k] = (double)c.f;
      break;
    }
    case MXP_DTYPE_F8_E4M3:
    case MXP_DTYPE_F8_E5M2: {
      const uint32_t v = (uint32_t)(mix64(seed + k * 0x9E3779B97F4A7C15ull) % 254ull);
      static_cast<uint8_t*>(dst)[k] = (uint8_t)(v < 127u ? v : v + 1u);
      break;
    }
    case MXP_DTYPE_I64:
      static_cast<uint64_t*>(dst)[k] = mix64(seed + k * 0x9E3779B97F4A7C15ull);
      break;
    case MXP_DTYPE_I32:
      static_cast<uint32_t*>(dst)[k] = (uint32_t)mix64(seed + k * 0x9E3779B97F4A7C15ull);
      break;
    case MXP_DTYPE_I16:
      static_cast<uint16_t*>(dst)[k] = (uint16_t)mix64(seed + k * 0x9E3779B97F4A7C15ull);
      break;
    default:  // I8, U8, BOOL
      static_cast<uint8_t*>(dst)[k] =
          (uint8_t)(dtype == MXP_DTYPE_BOOL ? (mix64(seed + k * 0x9E3779B97F4A7C15ull) & 1u)
                                            : mix64(seed + k * 0x9E3779B97F4A7C15ull));
      break;
  }
}

__global__ __launch_bounds__(256) void synth_kernel(void* dst, uint64_t n, uint32_t dtype,
                                                    uint32_t kind, uint64_t seed) {
  for (uint64_t k = blockIdx.x * 256ull + threadIdx.x; k < n; k += (uint64_t)gridDim.x * 256ull)
    synth_store(dst, k, dtype, kind, seed, 0);
}

hipError_t launch_synth(void* dst, uint64_t n_elems, uint32_t dtype_code, uint32_t kind,
                        uint64_t seed, hipStream_t stream) {
  if (n_elems == 0) return hipSuccess;
  const uint64_t blocks = (n_elems + 255) / 256;
  hipLaunchKernelGGL(synth_kernel, dim3((uint32_t)(blocks > 65536 ? 65536 : blocks)), dim3(256), 0,
                     stream, dst, n_elems, dtype_code, kind, seed);
  return hipGetLastError();
}

void synth_host(void* dst, uint64_t n_elems, uint32_t dtype_code, uint32_t kind, uint64_t seed,
                int threads) {
  if (threads < 1) threads = 1;
  const uint64_t min_chunk = 1 << 16;
  const uint64_t want = (n_elems + min_chunk - 1) / min_chunk;
  const int n_thr = (int)std::min<uint64_t>((uint64_t)threads, want ? want : 1);
  auto body = [&](uint64_t lo, uint64_t hi) {
    for (uint64_t k = lo; k < hi; ++k) synth_store(dst, k, dtype_code, kind, seed, 0);
  };
  if (n_thr <= 1) {
    body(0, n_elems);
    return;
  }
  std::vector<std::thread> pool;
  const uint64_t per = (n_elems + n_thr - 1) / n_thr;
  for (int t = 0; t < n_thr; ++t) {
    const uint64_t lo = std::min<uint64_t>(n_elems, per * t), hi = std::min<uint64_t>(n_elems, lo + per);
    if (lo < hi) pool.emplace_back(body, lo, hi);
  }
  for (auto& th : pool) th.join();
}

// ---------------------------------------------------------------------------
// Measurement support: a bare row gather with the placement kernel's workgroup shape (1024 lanes,
// eight 16-byte units per lane, all loads before all stores, non-temporal accesses, one workgroup
// per compute unit) and nothing else - no descriptor tables, no checksum, no conversion.  What it
// reaches for an access shape on a given box is what the memory system gives that shape; the
// library's kernels are compared with it (mxp_measure_gather).
// ---------------------------------------------------------------------------
namespace {
typedef uint32_t probe_u32x4 __attribute__((ext_vector_type(4)));
constexpr int kProbeThreads = 1024, kProbeBatch = 8;

// NARROW: the rows are fp32 and are stored as bf16 (round to nearest even; the probe's inputs hold no NaN):
// 16 bytes in and 8 bytes out per unit, the shape of the placement kernel's narrowing path.
typedef uint32_t probe_u32x2 __attribute__((ext_vector_type(2)));
template <bool NARROW>
__global__ __launch_bounds__(kProbeThreads) void probe_gather_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                                     uint32_t units_per_row, uint32_t magic, uint32_t src_pitch,
                                                                     uint32_t rows_per_tile) {
  constexpr uint32_t kOut = NARROW ? 8u : 16u;  // destination bytes per unit (a unit reads 16 source bytes)
  const uint64_t t = blockIdx.x;
  const uint8_t* s = src + t * rows_per_tile * (uint64_t)src_pitch;
  uint8_t* d = dst + t * rows_per_tile * (uint64_t)units_per_row * kOut;
  const uint32_t n_units = rows_per_tile * units_per_row;
  probe_u32x4 a[kProbeBatch];
  uint32_t so[kProbeBatch], d_o[kProbeBatch];
  bool ok[kProbeBatch];
#pragma unroll
  for (int k = 0; k < kProbeBatch; ++k) {
    const uint32_t v0 = threadIdx.x + (uint32_t)k * kProbeThreads;
    ok[k] = v0 < n_units;
    const uint32_t v = ok[k] ? v0 : 0u;
    const uint32_t row = units_per_row == 1u ? v : __umulhi(v, magic);
    const uint32_t col = v - row * units_per_row;
    so[k] = row * src_pitch + col * 16u;
    d_o[k] = v * kOut;
  }
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int k = 0; k < kProbeBatch; ++k) a[k] = __builtin_nontemporal_load(reinterpret_cast<const probe_u32x4*>(s + so[k]));
  __builtin_amdgcn_sched_barrier(0);
#pragma unroll
  for (int k = 0; k < kProbeBatch; ++k) {
    if (!ok[k]) continue;
    if constexpr (NARROW) {
      auto rne = [](uint32_t u) { return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16; };
      probe_u32x2 o;
      o.x = rne(a[k].x) | (rne(a[k].y) << 16);
      o.y = rne(a[k].z) | (rne(a[k].w) << 16);
      __builtin_nontemporal_store(o, reinterpret_cast<probe_u32x2*>(d + d_o[k]));
    } else {
      __builtin_nontemporal_store(a[k], reinterpret_cast<probe_u32x4*>(d + d_o[k]));
    }
  }
}
}  // namespace

// Gathers n_tiles * rows_per_tile rows of units_per_row * 16 source bytes, `src_pitch` bytes apart, into a
// contiguous destination (as they are, or narrowed from fp32 to bf16).  rows_per_tile * units_per_row <= 8192;
// both buffers 16-byte aligned.
hipError_t launch_probe_gather(const void* src, void* dst, uint32_t units_per_row, uint32_t src_pitch, uint32_t rows_per_tile,
                               uint32_t n_tiles, bool narrow, hipStream_t stream) {
  if (n_tiles == 0) return hipSuccess;
  if (units_per_row == 0 || rows_per_tile == 0 || (uint64_t)rows_per_tile * units_per_row > (uint64_t)kProbeThreads * kProbeBatch ||
      (uint64_t)rows_per_tile * src_pitch >= (1ull << 32) || src_pitch % 16u || (uint64_t)units_per_row * 16u > src_pitch)
    return hipErrorInvalidValue;
  constexpr int kOnePerCu = 96 * 1024;  // more than half a compute unit's LDS: one resident workgroup
  static bool configured = false;
  if (!configured) {
    for (const void* f : {reinterpret_cast<const void*>(probe_gather_kernel<false>), reinterpret_cast<const void*>(probe_gather_kernel<true>)})
      if (hipError_t e = hipFuncSetAttribute(f, hipFuncAttributeMaxDynamicSharedMemorySize, kOnePerCu); e != hipSuccess) return e;
    configured = true;
  }
  const uint32_t magic = units_per_row > 1 ? (uint32_t)((1ull << 32) / units_per_row) + 1u : 0u;
  if (narrow)
    hipLaunchKernelGGL(probe_gather_kernel<true>, dim3(n_tiles), dim3(kProbeThreads), kOnePerCu, stream, static_cast<const uint8_t*>(src),
                       static_cast<uint8_t*>(dst), units_per_row, magic, src_pitch, rows_per_tile);
  else
    hipLaunchKernelGGL(probe_gather_kernel<false>, dim3(n_tiles), dim3(kProbeThreads), kOnePerCu, stream, static_cast<const uint8_t*>(src),
                       static_cast<uint8_t*>(dst), units_per_row, magic, src_pitch, rows_per_tile);
  return hipGetLastError();
}

}  // namespace mxp
