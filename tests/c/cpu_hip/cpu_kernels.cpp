// CPU stand-ins for the kernel launches the host engine issues (declared in csrc/mxp_device.h), queued on the
// CPU streams of cpu_hip.cpp.  Test infrastructure: they exist so that the engine's ring, reader threads, descriptor
// arenas and stream ordering run under ThreadSanitizer / AddressSanitizer with every "device" access a real memory access.
// A segment is executed by its meaning (a pitched box, a conversion, a position-weighted checksum of the bytes
// written), not by the kernel's lane arithmetic - that is checked elsewhere (tests/c/lower_check.cpp, the GPU tests).
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <utility>
#include <vector>

#include "mxp_device.h"

namespace mxp {

namespace {

uint32_t f32_to_bf16(uint32_t u, uint32_t nan_bits) {
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return nan_bits;
  return (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
}

[[noreturn]] void unsupported(const char* what) {
  std::fprintf(stderr, "cpu stand-in: %s is not implemented\n", what);
  std::abort();
}

void run_item(const Seg* segs, const WorkItem& w, uint32_t block, const void* const* src_bases, void* const* dst_bases,
              uint32_t* sums, Fan fan, uint32_t nan_bits) {
  const Seg& s = segs[w.seg];
  const uint64_t r0 = (uint64_t)w.tile * s.rows_per_tile;
  if (r0 >= s.rows) unsupported("a work item past the end of its segment");
  const uint64_t nrows = s.rows - r0 < s.rows_per_tile ? s.rows - r0 : s.rows_per_tile;
  const uint8_t* src_base = static_cast<const uint8_t*>(s.src_buf == kSrcIsDestination ? dst_bases[s.dst_buf] : src_bases[s.src_buf]);
  uint8_t* dst_base = s.op == kOpChecksumOnly ? nullptr : static_cast<uint8_t*>(dst_bases[s.dst_buf]);
  uint32_t sum = 0;
  for (uint64_t r = r0; r < r0 + nrows; ++r) {
    const uint8_t* sp = src_base + s.src_off + r * s.src_pitch;
    uint8_t* dp = dst_base ? dst_base + s.dst_off + r * s.dst_pitch : nullptr;
    const uint8_t* written = nullptr;
    switch (s.op) {
      case kOpCopy:
        std::memcpy(dp, sp, s.row_bytes);
        written = dp;
        break;
      case kOpChecksumOnly:
        written = sp;
        break;
      case kOpCastF32Bf16:
        for (uint32_t e = 0; e < s.row_bytes / 2; ++e) {
          uint32_t u;
          std::memcpy(&u, sp + 4ull * e, 4);
          const uint16_t h = (uint16_t)f32_to_bf16(u, nan_bits);
          std::memcpy(dp + 2ull * e, &h, 2);
        }
        written = dp;
        break;
      case kOpCastBf16F32:
        for (uint32_t e = 0; e < s.row_bytes / 4; ++e) {
          uint16_t h;
          std::memcpy(&h, sp + 2ull * e, 2);
          const uint32_t u = (uint32_t)h << 16;
          std::memcpy(dp + 4ull * e, &u, 4);
        }
        written = dp;
        break;
      default:
        unsupported("this conversion");
    }
    if (s.csum_slot != 0xFFFFFFFFu) {
      const uint32_t pos0 = (uint32_t)(s.dst_off + r * s.dst_pitch) + s.csum_bias;
      for (uint32_t i = 0; i < s.row_bytes; ++i) sum += written[i] * ((pos0 + i) * kKnuth + 1u);
    }
  }
  if (s.csum_slot != 0xFFFFFFFFu)
    __atomic_fetch_add(&sums[(block & fan.mask) * fan.pitch + s.csum_slot], sum, __ATOMIC_RELAXED);
}

}  // namespace

hipError_t configure_place_kernels() { return hipSuccess; }

hipError_t launch_place(const Seg* segs_dev, const WorkItem* work_dev, uint32_t n_work, const void* const* src_bases_dev,
                        void* const* dst_bases_dev, uint32_t* sums_dev, Fan fan, uint16_t nan_bits, hipStream_t stream, bool,
                        uint32_t* zero_dev, uint32_t zero_words, bool) {
  if (n_work == 0 && zero_words == 0) return hipSuccess;
  cpu_hip::enqueue(stream, [=] {
    for (uint32_t i = 0; i < zero_words; ++i) zero_dev[i] = 0u;
    for (uint32_t b = 0; b < n_work; ++b) run_item(segs_dev, work_dev[b], b, src_bases_dev, dst_bases_dev, sums_dev, fan, nan_bits);
  });
  return hipSuccess;
}

hipError_t launch_fill_u32(uint32_t* ptr, uint64_t n, uint32_t value, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  cpu_hip::enqueue(stream, [=] {
    for (uint64_t i = 0; i < n; ++i) ptr[i] = value;
  });
  return hipSuccess;
}

hipError_t launch_copy_table(void* dst, const void* src, size_t bytes, hipStream_t stream) {
  if (bytes == 0) return hipSuccess;
  cpu_hip::enqueue(stream, [=] { std::memcpy(dst, src, bytes); });
  return hipSuccess;
}

template <typename T>
hipError_t launch_fold_fan(T* fanned_dev, Fan fan, uint32_t per_slot, uint64_t n, T* out_dev, bool clear, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  cpu_hip::enqueue(stream, [=] {
    for (uint64_t k = 0; k < n; ++k) {
      T t = 0;
      for (uint32_t l = 0; l < fan.lanes(); ++l) {
        T& x = fanned_dev[(uint64_t)l * fan.pitch * per_slot + k];
        t += x;
        if (clear) x = 0;
      }
      out_dev[k] = t;
    }
  });
  return hipSuccess;
}
template hipError_t launch_fold_fan<uint32_t>(uint32_t*, Fan, uint32_t, uint64_t, uint32_t*, bool, hipStream_t);
template hipError_t launch_fold_fan<unsigned long long>(unsigned long long*, Fan, uint32_t, uint64_t, unsigned long long*, bool,
                                                        hipStream_t);

// Not exercised by the sanitizer driver: refused, so that a call that reached them is noticed.
hipError_t launch_place_digest(const Seg*, const WorkItem*, uint32_t, const void* const*, void* const*, uint32_t*, Fan,
                               const unsigned long long*, unsigned long long*, uint16_t, hipStream_t, uint32_t*, uint32_t) {
  return hipErrorNotSupported;
}
hipError_t launch_digest(const DigestJob*, uint32_t, uint32_t, unsigned long long*, Fan, hipStream_t) { return hipErrorNotSupported; }
hipError_t launch_probe_gather(const void*, void*, uint32_t, uint32_t, uint32_t, uint32_t, bool, hipStream_t) { return hipErrorNotSupported; }
namespace {

// dst[b..., j, i] = convert(src[b..., i, j]) for every batch index, as the descriptor says it (strides in elements).
void run_transpose(const uint8_t* src, uint8_t* dst, const TransposeDesc& d, int es, uint32_t op, uint32_t nan_bits, uint32_t* sum_out) {
  const int eo = op == kOpCopy ? es : (int)op_dst_elem(op);
  if (op != kOpCopy && op != kOpCastF32Bf16 && op != kOpCastBf16F32) unsupported("this conversion in a transpose");
  uint64_t batches = 1;
  for (int k = 0; k < kMaxBatchDims; ++k) batches *= d.batch_size[k];
  uint32_t sum = 0;
  for (uint64_t b = 0; b < batches; ++b) {
    uint64_t rest = b, s_off = 0, d_off = 0;
    for (int k = kMaxBatchDims - 1; k >= 0; --k) {
      const uint64_t idx = rest % d.batch_size[k];
      rest /= d.batch_size[k];
      s_off += idx * d.batch_sstride[k];
      d_off += idx * d.batch_dstride[k];
    }
    for (uint64_t i = 0; i < d.ni; ++i)
      for (uint64_t j = 0; j < d.nj; ++j) {
        const uint8_t* sp = src + (s_off + i * d.si + j) * (uint64_t)es;
        const uint64_t del = d_off + j * d.dj + i;
        uint8_t* dp = dst + del * (uint64_t)eo;
        if (op == kOpCopy) {
          std::memcpy(dp, sp, (size_t)es);
        } else if (op == kOpCastF32Bf16) {
          uint32_t u;
          std::memcpy(&u, sp, 4);
          const uint16_t h = (uint16_t)f32_to_bf16(u, nan_bits);
          std::memcpy(dp, &h, 2);
        } else {
          uint16_t h;
          std::memcpy(&h, sp, 2);
          const uint32_t u = (uint32_t)h << 16;
          std::memcpy(dp, &u, 4);
        }
        if (sum_out) {
          const uint32_t pos0 = (uint32_t)(del * (uint64_t)eo) + d.csum_bias;
          for (int e = 0; e < eo; ++e) sum += dp[e] * ((pos0 + (uint32_t)e) * kKnuth + 1u);
        }
      }
  }
  if (sum_out) __atomic_fetch_add(sum_out, sum, __ATOMIC_RELAXED);
}

}  // namespace

hipError_t launch_transpose(const void* src, void* dst, const TransposeDesc& d, int elem_size, uint32_t op, uint32_t nan_bits,
                            uint32_t* sum_out, Fan, hipStream_t stream) {
  if (d.n_tiles == 0) return hipSuccess;
  if (!transpose_desc_ok(d)) return hipErrorInvalidValue;
  const TransposeDesc desc = d;  // a kernel argument: copied when the launch is issued
  cpu_hip::enqueue(stream, [=] { run_transpose(static_cast<const uint8_t*>(src), static_cast<uint8_t*>(dst), desc, elem_size, op, nan_bits, sum_out); });
  return hipSuccess;
}
hipError_t launch_transpose_batch(const TransposeItem* items_dev, uint32_t n_items, uint64_t total_tiles, uint32_t, int elem_size,
                                  uint32_t op, uint32_t nan_bits, hipStream_t stream, uint32_t, uint32_t uniform_tiles,
                                  const TransposeDesc* common, const TransposeItem* items_host) {
  if (n_items == 0 || total_tiles == 0) return hipSuccess;
  if (uniform_tiles && common && items_host) {
    // descriptor and pointers travel as kernel arguments: read now
    std::vector<std::pair<const uint8_t*, uint8_t*>> ptrs;
    for (uint32_t k = 0; k < n_items; ++k) ptrs.emplace_back(items_host[k].src, items_host[k].dst);
    const TransposeDesc desc = *common;
    cpu_hip::enqueue(stream, [=] {
      for (const auto& pr : ptrs) run_transpose(pr.first, pr.second, desc, elem_size, op, nan_bits, nullptr);
    });
    return hipSuccess;
  }
  // the item table is device memory: read when the launch runs
  cpu_hip::enqueue(stream, [=] {
    for (uint32_t k = 0; k < n_items; ++k) run_transpose(items_dev[k].src, items_dev[k].dst, items_dev[k].d, elem_size, op, nan_bits, nullptr);
  });
  return hipSuccess;
}
hipError_t launch_synth(void*, uint64_t, uint32_t, uint32_t, uint64_t, hipStream_t) { return hipErrorNotSupported; }
void synth_host(void*, uint64_t, uint32_t, uint32_t, uint64_t, int) { unsupported("the synthetic-checkpoint generator"); }

}  // namespace mxp
