// The CPU stand-in declared in hip/hip_runtime.h: streams as worker threads, events, memory.  Test infrastructure.
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <condition_variable>
#include <cstdlib>
#include <cstring>
#include <deque>
#include <future>
#include <map>
#include <memory>
#include <mutex>
#include <thread>
#include <vector>

namespace {

struct EventState {
  std::mutex mu;
  std::condition_variable cv;
  uint64_t recorded = 0, done = 0;
  std::chrono::steady_clock::time_point when{};
};

}  // namespace

struct ihipEvent_t {
  std::shared_ptr<EventState> st = std::make_shared<EventState>();
};

struct ihipStream_t {
  std::mutex mu;
  std::condition_variable cv;
  std::deque<std::function<void()>> q;
  bool stop = false;
  std::thread worker;
  ihipStream_t() : worker([this] { run(); }) {}
  ~ihipStream_t() {
    {
      std::lock_guard<std::mutex> lk(mu);
      stop = true;
    }
    cv.notify_all();
    worker.join();
  }
  void run() {
    for (;;) {
      std::function<void()> f;
      {
        std::unique_lock<std::mutex> lk(mu);
        cv.wait(lk, [&] { return stop || !q.empty(); });
        if (q.empty()) return;  // stop: everything queued has run
        f = std::move(q.front());
        q.pop_front();
      }
      f();
    }
  }
  void push(std::function<void()> f) {
    {
      std::lock_guard<std::mutex> lk(mu);
      q.push_back(std::move(f));
    }
    cv.notify_one();
  }
  void drain() {
    std::promise<void> p;
    auto fut = p.get_future();
    push([&p] { p.set_value(); });
    fut.wait();
  }
};

namespace {

std::atomic<uint64_t> g_ops{0};
std::atomic<unsigned> g_copy_delay_us{0};
// Self-check of the harness: with CPU_HIP_EVENTS_COMPLETE_EARLY set, waiting for an event returns at once, as if
// the device were already done - the engine then reuses ring slots whose copies are still queued, which the
// sanitizer must report (tests/test_host_sanitizers.py expects that run to fail).
const bool g_events_lie = std::getenv("CPU_HIP_EVENTS_COMPLETE_EARLY") != nullptr;

struct Runtime {
  std::mutex mu;
  std::vector<ihipStream_t*> streams;            // created and not yet destroyed
  std::unique_ptr<ihipStream_t> null_stream;     // made on first use
  std::map<uintptr_t, size_t> pinned;            // hipHostMalloc blocks
  ihipStream_t* of(hipStream_t s) {
    if (s) return s;
    std::lock_guard<std::mutex> lk(mu);
    if (!null_stream) null_stream = std::make_unique<ihipStream_t>();
    return null_stream.get();
  }
  bool is_pinned(const void* p, size_t n) {
    std::lock_guard<std::mutex> lk(mu);
    const uintptr_t a = reinterpret_cast<uintptr_t>(p);
    auto it = pinned.upper_bound(a);
    if (it == pinned.begin()) return false;
    --it;
    return a >= it->first && a + n <= it->first + it->second;
  }
  void sync_all() {
    std::vector<ihipStream_t*> all;
    {
      std::lock_guard<std::mutex> lk(mu);
      all = streams;
      if (null_stream) all.push_back(null_stream.get());
    }
    for (auto* s : all) s->drain();
  }
};
Runtime& rt() {
  static Runtime r;
  return r;
}

void* alloc_aligned(size_t n, size_t align) {
  const size_t bytes = (n ? n : 1) + align - 1;
  return std::aligned_alloc(align, bytes / align * align);
}

}  // namespace

namespace cpu_hip {
void enqueue(hipStream_t stream, std::function<void()> work) {
  rt().of(stream)->push([w = std::move(work)] {
    w();
    g_ops.fetch_add(1, std::memory_order_relaxed);
  });
}
uint64_t operations_run() { return g_ops.load(); }
void set_copy_delay_us(unsigned us) { g_copy_delay_us.store(us); }
}  // namespace cpu_hip

const char* hipGetErrorString(hipError_t e) {
  switch (e) {
    case hipSuccess: return "no error";
    case hipErrorInvalidValue: return "invalid argument";
    case hipErrorOutOfMemory: return "out of memory";
    case hipErrorNotReady: return "device not ready";
    case hipErrorNotSupported: return "operation not supported by the CPU stand-in";
  }
  return "unknown error";
}
hipError_t hipGetLastError(void) { return hipSuccess; }
hipError_t hipGetDeviceCount(int* n) {
  *n = 1;
  return hipSuccess;
}
hipError_t hipSetDevice(int device) { return device == 0 ? hipSuccess : hipErrorInvalidValue; }
hipError_t hipDeviceSynchronize(void) {
  rt().sync_all();
  return hipSuccess;
}

hipError_t hipMalloc(void** p, size_t n) {
  *p = alloc_aligned(n, 256);
  return *p ? hipSuccess : hipErrorOutOfMemory;
}
hipError_t hipFree(void* p) {
  rt().sync_all();  // as the runtime does: nothing in flight may still use the block
  std::free(p);
  return hipSuccess;
}
hipError_t hipHostMalloc(void** p, size_t n, unsigned) {
  *p = alloc_aligned(n, 4096);
  if (!*p) return hipErrorOutOfMemory;
  std::lock_guard<std::mutex> lk(rt().mu);
  rt().pinned[reinterpret_cast<uintptr_t>(*p)] = n;
  return hipSuccess;
}
hipError_t hipHostFree(void* p) {
  if (!p) return hipSuccess;
  rt().sync_all();
  {
    std::lock_guard<std::mutex> lk(rt().mu);
    rt().pinned.erase(reinterpret_cast<uintptr_t>(p));
  }
  std::free(p);
  return hipSuccess;
}
hipError_t hipHostGetDevicePointer(void** dev, void* host, unsigned) {
  *dev = host;
  return hipSuccess;
}
hipError_t hipMemset(void* p, int value, size_t n) {
  std::memset(p, value, n);
  return hipSuccess;
}
hipError_t hipMemcpy(void* dst, const void* src, size_t n, hipMemcpyKind) {
  std::memcpy(dst, src, n);
  return hipSuccess;
}
hipError_t hipMemcpyAsync(void* dst, const void* src, size_t n, hipMemcpyKind kind, hipStream_t stream) {
  if (n == 0) return hipSuccess;
  auto delay = [] {
    if (const unsigned us = g_copy_delay_us.load()) std::this_thread::sleep_for(std::chrono::microseconds(us));
  };
  if (kind == hipMemcpyHostToDevice && !rt().is_pinned(src, n)) {
    // pageable source: the runtime stages it before the call returns
    auto staged = std::make_shared<std::vector<uint8_t>>(static_cast<const uint8_t*>(src), static_cast<const uint8_t*>(src) + n);
    cpu_hip::enqueue(stream, [dst, staged, delay] {
      delay();
      std::memcpy(dst, staged->data(), staged->size());
    });
    return hipSuccess;
  }
  cpu_hip::enqueue(stream, [dst, src, n, delay] {
    delay();
    std::memcpy(dst, src, n);
  });
  if (kind == hipMemcpyDeviceToHost && !rt().is_pinned(dst, n)) rt().of(stream)->drain();  // pageable destination: synchronous
  return hipSuccess;
}
hipError_t hipGetSymbolAddress(void** p, const void* symbol) {
  *p = const_cast<void*>(symbol);
  return hipSuccess;
}

hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned) {
  *s = new ihipStream_t();
  std::lock_guard<std::mutex> lk(rt().mu);
  rt().streams.push_back(*s);
  return hipSuccess;
}
hipError_t hipStreamDestroy(hipStream_t s) {
  if (!s) return hipErrorInvalidValue;
  {
    std::lock_guard<std::mutex> lk(rt().mu);
    auto& v = rt().streams;
    for (size_t i = 0; i < v.size(); ++i)
      if (v[i] == s) {
        v.erase(v.begin() + (long)i);
        break;
      }
  }
  delete s;  // runs what is queued, then joins
  return hipSuccess;
}
hipError_t hipStreamSynchronize(hipStream_t s) {
  rt().of(s)->drain();
  return hipSuccess;
}
hipError_t hipStreamIsCapturing(hipStream_t, hipStreamCaptureStatus* status) {
  *status = hipStreamCaptureStatusNone;
  return hipSuccess;
}

hipError_t hipEventCreate(hipEvent_t* ev) {
  *ev = new ihipEvent_t();
  return hipSuccess;
}
hipError_t hipEventCreateWithFlags(hipEvent_t* ev, unsigned) { return hipEventCreate(ev); }
hipError_t hipEventDestroy(hipEvent_t ev) {
  delete ev;  // operations already queued keep the state alive
  return hipSuccess;
}
hipError_t hipEventRecord(hipEvent_t ev, hipStream_t s) {
  if (!ev) return hipErrorInvalidValue;
  auto st = ev->st;
  uint64_t gen;
  {
    std::lock_guard<std::mutex> lk(st->mu);
    gen = ++st->recorded;
  }
  cpu_hip::enqueue(s, [st, gen] {
    {
      std::lock_guard<std::mutex> lk(st->mu);
      if (gen > st->done) st->done = gen;
      st->when = std::chrono::steady_clock::now();
    }
    st->cv.notify_all();
  });
  return hipSuccess;
}
hipError_t hipEventQuery(hipEvent_t ev) {
  if (!ev) return hipErrorInvalidValue;
  if (g_events_lie) return hipSuccess;
  std::lock_guard<std::mutex> lk(ev->st->mu);
  return ev->st->done >= ev->st->recorded ? hipSuccess : hipErrorNotReady;
}
hipError_t hipEventSynchronize(hipEvent_t ev) {
  if (!ev) return hipErrorInvalidValue;
  if (g_events_lie) return hipSuccess;
  auto st = ev->st;
  std::unique_lock<std::mutex> lk(st->mu);
  const uint64_t target = st->recorded;
  st->cv.wait(lk, [&] { return st->done >= target; });
  return hipSuccess;
}
hipError_t hipStreamWaitEvent(hipStream_t s, hipEvent_t ev, unsigned) {
  if (!ev) return hipErrorInvalidValue;
  auto st = ev->st;
  uint64_t target;
  {
    std::lock_guard<std::mutex> lk(st->mu);
    target = st->recorded;  // the record that has been issued when this call is made
  }
  cpu_hip::enqueue(s, [st, target] {
    std::unique_lock<std::mutex> lk(st->mu);
    st->cv.wait(lk, [&] { return st->done >= target; });
  });
  return hipSuccess;
}
hipError_t hipEventElapsedTime(float* ms, hipEvent_t a, hipEvent_t b) {
  if (!a || !b) return hipErrorInvalidValue;
  std::chrono::steady_clock::time_point ta, tb;
  {
    std::lock_guard<std::mutex> lk(a->st->mu);
    if (a->st->done < a->st->recorded || !a->st->recorded) return hipErrorNotReady;
    ta = a->st->when;
  }
  {
    std::lock_guard<std::mutex> lk(b->st->mu);
    if (b->st->done < b->st->recorded || !b->st->recorded) return hipErrorNotReady;
    tb = b->st->when;
  }
  *ms = std::chrono::duration<float, std::milli>(tb - ta).count();
  return hipSuccess;
}
