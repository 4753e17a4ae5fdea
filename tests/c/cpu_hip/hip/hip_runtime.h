// A stand-in for the part of the HIP runtime that the host engine (modelexpress_amd/csrc/mxp_engine.cpp)
// calls, on the CPU: test infrastructure for running the engine's threads, ring and stream logic under
// ThreadSanitizer and AddressSanitizer (tests/test_host_sanitizers.py).  Not part of the product.
//
// Model (cpu_hip.cpp): "device memory" is host memory; a stream is a worker thread that runs what was
// queued on it in order; an event completes when the worker reaches its record; a copy out of pageable
// memory is staged at the call, a copy out of hipHostMalloc memory reads it when the worker gets there -
// so a slot that is overwritten before its copy ran is a data race the sanitizer sees, as it would be a
// wrong transfer on the GPU.
#pragma once
#include <stddef.h>
#include <stdint.h>

#define __host__
#define __device__
#define __global__
#define __forceinline__ inline
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) x

typedef enum hipError_t {
  hipSuccess = 0,
  hipErrorInvalidValue = 1,
  hipErrorOutOfMemory = 2,
  hipErrorNotReady = 600,
  hipErrorNotSupported = 801
} hipError_t;

typedef struct ihipStream_t* hipStream_t;
typedef struct ihipEvent_t* hipEvent_t;

typedef enum hipMemcpyKind {
  hipMemcpyHostToHost = 0,
  hipMemcpyHostToDevice = 1,
  hipMemcpyDeviceToHost = 2,
  hipMemcpyDeviceToDevice = 3,
  hipMemcpyDefault = 4
} hipMemcpyKind;

typedef enum hipStreamCaptureStatus {
  hipStreamCaptureStatusNone = 0,
  hipStreamCaptureStatusActive = 1,
  hipStreamCaptureStatusInvalidated = 2
} hipStreamCaptureStatus;

#define hipStreamNonBlocking 0x01
#define hipEventDisableTiming 0x02
#define hipHostMallocDefault 0x0

const char* hipGetErrorString(hipError_t e);
hipError_t hipGetLastError(void);
hipError_t hipGetDeviceCount(int* n);
hipError_t hipSetDevice(int device);
hipError_t hipDeviceSynchronize(void);

hipError_t hipMalloc(void** p, size_t n);
hipError_t hipFree(void* p);
hipError_t hipHostMalloc(void** p, size_t n, unsigned flags);
hipError_t hipHostFree(void* p);
hipError_t hipHostGetDevicePointer(void** dev, void* host, unsigned flags);
hipError_t hipMemset(void* p, int value, size_t n);
hipError_t hipMemcpy(void* dst, const void* src, size_t n, hipMemcpyKind kind);
hipError_t hipMemcpyAsync(void* dst, const void* src, size_t n, hipMemcpyKind kind, hipStream_t stream);
hipError_t hipGetSymbolAddress(void** p, const void* symbol);

hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned flags);
hipError_t hipStreamDestroy(hipStream_t s);
hipError_t hipStreamSynchronize(hipStream_t s);
hipError_t hipStreamWaitEvent(hipStream_t s, hipEvent_t ev, unsigned flags);
hipError_t hipStreamIsCapturing(hipStream_t s, hipStreamCaptureStatus* status);

hipError_t hipEventCreate(hipEvent_t* ev);
hipError_t hipEventCreateWithFlags(hipEvent_t* ev, unsigned flags);
hipError_t hipEventDestroy(hipEvent_t ev);
hipError_t hipEventRecord(hipEvent_t ev, hipStream_t s);
hipError_t hipEventQuery(hipEvent_t ev);
hipError_t hipEventSynchronize(hipEvent_t ev);
hipError_t hipEventElapsedTime(float* ms, hipEvent_t a, hipEvent_t b);

#ifdef __cplusplus
#include <functional>
namespace cpu_hip {
// Queues `work` on `stream` (null = the default stream); it runs on that stream's worker thread after
// everything queued before it.  What the stand-ins for the kernel launches use.
void enqueue(hipStream_t stream, std::function<void()> work);
// Counters for the test driver: operations run so far, and a delay (microseconds) every copy sleeps
// before it reads its source, which widens the window in which a slot could be overwritten too early.
uint64_t operations_run();
void set_copy_delay_us(unsigned us);
}  // namespace cpu_hip
#endif
