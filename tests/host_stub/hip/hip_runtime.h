// A stand-in for the HIP runtime API, for building the library's host runtime
// (mooncake_amd/csrc/ep_runtime.hip) without a GPU: tests/test_host_runtime_tsan.py compiles the
// runtime against this header with the host compiler and ThreadSanitizer and drives its per-rank
// collectives from many threads.  Streams and events are counters, device memory is host memory,
// kernel launches (tests/host_stub/kernels_stub.cpp) are counted and do nothing.
//
// The real runtime is thread-safe, so this one is too - but with relaxed atomics only, never a lock:
// a lock in here would order the library's threads and hide a data race from the sanitizer.
#pragma once

#include <atomic>
#include <cstdint>
#include <cstdlib>
#include <cstring>

#define __device__
#define __host__
#define __global__
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (&(x))

typedef enum hipError_t {
    hipSuccess = 0,
    hipErrorInvalidValue = 1,
    hipErrorOutOfMemory = 2,
    hipErrorNotReady = 600,
} hipError_t;

struct ihipStream_t {
    std::atomic<long> enqueued{0};        // operations put on the stream so far
};
struct ihipEvent_t {
    std::atomic<long> recorded{-1};       // the stream's count when the event was last recorded
    std::atomic<long> waits{0};
};
typedef ihipStream_t* hipStream_t;
typedef ihipEvent_t* hipEvent_t;

enum { hipStreamNonBlocking = 1, hipEventDisableTiming = 2 };
typedef enum hipStreamCaptureStatus {
    hipStreamCaptureStatusNone = 0,
    hipStreamCaptureStatusActive = 1,
    hipStreamCaptureStatusInvalidated = 2,
} hipStreamCaptureStatus;
typedef enum hipStreamCaptureMode {
    hipStreamCaptureModeGlobal = 0,
    hipStreamCaptureModeThreadLocal = 1,
    hipStreamCaptureModeRelaxed = 2,
} hipStreamCaptureMode;

namespace hip_stub {
// what the driver reads afterwards
inline std::atomic<long> g_calls{0};          // API calls of any kind
inline std::atomic<long> g_live_events{0};    // created and not yet destroyed
inline std::atomic<long> g_live_streams{0};
inline std::atomic<long> g_live_allocs{0};
inline ihipStream_t g_null_stream;
inline ihipStream_t* resolve(hipStream_t s) { return s ? s : &g_null_stream; }
inline void touch() { g_calls.fetch_add(1, std::memory_order_relaxed); }
}  // namespace hip_stub

inline const char* hipGetErrorString(hipError_t e) { return e == hipSuccess ? "no error" : "stub error"; }
inline hipError_t hipGetLastError() { return hipSuccess; }
inline hipError_t hipGetDevice(int* d) { hip_stub::touch(); *d = 0; return hipSuccess; }
inline hipError_t hipSetDevice(int) { hip_stub::touch(); return hipSuccess; }
inline hipError_t hipDeviceSynchronize() { hip_stub::touch(); return hipSuccess; }

inline hipError_t hipMalloc(void** p, size_t n) {
    hip_stub::touch();
    *p = std::malloc(n ? n : 1);
    if (!*p) return hipErrorOutOfMemory;
    hip_stub::g_live_allocs.fetch_add(1, std::memory_order_relaxed);
    return hipSuccess;
}
template <typename T>
inline hipError_t hipMalloc(T** p, size_t n) { return hipMalloc((void**)p, n); }
inline hipError_t hipFree(void* p) {
    hip_stub::touch();
    if (p) hip_stub::g_live_allocs.fetch_sub(1, std::memory_order_relaxed);
    std::free(p);
    return hipSuccess;
}
inline hipError_t hipMemset(void* p, int v, size_t n) { hip_stub::touch(); std::memset(p, v, n); return hipSuccess; }
inline hipError_t hipGetSymbolAddress(void** p, const void* symbol) { hip_stub::touch(); *p = (void*)symbol; return hipSuccess; }

inline hipError_t hipStreamCreateWithFlags(hipStream_t* s, unsigned) {
    hip_stub::touch();
    *s = new ihipStream_t();
    hip_stub::g_live_streams.fetch_add(1, std::memory_order_relaxed);
    return hipSuccess;
}
inline hipError_t hipStreamDestroy(hipStream_t s) {
    hip_stub::touch();
    hip_stub::g_live_streams.fetch_sub(1, std::memory_order_relaxed);
    delete s;
    return hipSuccess;
}
inline hipError_t hipStreamSynchronize(hipStream_t) { hip_stub::touch(); return hipSuccess; }
// a stream is "busy" every other time it is asked, so that both answers are exercised
inline hipError_t hipStreamQuery(hipStream_t s) {
    hip_stub::touch();
    return (hip_stub::resolve(s)->enqueued.fetch_add(1, std::memory_order_relaxed) & 1) ? hipErrorNotReady : hipSuccess;
}
inline hipError_t hipStreamGetCaptureInfo(hipStream_t, hipStreamCaptureStatus* status, unsigned long long* id) {
    hip_stub::touch();
    *status = hipStreamCaptureStatusNone;
    if (id) *id = 0;
    return hipSuccess;
}
inline hipError_t hipThreadExchangeStreamCaptureMode(hipStreamCaptureMode*) { hip_stub::touch(); return hipSuccess; }

inline hipError_t hipEventCreateWithFlags(hipEvent_t* e, unsigned) {
    hip_stub::touch();
    *e = new ihipEvent_t();
    hip_stub::g_live_events.fetch_add(1, std::memory_order_relaxed);
    return hipSuccess;
}
inline hipError_t hipEventCreate(hipEvent_t* e) { return hipEventCreateWithFlags(e, 0); }
inline hipError_t hipEventDestroy(hipEvent_t e) {
    hip_stub::touch();
    hip_stub::g_live_events.fetch_sub(1, std::memory_order_relaxed);
    delete e;
    return hipSuccess;
}
inline hipError_t hipEventRecord(hipEvent_t e, hipStream_t s) {
    hip_stub::touch();
    e->recorded.store(hip_stub::resolve(s)->enqueued.fetch_add(1, std::memory_order_relaxed) + 1,
                      std::memory_order_relaxed);
    return hipSuccess;
}
inline hipError_t hipStreamWaitEvent(hipStream_t s, hipEvent_t e, unsigned) {
    hip_stub::touch();
    e->waits.fetch_add(1, std::memory_order_relaxed);
    hip_stub::resolve(s)->enqueued.fetch_add(1, std::memory_order_relaxed);
    return hipSuccess;
}
inline hipError_t hipEventSynchronize(hipEvent_t e) {
    hip_stub::touch();
    return e->recorded.load(std::memory_order_relaxed) >= 0 ? hipSuccess : hipErrorNotReady;
}
inline hipError_t hipEventElapsedTime(float* ms, hipEvent_t, hipEvent_t) { hip_stub::touch(); *ms = 0.0f; return hipSuccess; }
