// Kernel launchers of the host-only build (see hip/hip_runtime.h beside this file): every launch is
// counted on its stream and does nothing.  The planning arithmetic is the library's own
// (mooncake_amd/csrc/ep_plan.cpp is compiled into the same program).
#include "ep_kernels.h"

namespace mcep {

std::atomic<long> g_stub_launches{0};

static hipError_t launched(hipStream_t stream) {
    g_stub_launches.fetch_add(1, std::memory_order_relaxed);
    hip_stub::resolve(stream)->enqueued.fetch_add(1, std::memory_order_relaxed);
    return hipSuccess;
}

hipError_t launch_table_write(uint64_t*, const uint64_t*, int, hipStream_t s) { return launched(s); }
hipError_t launch_count(const uint64_t*, const RoutingScratch&, const DispatchSource&, const Dims&, hipStream_t s) {
    return launched(s);
}
hipError_t launch_pack(const uint64_t*, const RoutingScratch&, const DispatchSource&, float*, const Dims&, bool,
                       const Tuning&, bool, bool, hipStream_t s) {
    return launched(s);
}
hipError_t launch_dispatch_small(const SmallTable&, int32_t*, const Dims&, bool, const Tuning&, hipStream_t s) {
    return launched(s);
}
hipError_t launch_resolve(const uint64_t*, CombineRoute*, uint32_t, bool, const Dims&, const Tuning&, hipStream_t s) {
    return launched(s);
}
hipError_t launch_reduce(const uint64_t*, const CombineRoute*, uint32_t, const RoutingScratch&, bool,
                         const CombineSource&, const void*, const Dims&, const Tuning&, hipStream_t s) {
    return launched(s);
}
hipError_t launch_reduce_packed(const uint64_t*, const CombineRoute*, uint32_t, const RoutingScratch&, bool,
                                const CombineSource&, const void*, const float*, bool, const Dims&, const Tuning&,
                                hipStream_t s) {
    return launched(s);
}
hipError_t launch_cast_back(const uint64_t*, void*, const float*, bool, long long, const Dims&, hipStream_t s) {
    return launched(s);
}
hipError_t launch_copy(void*, const void*, size_t, hipStream_t s) { return launched(s); }
void set_stream_occupancy(int) {}
hipError_t launch_stream(int, void*, const void*, size_t, hipStream_t s) { return launched(s); }
hipError_t launch_stream_rows(void*, const void*, int, long long, int, long long, int, hipStream_t s) {
    return launched(s);
}
hipError_t launch_stream_rows_scatter(void*, const void*, int, long long, int, long long, int, hipStream_t s) {
    return launched(s);
}
hipError_t launch_clear_words(const uint64_t*, int, int, hipStream_t s) { return launched(s); }
hipError_t launch_fill_u32(void*, uint32_t, size_t, hipStream_t s) { return launched(s); }

}  // namespace mcep
