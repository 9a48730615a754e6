// Host runtime behind the C ABI (include/mooncake_ep_hip.h): the logical EP
// world, per-rank buffers with the reference's call signatures, event and
// hook objects.  Mirrors the host side of the reference
// (mooncake-ep/src/mooncake_ep_buffer.cpp:193-474) minus everything that
// exists only to move bytes between GPUs: there is no communication buffer,
// no double buffering, no peer bootstrap.
#include "../../include/mooncake_ep_hip.h"

#include <hip/hip_runtime.h>

#include <linux/futex.h>
#include <sched.h>
#include <sys/syscall.h>
#include <unistd.h>

#include <atomic>
#include <chrono>
#include <climits>
#include <cstdio>
#include <cstring>
#include <deque>
#include <functional>
#include <memory>
#include <mutex>
#include <string>
#include <vector>

#include "ep_debug.h"
#include "ep_kernels.h"

using namespace mcep;

// Scratch of the allocation-free dispatch (mc_ep_world_dispatch_noalloc): the routing state, the fp8
// scale staging rows and the rank table of one call, carved out of one array that every GPU the
// library runs on holds until the process ends.  Host code never passes the array's name to a
// kernel: the device address is fetched once per device with hipGetSymbolAddress (world creation)
// and kept in g_scratch_ptr.
constexpr size_t kStaticScratchBytes = (size_t)16 << 20;
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

namespace {

constexpr int kMaxDevices = 64;
unsigned char* g_scratch_ptr[kMaxDevices] = {};

thread_local std::string g_last_error;

// One lock for the host bookkeeping of every world, buffer, round, event and hook of the process (an
// EventHandle may outlive its world, so the lock cannot live in the world): entry points take it for as
// long as they touch that state and enqueue work, not while they wait for a collective's peers or for
// its results (the short waits of set-up - a world's destruction, scratch that grows - are inside).  Per-rank
// callers that block until their collective is complete (option "blocking") sleep on their round's own
// word (Round::published) with the lock given up, and return without taking it again: when a round of 32
// ranks completes, its 31 sleepers wake side by side instead of queueing for one mutex (which is what a
// condition variable makes of a broadcast, and took most of a millisecond per step).
std::mutex g_mu;
using Lock = std::unique_lock<std::mutex>;

long futex_call(std::atomic<int>* word, int op, int value, const timespec* timeout) {
    static_assert(sizeof(std::atomic<int>) == sizeof(int), "the futex word is the atomic's storage");
    return syscall(SYS_futex, reinterpret_cast<int*>(word), op, value, timeout, nullptr, 0);
}

int fail(int code, const std::string& msg) {
    g_last_error = msg;
    return code;
}

#define MC_ASSERT(cond)                                                                                        \
    do {                                                                                                       \
        if (!(cond))                                                                                           \
            return fail(MC_EP_ERR_ASSERT, std::string("Failed: Assertion error ") + __FILE__ + ":" +          \
                                              std::to_string(__LINE__) + " '" #cond "'");                      \
    } while (0)

#define MC_HIP(cmd)                                                                                            \
    do {                                                                                                       \
        hipError_t e_ = (cmd);                                                                                 \
        if (e_ != hipSuccess)                                                                                  \
            return fail(MC_EP_ERR_HIP, std::string("Failed: HIP error ") + __FILE__ + ":" +                   \
                                           std::to_string(__LINE__) + " '" + hipGetErrorString(e_) + "'");    \
    } while (0)

// Events are reused: a collective needs one or two per round, and creating and destroying them costs
// more host time than the rest of a per-rank call.  Shared by a world and its rounds, which may outlive it
// (an EventHandle still held by the caller).
struct EventPool {
    std::vector<hipEvent_t> idle;
    int take(hipEvent_t* out) {
        if (!idle.empty()) {
            *out = idle.back();
            idle.pop_back();
            return MC_EP_OK;
        }
        MC_HIP(hipEventCreateWithFlags(out, hipEventDisableTiming));
        return MC_EP_OK;
    }
    void give(hipEvent_t e) { idle.push_back(e); }
    ~EventPool() {
        for (hipEvent_t e : idle) (void)hipEventDestroy(e);
    }
};

// One collective call (a "round"): the j-th dispatch (or combine) of every live rank.
struct Round {
    bool launched = false;
    std::string failure;          // why the round's launch failed, if it did
    // For callers that sleep until the round is decided (option "blocking"): 0 while ranks are missing, then
    // 1 (launched) or 2 (the launch failed; `failure` was written before).  Written once, with the lock held;
    // read without it.
    std::atomic<int> published{0};
    std::atomic<int> sleepers{0};
    void publish() {
        published.store(failure.empty() ? 1 : 2, std::memory_order_seq_cst);
        if (sleepers.load(std::memory_order_seq_cst) > 0) futex_call(&published, FUTEX_WAKE_PRIVATE, INT_MAX, nullptr);
    }
    // false: still undecided after `ms` milliseconds.  The first `spin_us` microseconds are spent looking at
    // the word and offering the core to other threads in turn, not asleep: when every rank's thread is on its
    // way, the round is decided within tens of microseconds, and putting a thread to sleep and waking it costs
    // about as much again per thread (more inside a virtual machine).
    bool wait_published(int ms, int spin_us) {
        if (published.load(std::memory_order_acquire) != 0) return true;
        const auto start = std::chrono::steady_clock::now();
        const auto deadline = start + std::chrono::milliseconds(ms < 0 ? 0 : ms);
        const auto spin_end = start + std::chrono::microseconds(spin_us < 0 ? 0 : spin_us);
        while (std::chrono::steady_clock::now() < spin_end) {
            if (published.load(std::memory_order_acquire) != 0) return true;
            sched_yield();
        }
        sleepers.fetch_add(1, std::memory_order_seq_cst);
        bool decided = true;
        while (published.load(std::memory_order_seq_cst) == 0) {
            const auto left = std::chrono::duration_cast<std::chrono::nanoseconds>(deadline - std::chrono::steady_clock::now());
            if (left.count() <= 0) {
                decided = false;
                break;
            }
            timespec ts;
            ts.tv_sec = (time_t)(left.count() / 1000000000ll);
            ts.tv_nsec = (long)(left.count() % 1000000000ll);
            futex_call(&published, FUTEX_WAIT_PRIVATE, 0, &ts);   // returns at once if the word is no longer 0
        }
        sleepers.fetch_sub(1, std::memory_order_seq_cst);
        return decided || published.load(std::memory_order_acquire) != 0;
    }
    hipEvent_t done = nullptr;
    std::shared_ptr<EventPool> pool;       // where `done` came from and goes back to
    std::vector<hipStream_t> waited;       // streams that already wait for `done`: a second wait adds nothing
    // A round whose callers all asked for a receive hook is launched in two parts, like the
    // reference's SEND / RECV phases (mooncake_ep_buffer.cpp:303-305, :330-335): the call that
    // completes it enqueues the layout and data kernels, the first hook that is called enqueues the
    // rest (`finish`) and records `done`; every hook then makes its rank's stream wait for `done`.
    std::function<int()> finish;
    hipStream_t launch_stream = nullptr;
    ~Round() {
        if (done && pool) pool->give(done);
        else if (done) (void)hipEventDestroy(done);
    }
    // makes `stream` wait for the round's completion, once
    int make_wait(hipStream_t stream) {
        for (hipStream_t s : waited)
            if (s == stream) return MC_EP_OK;
        if (done == nullptr)
            return fail(MC_EP_ERR_ASSERT, "Failed: a stream that took no part in the collective asks to wait for "
                                          "it, and no caller of the round asked for a completion event");
        MC_HIP(hipStreamWaitEvent(stream, done, 0));
        waited.push_back(stream);
        return MC_EP_OK;
    }
};

// How a blocking caller (a thread per rank) takes its share of a round's stream hand-offs off the thread
// that launches the round: it looks at its own stream when it posts (an event recorded there if anything is
// in flight, for the launch stream to wait on), and makes its own stream wait for the round when it wakes.
// The launching thread - the last rank to arrive, with every other rank waiting for it - is left with one wait
// per busy stream instead of a query, a record and two waits per rank.
struct StreamHandOff {
    bool by_caller = false;       // the caller did / does its part itself
    hipEvent_t before = nullptr;  // what the caller's stream held at the call; null: it was idle
};

struct DispatchPost {
    bool present = false;
    uint64_t x = 0, topk_idx = 0, active_ranks = 0;
    int num_tokens = 0, hidden = 0, num_topk = 0, max_tokens = 0, num_experts = 0, timeout_us = -1, use_fp8 = 0;
    uint64_t recv_x = 0, recv_scales = 0, recv_count = 0, src_info = 0, layout_range = 0;
    bool async = false, hook = false;
    hipStream_t stream = nullptr;
    StreamHandOff hand;
};

struct CombinePost {
    bool present = false;
    uint64_t x = 0, topk_idx = 0, topk_weights = 0, src_info = 0, layout_range = 0, active_ranks = 0, out = 0;
    int num_tokens = 0, hidden = 0, num_topk = 0, max_tokens = 0, num_experts = 0, timeout_us = -1;
    bool async = false, hook = false;
    hipStream_t stream = nullptr;
    StreamHandOff hand;
};

template <typename Post>
struct PendingRound {
    std::vector<Post> posts;
    std::shared_ptr<Round> state;
};

}  // namespace

struct mc_ep_world {
    int device = 0;
    int R = 0;
    hipStream_t comm_stream = nullptr;
    // Launch sequences of one world share its rank tables, routing state, routes and staged scales,
    // so they are serialised: a sequence that runs on another stream than the one before it first
    // waits for what that stream holds (order_begin).
    hipEvent_t ordered = nullptr;
    hipStream_t ordered_stream = nullptr;                // where the world's last eager sequence ran
    hipEvent_t fence = nullptr;                          // callers' streams -> launch stream, re-recorded per use
    std::shared_ptr<EventPool> events = std::make_shared<EventPool>();
    bool ordered_valid = false;
    uint64_t* d_tbl[3] = {nullptr, nullptr, nullptr};   // dispatch, combine, consumer pointer tables
    std::vector<uint64_t> tbl_cache[3];                  // what the device tables hold
    // Calls recorded into a HIP graph get tables of their own (a replay must not depend on what later
    // eager calls leave in the shared ones); calls with equal tables share a slot.
    uint64_t* d_captured_tbl[3] = {nullptr, nullptr, nullptr};
    std::vector<std::vector<uint64_t>> captured_tbls[3];
    bool dispatch_captured = false;                      // some dispatch of this world lives in a graph
    // routing state of the last dispatch (see RoutingScratch)
    int32_t* d_ucount = nullptr;
    size_t ucount_cap = 0;
    int32_t* d_ubegin = nullptr;
    size_t ubegin_cap = 0;
    int32_t* d_ucount_t = nullptr;
    size_t ucount_t_cap = 0;
    int32_t* d_selpos = nullptr;
    size_t selpos_cap = 0;
    int32_t* d_selrow = nullptr;
    size_t selrow_cap = 0;
    int32_t* d_row_src = nullptr;
    size_t row_src_cap = 0;
    int32_t* d_counts = nullptr;
    size_t counts_cap = 0;
    uint32_t* d_chunk_map = nullptr;     // work list of the cast-back kernel, 4 words per entry
    size_t chunk_map_cap = 0;
    // what the last dispatch was called with, so that a combine given that
    // dispatch's handle can reuse its routing state instead of re-deriving rows
    struct LastDispatch {
        bool valid = false;
        int hidden = 0, num_topk = 0, max_tokens = 0, num_experts = 0;
        std::vector<uint64_t> topk_idx, recv_x, src_info, layout_range;
        std::vector<int32_t> num_tokens;
        bool data_done = false;                   // its pack phase has been launched too (and did not fail)
        bool captured = false;                    // recorded into a graph, and which capture
        unsigned long long capture_id = 0;
    } last;
    CombineRoute* d_routes = nullptr;             // combine's general path: one route per selection
    size_t route_cap = 0;                         // capacity in selections
    uint32_t stamp = 0;                           // launch counter the routes are stamped with
    float* d_scale_stage = nullptr;               // fp8 scales of each token before transposition
    size_t scale_stage_cap = 0;                   // capacity in floats
    void* d_zero_row = nullptr;
    std::vector<void*> retired;                   // outgrown scratch, freed with the world
    Tuning tuning;
    int launches = 0;                             // kernels the call in progress has enqueued (see last_*_launches)
    std::vector<char> silent;
    // per-rank collective bookkeeping
    std::deque<PendingRound<DispatchPost>> dispatch_rounds;
    std::deque<PendingRound<CombinePost>> combine_rounds;
    std::vector<long long> dispatch_calls, combine_calls;   // calls made per rank
    long long dispatch_base = 0, combine_base = 0;          // index of the front round
    std::shared_ptr<Round> unfinished;                      // the dispatch round whose second part no hook has enqueued yet

    mc_ep_world() = default;
    mc_ep_world(const mc_ep_world&) = delete;
    mc_ep_world& operator=(const mc_ep_world&) = delete;
    // also runs when creation fails half way
    ~mc_ep_world() {
        int prev = -1;
        const bool switched = hipGetDevice(&prev) == hipSuccess && prev != device && hipSetDevice(device) == hipSuccess;
        (void)hipDeviceSynchronize();
        void* owned[] = {d_tbl[0], d_tbl[1], d_tbl[2], d_captured_tbl[0], d_captured_tbl[1], d_captured_tbl[2],
                         d_ucount, d_ucount_t, d_ubegin, d_selpos, d_selrow, d_row_src, d_counts, d_chunk_map, d_routes,
                         d_scale_stage, d_zero_row};
        for (void* p : owned)
            if (p) (void)hipFree(p);
        for (void* p : retired) (void)hipFree(p);
        if (comm_stream) (void)hipStreamDestroy(comm_stream);
        if (ordered) (void)hipEventDestroy(ordered);
        if (fence) (void)hipEventDestroy(fence);
        if (switched) (void)hipSetDevice(prev);
    }
};

struct mc_ep_buffer {
    mc_ep_world* world = nullptr;
    int rank = 0;
    int64_t num_ep_buffer_bytes = 0;
    bool p2p_enabled = true;
    hipEvent_t before = nullptr;    // see StreamHandOff; re-recorded by every blocking call of the rank
    ~mc_ep_buffer() {
        if (before) (void)hipEventDestroy(before);
    }
};

struct mc_ep_event {
    std::shared_ptr<Round> round;   // deferred: completion of a collective
    hipEvent_t own = nullptr;       // immediate: recorded at creation
};

struct mc_ep_hook {
    mc_ep_world* world = nullptr;
    std::shared_ptr<Round> round;
    hipStream_t stream = nullptr;
};

namespace {

struct DeviceGuard {
    int prev = -1;
    bool changed = false;
    explicit DeviceGuard(int dev) {
        if (hipGetDevice(&prev) == hipSuccess && prev != dev) changed = (hipSetDevice(dev) == hipSuccess);
    }
    ~DeviceGuard() {
        if (changed) (void)hipSetDevice(prev);
    }
};

// Tables a world keeps for calls recorded into graphs, per kind of call.
constexpr int kCapturedTables = 256;

struct Capture {
    bool active = false;
    unsigned long long id = 0;
};

// Whether work issued to `stream` is being recorded into a graph rather than run.
int capture_of(hipStream_t stream, Capture* out) {
    *out = Capture{};
    if (stream == nullptr) return MC_EP_OK;   // the null stream cannot be captured
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    unsigned long long id = 0;
    MC_HIP(hipStreamGetCaptureInfo(stream, &status, &id));
    MC_ASSERT(status != hipStreamCaptureStatusInvalidated);
    out->active = status == hipStreamCaptureStatusActive;
    out->id = id;
    return MC_EP_OK;
}

// Set while a call is being recorded: scratch cannot be allocated then.
thread_local bool t_recording = false;

struct RecordingScope {
    bool prev;
    explicit RecordingScope(bool on) : prev(t_recording) { t_recording = on; }
    ~RecordingScope() { t_recording = prev; }
};

#define MC_NO_GROWTH_WHILE_RECORDING()                                                                         \
    do {                                                                                                       \
        if (t_recording)                                                                                       \
            return fail(MC_EP_ERR_ASSERT,                                                                      \
                        "Failed: the library's scratch memory would have to grow during stream capture; make "  \
                        "the same call once outside the capture first");                                        \
    } while (0)

// Scratch grows by replacement.  The outgrown allocation is kept until the world is destroyed
// (`retired`): kernels already queued, and graphs instantiated while it was current, hold its address
// in their arguments and go on using it - a graph's calls are self-contained (a recorded combine
// reuses only a dispatch of its own capture), so they stay right on the old memory.  Sizes grow
// geometrically, so the retired total stays below twice the live one.
template <typename T>
int grow_scratch(mc_ep_world* w, T** ptr, size_t* cap, size_t count, bool zero) {
    if (count <= *cap) return MC_EP_OK;
    MC_NO_GROWTH_WHILE_RECORDING();
    const size_t grown = count + count / 2 + 1024;
    T* fresh = nullptr;
    MC_HIP(hipMalloc((void**)&fresh, grown * sizeof(T)));
    if (zero) {
        const hipError_t e = hipMemset(fresh, 0, grown * sizeof(T));
        // the fill must have landed before a kernel on any stream reads the new memory
        const hipError_t e2 = e == hipSuccess ? hipStreamSynchronize(nullptr) : e;
        if (e2 != hipSuccess) {
            (void)hipFree(fresh);
            MC_HIP(e2);
        }
    }
    if (*ptr) w->retired.push_back(*ptr);
    *ptr = fresh;
    *cap = grown;
    return MC_EP_OK;
}

// stamps start at 1 and are never reset, so a zeroed route table holds no valid route
int ensure_routes(mc_ep_world* w, size_t selections) {
    return grow_scratch(w, &w->d_routes, &w->route_cap, selections, true);
}

template <typename T>
int ensure_scratch(mc_ep_world* w, T** ptr, size_t* cap, size_t count) {
    return grow_scratch(w, ptr, cap, count, true);
}

int ensure_scale_stage(mc_ep_world* w, size_t floats) {
    return grow_scratch(w, &w->d_scale_stage, &w->scale_stage_cap, floats, false);
}

// Puts the call's rank table on the device and returns where.  Eager calls share one table per kind,
// rewritten only when its contents change.  A call being recorded into a graph gets a slot that no
// eager call touches and that is never rewritten; it is filled right away on the world's own
// (non-capturing) stream, so the graph holds the call's kernels and nothing else.
int upload_table(mc_ep_world* w, int which, const std::vector<uint64_t>& tbl, const Capture& cap,
                 hipStream_t stream, const uint64_t** d_out) {
    if (!cap.active) {
        *d_out = w->d_tbl[which];
        if (w->tbl_cache[which] == tbl) return MC_EP_OK;
        MC_HIP(launch_table_write(w->d_tbl[which], tbl.data(), (int)tbl.size(), stream));
        w->launches += ((int)tbl.size() + kTableChunk - 1) / kTableChunk;
        w->tbl_cache[which] = tbl;
        return MC_EP_OK;
    }
    auto& known = w->captured_tbls[which];
    size_t slot = 0;
    while (slot < known.size() && known[slot] != tbl) ++slot;
    if (slot == known.size()) {
        if ((int)known.size() >= kCapturedTables)
            return fail(MC_EP_ERR_ASSERT, "Failed: too many distinct calls of one world recorded into graphs (" +
                                              std::to_string(kCapturedTables) + " sets of tensors per kind of call)");
        uint64_t* d_new = w->d_captured_tbl[which] + slot * tbl.size();
        MC_HIP(launch_table_write(d_new, tbl.data(), (int)tbl.size(), w->comm_stream));
        // waiting for another stream is among the calls a capture in progress forbids by default; this
        // one is safe (the world's stream takes no part in the capture), so say so for its duration
        hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
        MC_HIP(hipThreadExchangeStreamCaptureMode(&mode));
        const hipError_t waited = hipStreamSynchronize(w->comm_stream);
        (void)hipThreadExchangeStreamCaptureMode(&mode);
        MC_HIP(waited);
        known.push_back(tbl);
    }
    *d_out = w->d_captured_tbl[which] + slot * tbl.size();
    return MC_EP_OK;
}

// the reference's host assertions on shapes (mooncake_ep_buffer.cpp:202-206,
// :246-251, :351-354; mooncake_ep_kernel.cu:505, :781)
int check_dims(const mc_ep_world* w, int hidden, int num_topk, int max_tokens, int num_experts) {
    MC_ASSERT(num_experts > 0 && num_experts % w->R == 0);
    MC_ASSERT(hidden > 0 && hidden % 16 == 0 && hidden % 128 == 0);
    MC_ASSERT((size_t)hidden * 2 <= kZeroRowBytes);
    MC_ASSERT(num_topk > 0 && num_topk <= kMaxTopK);
    MC_ASSERT(max_tokens > 0);
    return MC_EP_OK;
}

// Evenly spaced per-rank tensors (every rank present) can be addressed from
// kernel arguments; otherwise base stays 0 and kernels use the rank table.
RankPtr uniform_ptr(const uint64_t* p, int R, bool enabled) {
    RankPtr u;
    if (!enabled || p[0] == 0) return u;
    const int64_t stride = R > 1 ? (int64_t)(p[1] - p[0]) : 0;
    for (int r = 0; r < R; ++r)
        if (p[r] == 0 || p[r] != p[0] + (uint64_t)(stride * r)) return u;
    u.base = p[0];
    u.stride = stride;
    return u;
}

int uniform_tokens(const int32_t* n, int R, bool enabled) {
    if (!enabled) return -1;
    for (int r = 1; r < R; ++r)
        if (n[r] != n[0]) return -1;
    return n[0];
}

RoutingScratch routing_scratch(const mc_ep_world* w) {
    return RoutingScratch{w->d_ucount, w->d_ucount_t, w->d_ubegin, w->d_selpos, w->d_selrow, w->d_counts, w->d_row_src};
}

// Enqueues what is left of a round that was launched in two parts (see Round::finish).
int finish_round(mc_ep_world* w, Round* round) {
    if (!round->finish) return MC_EP_OK;
    const std::function<int()> rest = std::move(round->finish);
    round->finish = nullptr;
    // the world's reference may be the last one (every hook of the round dropped without being called):
    // it is held here until the second part has been enqueued and its outcome recorded in the round
    std::shared_ptr<Round> keep;
    if (w->unfinished.get() == round) keep = std::move(w->unfinished);
    const int e = rest();
    if (e) round->failure = g_last_error;
    return e;
}

// Serialisation of a world's launch sequences across streams (see mc_ep_world::ordered).  Nothing is
// recorded while the world stays on one stream (an event per call costs 3-4 us of device time each);
// when a sequence arrives on another stream, the event is recorded on the previous stream then - it
// covers everything queued there so far, the world's earlier sequences included - and the new stream
// waits for it.  Calls being recorded into a graph take no part: a graph's order is its capturing
// stream's, and a stream that is capturing cannot be asked for an event of eager work.
int order_begin(mc_ep_world* w, hipStream_t stream, const Capture& cap) {
    if (cap.active) return MC_EP_OK;
    if (w->ordered_valid && w->ordered_stream != stream) {
        Capture prev;
        if (int rc = capture_of(w->ordered_stream, &prev)) return rc;
        if (!prev.active) {
            MC_HIP(hipEventRecord(w->ordered, w->ordered_stream));
            MC_HIP(hipStreamWaitEvent(stream, w->ordered, 0));
        }
    }
    w->ordered_stream = stream;
    w->ordered_valid = true;
    return MC_EP_OK;
}

int world_dispatch_impl(mc_ep_world* w, const uint64_t* x, const uint64_t* topk_idx, const int32_t* num_tokens,
                        int hidden, int num_topk, int max_tokens, int num_experts, int use_fp8,
                        const uint64_t* recv_x, const uint64_t* recv_scales, const uint64_t* recv_count,
                        const uint64_t* src_info, const uint64_t* layout_range, int phases, hipStream_t stream,
                        bool static_scratch = false) {
    const int R = w->R;
    if (int rc = check_dims(w, hidden, num_topk, max_tokens, num_experts)) return rc;
    MC_ASSERT(x != nullptr && topk_idx != nullptr && num_tokens != nullptr);
    MC_ASSERT(recv_x != nullptr && recv_count != nullptr && src_info != nullptr && layout_range != nullptr);
    if (use_fp8) {
        MC_ASSERT(((long long)R * max_tokens) % 4 == 0);
        MC_ASSERT(recv_scales != nullptr);
    }
    int tgrid = 0;
    long long selections = 0, list_rounds = 0;
    // the rank table: on the stack, so that the allocation-free variant touches no heap either
    uint64_t tbl[(size_t)DF_COUNT * MC_EP_MAX_QP_COUNT];
    const size_t tbl_words = (size_t)DF_COUNT * R;
    for (int r = 0; r < R; ++r) {
        MC_ASSERT(num_tokens[r] >= 0 && num_tokens[r] <= max_tokens);
        MC_ASSERT(num_tokens[r] == 0 || (x[r] != 0 && topk_idx[r] != 0));
        if (recv_x[r] != 0) {
            MC_ASSERT(recv_count[r] != 0 && src_info[r] != 0 && layout_range[r] != 0);
            if (use_fp8) MC_ASSERT(recv_scales[r] != 0);
        }
        tbl[DF_X * R + r] = x[r];
        tbl[DF_TOPK_IDX * R + r] = topk_idx[r];
        tbl[DF_RECV_X * R + r] = recv_x[r];
        tbl[DF_RECV_SCALES * R + r] = (use_fp8 && recv_scales) ? recv_scales[r] : 0;
        tbl[DF_RECV_COUNT * R + r] = recv_count[r];
        tbl[DF_SRC_INFO * R + r] = src_info[r];
        tbl[DF_LAYOUT_RANGE * R + r] = layout_range[r];
        tbl[DF_NUM_TOKENS * R + r] = (uint64_t)num_tokens[r];
        if (num_tokens[r] > tgrid) tgrid = num_tokens[r];
        selections += (long long)num_tokens[r] * num_topk;
        list_rounds += ((long long)num_tokens[r] * num_topk + kSmallListRound - 1) / kSmallListRound;
    }
    // A world that names few selections is dispatched in one launch, every wave rebuilding the routing it
    // needs from the index lists (dispatch_small_kernel); the rank table then travels in kernel arguments.
    // What that costs grows with the rounds of index-list entries a late wave reads one after another (every
    // rank's list is at least one round); measured against the launches it saves - two for an fp8 payload,
    // one for bf16 - it pays up to six rounds and four.
    const int rounds_limit = w->tuning.fused_small_rounds >= 0 ? w->tuning.fused_small_rounds : (use_fp8 ? 6 : 4);
    const bool fused = w->tuning.fused_small != 0 && phases == MC_EP_PHASE_ALL && R <= kSmallRanks && tgrid > 0 &&
                       selections <= (long long)w->tuning.fused_small_max && list_rounds <= (long long)rounds_limit;
    DeviceGuard guard(w->device);
    w->launches = 0;
    struct Tally {                                // the option "last_dispatch_launches", on every way out
        mc_ep_world* w;
        ~Tally() { w->tuning.last_dispatch_launches = w->launches; }
    } tally{w};
    // a new dispatch overwrites the staged scales and the routing state: the second part of a round
    // that still waits for its hook has to be enqueued first
    if (!static_scratch && (phases & MC_EP_PHASE_LAYOUT) && w->unfinished)
        if (int rc = finish_round(w, w->unfinished.get())) return rc;
    Dims d{R, num_experts, num_topk, hidden, max_tokens, tgrid};
    plan_units(d, w->tuning);
    // the count kernel keeps per-wave counts and prefixes of every expert in LDS
    MC_ASSERT(fused || count_lds_bytes(d) <= kMaxCountLdsBytes);
    MC_ASSERT(fused || d.units() <= kMaxUnits);
    const size_t UE = (size_t)d.units() * num_experts;
    const size_t stage_floats = use_fp8 ? (size_t)R * max_tokens * (hidden / 128) : 0;

    RoutingScratch sc{};
    float* stage = nullptr;
    const uint64_t* d_tbl = nullptr;
    Capture cap;
    if (static_scratch) {
        // every piece comes out of the device's static array; nothing is allocated, whatever the shape
        unsigned char* base = (w->device >= 0 && w->device < kMaxDevices) ? g_scratch_ptr[w->device] : nullptr;
        MC_ASSERT(base != nullptr);
        size_t used = 0;
        auto carve = [&](size_t bytes) {
            unsigned char* p = base + used;
            used += (bytes + 255) & ~(size_t)255;
            return p;
        };
        uint64_t* s_tbl = (uint64_t*)carve(tbl_words * sizeof(uint64_t));
        sc.ucount = (int32_t*)carve(UE * 4);
        sc.ucount_t = (int32_t*)carve((size_t)num_experts * kMaxSummedUnits * 4);
        sc.ubegin = (int32_t*)carve(UE * 4);
        sc.selpos = (int32_t*)carve((size_t)R * max_tokens * num_topk * 4);
        sc.selrow = (int32_t*)carve((size_t)R * max_tokens * num_topk * 4);
        sc.counts = (int32_t*)carve((size_t)num_experts * 4);
        sc.row_src = (int32_t*)carve((size_t)num_experts * R * max_tokens * 4);
        stage = (float*)carve(stage_floats * 4);
        if (used > kStaticScratchBytes)
            return fail(MC_EP_ERR_ASSERT,
                        "Failed: this shape needs " + std::to_string(used) + " bytes of scratch; the allocation-free "
                        "dispatch holds " + std::to_string(kStaticScratchBytes) + " (use mc_ep_world_dispatch)");
        // the table travels in kernel arguments on the call's own stream, every time: a recorded call
        // then carries its own copy, and nothing of the world's eager state is involved
        if (!fused) {
            MC_HIP(launch_table_write(s_tbl, tbl, (int)tbl_words, stream));
            w->launches += ((int)tbl_words + kTableChunk - 1) / kTableChunk;
        }
        d_tbl = s_tbl;
        // the world's own routing state is no longer that of "the last dispatch": combines resolve their handle
        w->last.valid = false;
    } else {
        if (int rc = capture_of(stream, &cap)) return rc;
        RecordingScope recording(cap.active);
        if (int rc = order_begin(w, stream, cap)) return rc;
        if (int rc = ensure_scratch(w, &w->d_selrow, &w->selrow_cap, (size_t)R * max_tokens * num_topk)) return rc;
        if (!fused) {
            // (the one-launch dispatch keeps no routing state but selrow, and needs no table in memory)
            if (int rc = ensure_scratch(w, &w->d_ucount, &w->ucount_cap, UE)) return rc;
            if (int rc = ensure_scratch(w, &w->d_ubegin, &w->ubegin_cap, UE)) return rc;
            if (int rc = ensure_scratch(w, &w->d_ucount_t, &w->ucount_t_cap, (size_t)num_experts * kMaxSummedUnits)) return rc;
            if (int rc = ensure_scratch(w, &w->d_selpos, &w->selpos_cap, (size_t)R * max_tokens * num_topk)) return rc;
            if (int rc = ensure_scratch(w, &w->d_row_src, &w->row_src_cap, (size_t)num_experts * R * max_tokens)) return rc;
            if (int rc = ensure_scratch(w, &w->d_counts, &w->counts_cap, (size_t)num_experts)) return rc;
            if (stage_floats > 0 && (phases & (MC_EP_PHASE_DATA | MC_EP_PHASE_FINISH)) && tgrid > 0) {
                if (int rc = ensure_scale_stage(w, stage_floats)) return rc;
                stage = w->d_scale_stage;
            }
            const std::vector<uint64_t> tbl_vec(tbl, tbl + tbl_words);
            if (int rc = upload_table(w, 0, tbl_vec, cap, stream, &d_tbl)) return rc;
        }
        sc = routing_scratch(w);
    }
    // what a combine has to know to recognise this dispatch's handle (see mc_ep_world::LastDispatch)
    auto remember = [&](bool data_done) {
        auto& ld = w->last;
        ld.valid = true;
        ld.hidden = hidden; ld.num_topk = num_topk; ld.max_tokens = max_tokens; ld.num_experts = num_experts;
        ld.topk_idx.assign(topk_idx, topk_idx + R);
        ld.recv_x.assign(recv_x, recv_x + R);
        ld.src_info.assign(src_info, src_info + R);
        ld.layout_range.assign(layout_range, layout_range + R);
        ld.num_tokens.assign(num_tokens, num_tokens + R);
        ld.captured = cap.active;
        ld.capture_id = cap.id;
        ld.data_done = data_done;
        if (cap.active) w->dispatch_captured = true;
    };
    if (fused) {
        SmallTable st{};
        memcpy(st.v, tbl, tbl_words * sizeof(uint64_t));
        MC_HIP(launch_dispatch_small(st, sc.selrow, d, use_fp8 != 0, w->tuning, stream));
        w->launches += 1;
        if (!static_scratch) remember(true);
        return MC_EP_OK;
    }

    const bool uni = w->tuning.uniform != 0;
    DispatchSource src;
    src.x = uniform_ptr(x, R, uni);
    src.topk_idx = uniform_ptr(topk_idx, R, uni);
    src.tokens = uniform_tokens(num_tokens, R, uni);
    if (phases & MC_EP_PHASE_LAYOUT) {
        MC_HIP(launch_count(d_tbl, sc, src, d, stream));
        w->launches += d.plan.carried ? 1 : 2;    // the prefix pass is a launch of its own unless it rides in pack's
        if (!static_scratch) remember(false);
    }
    if ((phases & (MC_EP_PHASE_DATA | MC_EP_PHASE_FINISH)) && tgrid > 0) {
        MC_HIP(launch_pack(d_tbl, sc, src, stage, d, use_fp8 != 0, w->tuning,
                           (phases & MC_EP_PHASE_DATA) != 0, (phases & MC_EP_PHASE_FINISH) != 0, stream));
        w->launches += ((phases & MC_EP_PHASE_DATA) ? 1 : 0) + (((phases & MC_EP_PHASE_FINISH) && use_fp8) ? 1 : 0);
    }
    // under the carried plan the pack launch also produces ubegin and the counts: only now is the
    // routing state complete for a combine to reuse
    if (!static_scratch && (phases & MC_EP_PHASE_DATA)) w->last.data_done = true;
    return MC_EP_OK;
}

// What combine reads its rows from: bf16 expert outputs (the reference's combine), or, for the packed
// combine, the payload dispatch wrote (fp8 with scales, or bf16) times an optional per-expert factor.
struct PackedSource {
    bool packed = false;
    const uint64_t* scales = nullptr;   // per-rank addresses; null: the payload is bf16
    const float* factor = nullptr;      // device f32 [num_experts]; null: no factor
};

int world_combine_impl(mc_ep_world* w, const uint64_t* x, const uint64_t* topk_idx, const uint64_t* topk_weights,
                       const uint64_t* src_info, const uint64_t* layout_range, const uint64_t* active_ranks,
                       const int32_t* num_tokens, int hidden, int num_topk, int max_tokens, int num_experts,
                       const uint64_t* out, int phases, hipStream_t stream, const PackedSource& ps = PackedSource()) {
    const int R = w->R;
    if (int rc = check_dims(w, hidden, num_topk, max_tokens, num_experts)) return rc;
    MC_ASSERT(x != nullptr && topk_idx != nullptr && topk_weights != nullptr && num_tokens != nullptr);
    MC_ASSERT(src_info != nullptr && layout_range != nullptr && active_ranks != nullptr && out != nullptr);
    int tgrid = 0;
    std::vector<uint64_t> tbl((size_t)CF_COUNT * R, 0);
    for (int r = 0; r < R; ++r) {
        MC_ASSERT(num_tokens[r] >= 0 && num_tokens[r] <= max_tokens);
        if (num_tokens[r] > 0) {
            MC_ASSERT(topk_idx[r] != 0 && topk_weights[r] != 0);
            MC_ASSERT(active_ranks[r] != 0);
            MC_ASSERT(out[r] != 0);
        }
        if (x[r] != 0) MC_ASSERT(src_info[r] != 0 && layout_range[r] != 0);
        if (x[r] != 0 && ps.scales != nullptr) MC_ASSERT(ps.scales[r] != 0);
        tbl[CF_SCALES * R + r] = (ps.scales != nullptr && x[r] != 0) ? ps.scales[r] : 0;
        tbl[CF_X * R + r] = x[r];
        tbl[CF_TOPK_IDX * R + r] = topk_idx[r];
        tbl[CF_TOPK_W * R + r] = topk_weights[r];
        tbl[CF_SRC_INFO * R + r] = x[r] ? src_info[r] : 0;
        tbl[CF_LAYOUT_RANGE * R + r] = x[r] ? layout_range[r] : 0;
        tbl[CF_ACTIVE * R + r] = active_ranks[r];
        tbl[CF_OUT * R + r] = out[r];
        tbl[CF_NUM_TOKENS * R + r] = (uint64_t)num_tokens[r];
        if (num_tokens[r] > tgrid) tgrid = num_tokens[r];
    }
    if (tgrid == 0) return MC_EP_OK;
    DeviceGuard guard(w->device);
    w->launches = 0;
    struct Tally {                                // the option "last_combine_launches", on every way out
        mc_ep_world* w;
        ~Tally() { w->tuning.last_combine_launches = w->launches; }
    } tally{w};
    Capture cap;
    if (int rc = capture_of(stream, &cap)) return rc;
    RecordingScope recording(cap.active);
    if (int rc = order_begin(w, stream, cap)) return rc;
    const uint64_t* d_tbl = nullptr;
    if (int rc = upload_table(w, 1, tbl, cap, stream, &d_tbl)) return rc;
    Dims d{R, num_experts, num_topk, hidden, max_tokens, tgrid};

    // Is this the handle (and the routing input) of the last dispatch?  Then the
    // packed row of every selection is already known on the device.  The kernel
    // still reads topk_idx as combine is given it, as the reference's does
    // (mooncake_ep_kernel.cu:719-732): a selection that no longer names the
    // expert it was dispatched to (masked to -1 in place, say) contributes nothing.
    const auto& ld = w->last;
    bool direct = w->tuning.combine_direct != 0 && ld.valid && ld.data_done && ld.hidden == hidden &&
                  (long long)num_experts * R * max_tokens < 0x7fffffffll && ld.num_topk == num_topk &&
                  ld.max_tokens == max_tokens && ld.num_experts == num_experts;
    // "Last" is about the order on the device.  Graph replays run dispatches the host never sees, so: a
    // recorded combine trusts only a dispatch recorded in the same capture, and once a dispatch of this
    // world lives in a graph, eager combines resolve their handle (always right) instead.
    direct = direct && (cap.active ? (ld.captured && ld.capture_id == cap.id) : !w->dispatch_captured);
    for (int r = 0; r < R && direct; ++r) {
        if (num_tokens[r] > 0) direct = topk_idx[r] == ld.topk_idx[r] && num_tokens[r] == ld.num_tokens[r];
        if (direct && x[r] != 0)
            direct = ld.recv_x[r] != 0 && src_info[r] == ld.src_info[r] && layout_range[r] == ld.layout_range[r];
    }

    const bool uni = w->tuning.uniform != 0;
    CombineSource src;
    src.topk_idx = uniform_ptr(topk_idx, R, uni);
    src.topk_weights = uniform_ptr(topk_weights, R, uni);
    src.out = uniform_ptr(out, R, uni);
    src.x = uniform_ptr(x, R, uni);
    if (ps.scales != nullptr) src.scales = uniform_ptr(ps.scales, R, uni);
    src.tokens = uniform_tokens(num_tokens, R, uni);
    // sized on every path, so that an eager call prepares the world for any recorded one of the same shape
    if (int rc = ensure_routes(w, (size_t)R * max_tokens * num_topk)) return rc;
    if (!direct) {
        if (phases & MC_EP_PHASE_LAYOUT) {
            w->stamp += 1;
            // every replay of a recorded call carries the same stamp: clear the routes so that none of an
            // earlier replay passes for this one's
            if (cap.active) {
                MC_HIP(launch_fill_u32(w->d_routes, 0u, (size_t)R * max_tokens * num_topk * (sizeof(CombineRoute) / 4),
                                       stream));
                w->launches += 1;
            }
            MC_HIP(launch_resolve(d_tbl, w->d_routes, w->stamp, ps.packed, d, w->tuning, stream));
            w->launches += 1;
        }
    }
    if (phases & MC_EP_PHASE_DATA) w->launches += 1;
    if ((phases & MC_EP_PHASE_DATA) && ps.packed)
        MC_HIP(launch_reduce_packed(d_tbl, w->d_routes, w->stamp, routing_scratch(w), direct, src, w->d_zero_row,
                                    ps.factor, ps.scales != nullptr, d, w->tuning, stream));
    else if (phases & MC_EP_PHASE_DATA)
        MC_HIP(launch_reduce(d_tbl, w->d_routes, w->stamp, routing_scratch(w), direct, src, w->d_zero_row, d,
                             w->tuning, stream));
    return MC_EP_OK;
}

// Streams of a round.  When every caller of the round is on one stream, the round runs there: an
// async_finish caller still gets its event (recorded behind the round's kernels), a hook caller its
// hook, and nothing has to cross streams - on one GPU there is no link transfer for later work of that
// stream to overlap with, while every cross-stream hand-off costs about 10 us of device time.  With
// callers on different streams, or with the option "comm_stream" set, the round runs on the world's
// communication stream, fenced against every caller's stream before and after, which is the reference's
// arrangement (mooncake_ep_buffer.cpp:225-227, :318-327).
template <typename Post>
hipStream_t pick_launch_stream(mc_ep_world* w, const std::vector<Post>& posts, bool* shared) {
    hipStream_t first = nullptr;
    bool have = false, same = true;
    for (const auto& p : posts) {
        if (!p.present) continue;
        if (!have) {
            first = p.stream;
            have = true;
        } else if (p.stream != first) {
            same = false;
        }
    }
    *shared = have && same && w->tuning.comm_stream == 0;
    return *shared ? first : w->comm_stream;
}

template <typename Post>
int fence_before(mc_ep_world* w, const std::vector<Post>& posts, hipStream_t launch) {
    std::vector<hipStream_t> seen;
    for (const auto& p : posts) {
        if (!p.present || p.stream == launch) continue;
        if (p.hand.by_caller) {
            if (p.hand.before) MC_HIP(hipStreamWaitEvent(launch, p.hand.before, 0));
            continue;
        }
        bool dup = false;
        for (auto s : seen) dup |= (s == p.stream);
        if (dup) continue;
        seen.push_back(p.stream);
        // a stream with nothing in flight has nothing to wait for (a rank that waits for its own stream after
        // every step, as the reference's tests do): asking costs a microsecond of host time, a cross-stream
        // hand-off about ten of the device's
        if (hipStreamQuery(p.stream) == hipSuccess) continue;
        // a wait refers to what the event held when the wait was issued, so one event serves every stream
        MC_HIP(hipEventRecord(w->fence, p.stream));
        MC_HIP(hipStreamWaitEvent(launch, w->fence, 0));
    }
    return MC_EP_OK;
}

template <typename Post>
int fence_after(mc_ep_world* w, const std::vector<Post>& posts, hipStream_t launch, Round* round) {
    round->waited.assign(1, launch);      // work queued on the launch stream is behind the round anyway
    // the completion event is recorded only when somebody can ask for it: an async caller's
    // EventHandle, or a caller on another stream (a record costs a few us of device time)
    bool needed = false;
    for (const auto& p : posts) needed |= p.present && (p.async || p.stream != launch);
    if (needed) {
        round->pool = w->events;
        if (int e = round->pool->take(&round->done)) return e;
        MC_HIP(hipEventRecord(round->done, launch));
    }
    for (const auto& p : posts) {
        // default mode: the caller's stream waits for the result (a blocking caller sees to that itself
        // when it wakes); async and hook callers wait through their event / hook
        if (!p.present || p.async || p.hook || p.hand.by_caller) continue;
        if (int e = round->make_wait(p.stream)) return e;
    }
    round->launched = true;
    return MC_EP_OK;
}

// A silent source rank has "timed out": each live rank's active_ranks entry
// for it drops to 0 when that rank asked for a timeout
// (mooncake_ep_kernel.cu:421-423, :692-694).
template <typename Post>
int mark_silent_inactive(mc_ep_world* w, const std::vector<Post>& posts, hipStream_t launch) {
    for (int r = 0; r < w->R; ++r) {
        const auto& p = posts[r];
        if (!p.present || p.timeout_us == -1 || p.active_ranks == 0) continue;
        for (int j = 0; j < w->R; ++j) {
            if (posts[j].present) continue;
            MC_HIP(launch_fill_u32((void*)(p.active_ranks + (uint64_t)j * 4), 0u, 1, launch));
        }
    }
    return MC_EP_OK;
}

int launch_dispatch_round(mc_ep_world* w, PendingRound<DispatchPost>& pr) {
    const int R = w->R;
    const DispatchPost* first = nullptr;
    for (const auto& p : pr.posts)
        if (p.present && !first) first = &p;
    if (!first) return MC_EP_OK;
    for (const auto& p : pr.posts) {
        if (!p.present) continue;
        // every rank of a collective names the same problem shape
        MC_ASSERT(p.hidden == first->hidden && p.num_topk == first->num_topk);
        MC_ASSERT(p.max_tokens == first->max_tokens && p.num_experts == first->num_experts);
        MC_ASSERT(p.use_fp8 == first->use_fp8);
    }
    std::vector<uint64_t> x(R, 0), idx(R, 0), rx(R, 0), rs(R, 0), rc(R, 0), si(R, 0), lr(R, 0);
    std::vector<int32_t> nt(R, 0);
    for (int r = 0; r < R; ++r) {
        const auto& p = pr.posts[r];
        if (!p.present) continue;
        x[r] = p.x; idx[r] = p.topk_idx; nt[r] = p.num_tokens;
        rx[r] = p.recv_x; rs[r] = p.recv_scales; rc[r] = p.recv_count; si[r] = p.src_info; lr[r] = p.layout_range;
    }
    DeviceGuard guard(w->device);
    bool shared = false;
    hipStream_t launch = pick_launch_stream(w, pr.posts, &shared);
    if (int e = fence_before(w, pr.posts, launch)) return e;
    if (int e = mark_silent_inactive(w, pr.posts, launch)) return e;
    bool all_hook = true;
    for (const auto& p : pr.posts)
        if (p.present && !p.hook) all_hook = false;
    // only an fp8 dispatch has a second part (the scales' move into their column-major layout)
    const bool two_part = all_hook && first->use_fp8;
    const int hidden = first->hidden, num_topk = first->num_topk, max_tokens = first->max_tokens,
              num_experts = first->num_experts, use_fp8 = first->use_fp8;
    if (int e = world_dispatch_impl(w, x.data(), idx.data(), nt.data(), hidden, num_topk, max_tokens, num_experts,
                                    use_fp8, rx.data(), rs.data(), rc.data(), si.data(), lr.data(),
                                    two_part ? (MC_EP_PHASE_LAYOUT | MC_EP_PHASE_DATA) : MC_EP_PHASE_ALL, launch))
        return e;
    Round* round = pr.state.get();
    round->launch_stream = launch;
    if (!two_part) return fence_after(w, pr.posts, launch, round);
    bool needed = false;
    for (const auto& p : pr.posts) needed |= p.present && p.stream != launch;
    if (needed) {
        round->pool = w->events;
        if (int e = round->pool->take(&round->done)) return e;
    }
    round->finish = [=]() -> int {
        DeviceGuard g(w->device);
        if (int e = world_dispatch_impl(w, x.data(), idx.data(), nt.data(), hidden, num_topk, max_tokens, num_experts,
                                        use_fp8, rx.data(), rs.data(), rc.data(), si.data(), lr.data(),
                                        MC_EP_PHASE_FINISH, launch))
            return e;
        if (round->done) MC_HIP(hipEventRecord(round->done, launch));
        round->waited.assign(1, launch);
        return MC_EP_OK;
    };
    w->unfinished = pr.state;
    round->launched = true;
    return MC_EP_OK;
}

int launch_combine_round(mc_ep_world* w, PendingRound<CombinePost>& pr) {
    const int R = w->R;
    const CombinePost* first = nullptr;
    for (const auto& p : pr.posts)
        if (p.present && !first) first = &p;
    if (!first) return MC_EP_OK;
    for (const auto& p : pr.posts) {
        if (!p.present) continue;
        MC_ASSERT(p.hidden == first->hidden && p.num_topk == first->num_topk);
        MC_ASSERT(p.max_tokens == first->max_tokens && p.num_experts == first->num_experts);
    }
    std::vector<uint64_t> x(R, 0), idx(R, 0), tw(R, 0), si(R, 0), lr(R, 0), ar(R, 0), out(R, 0);
    std::vector<int32_t> nt(R, 0);
    for (int r = 0; r < R; ++r) {
        const auto& p = pr.posts[r];
        if (!p.present) continue;
        x[r] = p.x; idx[r] = p.topk_idx; tw[r] = p.topk_weights; si[r] = p.src_info; lr[r] = p.layout_range;
        ar[r] = p.active_ranks; out[r] = p.out; nt[r] = p.num_tokens;
    }
    DeviceGuard guard(w->device);
    bool shared = false;
    hipStream_t launch = pick_launch_stream(w, pr.posts, &shared);
    if (int e = fence_before(w, pr.posts, launch)) return e;
    if (int e = mark_silent_inactive(w, pr.posts, launch)) return e;
    if (int e = world_combine_impl(w, x.data(), idx.data(), tw.data(), si.data(), lr.data(), ar.data(), nt.data(),
                                   first->hidden, first->num_topk, first->max_tokens, first->num_experts,
                                   out.data(), MC_EP_PHASE_ALL, launch))
        return e;
    pr.state->launch_stream = launch;
    return fence_after(w, pr.posts, launch, pr.state.get());
}

template <typename Post>
bool round_complete(const mc_ep_world* w, const PendingRound<Post>& pr) {
    for (int r = 0; r < w->R; ++r)
        if (!pr.posts[r].present && !w->silent[r]) return false;
    return true;
}

// Launch every leading round that has all its live ranks.
int drain_dispatch(mc_ep_world* w) {
    while (!w->dispatch_rounds.empty() && round_complete(w, w->dispatch_rounds.front())) {
        int e = launch_dispatch_round(w, w->dispatch_rounds.front());
        const std::shared_ptr<Round> state = w->dispatch_rounds.front().state;
        if (e) state->failure = g_last_error;
        w->dispatch_rounds.pop_front();
        w->dispatch_base++;
        state->publish();
        if (e) return e;
    }
    return MC_EP_OK;
}

int drain_combine(mc_ep_world* w) {
    while (!w->combine_rounds.empty() && round_complete(w, w->combine_rounds.front())) {
        int e = launch_combine_round(w, w->combine_rounds.front());
        const std::shared_ptr<Round> state = w->combine_rounds.front().state;
        if (e) state->failure = g_last_error;
        w->combine_rounds.pop_front();
        w->combine_base++;
        state->publish();
        if (e) return e;
    }
    return MC_EP_OK;
}

// The round a rank's call_index-th call belongs to (opened on demand), or null for a call index that
// lies before the front round, which the callers turn into an assertion failure.
template <typename Post>
PendingRound<Post>* round_for_call(mc_ep_world* w, std::deque<PendingRound<Post>>& rounds, long long base,
                                   long long call_index) {
    if (call_index < base) return nullptr;
    while ((long long)rounds.size() <= call_index - base) {
        PendingRound<Post> pr;
        pr.posts.resize(w->R);
        pr.state = std::make_shared<Round>();
        rounds.push_back(std::move(pr));
    }
    return &rounds[(size_t)(call_index - base)];
}

// What a waiter on a round that cannot complete is told: either the launch failed (the call that
// completed the round got the error; the other ranks learn it here), or ranks are still missing.
int round_not_ready(const Round* round) {
    if (round != nullptr && !round->failure.empty())
        return fail(MC_EP_ERR_ASSERT, "Failed: the collective could not be launched: " + round->failure);
    return fail(MC_EP_ERR_PENDING,
                "Failed: the call is a collective over the world's live ranks and not every one of them has "
                "called it yet");
}

// Option "blocking": the caller is one of several threads, one per rank, each of which goes on to use its
// results as soon as its call returns, as a process of the reference does.  The call therefore returns
// only when the round has been launched (by the thread whose call completed it), so that whatever the
// caller enqueues next on its stream is ordered behind the round.  Called with the lock held; a blocking
// caller gives it up here and comes back without it (what the entry points do afterwards touches nothing
// that is shared).
int wait_for_round(mc_ep_world* w, const std::shared_ptr<Round>& round, Lock& lock) {
    if (w->tuning.blocking == 0) return MC_EP_OK;
    const int ms = w->tuning.block_timeout_ms;
    lock.unlock();
    if (!round->wait_published(ms, w->tuning.block_spin_us))
        return fail(MC_EP_ERR_PENDING, "Failed: the call waited " + std::to_string(ms) + " ms for the other live ranks "
                                       "of its collective (option block_timeout_ms); it stays posted");
    if (round->published.load(std::memory_order_acquire) == 2) {
        lock.lock();                       // `failure` may be appended to by a later second part
        return round_not_ready(round.get());
    }
    return MC_EP_OK;
}

// A blocking caller's part before the round (see StreamHandOff); with the lock held.
int hand_off_before(mc_ep_buffer* b, hipStream_t stream, StreamHandOff* hand) {
    hand->by_caller = true;
    hand->before = nullptr;
    if (hipStreamQuery(stream) == hipSuccess) return MC_EP_OK;       // nothing in flight: nothing to wait for
    if (b->before == nullptr) MC_HIP(hipEventCreateWithFlags(&b->before, hipEventDisableTiming));
    // the rank's one event serves every round: a wait issued for an earlier round refers to what the event
    // held then or, if the rank has run ahead and recorded again, to more of the same stream
    MC_HIP(hipEventRecord(b->before, stream));
    hand->before = b->before;
    return MC_EP_OK;
}

// ... and after it: the default mode's "the caller's stream waits for the result", by the caller, without
// the lock (the round's event and launch stream were set before the round was published).
int hand_off_after(const Round* round, hipStream_t stream, bool default_mode) {
    if (!default_mode || round->launch_stream == stream || round->done == nullptr) return MC_EP_OK;
    MC_HIP(hipStreamWaitEvent(stream, round->done, 0));
    return MC_EP_OK;
}

// The per-rank calls form a round out of several host calls, with events between streams: that
// bookkeeping is not something a graph can hold.  Whole-world calls can be recorded.
int refuse_capture(uint64_t stream_ptr) {
    Capture cap;
    if (int rc = capture_of((hipStream_t)stream_ptr, &cap)) return rc;
    if (cap.active)
        return fail(MC_EP_ERR_UNSUPPORTED,
                    "Failed: per-rank Buffer calls cannot be recorded into a graph; record mc_ep_world_dispatch / "
                    "mc_ep_world_combine instead");
    return MC_EP_OK;
}

}  // namespace

// ---------------------------------------------------------------------------
// C ABI
// ---------------------------------------------------------------------------

extern "C" {

const char* mc_ep_last_error(void) { return g_last_error.c_str(); }

uint64_t mc_ep_get_buffer_size_hint(int max_tokens, int hidden, int num_ranks, int num_experts) {
    (void)num_ranks;
    // two buffers, each: two signalling areas of num_experts ints and two data
    // areas of num_experts * max_tokens messages of (2 * 16 + hidden * 2) bytes
    const uint64_t signaling = (uint64_t)num_experts * sizeof(int);
    const uint64_t data = (uint64_t)num_experts * (uint64_t)max_tokens * (2 * 16 + (uint64_t)hidden * 2);
    return 4 * signaling + 4 * data;
}

int mc_ep_world_create(int num_ranks, mc_ep_world_t** out) {
    MC_ASSERT(out != nullptr);
    MC_ASSERT(num_ranks > 0 && num_ranks <= MC_EP_MAX_QP_COUNT);
    Lock lock(g_mu);
    auto w = std::make_unique<mc_ep_world>();
    w->R = num_ranks;
    MC_HIP(hipGetDevice(&w->device));
    // the device's copy of the static scratch array: its address is asked for once per device, here,
    // with that device current; host code uses the pointer, never the array's name
    if (w->device >= 0 && w->device < kMaxDevices && g_scratch_ptr[w->device] == nullptr) {
        void* ptr = nullptr;
        MC_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        MC_ASSERT(ptr != nullptr);
        g_scratch_ptr[w->device] = (unsigned char*)ptr;
    }
    MC_HIP(hipStreamCreateWithFlags(&w->comm_stream, hipStreamNonBlocking));
    MC_HIP(hipEventCreateWithFlags(&w->ordered, hipEventDisableTiming));
    MC_HIP(hipEventCreateWithFlags(&w->fence, hipEventDisableTiming));
    for (int i = 0; i < 3; ++i) {
        const int fields[3] = {(int)DF_COUNT, (int)CF_COUNT, (int)XF_COUNT};
        const size_t words = (size_t)fields[i] * num_ranks;
        MC_HIP(hipMalloc((void**)&w->d_tbl[i], words * sizeof(uint64_t)));
        MC_HIP(hipMalloc((void**)&w->d_captured_tbl[i], (size_t)kCapturedTables * words * sizeof(uint64_t)));
    }
    MC_HIP(hipMalloc(&w->d_zero_row, kZeroRowBytes));
    MC_HIP(hipMemset(w->d_zero_row, 0, kZeroRowBytes));
    w->silent.assign(num_ranks, 0);
    w->dispatch_calls.assign(num_ranks, 0);
    w->combine_calls.assign(num_ranks, 0);
    *out = w.release();
    return MC_EP_OK;
}

int mc_ep_world_destroy(mc_ep_world_t* w) {
    Lock lock(g_mu);
    delete w;   // ~mc_ep_world waits for the device and releases what the world owns
    return MC_EP_OK;
}

int mc_ep_world_num_ranks(const mc_ep_world_t* w) { return w ? w->R : 0; }

int mc_ep_world_set_rank_silent(mc_ep_world_t* w, int rank, int silent) {
    MC_ASSERT(w != nullptr && rank >= 0 && rank < w->R);
    Lock lock(g_mu);
    const bool was_silent = w->silent[rank] != 0;
    w->silent[rank] = silent ? 1 : 0;
    if (was_silent && !silent) {
        // A rank that comes back (the reference's update_ep_member after a restart) has missed the
        // rounds that completed without it and the ones its peers have already opened: its next call
        // joins the first round nobody has opened yet.
        w->dispatch_calls[rank] = w->dispatch_base + (long long)w->dispatch_rounds.size();
        w->combine_calls[rank] = w->combine_base + (long long)w->combine_rounds.size();
        return MC_EP_OK;
    }
    // rounds that were only waiting for this rank can go now
    if (int e = drain_dispatch(w)) return e;
    return drain_combine(w);
}

static int* option_slot(Tuning& t, const char* name) {
    if (!strcmp(name, "pack_waves")) return &t.pack_waves;
    if (!strcmp(name, "pack_nt")) return &t.pack_nt;
    if (!strcmp(name, "uniform")) return &t.uniform;
    if (!strcmp(name, "fp8_arith")) return &t.fp8_arith;
    if (!strcmp(name, "comm_stream")) return &t.comm_stream;
    if (!strcmp(name, "combine_direct")) return &t.combine_direct;
    if (!strcmp(name, "combine_chunks")) return &t.combine_chunks;
    if (!strcmp(name, "packed_map")) return &t.packed_map;
    if (!strcmp(name, "combine_occupancy")) return &t.combine_occupancy;
    if (!strcmp(name, "routing_sum")) return &t.routing_sum;
    if (!strcmp(name, "combine_waves")) return &t.combine_waves;
    if (!strcmp(name, "combine_nt")) return &t.combine_nt;
    if (!strcmp(name, "last_dispatch_launches")) return &t.last_dispatch_launches;
    if (!strcmp(name, "last_combine_launches")) return &t.last_combine_launches;
    if (!strcmp(name, "fused_small")) return &t.fused_small;
    if (!strcmp(name, "fused_small_max")) return &t.fused_small_max;
    if (!strcmp(name, "fused_small_rounds")) return &t.fused_small_rounds;
    if (!strcmp(name, "blocking")) return &t.blocking;
    if (!strcmp(name, "block_timeout_ms")) return &t.block_timeout_ms;
    if (!strcmp(name, "block_spin_us")) return &t.block_spin_us;
    return nullptr;
}

int mc_ep_world_set_option(mc_ep_world_t* w, const char* name, int value) {
    MC_ASSERT(w != nullptr && name != nullptr);
    Lock lock(g_mu);
    int* slot = option_slot(w->tuning, name);
    if (!slot) return fail(MC_EP_ERR_ASSERT, std::string("Failed: unknown option '") + name + "'");
    *slot = value;
    return MC_EP_OK;
}

int mc_ep_world_get_option(const mc_ep_world_t* w, const char* name, int* value) {
    MC_ASSERT(w != nullptr && name != nullptr && value != nullptr);
    Lock lock(g_mu);
    Tuning t = w->tuning;
    int* slot = option_slot(t, name);
    if (!slot) return fail(MC_EP_ERR_ASSERT, std::string("Failed: unknown option '") + name + "'");
    *value = *slot;
    return MC_EP_OK;
}

int mc_ep_world_dispatch(mc_ep_world_t* w, const uint64_t* x_ptrs, const uint64_t* topk_idx_ptrs,
                         const int32_t* num_tokens, int hidden, int num_topk, int max_tokens, int num_experts,
                         int use_fp8, const uint64_t* recv_x_ptrs, const uint64_t* recv_scales_ptrs,
                         const uint64_t* recv_count_ptrs, const uint64_t* src_info_ptrs,
                         const uint64_t* layout_range_ptrs, int phases, uint64_t stream_ptr) {
    MC_ASSERT(w != nullptr);
    Lock lock(g_mu);
    return world_dispatch_impl(w, x_ptrs, topk_idx_ptrs, num_tokens, hidden, num_topk, max_tokens, num_experts,
                               use_fp8, recv_x_ptrs, recv_scales_ptrs, recv_count_ptrs, src_info_ptrs,
                               layout_range_ptrs, phases, (hipStream_t)stream_ptr);
}

int mc_ep_world_dispatch_noalloc(mc_ep_world_t* w, const uint64_t* x_ptrs, const uint64_t* topk_idx_ptrs,
                                 const int32_t* num_tokens, int hidden, int num_topk, int max_tokens,
                                 int num_experts, int use_fp8, const uint64_t* recv_x_ptrs,
                                 const uint64_t* recv_scales_ptrs, const uint64_t* recv_count_ptrs,
                                 const uint64_t* src_info_ptrs, const uint64_t* layout_range_ptrs,
                                 uint64_t stream_ptr) {
    MC_ASSERT(w != nullptr);
    Lock lock(g_mu);
    return world_dispatch_impl(w, x_ptrs, topk_idx_ptrs, num_tokens, hidden, num_topk, max_tokens, num_experts,
                               use_fp8, recv_x_ptrs, recv_scales_ptrs, recv_count_ptrs, src_info_ptrs,
                               layout_range_ptrs, MC_EP_PHASE_ALL, (hipStream_t)stream_ptr, true);
}

int mc_ep_world_combine(mc_ep_world_t* w, const uint64_t* x_ptrs, const uint64_t* topk_idx_ptrs,
                        const uint64_t* topk_weights_ptrs, const uint64_t* src_info_ptrs,
                        const uint64_t* layout_range_ptrs, const uint64_t* active_ranks_ptrs,
                        const int32_t* num_combined_tokens, int hidden, int num_topk, int max_tokens,
                        int num_experts, const uint64_t* combined_x_ptrs, int phases, uint64_t stream_ptr) {
    MC_ASSERT(w != nullptr);
    Lock lock(g_mu);
    return world_combine_impl(w, x_ptrs, topk_idx_ptrs, topk_weights_ptrs, src_info_ptrs, layout_range_ptrs,
                              active_ranks_ptrs, num_combined_tokens, hidden, num_topk, max_tokens, num_experts,
                              combined_x_ptrs, phases, (hipStream_t)stream_ptr);
}

int mc_ep_world_combine_packed(mc_ep_world_t* w, const uint64_t* recv_x_ptrs, const uint64_t* recv_scales_ptrs,
                               uint64_t expert_factor_ptr, const uint64_t* topk_idx_ptrs,
                               const uint64_t* topk_weights_ptrs, const uint64_t* src_info_ptrs,
                               const uint64_t* layout_range_ptrs, const uint64_t* active_ranks_ptrs,
                               const int32_t* num_combined_tokens, int hidden, int num_topk, int max_tokens,
                               int num_experts, const uint64_t* combined_x_ptrs, int phases, uint64_t stream_ptr) {
    MC_ASSERT(w != nullptr);
    Lock lock(g_mu);
    PackedSource ps;
    ps.packed = true;
    ps.scales = recv_scales_ptrs;
    ps.factor = (const float*)expert_factor_ptr;
    return world_combine_impl(w, recv_x_ptrs, topk_idx_ptrs, topk_weights_ptrs, src_info_ptrs, layout_range_ptrs,
                              active_ranks_ptrs, num_combined_tokens, hidden, num_topk, max_tokens, num_experts,
                              combined_x_ptrs, phases, (hipStream_t)stream_ptr, ps);
}

int mc_ep_world_cast_back(mc_ep_world_t* w, const uint64_t* recv_x_ptrs, const uint64_t* recv_scales_ptrs,
                          const uint64_t* recv_count_ptrs, uint64_t expert_factor_ptr, const uint64_t* out_ptrs,
                          int hidden, int num_topk, int max_tokens, int num_experts, uint64_t stream_ptr) {
    MC_ASSERT(w != nullptr);
    Lock lock(g_mu);
    const int R = w->R;
    MC_ASSERT(num_experts > 0 && num_experts % R == 0);
    MC_ASSERT(hidden > 0 && hidden % 128 == 0);
    MC_ASSERT(max_tokens > 0 && num_topk >= 0);
    MC_ASSERT(recv_x_ptrs != nullptr && recv_count_ptrs != nullptr && out_ptrs != nullptr);
    const bool use_fp8 = recv_scales_ptrs != nullptr;
    std::vector<uint64_t> tbl((size_t)XF_COUNT * R, 0);
    for (int r = 0; r < R; ++r) {
        if (recv_x_ptrs[r] != 0) {
            MC_ASSERT(recv_count_ptrs[r] != 0 && out_ptrs[r] != 0);
            MC_ASSERT(out_ptrs[r] != recv_x_ptrs[r] || !use_fp8);   // fp8 rows cannot be widened in place
            if (use_fp8) MC_ASSERT(recv_scales_ptrs[r] != 0);
        }
        tbl[XF_RECV_X * R + r] = recv_x_ptrs[r];
        tbl[XF_RECV_SCALES * R + r] = use_fp8 ? recv_scales_ptrs[r] : 0;
        tbl[XF_RECV_COUNT * R + r] = recv_count_ptrs[r];
        tbl[XF_OUT * R + r] = recv_x_ptrs[r] != 0 ? out_ptrs[r] : 0;
    }
    DeviceGuard guard(w->device);
    hipStream_t stream = (hipStream_t)stream_ptr;
    Capture cap;
    if (int rc = capture_of(stream, &cap)) return rc;
    RecordingScope recording(cap.active);
    if (int rc = order_begin(w, stream, cap)) return rc;
    const uint64_t* d_tbl = nullptr;
    if (int rc = upload_table(w, 2, tbl, cap, stream, &d_tbl)) return rc;
    Dims d{R, num_experts, num_topk, hidden, max_tokens, max_tokens};
    // valid rows of the world: at most one per selection, and no more than the layout holds
    long long max_rows = (long long)num_experts * R * max_tokens;
    if (num_topk > 0 && (long long)R * max_tokens * num_topk < max_rows) max_rows = (long long)R * max_tokens * num_topk;
    const size_t map_words = (size_t)(cast_back_chunks(max_rows, num_experts) + 1) * 4;
    if (int rc = ensure_scratch(w, &w->d_chunk_map, &w->chunk_map_cap, map_words)) return rc;
    MC_HIP(launch_cast_back(d_tbl, w->d_chunk_map, (const float*)expert_factor_ptr, use_fp8, max_rows, d,
                            stream));
    return MC_EP_OK;
}

int mc_ep_world_legacy_buffer_perf(mc_ep_world_t* w, const mc_ep_legacy_perf_tensors_t* t,
                                   const mc_ep_legacy_perf_config_t* c, mc_ep_legacy_perf_result_t* result) {
    MC_ASSERT(w != nullptr && t != nullptr && c != nullptr && result != nullptr);
    if (c->num_tokens <= 0 || c->hidden <= 0 || c->num_topk <= 0 ||
        c->num_max_dispatch_tokens_per_rank < c->num_tokens || c->num_experts <= 0 || c->num_local_experts <= 0 ||
        c->warmups < 0 || c->iterations <= 1)
        return fail(MC_EP_ERR_INVALID, "invalid legacy EP benchmark configuration");
    const uint64_t* const fields[] = {t->x_ptrs,
                                      t->topk_idx_ptrs,
                                      t->topk_weights_ptrs,
                                      t->active_ranks_ptrs,
                                      t->expert_x_ptrs,
                                      t->packed_recv_x_ptrs,
                                      t->packed_recv_count_ptrs,
                                      t->packed_recv_src_info_ptrs,
                                      t->packed_recv_layout_range_ptrs,
                                      t->combined_x_ptrs};
    for (const uint64_t* f : fields) {
        if (f == nullptr) return fail(MC_EP_ERR_INVALID, "legacy EP benchmark received a null tensor pointer");
        for (int r = 0; r < w->R; ++r)
            if (f[r] == 0) return fail(MC_EP_ERR_INVALID, "legacy EP benchmark received a null tensor pointer");
    }
    MC_ASSERT(c->num_local_experts * w->R == c->num_experts);

    DeviceGuard guard(w->device);
    hipStream_t stream = (hipStream_t)c->compute_stream_ptr;
    const std::vector<int32_t> tokens((size_t)w->R, c->num_tokens);

    auto run_once = [&]() -> int {
        Lock lock(g_mu);   // per step: the waits for the GPU below happen without it
        // the reference's cudaMemsetAsync(packed_recv_count) of every rank, in one launch
        MC_HIP(launch_clear_words(t->packed_recv_count_ptrs, w->R, c->num_local_experts, stream));
        int rc = world_dispatch_impl(w, t->x_ptrs, t->topk_idx_ptrs, tokens.data(), c->hidden, c->num_topk,
                                     c->num_max_dispatch_tokens_per_rank, c->num_experts, 0, t->packed_recv_x_ptrs,
                                     nullptr, t->packed_recv_count_ptrs, t->packed_recv_src_info_ptrs,
                                     t->packed_recv_layout_range_ptrs, MC_EP_PHASE_ALL, stream);
        if (rc != MC_EP_OK) return rc;
        return world_combine_impl(w, t->expert_x_ptrs, t->topk_idx_ptrs, t->topk_weights_ptrs,
                                  t->packed_recv_src_info_ptrs, t->packed_recv_layout_range_ptrs,
                                  t->active_ranks_ptrs, tokens.data(), c->hidden, c->num_topk,
                                  c->num_max_dispatch_tokens_per_rank, c->num_experts, t->combined_x_ptrs,
                                  MC_EP_PHASE_ALL, stream);
    };

    for (int i = 0; i < c->warmups; ++i) {
        const int rc = run_once();
        if (rc != MC_EP_OK) return rc;
    }
    MC_HIP(hipStreamSynchronize(stream));

    // events are released on every way out
    struct Events {
        std::vector<hipEvent_t> v;
        ~Events() {
            for (hipEvent_t e : v) (void)hipEventDestroy(e);
        }
    } starts, ends;
    for (int i = 0; i < c->iterations; ++i) {
        hipEvent_t s = nullptr, e = nullptr;
        MC_HIP(hipEventCreate(&s));
        starts.v.push_back(s);
        MC_HIP(hipEventCreate(&e));
        ends.v.push_back(e);
        MC_HIP(hipEventRecord(s, stream));
        const int rc = run_once();
        if (rc != MC_EP_OK) return rc;
        MC_HIP(hipEventRecord(e, stream));
    }
    MC_HIP(hipEventSynchronize(ends.v.back()));

    // the first timed iteration is dropped, as in the reference
    double total = 0.0, lo = 0.0, hi = 0.0;
    for (int i = 1; i < c->iterations; ++i) {
        float ms = 0.0f;
        MC_HIP(hipEventElapsedTime(&ms, starts.v[i], ends.v[i]));
        const double us = (double)ms * 1000.0;
        total += us;
        if (i == 1 || us < lo) lo = us;
        if (i == 1 || us > hi) hi = us;
    }
    result->average_us = total / (c->iterations - 1);
    result->min_us = lo;
    result->max_us = hi;
    return MC_EP_OK;
}

int mc_ep_buffer_create(mc_ep_world_t* w, int rank, int64_t num_ep_buffer_bytes, int disable_p2p,
                        mc_ep_buffer_t** out) {
    MC_ASSERT(w != nullptr && out != nullptr);
    Lock lock(g_mu);
    MC_ASSERT(rank >= 0 && rank < w->R);
    MC_ASSERT(num_ep_buffer_bytes >= 0);
    auto* b = new mc_ep_buffer();
    b->world = w;
    b->rank = rank;
    b->num_ep_buffer_bytes = num_ep_buffer_bytes;
    b->p2p_enabled = !disable_p2p;
    *out = b;
    return MC_EP_OK;
}

int mc_ep_buffer_destroy(mc_ep_buffer_t* b) {
    Lock lock(g_mu);
    delete b;
    return MC_EP_OK;
}

int mc_ep_buffer_pending_calls(const mc_ep_buffer_t* b, int* dispatch_pending, int* combine_pending) {
    MC_ASSERT(b != nullptr && dispatch_pending != nullptr && combine_pending != nullptr);
    Lock lock(g_mu);
    const mc_ep_world* w = b->world;
    long long d = w->dispatch_calls[b->rank] - w->dispatch_base;
    long long c = w->combine_calls[b->rank] - w->combine_base;
    if (d < 0) d = 0;
    if (c < 0) c = 0;
    if (w->unfinished) d += 1;   // launched in part: its second part still reads the round's tensors
    *dispatch_pending = (int)d;
    *combine_pending = (int)c;
    return MC_EP_OK;
}

int mc_ep_buffer_ibgda_disabled(const mc_ep_buffer_t*) { return 1; }
int mc_ep_buffer_p2p_enabled(const mc_ep_buffer_t* b) { return b && b->p2p_enabled ? 1 : 0; }
int mc_ep_buffer_use_fast_path(const mc_ep_buffer_t*) { return 1; }
int mc_ep_buffer_is_roce(const mc_ep_buffer_t*) { return 0; }

int mc_ep_buffer_dispatch(mc_ep_buffer_t* b, uint64_t x_ptr, uint64_t topk_idx_ptr, uint64_t active_ranks_ptr,
                          int num_tokens, int hidden, int num_topk, int max_tokens, int num_experts,
                          int timeout_us, int use_fp8, uint64_t recv_x_ptr, uint64_t recv_scales_ptr,
                          uint64_t recv_count_ptr, uint64_t src_info_ptr, uint64_t layout_range_ptr, int async,
                          int return_recv_hook, uint64_t compute_stream_ptr, mc_ep_event_t** event_out,
                          mc_ep_hook_t** hook_out) {
    MC_ASSERT(b != nullptr && event_out != nullptr && hook_out != nullptr);
    *event_out = nullptr;
    *hook_out = nullptr;
    if (int rc = refuse_capture(compute_stream_ptr)) return rc;
    Lock lock(g_mu);
    mc_ep_world* w = b->world;
    const int num_ranks = w->R;
    // mooncake_ep_buffer.cpp:202-206
    MC_ASSERT(num_experts % num_ranks == 0);
    MC_ASSERT(hidden % 16 == 0 && hidden % 128 == 0);
    MC_ASSERT(num_tokens <= max_tokens);
    // :212-214: the reference's communication buffer must hold this shape
    MC_ASSERT(mc_ep_get_buffer_size_hint(max_tokens, hidden, num_ranks, num_experts) <=
              (uint64_t)b->num_ep_buffer_bytes);
    MC_ASSERT(!(async && return_recv_hook));   // :226
    // :241-251
    MC_ASSERT(active_ranks_ptr != 0);
    MC_ASSERT(num_tokens == 0 || (x_ptr != 0 && topk_idx_ptr != 0));
    MC_ASSERT(recv_x_ptr != 0 && recv_count_ptr != 0);
    MC_ASSERT(src_info_ptr != 0 && layout_range_ptr != 0);
    if (use_fp8) {
        MC_ASSERT(((long long)num_ranks * max_tokens) % 4 == 0);
        MC_ASSERT(recv_scales_ptr != 0);
    }
    MC_ASSERT(num_topk <= kMaxTopK);
    MC_ASSERT(!w->silent[b->rank]);

    const long long call = w->dispatch_calls[b->rank];
    auto* prp = round_for_call(w, w->dispatch_rounds, w->dispatch_base, call);
    MC_ASSERT(prp != nullptr);
    w->dispatch_calls[b->rank] = call + 1;
    auto& pr = *prp;
    DispatchPost& p = pr.posts[b->rank];
    p.present = true;
    p.x = x_ptr; p.topk_idx = topk_idx_ptr; p.active_ranks = active_ranks_ptr;
    p.num_tokens = num_tokens; p.hidden = hidden; p.num_topk = num_topk; p.max_tokens = max_tokens;
    p.num_experts = num_experts; p.timeout_us = timeout_us; p.use_fp8 = use_fp8 ? 1 : 0;
    p.recv_x = recv_x_ptr; p.recv_scales = recv_scales_ptr; p.recv_count = recv_count_ptr;
    p.src_info = src_info_ptr; p.layout_range = layout_range_ptr;
    p.async = async != 0; p.hook = return_recv_hook != 0;
    p.stream = (hipStream_t)compute_stream_ptr;
    const bool blocking = w->tuning.blocking != 0;
    if (blocking)
        if (int e = hand_off_before(b, p.stream, &p.hand)) return e;
    std::shared_ptr<Round> state = pr.state;

    if (int e = drain_dispatch(w)) return e;
    if (int e = wait_for_round(w, state, lock)) return e;
    if (blocking)
        if (int e = hand_off_after(state.get(), (hipStream_t)compute_stream_ptr, !async && !return_recv_hook)) return e;
    if (async) {
        auto* ev = new mc_ep_event();
        ev->round = state;
        *event_out = ev;
    }
    if (return_recv_hook) {
        auto* h = new mc_ep_hook();
        h->world = w;
        h->round = state;
        h->stream = (hipStream_t)compute_stream_ptr;
        *hook_out = h;
    }
    return MC_EP_OK;
}

int mc_ep_buffer_combine(mc_ep_buffer_t* b, uint64_t x_ptr, uint64_t topk_idx_ptr, uint64_t topk_weights_ptr,
                         uint64_t src_info_ptr, uint64_t layout_range_ptr, uint64_t active_ranks_ptr,
                         int num_local_experts, int num_combined_tokens, int hidden, int num_topk, int max_tokens,
                         int num_experts, int timeout_us, int zero_copy, uint64_t combined_x_ptr, int async,
                         int return_recv_hook, uint64_t compute_stream_ptr, mc_ep_event_t** event_out,
                         mc_ep_hook_t** hook_out) {
    MC_ASSERT(b != nullptr && event_out != nullptr && hook_out != nullptr);
    *event_out = nullptr;
    *hook_out = nullptr;
    if (int rc = refuse_capture(compute_stream_ptr)) return rc;
    Lock lock(g_mu);
    mc_ep_world* w = b->world;
    const int num_ranks = w->R;
    if (zero_copy)
        return fail(MC_EP_ERR_UNSUPPORTED,
                    "Mooncake EP zero-copy combine is not supported; pass the expert output tensor to combine() "
                    "with zero_copy=False");
    // mooncake_ep_buffer.cpp:351-367
    MC_ASSERT(num_experts % num_ranks == 0);
    MC_ASSERT(num_local_experts == num_experts / num_ranks);
    MC_ASSERT(hidden % 16 == 0 && hidden % 128 == 0);
    MC_ASSERT(num_combined_tokens <= max_tokens);
    MC_ASSERT(num_combined_tokens == 0 || (x_ptr != 0 && topk_idx_ptr != 0 && topk_weights_ptr != 0));
    MC_ASSERT(src_info_ptr != 0 && layout_range_ptr != 0);
    MC_ASSERT(active_ranks_ptr != 0);
    MC_ASSERT(num_combined_tokens == 0 || combined_x_ptr != 0);
    MC_ASSERT(mc_ep_get_buffer_size_hint(max_tokens, hidden, num_ranks, num_experts) <=
              (uint64_t)b->num_ep_buffer_bytes);   // :370-372
    MC_ASSERT(!(async && return_recv_hook));       // :384
    MC_ASSERT(num_topk <= kMaxTopK);
    MC_ASSERT(!w->silent[b->rank]);

    const long long call = w->combine_calls[b->rank];
    auto* prp = round_for_call(w, w->combine_rounds, w->combine_base, call);
    MC_ASSERT(prp != nullptr);
    w->combine_calls[b->rank] = call + 1;
    auto& pr = *prp;
    CombinePost& p = pr.posts[b->rank];
    p.present = true;
    p.x = x_ptr; p.topk_idx = topk_idx_ptr; p.topk_weights = topk_weights_ptr; p.src_info = src_info_ptr;
    p.layout_range = layout_range_ptr; p.active_ranks = active_ranks_ptr; p.out = combined_x_ptr;
    p.num_tokens = num_combined_tokens; p.hidden = hidden; p.num_topk = num_topk; p.max_tokens = max_tokens;
    p.num_experts = num_experts; p.timeout_us = timeout_us;
    p.async = async != 0; p.hook = return_recv_hook != 0;
    p.stream = (hipStream_t)compute_stream_ptr;
    const bool blocking = w->tuning.blocking != 0;
    if (blocking)
        if (int e = hand_off_before(b, p.stream, &p.hand)) return e;
    std::shared_ptr<Round> state = pr.state;

    if (int e = drain_combine(w)) return e;
    if (int e = wait_for_round(w, state, lock)) return e;
    if (blocking)
        if (int e = hand_off_after(state.get(), (hipStream_t)compute_stream_ptr, !async && !return_recv_hook)) return e;
    if (async) {
        auto* ev = new mc_ep_event();
        ev->round = state;
        *event_out = ev;
    }
    if (return_recv_hook) {
        auto* h = new mc_ep_hook();
        h->world = w;
        h->round = state;
        h->stream = (hipStream_t)compute_stream_ptr;
        *hook_out = h;
    }
    return MC_EP_OK;
}

int mc_ep_event_create(uint64_t stream_ptr, mc_ep_event_t** out) {
    MC_ASSERT(out != nullptr);
    auto ev = std::make_unique<mc_ep_event>();
    MC_HIP(hipEventCreateWithFlags(&ev->own, hipEventDisableTiming));
    MC_HIP(hipEventRecord(ev->own, (hipStream_t)stream_ptr));
    *out = ev.release();
    return MC_EP_OK;
}

int mc_ep_event_current_stream_wait(mc_ep_event_t* ev, uint64_t stream_ptr) {
    MC_ASSERT(ev != nullptr);
    if (ev->own) {
        MC_HIP(hipStreamWaitEvent((hipStream_t)stream_ptr, ev->own, 0));
        return MC_EP_OK;
    }
    Lock lock(g_mu);
    if (!ev->round || !ev->round->launched) return round_not_ready(ev->round.get());
    return ev->round->make_wait((hipStream_t)stream_ptr);
}

int mc_ep_event_synchronize(mc_ep_event_t* ev) {
    MC_ASSERT(ev != nullptr);
    if (ev->own) {
        MC_HIP(hipEventSynchronize(ev->own));
        return MC_EP_OK;
    }
    hipEvent_t done = nullptr;
    hipStream_t launch = nullptr;
    {
        Lock lock(g_mu);
        if (!ev->round || !ev->round->launched) return round_not_ready(ev->round.get());
        done = ev->round->done;
        launch = ev->round->launch_stream;
    }
    // the wait itself happens without the lock; the handle keeps the round, and so its event, alive.
    // An async caller's round always has its event; without one, the round's stream says the same.
    if (done) MC_HIP(hipEventSynchronize(done));
    else MC_HIP(hipStreamSynchronize(launch));
    return MC_EP_OK;
}

int mc_ep_event_destroy(mc_ep_event_t* ev) {
    if (!ev) return MC_EP_OK;
    if (ev->own) (void)hipEventDestroy(ev->own);
    Lock lock(g_mu);   // the last handle of a round gives its event back to the pool
    delete ev;
    return MC_EP_OK;
}

int mc_ep_hook_call(mc_ep_hook_t* h) {
    MC_ASSERT(h != nullptr);
    Lock lock(g_mu);
    if (!h->round || !h->round->launched) return round_not_ready(h->round.get());
    // the first hook of a round launched in two parts enqueues the second part (the reference's
    // RECV phase, mooncake_ep_buffer.cpp:330-335)
    if (h->round->finish)
        if (int e = finish_round(h->world, h->round.get())) return e;
    if (!h->round->failure.empty()) return round_not_ready(h->round.get());
    return h->round->make_wait(h->stream);
}

int mc_ep_hook_destroy(mc_ep_hook_t* h) {
    Lock lock(g_mu);
    delete h;
    return MC_EP_OK;
}

int mc_ep_debug_set_stream_occupancy(int waves_per_cu) {
    set_stream_occupancy(waves_per_cu);
    return MC_EP_OK;
}

int mc_ep_debug_stream(int kind, uint64_t dst_ptr, uint64_t src_ptr, uint64_t unit_bytes, uint64_t stream_ptr) {
    MC_ASSERT(dst_ptr != 0 && src_ptr != 0 && unit_bytes % 16 == 0 && kind >= 0 && kind <= 5);
    MC_HIP(launch_stream(kind, (void*)dst_ptr, (const void*)src_ptr, (size_t)unit_bytes, (hipStream_t)stream_ptr));
    return MC_EP_OK;
}

int mc_ep_debug_gather_rows(uint64_t dst_ptr, uint64_t src_ptr, int row_bytes, int64_t out_rows, int regions,
                            int64_t region_rows, int used, uint64_t stream_ptr) {
    MC_ASSERT(dst_ptr != 0 && src_ptr != 0 && row_bytes > 0 && row_bytes % 1024 == 0 && out_rows >= 0);
    MC_ASSERT(regions > 0 && used > 0 && region_rows >= used && out_rows < (1ll << 28));
    MC_HIP(launch_stream_rows((void*)dst_ptr, (const void*)src_ptr, row_bytes, (long long)out_rows, regions,
                              (long long)region_rows, used, (hipStream_t)stream_ptr));
    return MC_EP_OK;
}

int mc_ep_debug_scatter_rows(uint64_t dst_ptr, uint64_t src_ptr, int row_bytes, int64_t in_rows, int regions,
                             int64_t region_rows, int used, uint64_t stream_ptr) {
    MC_ASSERT(dst_ptr != 0 && src_ptr != 0 && row_bytes > 0 && row_bytes % 1024 == 0 && in_rows >= 0);
    MC_ASSERT(regions > 0 && used > 0 && region_rows >= used && in_rows < (1ll << 28));
    MC_HIP(launch_stream_rows_scatter((void*)dst_ptr, (const void*)src_ptr, row_bytes, (long long)in_rows, regions,
                                      (long long)region_rows, used, (hipStream_t)stream_ptr));
    return MC_EP_OK;
}

int mc_ep_debug_copy(uint64_t dst_ptr, uint64_t src_ptr, uint64_t bytes, uint64_t stream_ptr) {
    MC_ASSERT(dst_ptr != 0 && src_ptr != 0 && bytes % 16 == 0);
    MC_HIP(launch_copy((void*)dst_ptr, (const void*)src_ptr, (size_t)bytes, (hipStream_t)stream_ptr));
    return MC_EP_OK;
}

}  // extern "C"
