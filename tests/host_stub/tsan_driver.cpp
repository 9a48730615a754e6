// Drives the per-rank collectives of the library's host runtime from many threads, in a host-only build
// (see hip/hip_runtime.h beside this file) under ThreadSanitizer: the thread-per-rank mode (option
// "blocking") in its three completion modes, a late rank, a rank that goes silent while its peers wait for
// it, a call that times out and stays posted, a rank whose call fails, events and hooks released on other
// threads than the ones that made them, and readers of a world's state beside its callers.  Uses nothing
// but the public C ABI; device addresses are made-up numbers (nothing on the host dereferences them).
//
//   tsan_driver              every scenario once; exit status 0 when all checks hold
//   tsan_driver --time R N   N steps of R threads, one per rank: prints microseconds per step of host time
#include <atomic>
#include <chrono>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <vector>

#include <hip/hip_runtime.h>

#include "mooncake_ep_hip.h"

namespace {

int g_failures = 0;
std::atomic<int> g_thread_failures{0};

#define CHECK(cond)                                                                        \
    do {                                                                                   \
        if (!(cond)) {                                                                     \
            std::fprintf(stderr, "CHECK failed %s:%d: %s (last error: %s)\n", __FILE__, __LINE__, #cond, \
                         mc_ep_last_error());                                              \
            ++g_failures;                                                                  \
        }                                                                                  \
    } while (0)
#define TCHECK(cond)                                                                       \
    do {                                                                                   \
        if (!(cond)) {                                                                     \
            std::fprintf(stderr, "CHECK failed %s:%d: %s (last error: %s)\n", __FILE__, __LINE__, #cond, \
                         mc_ep_last_error());                                              \
            g_thread_failures.fetch_add(1);                                                \
        }                                                                                  \
    } while (0)

struct Shape {
    int R, T, H, K, E;
    int L() const { return E / R; }
};

// made-up, 256-byte aligned "device addresses", distinct per (rank, field, generation)
uint64_t fake(int rank, int field, int gen = 0) {
    return 0x100000000ull + ((uint64_t)rank << 24) + ((uint64_t)field << 16) + ((uint64_t)(gen & 0xff) << 8);
}

struct World {
    Shape s;
    mc_ep_world_t* w = nullptr;
    std::vector<mc_ep_buffer_t*> bufs;
    explicit World(const Shape& shape, bool blocking, int timeout_ms = 30000) : s(shape) {
        CHECK(mc_ep_world_create(s.R, &w) == MC_EP_OK);
        if (blocking) CHECK(mc_ep_world_set_option(w, "blocking", 1) == MC_EP_OK);
        CHECK(mc_ep_world_set_option(w, "block_timeout_ms", timeout_ms) == MC_EP_OK);
        const uint64_t bytes = mc_ep_get_buffer_size_hint(s.T, s.H, s.R, s.E);
        bufs.resize(s.R);
        for (int r = 0; r < s.R; ++r) CHECK(mc_ep_buffer_create(w, r, (int64_t)bytes, 0, &bufs[r]) == MC_EP_OK);
    }
    ~World() {
        for (auto* b : bufs) mc_ep_buffer_destroy(b);
        mc_ep_world_destroy(w);
    }
};

enum Mode { kDefault = 0, kAsync = 1, kHook = 2 };

// one rank's dispatch in the given completion mode, waited for the way a caller of the reference does
int rank_dispatch(World& W, int r, int gen, bool fp8, Mode mode, hipStream_t stream, mc_ep_event_t** keep_event = nullptr) {
    const Shape& s = W.s;
    mc_ep_event_t* ev = nullptr;
    mc_ep_hook_t* hook = nullptr;
    int rc = mc_ep_buffer_dispatch(W.bufs[r], fake(r, 1), fake(r, 2), fake(r, 3), s.T, s.H, s.K, s.T, s.E, -1, fp8 ? 1 : 0,
                                   fake(r, 4, gen), fp8 ? fake(r, 5, gen) : 0, fake(r, 6, gen), fake(r, 7, gen),
                                   fake(r, 8, gen), mode == kAsync, mode == kHook, (uint64_t)stream, &ev, &hook);
    if (rc != MC_EP_OK) return rc;
    if (mode == kAsync) {
        if (!ev) return -1;
        rc = mc_ep_event_current_stream_wait(ev, (uint64_t)stream);
        if (keep_event) *keep_event = ev;
        else mc_ep_event_destroy(ev);
    }
    if (mode == kHook) {
        if (!hook) return -1;
        rc = mc_ep_hook_call(hook);
        mc_ep_hook_destroy(hook);
    }
    return rc;
}

int rank_combine(World& W, int r, int gen, Mode mode, hipStream_t stream) {
    const Shape& s = W.s;
    mc_ep_event_t* ev = nullptr;
    mc_ep_hook_t* hook = nullptr;
    int rc = mc_ep_buffer_combine(W.bufs[r], fake(r, 9, gen), fake(r, 2), fake(r, 10), fake(r, 7, gen), fake(r, 8, gen),
                                  fake(r, 3), s.L(), s.T, s.H, s.K, s.T, s.E, -1, 0, fake(r, 11, gen), mode == kAsync,
                                  mode == kHook, (uint64_t)stream, &ev, &hook);
    if (rc != MC_EP_OK) return rc;
    if (mode == kAsync) {
        if (!ev) return -1;
        rc = mc_ep_event_synchronize(ev);
        mc_ep_event_destroy(ev);
    }
    if (mode == kHook) {
        if (!hook) return -1;
        rc = mc_ep_hook_call(hook);
        mc_ep_hook_destroy(hook);
    }
    return rc;
}

void expect_drained(World& W) {
    for (int r = 0; r < W.s.R; ++r) {
        int d = -1, c = -1;
        CHECK(mc_ep_buffer_pending_calls(W.bufs[r], &d, &c) == MC_EP_OK);
        CHECK(d == 0 && c == 0);
    }
}

// ---- scenarios ---------------------------------------------------------------------------------------

// a thread per rank, every completion mode in turn, fp8 and bf16, one rank late now and then
void scenario_thread_per_rank() {
    std::puts("scenario: a thread per rank, three completion modes, a late rank");
    World W({4, 32, 1024, 4, 16}, true);
    const int steps = 60;
    std::vector<std::thread> threads;
    for (int r = 0; r < W.s.R; ++r)
        threads.emplace_back([&, r] {
            hipStream_t stream = nullptr;
            TCHECK(hipStreamCreateWithFlags(&stream, hipStreamNonBlocking) == hipSuccess);
            for (int i = 0; i < steps; ++i) {
                const Mode mode = (Mode)(i % 3);
                if (r == 2 && i % 7 == 3) std::this_thread::sleep_for(std::chrono::milliseconds(2));
                TCHECK(rank_dispatch(W, r, i, (i & 1) == 0, mode, stream) == MC_EP_OK);
                TCHECK(rank_combine(W, r, i, mode, stream) == MC_EP_OK);
                TCHECK(hipStreamSynchronize(stream) == hipSuccess);
            }
            TCHECK(hipStreamDestroy(stream) == hipSuccess);
        });
    for (auto& t : threads) t.join();
    expect_drained(W);
}

// one rank stops calling; another thread marks it silent while its peers are blocked waiting for it
void scenario_rank_goes_silent() {
    std::puts("scenario: a rank goes silent while its peers wait");
    World W({4, 16, 512, 2, 8}, true, 20000);
    const int steps = 24, dies_after = 5, dead = 3;
    std::vector<std::thread> threads;
    std::atomic<bool> stopped{false};
    for (int r = 0; r < W.s.R; ++r)
        threads.emplace_back([&, r] {
            for (int i = 0; i < steps; ++i) {
                if (r == dead && i == dies_after) {
                    stopped.store(true);
                    return;                                            // the rank's process is gone
                }
                TCHECK(rank_dispatch(W, r, i, false, kDefault, nullptr) == MC_EP_OK);
                TCHECK(rank_combine(W, r, i, kDefault, nullptr) == MC_EP_OK);
            }
        });
    while (!stopped.load()) std::this_thread::sleep_for(std::chrono::milliseconds(1));
    std::this_thread::sleep_for(std::chrono::milliseconds(5));         // the peers are blocked in their next call by now
    CHECK(mc_ep_world_set_rank_silent(W.w, dead, 1) == MC_EP_OK);
    for (auto& t : threads) t.join();
    for (int r = 0; r < W.s.R; ++r) {
        if (r == dead) continue;
        int d = -1, c = -1;
        CHECK(mc_ep_buffer_pending_calls(W.bufs[r], &d, &c) == MC_EP_OK && d == 0 && c == 0);
    }
}

// a call that waits longer than block_timeout_ms fails with MC_EP_ERR_PENDING and stays posted: the round
// goes when the peer arrives
void scenario_timeout_stays_posted() {
    std::puts("scenario: a blocking call times out and stays posted");
    World W({2, 16, 512, 2, 8}, true, 30);
    std::atomic<int> first_rc{-100};
    std::thread a([&] { first_rc.store(rank_dispatch(W, 0, 0, true, kDefault, nullptr)); });
    a.join();
    CHECK(first_rc.load() == MC_EP_ERR_PENDING);
    CHECK(std::strstr(mc_ep_last_error(), "") != nullptr);
    int d = -1, c = -1;
    CHECK(mc_ep_buffer_pending_calls(W.bufs[0], &d, &c) == MC_EP_OK && d == 1 && c == 0);
    std::thread b([&] { TCHECK(rank_dispatch(W, 1, 0, true, kDefault, nullptr) == MC_EP_OK); });
    b.join();
    CHECK(mc_ep_buffer_pending_calls(W.bufs[0], &d, &c) == MC_EP_OK && d == 0 && c == 0);
    // both go on together
    std::thread t0([&] { TCHECK(rank_combine(W, 0, 0, kDefault, nullptr) == MC_EP_OK); });
    std::thread t1([&] { TCHECK(rank_combine(W, 1, 0, kDefault, nullptr) == MC_EP_OK); });
    t0.join();
    t1.join();
    expect_drained(W);
}

// a rank whose call fails its host checks (the reference raises there) takes itself out; the others go on
void scenario_rank_raises() {
    std::puts("scenario: a rank's call fails and the rank leaves the world");
    World W({4, 16, 512, 2, 8}, true, 20000);
    const int steps = 12, bad = 1, fails_at = 4;
    std::vector<std::thread> threads;
    for (int r = 0; r < W.s.R; ++r)
        threads.emplace_back([&, r] {
            for (int i = 0; i < steps; ++i) {
                if (r == bad && i == fails_at) {
                    mc_ep_event_t* ev = nullptr;
                    mc_ep_hook_t* hook = nullptr;
                    // more tokens than num_max_dispatch_tokens_per_rank: a host assertion of the reference
                    const int rc = mc_ep_buffer_dispatch(W.bufs[r], fake(r, 1), fake(r, 2), fake(r, 3), W.s.T + 1, W.s.H,
                                                         W.s.K, W.s.T, W.s.E, -1, 0, fake(r, 4), 0, fake(r, 6), fake(r, 7),
                                                         fake(r, 8), 0, 0, 0, &ev, &hook);
                    TCHECK(rc == MC_EP_ERR_ASSERT);
                    TCHECK(mc_ep_world_set_rank_silent(W.w, r, 1) == MC_EP_OK);
                    return;
                }
                TCHECK(rank_dispatch(W, r, i, false, (Mode)(i % 3), nullptr) == MC_EP_OK);
                TCHECK(rank_combine(W, r, i, (Mode)(i % 3), nullptr) == MC_EP_OK);
            }
        });
    for (auto& t : threads) t.join();
}

// events handed to other threads, released there while rounds go on; one outlives its world
void scenario_handles_cross_threads() {
    std::puts("scenario: events and hooks released on other threads, an event that outlives its world");
    mc_ep_event_t* survivor = nullptr;
    {
        World W({2, 16, 512, 2, 8}, true);
        const int steps = 40;
        std::vector<mc_ep_event_t*> handed[2];
        for (auto& v : handed) v.assign(steps, nullptr);
        std::atomic<int> produced[2] = {{0}, {0}};
        std::vector<std::thread> threads;
        for (int r = 0; r < 2; ++r)
            threads.emplace_back([&, r] {
                for (int i = 0; i < steps; ++i) {
                    mc_ep_event_t* ev = nullptr;
                    TCHECK(rank_dispatch(W, r, i, false, kAsync, nullptr, &ev) == MC_EP_OK);
                    handed[r][i] = ev;
                    produced[r].store(i + 1, std::memory_order_release);
                    TCHECK(rank_combine(W, r, i, kDefault, nullptr) == MC_EP_OK);
                }
            });
        // a third thread waits on and releases what the rank threads made
        std::thread reaper([&] {
            for (int i = 0; i < steps; ++i)
                for (int r = 0; r < 2; ++r) {
                    while (produced[r].load(std::memory_order_acquire) <= i) std::this_thread::yield();
                    mc_ep_event_t* ev = handed[r][i];
                    TCHECK(ev != nullptr);
                    TCHECK(mc_ep_event_synchronize(ev) == MC_EP_OK);
                    if (r == 0 && i == steps - 1) survivor = ev;
                    else TCHECK(mc_ep_event_destroy(ev) == MC_EP_OK);
                }
        });
        for (auto& t : threads) t.join();
        reaper.join();
        expect_drained(W);
    }
    CHECK(survivor != nullptr);
    CHECK(mc_ep_event_synchronize(survivor) == MC_EP_OK);      // the handle keeps the round and its event alive
    CHECK(mc_ep_event_destroy(survivor) == MC_EP_OK);
}

// one driver thread for all ranks (the default, non-blocking mode) with two-part hook rounds whose hooks are
// dropped uncalled, while another thread reads and writes options and asks for pending calls
void scenario_driver_thread_with_readers() {
    std::puts("scenario: one driver thread, hooks dropped uncalled, readers beside it");
    World W({4, 16, 512, 2, 8}, false);
    std::atomic<bool> done{false};
    std::thread reader([&] {
        int v = 0, d = 0, c = 0;
        while (!done.load()) {
            TCHECK(mc_ep_world_get_option(W.w, "combine_direct", &v) == MC_EP_OK);
            TCHECK(mc_ep_world_set_option(W.w, "combine_waves", 4) == MC_EP_OK);
            TCHECK(mc_ep_buffer_pending_calls(W.bufs[1], &d, &c) == MC_EP_OK);
            TCHECK(mc_ep_world_get_option(W.w, "last_dispatch_launches", &v) == MC_EP_OK);
        }
    });
    const Shape& s = W.s;
    for (int i = 0; i < 50; ++i) {
        std::vector<mc_ep_hook_t*> hooks(s.R, nullptr);
        for (int r = 0; r < s.R; ++r) {
            mc_ep_event_t* ev = nullptr;
            CHECK(mc_ep_buffer_dispatch(W.bufs[r], fake(r, 1), fake(r, 2), fake(r, 3), s.T, s.H, s.K, s.T, s.E, -1, 1,
                                        fake(r, 4, i), fake(r, 5, i), fake(r, 6, i), fake(r, 7, i), fake(r, 8, i), 0, 1, 0,
                                        &ev, &hooks[r]) == MC_EP_OK);
        }
        if (i % 2 == 0) {
            for (auto* h : hooks) CHECK(mc_ep_hook_call(h) == MC_EP_OK);
        }
        // odd steps: the hooks go uncalled, and the next dispatch has to enqueue the second part itself
        for (auto* h : hooks) CHECK(mc_ep_hook_destroy(h) == MC_EP_OK);
        for (int r = 0; r < s.R; ++r) CHECK(rank_combine(W, r, i, kDefault, nullptr) == MC_EP_OK);
    }
    done.store(true);
    reader.join();
    // the last step's second part is still owed (its hooks were dropped): one more dispatch settles it
    for (int r = 0; r < s.R; ++r) CHECK(rank_dispatch(W, r, 99, false, kDefault, nullptr) == MC_EP_OK);
    expect_drained(W);
}

double time_thread_per_rank(int R, int steps) {
    World W({R, 128, 7168, 8, 8 * R}, true);
    std::vector<std::thread> threads;
    std::atomic<int> ready{0};
    std::atomic<bool> go{false};
    std::chrono::steady_clock::time_point t0;
    for (int r = 0; r < R; ++r)
        threads.emplace_back([&, r] {
            hipStream_t stream = nullptr;
            hipStreamCreateWithFlags(&stream, hipStreamNonBlocking);
            ready.fetch_add(1);
            while (!go.load()) std::this_thread::yield();
            for (int i = 0; i < steps; ++i) {
                TCHECK(rank_dispatch(W, r, 0, false, kDefault, stream) == MC_EP_OK);
                TCHECK(rank_combine(W, r, 0, kDefault, stream) == MC_EP_OK);
                hipStreamSynchronize(stream);
            }
            hipStreamDestroy(stream);
        });
    while (ready.load() < R) std::this_thread::yield();
    t0 = std::chrono::steady_clock::now();
    go.store(true);
    for (auto& t : threads) t.join();
    const double us = std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count();
    return us / steps;
}

}  // namespace

int main(int argc, char** argv) {
    if (argc == 4 && !std::strcmp(argv[1], "--time")) {
        const int R = std::atoi(argv[2]), steps = std::atoi(argv[3]);
        std::printf("thread per rank, host only: %d ranks, %d steps: %.1f us per step\n", R, steps,
                    time_thread_per_rank(R, steps));
        return g_thread_failures.load() ? 1 : 0;
    }
    scenario_thread_per_rank();
    scenario_rank_goes_silent();
    scenario_timeout_stays_posted();
    scenario_rank_raises();
    scenario_handles_cross_threads();
    scenario_driver_thread_with_readers();
    const long events = hip_stub::g_live_events.load(), streams = hip_stub::g_live_streams.load(),
               allocs = hip_stub::g_live_allocs.load();
    std::printf("api calls %ld, live events %ld, live streams %ld, live allocations %ld\n", hip_stub::g_calls.load(),
                events, streams, allocs);
    CHECK(events == 0 && streams == 0 && allocs == 0);       // everything the worlds made went with them
    const int failures = g_failures + g_thread_failures.load();
    std::printf("%s (%d failed checks)\n", failures ? "FAILED" : "ok", failures);
    return failures ? 1 : 0;
}
