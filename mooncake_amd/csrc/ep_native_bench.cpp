// A Python-free driver of libmooncake_ep_hip.so: everything it needs from the
// library is in include/mooncake_ep_hip.h.  It builds a synthetic world in
// device memory, checks the routing outputs against a host count, and times
//   * fp8 (or bf16) dispatch + combine steps, whole world, back to back, and
//   * the library's native loop (the reference's _benchmark_legacy_buffer:
//     recv_count clear + bf16 dispatch + combine, legacy_buffer_perf.cpp:84-146).
//
//   ep_native_bench [--ranks R] [--tokens T] [--hidden H] [--experts E] [--topk K]
//                   [--bf16] [--warmups W] [--iterations N] [--per-rank] [--opt name=value ...]
//
// With --per-rank it first drives the per-rank Buffer calls (the reference's binding:
// mc_ep_buffer_dispatch / mc_ep_buffer_combine, one call per rank and collective) in the three
// completion modes, with one rank a call ahead of the others, and compares the combined rows bit for
// bit with the same multiply-add chain on the host; then once more with a thread per rank, each on a
// stream of its own, under the world's option "blocking".
//
// Exit status 0 means the self-checks passed.  Built by `make bench`.
#include <hip/hip_runtime.h>

#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <string>
#include <thread>
#include <utility>
#include <vector>

#include "mooncake_ep_hip.h"

namespace {

#define HIP_OK(cmd)                                                                                  \
    do {                                                                                             \
        hipError_t e_ = (cmd);                                                                       \
        if (e_ != hipSuccess) {                                                                      \
            std::fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #cmd, hipGetErrorString(e_)); \
            std::exit(2);                                                                            \
        }                                                                                            \
    } while (0)

#define EP_OK(cmd)                                                                              \
    do {                                                                                        \
        if ((cmd) != MC_EP_OK) {                                                                \
            std::fprintf(stderr, "%s:%d %s: %s\n", __FILE__, __LINE__, #cmd, mc_ep_last_error()); \
            std::exit(2);                                                                       \
        }                                                                                       \
    } while (0)

struct Args {
    int ranks = 32, tokens = 128, hidden = 7168, experts = 256, topk = 8, warmups = 20, iterations = 30;
    bool fp8 = true, per_rank = false;
    std::vector<std::pair<std::string, int>> options;   // --opt name=value: options of the world
};

Args parse(int argc, char** argv) {
    Args a;
    for (int i = 1; i < argc; ++i) {
        const std::string f = argv[i];
        auto value = [&]() -> int {
            if (i + 1 >= argc) {
                std::fprintf(stderr, "%s needs a value\n", f.c_str());
                std::exit(2);
            }
            return std::atoi(argv[++i]);
        };
        if (f == "--ranks") a.ranks = value();
        else if (f == "--tokens") a.tokens = value();
        else if (f == "--hidden") a.hidden = value();
        else if (f == "--experts") a.experts = value();
        else if (f == "--topk") a.topk = value();
        else if (f == "--warmups") a.warmups = value();
        else if (f == "--iterations") a.iterations = value();
        else if (f == "--bf16") a.fp8 = false;
        else if (f == "--per-rank") a.per_rank = true;
        else if (f == "--opt" && i + 1 < argc) {
            const std::string kv = argv[++i];
            const size_t eq = kv.find('=');
            if (eq == std::string::npos) {
                std::fprintf(stderr, "--opt wants name=value\n");
                std::exit(2);
            }
            a.options.emplace_back(kv.substr(0, eq), std::atoi(kv.c_str() + eq + 1));
        }
        else {
            std::fprintf(stderr, "unknown flag %s\n", f.c_str());
            std::exit(2);
        }
    }
    if (a.ranks < 1 || a.experts % a.ranks || a.hidden % 128 || a.topk < 1 || a.topk > a.experts || a.tokens < 1 ||
        a.iterations < 2 || (a.fp8 && ((long long)a.ranks * a.tokens) % 4)) {
        std::fprintf(stderr, "unusable shape\n");
        std::exit(2);
    }
    return a;
}

// xorshift: a reproducible stream that needs no library
struct Rng {
    uint64_t s;
    explicit Rng(uint64_t seed) : s(seed * 0x9E3779B97F4A7C15ull + 1) {}
    uint64_t next() {
        s ^= s << 13;
        s ^= s >> 7;
        s ^= s << 17;
        return s;
    }
    float unit() { return (float)((next() >> 40) & 0xFFFFFF) / 16777216.0f; }
};

uint16_t to_bf16(float f) {
    uint32_t u;
    std::memcpy(&u, &f, 4);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

template <typename T>
T* device_copy(const std::vector<T>& host) {
    T* d = nullptr;
    HIP_OK(hipMalloc((void**)&d, host.size() * sizeof(T)));
    HIP_OK(hipMemcpy(d, host.data(), host.size() * sizeof(T), hipMemcpyHostToDevice));
    return d;
}

template <typename T>
std::vector<uint64_t> per_rank(const T* base, size_t stride_elems, int ranks) {
    std::vector<uint64_t> p((size_t)ranks);
    for (int r = 0; r < ranks; ++r) p[(size_t)r] = (uint64_t)(base + (size_t)r * stride_elems);
    return p;
}

float from_bf16(uint16_t h) {
    const uint32_t u = (uint32_t)h << 16;
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

// What the per-rank self-test works on: per-rank device addresses and the host copies it checks against.
struct PerRank {
    int R, T, H, E, K;
    bool fp8;
    std::vector<uint64_t> x, idx, w, active, recv, scales, recv16, count, src, range, out;
    const uint16_t* out_base;
    const std::vector<uint16_t>* hx;
    const std::vector<float>* hw;
};

// Compares the combined rows on the device with the host's chain: fp32 multiply-add over k, one rounding.
int check_combined(const PerRank& p, const char* what) {
    const int R = p.R, T = p.T, H = p.H, K = p.K;
    std::vector<uint16_t> got((size_t)R * T * H);
    HIP_OK(hipMemcpy(got.data(), p.out_base, got.size() * 2, hipMemcpyDeviceToHost));
    for (size_t n = 0; n < (size_t)R * T; ++n) {
        for (int h = 0; h < H; ++h) {
            const float v = from_bf16((*p.hx)[n * H + h]);
            float acc = 0.0f;
            for (int k = 0; k < K; ++k) acc = std::fmaf(v, (*p.hw)[n * K + k], acc);
            if (got[n * H + h] != to_bf16(acc)) {
                std::fprintf(stderr, "%s: token %zu element %d is 0x%04x, expected 0x%04x\n", what, n, h,
                             got[n * H + h], to_bf16(acc));
                return 1;
            }
        }
    }
    return 0;
}

// One dispatch + combine through the per-rank calls.  mode 0: the caller's stream waits inside the
// call; 1: async, an event per call; 2: receive hooks.  Rank 0 posts its dispatch first and, with
// `ahead`, a second one before any other rank has posted its first.
int per_rank_cycle(std::vector<mc_ep_buffer_t*>& bufs, const PerRank& p, int mode, bool fp8, bool ahead,
                   hipStream_t stream, std::vector<mc_ep_event_t*>& keep) {
    const int R = p.R, T = p.T, H = p.H, E = p.E, K = p.K, L = E / R;
    const uint64_t s = (uint64_t)stream;
    const int async = mode == 1, hook = mode == 2;
    HIP_OK(hipMemsetAsync((void*)p.out_base, 0xFF, (size_t)R * T * H * 2, stream));
    std::vector<mc_ep_event_t*> events;
    std::vector<mc_ep_hook_t*> hooks;
    auto post_dispatch = [&](int r) {
        mc_ep_event_t* ev = nullptr;
        mc_ep_hook_t* hk = nullptr;
        EP_OK(mc_ep_buffer_dispatch(bufs[(size_t)r], p.x[(size_t)r], p.idx[(size_t)r], p.active[(size_t)r], T, H, K, T, E,
                                    -1, fp8 ? 1 : 0, fp8 ? p.recv[(size_t)r] : p.recv16[(size_t)r],
                                    fp8 ? p.scales[(size_t)r] : 0, p.count[(size_t)r], p.src[(size_t)r],
                                    p.range[(size_t)r], async, hook, s, &ev, &hk));
        if ((ev != nullptr) != (async != 0) || (hk != nullptr) != (hook != 0)) {
            std::fprintf(stderr, "per-rank dispatch: event / hook do not follow the flags\n");
            std::exit(1);
        }
        if (ev) events.push_back(ev);
        if (hk) hooks.push_back(hk);
    };
    const int rounds = ahead ? 2 : 1;
    for (int j = 0; j < rounds; ++j) post_dispatch(0);
    if (R > 1) {
        int dp = -1, cp = -1;
        EP_OK(mc_ep_buffer_pending_calls(bufs[0], &dp, &cp));
        if (dp != rounds || cp != 0) {
            std::fprintf(stderr, "per-rank: rank 0 has %d dispatches pending, expected %d\n", dp, rounds);
            return 1;
        }
        // waiting for a collective that other ranks have not joined is an error, not a hang
        if (async && mc_ep_event_synchronize(events[0]) != MC_EP_ERR_PENDING) {
            std::fprintf(stderr, "per-rank: an incomplete round did not report MC_EP_ERR_PENDING\n");
            return 1;
        }
    }
    for (int j = 0; j < rounds; ++j)
        for (int r = 1; r < R; ++r) post_dispatch(r);
    for (mc_ep_hook_t* hk : hooks) EP_OK(mc_ep_hook_call(hk));
    for (mc_ep_event_t* ev : events) EP_OK(mc_ep_event_current_stream_wait(ev, s));

    // the dispatched rows are the expert outputs (bf16) - fp8 rounds only have their counts checked
    std::vector<mc_ep_event_t*> cevents;
    std::vector<mc_ep_hook_t*> chooks;
    if (!fp8) {
        for (int r = 0; r < R; ++r) {
            mc_ep_event_t* ev = nullptr;
            mc_ep_hook_t* hk = nullptr;
            EP_OK(mc_ep_buffer_combine(bufs[(size_t)r], p.recv16[(size_t)r], p.idx[(size_t)r], p.w[(size_t)r],
                                       p.src[(size_t)r], p.range[(size_t)r], p.active[(size_t)r], L, T, H, K, T, E, -1,
                                       0, p.out[(size_t)r], async, hook, s, &ev, &hk));
            if (ev) cevents.push_back(ev);
            if (hk) chooks.push_back(hk);
        }
        for (mc_ep_hook_t* hk : chooks) EP_OK(mc_ep_hook_call(hk));
        for (mc_ep_event_t* ev : cevents) EP_OK(mc_ep_event_synchronize(ev));
    }
    HIP_OK(hipStreamSynchronize(stream));
    for (mc_ep_hook_t* hk : hooks) EP_OK(mc_ep_hook_destroy(hk));
    for (mc_ep_hook_t* hk : chooks) EP_OK(mc_ep_hook_destroy(hk));
    // events are the caller's to release whenever it likes: main does, after the world is gone
    keep.insert(keep.end(), events.begin(), events.end());
    keep.insert(keep.end(), cevents.begin(), cevents.end());
    if (fp8) return 0;

    char what[32];
    std::snprintf(what, sizeof(what), "per-rank mode %d", mode);
    return check_combined(p, what);
}

// A thread per rank, as a process per rank of the reference: each makes its own calls on its own stream
// and waits for its own stream only.  With the world's option "blocking" a call returns when the
// collective has been launched, so the stream order of the caller is enough.
int thread_per_rank(mc_ep_world_t* world, std::vector<mc_ep_buffer_t*>& bufs, const PerRank& p, int steps) {
    const int R = p.R, T = p.T, H = p.H, E = p.E, K = p.K, L = E / R;
    EP_OK(mc_ep_world_set_option(world, "blocking", 1));
    HIP_OK(hipMemset((void*)p.out_base, 0xFF, (size_t)R * T * H * 2));
    std::vector<int> failed((size_t)R, 0);
    // where a rank's thread spends a step: inside its dispatch call (and the wait on its event / hook), inside
    // its combine call, waiting for its stream (microseconds, summed over the steps)
    std::vector<double> in_dispatch((size_t)R, 0.0), in_combine((size_t)R, 0.0), in_sync((size_t)R, 0.0);
    const auto now = [] { return std::chrono::steady_clock::now(); };
    const auto us_since = [](std::chrono::steady_clock::time_point a) {
        return std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - a).count();
    };
    std::vector<std::thread> threads;
    std::atomic<int> ready{0};
    std::chrono::steady_clock::time_point t0;
    std::vector<std::chrono::steady_clock::time_point> finished((size_t)R);
    for (int r = 0; r < R; ++r) {
        threads.emplace_back([&, r] {
            hipStream_t mine;
            if (hipStreamCreateWithFlags(&mine, hipStreamNonBlocking) != hipSuccess) {
                failed[(size_t)r] = 1;
                return;
            }
            const uint64_t s = (uint64_t)mine;
            // all threads start their steps together; the last one to get here starts the clock
            if (ready.fetch_add(1) + 1 == R) t0 = std::chrono::steady_clock::now();
            while (ready.load() < R) std::this_thread::yield();
            for (int j = 0; j < steps && !failed[(size_t)r]; ++j) {
                const int mode = j % 3;   // default, async, hook in turn: every rank the same mode per step
                mc_ep_event_t* ev = nullptr;
                mc_ep_hook_t* hk = nullptr;
                auto mark = now();
                int rc = mc_ep_buffer_dispatch(bufs[(size_t)r], p.x[(size_t)r], p.idx[(size_t)r], p.active[(size_t)r],
                                               T, H, K, T, E, -1, 0, p.recv16[(size_t)r], 0, p.count[(size_t)r],
                                               p.src[(size_t)r], p.range[(size_t)r], mode == 1, mode == 2, s, &ev, &hk);
                if (rc == MC_EP_OK && ev) rc = mc_ep_event_current_stream_wait(ev, s);
                if (rc == MC_EP_OK && hk) rc = mc_ep_hook_call(hk);
                mc_ep_event_destroy(ev);
                mc_ep_hook_destroy(hk);
                ev = nullptr;
                hk = nullptr;
                in_dispatch[(size_t)r] += us_since(mark);
                mark = now();
                if (rc == MC_EP_OK)
                    rc = mc_ep_buffer_combine(bufs[(size_t)r], p.recv16[(size_t)r], p.idx[(size_t)r], p.w[(size_t)r],
                                              p.src[(size_t)r], p.range[(size_t)r], p.active[(size_t)r], L, T, H, K, T,
                                              E, -1, 0, p.out[(size_t)r], mode == 1, mode == 2, s, &ev, &hk);
                if (rc == MC_EP_OK && ev) rc = mc_ep_event_current_stream_wait(ev, s);
                if (rc == MC_EP_OK && hk) rc = mc_ep_hook_call(hk);
                mc_ep_event_destroy(ev);
                mc_ep_hook_destroy(hk);
                if (rc != MC_EP_OK) {
                    std::fprintf(stderr, "rank %d step %d: %s\n", r, j, mc_ep_last_error());
                    failed[(size_t)r] = 1;
                }
                in_combine[(size_t)r] += us_since(mark);
                mark = now();
                // the next step's dispatch rewrites what this step's combine reads: a rank must not run
                // ahead of its own stream, exactly as with the reference's buffers
                if (hipStreamSynchronize(mine) != hipSuccess) failed[(size_t)r] = 1;
                in_sync[(size_t)r] += us_since(mark);
            }
            finished[(size_t)r] = now();
            (void)hipStreamDestroy(mine);        // (milliseconds for 32 streams: not part of the steps)
        });
    }
    for (auto& t : threads) t.join();
    auto last = finished[0];
    for (int r = 1; r < R; ++r) last = finished[(size_t)r] > last ? finished[(size_t)r] : last;
    const double us = std::chrono::duration<double, std::micro>(last - t0).count();
    std::printf("thread per rank: %d threads, each on a stream of its own that it waits for after every step: %.0f us "
                "per bf16 dispatch + combine step\n", R, us / steps);
    double d = 0.0, c = 0.0, y = 0.0;
    for (int r = 0; r < R; ++r) {
        d += in_dispatch[(size_t)r];
        c += in_combine[(size_t)r];
        y += in_sync[(size_t)r];
    }
    std::printf("  of which a rank's thread spends, on average: %.0f us in its dispatch call, %.0f us in its combine call, "
                "%.0f us waiting for its stream\n", d / R / steps, c / R / steps, y / R / steps);
    EP_OK(mc_ep_world_set_option(world, "blocking", 0));
    for (int r = 0; r < R; ++r)
        if (failed[(size_t)r]) return 1;
    HIP_OK(hipDeviceSynchronize());
    return check_combined(p, "thread per rank");
}

}  // namespace

int main(int argc, char** argv) {
    const Args a = parse(argc, argv);
    const int R = a.ranks, T = a.tokens, H = a.hidden, E = a.experts, K = a.topk, L = E / R;
    const size_t RM = (size_t)R * T;

    // inputs: x ~ uniform(-1, 1) as bf16; top-k = K distinct experts per token; weights sum to one
    std::vector<uint16_t> hx((size_t)R * T * H);
    std::vector<int64_t> hidx((size_t)R * T * K);
    std::vector<float> hw((size_t)R * T * K);
    std::vector<long long> expect((size_t)E, 0);
    Rng rng(2026);
    for (auto& v : hx) v = to_bf16(rng.unit() * 2.0f - 1.0f);
    std::vector<int> pool((size_t)E);
    for (size_t n = 0; n < (size_t)R * T; ++n) {
        for (int e = 0; e < E; ++e) pool[(size_t)e] = e;
        float wsum = 0.0f;
        for (int k = 0; k < K; ++k) {   // partial Fisher-Yates: K distinct experts
            const int j = k + (int)(rng.next() % (uint64_t)(E - k));
            std::swap(pool[(size_t)k], pool[(size_t)j]);
            hidx[n * K + k] = pool[(size_t)k];
            expect[(size_t)pool[(size_t)k]]++;
            hw[n * K + k] = 0.1f + rng.unit();
            wsum += hw[n * K + k];
        }
        for (int k = 0; k < K; ++k) hw[n * K + k] /= wsum;
    }

    uint16_t* x = device_copy(hx);
    int64_t* idx = device_copy(hidx);
    float* wts = device_copy(hw);
    std::vector<int32_t> ones((size_t)R * R, 1);
    int32_t* active = device_copy(ones);
    const size_t payload = a.fp8 ? 1 : 2;
    uint8_t* recv_x = nullptr;
    float* scales = nullptr;
    uint16_t *recv_bf16 = nullptr, *expert_x = nullptr, *out = nullptr;
    int32_t *recv_count = nullptr, *src_info = nullptr;
    int64_t* layout_range = nullptr;
    HIP_OK(hipMalloc((void**)&recv_x, (size_t)R * L * RM * H * payload));
    if (a.fp8) HIP_OK(hipMalloc((void**)&scales, (size_t)R * L * (H / 128) * RM * sizeof(float)));
    HIP_OK(hipMalloc((void**)&recv_bf16, (size_t)R * L * RM * H * 2));     // the native loop's bf16 receive layout
    HIP_OK(hipMalloc((void**)&expert_x, (size_t)R * L * RM * H * 2));
    HIP_OK(hipMemset(expert_x, 0, (size_t)R * L * RM * H * 2));
    HIP_OK(hipMalloc((void**)&out, (size_t)R * T * H * 2));
    HIP_OK(hipMalloc((void**)&recv_count, (size_t)R * L * sizeof(int32_t)));
    HIP_OK(hipMalloc((void**)&src_info, (size_t)R * L * RM * sizeof(int32_t)));
    HIP_OK(hipMalloc((void**)&layout_range, (size_t)R * L * R * sizeof(int64_t)));

    const auto px = per_rank(x, (size_t)T * H, R), pidx = per_rank(idx, (size_t)T * K, R);
    const auto pw = per_rank(wts, (size_t)T * K, R), pact = per_rank(active, (size_t)R, R);
    const auto precv = per_rank(recv_x, (size_t)L * RM * H * payload, R);
    const auto pscales = a.fp8 ? per_rank(scales, (size_t)L * (H / 128) * RM, R) : std::vector<uint64_t>();
    const auto precv16 = per_rank(recv_bf16, (size_t)L * RM * H, R), pexp = per_rank(expert_x, (size_t)L * RM * H, R);
    const auto pout = per_rank(out, (size_t)T * H, R), pcnt = per_rank(recv_count, (size_t)L, R);
    const auto psrc = per_rank(src_info, (size_t)L * RM, R), plr = per_rank(layout_range, (size_t)L * R, R);
    const std::vector<int32_t> tokens((size_t)R, T);

    mc_ep_world_t* world = nullptr;
    EP_OK(mc_ep_world_create(R, &world));
    for (const auto& o : a.options) EP_OK(mc_ep_world_set_option(world, o.first.c_str(), o.second));
    hipStream_t stream;
    HIP_OK(hipStreamCreate(&stream));
    const uint64_t s = (uint64_t)stream;

    std::vector<mc_ep_event_t*> kept_events;
    if (a.per_rank) {
        PerRank p{R, T, H, E, K, a.fp8, px, pidx, pw, pact, precv, pscales, precv16, pcnt, psrc, plr, pout, out, &hx, &hw};
        std::vector<mc_ep_buffer_t*> bufs((size_t)R, nullptr);
        const int64_t hint = (int64_t)mc_ep_get_buffer_size_hint(T, H, R, E);
        for (int r = 0; r < R; ++r) EP_OK(mc_ep_buffer_create(world, r, hint, 0, &bufs[(size_t)r]));
        for (int mode = 0; mode < 3; ++mode) {
            for (int ahead = 0; ahead < 2; ++ahead) {
                if (per_rank_cycle(bufs, p, mode, false, ahead != 0, stream, kept_events)) return 1;
                if (a.fp8 && per_rank_cycle(bufs, p, mode, true, ahead != 0, stream, kept_events)) return 1;
            }
        }
        if (thread_per_rank(world, bufs, p, a.iterations < 6 ? 6 : a.iterations)) return 1;
        for (mc_ep_buffer_t* b : bufs) EP_OK(mc_ep_buffer_destroy(b));
        std::printf("per-rank calls: 3 completion modes x (in step, rank 0 a call ahead), bf16%s, and a thread per "
                    "rank: combined rows equal the host chain\n", a.fp8 ? " and fp8" : "");
    }

    auto dispatch = [&] {
        EP_OK(mc_ep_world_dispatch(world, px.data(), pidx.data(), tokens.data(), H, K, T, E, a.fp8 ? 1 : 0, precv.data(),
                                   a.fp8 ? pscales.data() : nullptr, pcnt.data(), psrc.data(), plr.data(),
                                   MC_EP_PHASE_ALL, s));
    };
    auto combine = [&] {
        EP_OK(mc_ep_world_combine(world, pexp.data(), pidx.data(), pw.data(), psrc.data(), plr.data(), pact.data(),
                                  tokens.data(), H, K, T, E, pout.data(), MC_EP_PHASE_ALL, s));
    };

    // self-check: every expert received exactly the rows that name it
    dispatch();
    HIP_OK(hipStreamSynchronize(stream));
    std::vector<int32_t> got((size_t)E);
    HIP_OK(hipMemcpy(got.data(), recv_count, (size_t)E * sizeof(int32_t), hipMemcpyDeviceToHost));
    for (int e = 0; e < E; ++e) {
        if (got[(size_t)e] != expect[(size_t)e]) {
            std::fprintf(stderr, "self-check failed: expert %d received %d rows, %lld selections name it\n", e,
                         got[(size_t)e], expect[(size_t)e]);
            return 1;
        }
    }
    // the mock expert of the reference's tests, on valid rows only
    EP_OK(mc_ep_world_cast_back(world, precv.data(), a.fp8 ? pscales.data() : nullptr, pcnt.data(), 0, pexp.data(), H, K,
                                T, E, s));

    for (int i = 0; i < a.warmups; ++i) {
        dispatch();
        combine();
    }
    HIP_OK(hipStreamSynchronize(stream));
    const auto t0 = std::chrono::steady_clock::now();
    for (int i = 0; i < a.iterations; ++i) {
        dispatch();
        combine();
    }
    HIP_OK(hipStreamSynchronize(stream));
    const double step_us =
        std::chrono::duration<double, std::micro>(std::chrono::steady_clock::now() - t0).count() / a.iterations;

    const double N = (double)R * T, S = N * K;
    const double row = a.fp8 ? H + H / 128 * 4.0 : 2.0 * H;
    const double bytes = N * H * 2 + N * K * 8 + S * (row + 4) + E * 4.0 + (double)E * R * 8   // dispatch
                         + S * H * 2 + N * K * 12 + S * 4 + N * H * 2;                          // combine
    std::printf("%s dispatch + combine, %d ranks x %d tokens, hidden %d, %d experts, top-%d: %.1f us per step, "
                "%.0f GB/s (%.1f %% of 8 TB/s)\n",
                a.fp8 ? "fp8" : "bf16", R, T, H, E, K, step_us, bytes / step_us / 1e3, bytes / step_us / 1e3 / 80.0);

    mc_ep_legacy_perf_tensors_t lt = {px.data(),      pidx.data(), pw.data(),  pact.data(), pexp.data(),
                                      precv16.data(), pcnt.data(), psrc.data(), plr.data(),  pout.data()};
    mc_ep_legacy_perf_config_t lc = {T, H, K, L, T, E, -1, a.warmups, a.iterations, s};
    mc_ep_legacy_perf_result_t lr = {0, 0, 0};
    EP_OK(mc_ep_world_legacy_buffer_perf(world, &lt, &lc, &lr));
    std::printf("native loop (clear + bf16 dispatch + combine): avg_t=%.2f us, min_t=%.2f us, max_t=%.2f us\n",
                lr.average_us, lr.min_us, lr.max_us);

    EP_OK(mc_ep_world_destroy(world));
    // an EventHandle may outlive the world whose collective it stands for
    for (mc_ep_event_t* ev : kept_events) EP_OK(mc_ep_event_destroy(ev));
    HIP_OK(hipStreamDestroy(stream));
    const void* owned[] = {x, idx, wts, active, recv_x, scales, recv_bf16, expert_x, out, recv_count, src_info, layout_range};
    for (const void* d : owned)
        if (d) HIP_OK(hipFree((void*)d));
    return 0;
}
