// mooncake_amd._ep: the compiled Python module of this library, a drop-in for the
// reference's pybind11 module `mooncake._ep` on the low-latency dispatch / combine
// path (mooncake-ep/src/ep_py.cpp:14-46): get_ep_buffer_size_hint, MAX_QP_COUNT,
// EventHandle, Buffer with the bound names and argument order of the reference, and
// _benchmark_legacy_buffer with its three structs
// (mooncake-ep/benchmarks/legacy_buffer_perf.cpp:151-199).  Everything goes through
// the C ABI of include/mooncake_ep_hip.h; no torch type appears here either - device
// addresses and streams are integers, as in the reference's bindings.
//
// What the reference does not have: World (the expert-parallel world as logical ranks
// of one GPU; Buffer takes the one it belongs to as an optional fifth argument and
// otherwise joins a process-wide world of its num_ranks) and the whole-world calls.
#include <pybind11/functional.h>
#include <pybind11/pybind11.h>
#include <pybind11/stl.h>

#include <atomic>
#include <cstdint>
#include <deque>
#include <functional>
#include <map>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <tuple>
#include <vector>

#include "mooncake_ep_hip.h"

namespace py = pybind11;

namespace {

// EPException surfaces as RuntimeError through pybind11 in the reference; the paths
// its Python wrapper answers with NotImplementedError do so here too.
void check(int rc) {
    if (rc == MC_EP_OK) return;
    const char* msg = mc_ep_last_error();
    if (rc == MC_EP_ERR_UNSUPPORTED) {
        PyErr_SetString(PyExc_NotImplementedError, msg ? msg : "unsupported");
        throw py::error_already_set();
    }
    if (rc == MC_EP_ERR_INVALID) throw std::invalid_argument(msg ? msg : "invalid argument");   // ValueError
    if (rc == MC_EP_ERR_PENDING) {
        // a RuntimeError of its own, shared with the ctypes binding: callers tell "not every rank has called
        // yet" (the call stays posted) from a failure by the type, not by the text
        const std::string text = msg ? msg : "pending";
        py::object type = py::module_::import("mooncake_amd._lib").attr("PendingError");
        PyErr_SetString(type.ptr(), text.c_str());
        throw py::error_already_set();
    }
    throw std::runtime_error(msg ? msg : "mooncake_ep_hip: unknown failure");
}

using U64s = std::vector<uint64_t>;
using I32s = std::vector<int32_t>;

struct World {
    mc_ep_world_t* h = nullptr;
    int num_ranks = 0;
    explicit World(int n) : num_ranks(n) { check(mc_ep_world_create(n, &h)); }
    World(const World&) = delete;
    World& operator=(const World&) = delete;
    ~World() {
        if (h) mc_ep_world_destroy(h);
    }
    void need(const U64s& v, const char* what) const {
        if ((int)v.size() != num_ranks)
            throw std::invalid_argument(std::string(what) + ": one entry per logical rank expected");
    }
};

using WorldPtr = std::shared_ptr<World>;

// Buffers created without a world share one per num_ranks, like processes that join one group.
std::map<int, std::weak_ptr<World>>& default_worlds() {
    static std::map<int, std::weak_ptr<World>> worlds;
    return worlds;
}

WorldPtr default_world(int num_ranks) {
    auto& slot = default_worlds()[num_ranks];
    WorldPtr w = slot.lock();
    if (!w) {
        w = std::make_shared<World>(num_ranks);
        slot = w;
    }
    return w;
}

// EventHandle, mooncake_ep_event.h:9-42
struct Event {
    mc_ep_event_t* h = nullptr;
    WorldPtr keep;   // an event of a collective refers to its world's bookkeeping
    explicit Event(uint64_t stream_ptr) { check(mc_ep_event_create(stream_ptr, &h)); }
    Event(mc_ep_event_t* raw, WorldPtr w) : h(raw), keep(std::move(w)) {}
    Event(const Event&) = delete;
    Event& operator=(const Event&) = delete;
    ~Event() { mc_ep_event_destroy(h); }
    void current_stream_wait(uint64_t stream_ptr) { check(mc_ep_event_current_stream_wait(h, stream_ptr)); }
    void synchronize() { check(mc_ep_event_synchronize(h)); }
};

using CallResult = std::tuple<std::optional<std::shared_ptr<Event>>, std::optional<std::function<void()>>>;

CallResult wrap(mc_ep_event_t* ev, mc_ep_hook_t* hook, const WorldPtr& world) {
    CallResult r;
    if (ev) std::get<0>(r) = std::make_shared<Event>(ev, world);
    if (hook) {
        std::shared_ptr<mc_ep_hook_t> keep(hook, mc_ep_hook_destroy);
        WorldPtr w = world;   // the hook enqueues work of its world: keep it alive
        std::get<1>(r) = [keep, w] { check(mc_ep_hook_call(keep.get())); };
    }
    return r;
}

// A per-rank call may wait for other Python threads (one per rank, option "blocking" - which can be set
// through any binding of the C ABI, so nothing here tries to know): it always gives up the GIL for its
// duration.  The library reports its failure per thread, so the error text is still this call's.
template <typename F>
int without_gil(F&& f) {
    py::gil_scoped_release release;
    return f();
}

// MooncakeEpBuffer, mooncake_ep_buffer.h:66-194
struct Buffer {
    mc_ep_buffer_t* h = nullptr;
    WorldPtr world;
    int rank = 0, num_ranks = 0;
    Buffer(int rank_, int num_ranks_, int64_t num_ep_buffer_bytes, bool disable_p2p, WorldPtr w)
        : world(w ? std::move(w) : default_world(num_ranks_)), rank(rank_), num_ranks(num_ranks_) {
        if (world->num_ranks != num_ranks)
            throw std::runtime_error("world has " + std::to_string(world->num_ranks) + " ranks, Buffer asked for " +
                                     std::to_string(num_ranks));
        check(mc_ep_buffer_create(world->h, rank, num_ep_buffer_bytes, disable_p2p ? 1 : 0, &h));
    }
    Buffer(const Buffer&) = delete;
    Buffer& operator=(const Buffer&) = delete;
    ~Buffer() { mc_ep_buffer_destroy(h); }

    // A round's kernels are enqueued by the call of its last rank, from the raw addresses every rank
    // posted, so a call's tensors must outlive the call: whatever the caller hands over as `keep_alive`
    // (the reference's tensors_to_record) is held here until the library reports that the call's round
    // has been enqueued - also when the call itself gave up waiting for its peers (MC_EP_ERR_PENDING:
    // it stays posted).  kind 0: dispatch, 1: combine.  The GIL is held.
    std::deque<py::object> kept[2];
    void retain(int kind, int rc, py::object& keep_alive) {
        if (keep_alive.is_none() || (rc != MC_EP_OK && rc != MC_EP_ERR_PENDING)) return;
        kept[kind].push_back(std::move(keep_alive));
        int pending[2] = {0, 0};
        if (mc_ep_buffer_pending_calls(h, &pending[0], &pending[1]) != MC_EP_OK) return;
        while ((long long)kept[kind].size() > pending[kind]) kept[kind].pop_front();
    }
    std::pair<int, int> retained() const { return {(int)kept[0].size(), (int)kept[1].size()}; }

    CallResult dispatch(uint64_t x_ptr, uint64_t topk_idx_ptr, uint64_t active_ranks_ptr, int num_tokens, int hidden,
                        int num_topk, int num_max_dispatch_tokens_per_rank, int num_experts, int timeout_us,
                        bool use_fp8, uint64_t packed_recv_x_ptr, uint64_t packed_recv_x_scales_ptr,
                        uint64_t packed_recv_count_ptr, uint64_t packed_recv_src_info_ptr,
                        uint64_t packed_recv_layout_range_ptr, bool async, bool return_recv_hook,
                        uint64_t compute_stream_ptr, py::object keep_alive) {
        mc_ep_event_t* ev = nullptr;
        mc_ep_hook_t* hook = nullptr;
        const auto call = [&] {
            return mc_ep_buffer_dispatch(h, x_ptr, topk_idx_ptr, active_ranks_ptr, num_tokens, hidden, num_topk,
                                         num_max_dispatch_tokens_per_rank, num_experts, timeout_us, use_fp8 ? 1 : 0,
                                         packed_recv_x_ptr, packed_recv_x_scales_ptr, packed_recv_count_ptr,
                                         packed_recv_src_info_ptr, packed_recv_layout_range_ptr, async ? 1 : 0,
                                         return_recv_hook ? 1 : 0, compute_stream_ptr, &ev, &hook);
        };
        const int rc = without_gil(call);
        retain(0, rc, keep_alive);
        check(rc);
        return wrap(ev, hook, world);
    }

    CallResult combine(uint64_t x_ptr, uint64_t topk_idx_ptr, uint64_t topk_weights_ptr, uint64_t src_info_ptr,
                       uint64_t layout_range_ptr, uint64_t active_ranks_ptr, int num_local_experts,
                       int num_combined_tokens, int hidden, int num_topk, int num_max_dispatch_tokens_per_rank,
                       int num_experts, int timeout_us, bool zero_copy, uint64_t combined_x_ptr, bool async,
                       bool return_recv_hook, uint64_t compute_stream_ptr, py::object keep_alive) {
        mc_ep_event_t* ev = nullptr;
        mc_ep_hook_t* hook = nullptr;
        const auto call = [&] {
            return mc_ep_buffer_combine(h, x_ptr, topk_idx_ptr, topk_weights_ptr, src_info_ptr, layout_range_ptr,
                                        active_ranks_ptr, num_local_experts, num_combined_tokens, hidden, num_topk,
                                        num_max_dispatch_tokens_per_rank, num_experts, timeout_us, zero_copy ? 1 : 0,
                                        combined_x_ptr, async ? 1 : 0, return_recv_hook ? 1 : 0, compute_stream_ptr,
                                        &ev, &hook);
        };
        const int rc = without_gil(call);
        retain(1, rc, keep_alive);
        check(rc);
        return wrap(ev, hook, world);
    }

    std::pair<int, int> pending_calls() const {
        int d = 0, c = 0;
        check(mc_ep_buffer_pending_calls(h, &d, &c));
        return {d, c};
    }
};

// A whole-world call whose per-rank address arrays were marshalled once.
struct PreparedDispatch {
    WorldPtr world;
    U64s x, topk_idx, recv_x, recv_scales, recv_count, src_info, layout_range;
    I32s num_tokens;
    int hidden = 0, num_topk = 0, max_tokens = 0, num_experts = 0, use_fp8 = 0;
    void call(uint64_t stream_ptr, int phases) const {
        check(mc_ep_world_dispatch(world->h, x.data(), topk_idx.data(), num_tokens.data(), hidden, num_topk, max_tokens,
                                   num_experts, use_fp8, recv_x.data(), use_fp8 ? recv_scales.data() : nullptr,
                                   recv_count.data(), src_info.data(), layout_range.data(), phases, stream_ptr));
    }
    void call_noalloc(uint64_t stream_ptr) const {
        check(mc_ep_world_dispatch_noalloc(world->h, x.data(), topk_idx.data(), num_tokens.data(), hidden, num_topk,
                                           max_tokens, num_experts, use_fp8, recv_x.data(),
                                           use_fp8 ? recv_scales.data() : nullptr, recv_count.data(), src_info.data(),
                                           layout_range.data(), stream_ptr));
    }
};

struct PreparedCombine {
    WorldPtr world;
    U64s x, scales, topk_idx, topk_weights, src_info, layout_range, active_ranks, out;
    I32s num_tokens;
    uint64_t factor = 0;
    bool packed = false, has_scales = false;
    int hidden = 0, num_topk = 0, max_tokens = 0, num_experts = 0;
    void call(uint64_t stream_ptr, int phases) const {
        if (packed)
            check(mc_ep_world_combine_packed(world->h, x.data(), has_scales ? scales.data() : nullptr, factor,
                                             topk_idx.data(), topk_weights.data(), src_info.data(),
                                             layout_range.data(), active_ranks.data(), num_tokens.data(), hidden,
                                             num_topk, max_tokens, num_experts, out.data(), phases, stream_ptr));
        else
            check(mc_ep_world_combine(world->h, x.data(), topk_idx.data(), topk_weights.data(), src_info.data(),
                                      layout_range.data(), active_ranks.data(), num_tokens.data(), hidden, num_topk,
                                      max_tokens, num_experts, out.data(), phases, stream_ptr));
    }
};

// LegacyBufferPerfTensors / Config / Result of legacy_buffer_perf.cpp:18-49, with one device address
// per logical rank where the reference has one address.
struct LegacyTensors {
    U64s x_ptr, topk_idx_ptr, topk_weights_ptr, active_ranks_ptr, expert_x_ptr, packed_recv_x_ptr,
        packed_recv_count_ptr, packed_recv_src_info_ptr, packed_recv_layout_range_ptr, combined_x_ptr;
};

struct LegacyConfig {
    int num_tokens = 0, hidden = 0, num_topk = 0, num_local_experts = 0, num_max_dispatch_tokens_per_rank = 0,
        num_experts = 0, timeout_us = -1, warmups = 20, iterations = 30;
    uint64_t compute_stream_ptr = 0;
};

struct LegacyResult {
    double average_us = 0.0, min_us = 0.0, max_us = 0.0;
};

LegacyResult benchmark_legacy(const WorldPtr& world, const LegacyTensors& t, const LegacyConfig& c) {
    const U64s* fields[] = {&t.x_ptr,           &t.topk_idx_ptr,          &t.topk_weights_ptr,
                            &t.active_ranks_ptr, &t.expert_x_ptr,          &t.packed_recv_x_ptr,
                            &t.packed_recv_count_ptr, &t.packed_recv_src_info_ptr,
                            &t.packed_recv_layout_range_ptr, &t.combined_x_ptr};
    for (const U64s* f : fields)
        if ((int)f->size() != world->num_ranks)
            throw std::invalid_argument("legacy EP benchmark received a null tensor pointer");
    mc_ep_legacy_perf_tensors_t ct{t.x_ptr.data(),
                                   t.topk_idx_ptr.data(),
                                   t.topk_weights_ptr.data(),
                                   t.active_ranks_ptr.data(),
                                   t.expert_x_ptr.data(),
                                   t.packed_recv_x_ptr.data(),
                                   t.packed_recv_count_ptr.data(),
                                   t.packed_recv_src_info_ptr.data(),
                                   t.packed_recv_layout_range_ptr.data(),
                                   t.combined_x_ptr.data()};
    mc_ep_legacy_perf_config_t cc{c.num_tokens, c.hidden,     c.num_topk,   c.num_local_experts,
                                  c.num_max_dispatch_tokens_per_rank, c.num_experts, c.timeout_us,
                                  c.warmups,    c.iterations, c.compute_stream_ptr};
    mc_ep_legacy_perf_result_t cr{0, 0, 0};
    int rc;
    {
        py::gil_scoped_release release;   // as the reference's binding does for its timed loop
        rc = mc_ep_world_legacy_buffer_perf(world->h, &ct, &cc, &cr);
    }
    check(rc);
    return LegacyResult{cr.average_us, cr.min_us, cr.max_us};
}

}  // namespace

PYBIND11_MODULE(_ep, m) {
    m.doc() = "Low-latency MoE dispatch / combine on one AMD MI355X (C ABI: include/mooncake_ep_hip.h)";
    m.def("get_ep_buffer_size_hint", [](int max_tokens, int hidden, int num_ranks, int num_experts) {
        return mc_ep_get_buffer_size_hint(max_tokens, hidden, num_ranks, num_experts);
    });
    m.attr("MAX_QP_COUNT") = py::int_(MC_EP_MAX_QP_COUNT);
    m.attr("PHASE_LAYOUT") = py::int_(MC_EP_PHASE_LAYOUT);
    m.attr("PHASE_DATA") = py::int_(MC_EP_PHASE_DATA);
    m.attr("PHASE_FINISH") = py::int_(MC_EP_PHASE_FINISH);
    m.attr("PHASE_ALL") = py::int_(MC_EP_PHASE_ALL);

    py::class_<Event, std::shared_ptr<Event>>(m, "EventHandle")
        .def(py::init<uint64_t>(), py::arg("stream_ptr") = 0)
        .def("current_stream_wait", &Event::current_stream_wait, py::arg("stream_ptr"))
        .def("synchronize", &Event::synchronize);

    py::class_<PreparedDispatch>(m, "_PreparedDispatch")
        .def("__call__", &PreparedDispatch::call, py::arg("stream_ptr"), py::arg("phases") = MC_EP_PHASE_ALL)
        .def("noalloc", &PreparedDispatch::call_noalloc, py::arg("stream_ptr"));
    py::class_<PreparedCombine>(m, "_PreparedCombine")
        .def("__call__", &PreparedCombine::call, py::arg("stream_ptr"), py::arg("phases") = MC_EP_PHASE_ALL);

    py::class_<World, WorldPtr>(m, "World")
        .def(py::init<int>(), py::arg("num_ranks"))
        .def_readonly("num_ranks", &World::num_ranks)
        .def_property_readonly("handle", [](const World& w) { return (uintptr_t)w.h; },
                               "address of the mc_ep_world_t, for callers of the C ABI")
        .def("set_rank_silent",
             [](World& w, int rank, bool silent) { check(mc_ep_world_set_rank_silent(w.h, rank, silent ? 1 : 0)); },
             py::arg("rank"), py::arg("silent") = true)
        .def("set_option",
             [](World& w, const std::string& name, int value) {
                 check(mc_ep_world_set_option(w.h, name.c_str(), value));
             })
        .def("get_option",
             [](const World& w, const std::string& name) {
                 int v = 0;
                 check(mc_ep_world_get_option(w.h, name.c_str(), &v));
                 return v;
             })
        .def("prepare_dispatch",
             [](const WorldPtr& w, U64s x, U64s topk_idx, I32s num_tokens, int hidden, int num_topk, int max_tokens,
                int num_experts, bool use_fp8, U64s recv_x, std::optional<U64s> recv_scales, U64s recv_count,
                U64s src_info, U64s layout_range) {
                 PreparedDispatch p;
                 p.world = w;
                 w->need(x, "x_ptrs");
                 w->need(topk_idx, "topk_idx_ptrs");
                 w->need(recv_x, "packed_recv_x_ptrs");
                 w->need(recv_count, "packed_recv_count_ptrs");
                 w->need(src_info, "packed_recv_src_info_ptrs");
                 w->need(layout_range, "packed_recv_layout_range_ptrs");
                 if ((int)num_tokens.size() != w->num_ranks) throw std::invalid_argument("num_tokens: one per rank");
                 if (use_fp8) {
                     if (!recv_scales) throw std::invalid_argument("fp8 dispatch needs packed_recv_x_scales_ptrs");
                     w->need(*recv_scales, "packed_recv_x_scales_ptrs");
                     p.recv_scales = std::move(*recv_scales);
                 }
                 p.x = std::move(x); p.topk_idx = std::move(topk_idx); p.num_tokens = std::move(num_tokens);
                 p.recv_x = std::move(recv_x); p.recv_count = std::move(recv_count);
                 p.src_info = std::move(src_info); p.layout_range = std::move(layout_range);
                 p.hidden = hidden; p.num_topk = num_topk; p.max_tokens = max_tokens; p.num_experts = num_experts;
                 p.use_fp8 = use_fp8 ? 1 : 0;
                 return p;
             })
        .def("prepare_combine",
             [](const WorldPtr& w, U64s x, std::optional<U64s> scales, uint64_t expert_factor_ptr, bool packed,
                U64s topk_idx, U64s topk_weights, U64s src_info, U64s layout_range, U64s active_ranks,
                I32s num_tokens, int hidden, int num_topk, int max_tokens, int num_experts, U64s out) {
                 PreparedCombine p;
                 p.world = w;
                 w->need(x, "x_ptrs");
                 w->need(topk_idx, "topk_idx_ptrs");
                 w->need(topk_weights, "topk_weights_ptrs");
                 w->need(src_info, "src_info_ptrs");
                 w->need(layout_range, "layout_range_ptrs");
                 w->need(active_ranks, "active_ranks_ptrs");
                 w->need(out, "combined_x_ptrs");
                 if ((int)num_tokens.size() != w->num_ranks) throw std::invalid_argument("num_tokens: one per rank");
                 if (scales) {
                     w->need(*scales, "packed_recv_x_scales_ptrs");
                     p.scales = std::move(*scales);
                     p.has_scales = true;
                 }
                 p.packed = packed; p.factor = expert_factor_ptr;
                 p.x = std::move(x); p.topk_idx = std::move(topk_idx); p.topk_weights = std::move(topk_weights);
                 p.src_info = std::move(src_info); p.layout_range = std::move(layout_range);
                 p.active_ranks = std::move(active_ranks); p.out = std::move(out); p.num_tokens = std::move(num_tokens);
                 p.hidden = hidden; p.num_topk = num_topk; p.max_tokens = max_tokens; p.num_experts = num_experts;
                 return p;
             })
        .def("cast_back",
             [](const WorldPtr& w, U64s recv_x, std::optional<U64s> recv_scales, U64s recv_count,
                uint64_t expert_factor_ptr, U64s out, int hidden, int num_topk, int max_tokens, int num_experts,
                uint64_t stream_ptr) {
                 w->need(recv_x, "packed_recv_x_ptrs");
                 w->need(recv_count, "packed_recv_count_ptrs");
                 w->need(out, "out_ptrs");
                 if (recv_scales) w->need(*recv_scales, "packed_recv_x_scales_ptrs");
                 check(mc_ep_world_cast_back(w->h, recv_x.data(), recv_scales ? recv_scales->data() : nullptr,
                                             recv_count.data(), expert_factor_ptr, out.data(), hidden, num_topk,
                                             max_tokens, num_experts, stream_ptr));
             });

    py::class_<LegacyTensors>(m, "_LegacyBufferPerfTensors")
        .def(py::init<>())
        .def_readwrite("x_ptr", &LegacyTensors::x_ptr)
        .def_readwrite("topk_idx_ptr", &LegacyTensors::topk_idx_ptr)
        .def_readwrite("topk_weights_ptr", &LegacyTensors::topk_weights_ptr)
        .def_readwrite("active_ranks_ptr", &LegacyTensors::active_ranks_ptr)
        .def_readwrite("expert_x_ptr", &LegacyTensors::expert_x_ptr)
        .def_readwrite("packed_recv_x_ptr", &LegacyTensors::packed_recv_x_ptr)
        .def_readwrite("packed_recv_count_ptr", &LegacyTensors::packed_recv_count_ptr)
        .def_readwrite("packed_recv_src_info_ptr", &LegacyTensors::packed_recv_src_info_ptr)
        .def_readwrite("packed_recv_layout_range_ptr", &LegacyTensors::packed_recv_layout_range_ptr)
        .def_readwrite("combined_x_ptr", &LegacyTensors::combined_x_ptr);
    py::class_<LegacyConfig>(m, "_LegacyBufferPerfConfig")
        .def(py::init<>())
        .def_readwrite("num_tokens", &LegacyConfig::num_tokens)
        .def_readwrite("hidden", &LegacyConfig::hidden)
        .def_readwrite("num_topk", &LegacyConfig::num_topk)
        .def_readwrite("num_local_experts", &LegacyConfig::num_local_experts)
        .def_readwrite("num_max_dispatch_tokens_per_rank", &LegacyConfig::num_max_dispatch_tokens_per_rank)
        .def_readwrite("num_experts", &LegacyConfig::num_experts)
        .def_readwrite("timeout_us", &LegacyConfig::timeout_us)
        .def_readwrite("warmups", &LegacyConfig::warmups)
        .def_readwrite("iterations", &LegacyConfig::iterations)
        .def_readwrite("compute_stream_ptr", &LegacyConfig::compute_stream_ptr);
    py::class_<LegacyResult>(m, "_LegacyBufferPerfResult")
        .def_readonly("average_us", &LegacyResult::average_us)
        .def_readonly("min_us", &LegacyResult::min_us)
        .def_readonly("max_us", &LegacyResult::max_us);

    py::class_<Buffer>(m, "Buffer")
        .def(py::init<int, int, int64_t, bool, WorldPtr>(), py::arg("rank"), py::arg("num_ranks"),
             py::arg("num_ep_buffer_bytes"), py::arg("disable_p2p") = false, py::arg("world") = WorldPtr())
        .def_readonly("world", &Buffer::world)
        .def_readonly("rank", &Buffer::rank)
        .def_readonly("num_ranks", &Buffer::num_ranks)
        // transport introspection (ep_py.cpp:31-42): one address space, no NIC, no peer process
        .def("ibgda_disabled", [](const Buffer& b) { return mc_ep_buffer_ibgda_disabled(b.h) != 0; })
        .def("p2p_enabled", [](const Buffer& b) { return mc_ep_buffer_p2p_enabled(b.h) != 0; })
        .def("use_fast_path", [](const Buffer& b) { return mc_ep_buffer_use_fast_path(b.h) != 0; })
        .def("is_roce", [](const Buffer& b) { return mc_ep_buffer_is_roce(b.h) != 0; })
        .def("update_local_qpns", [](Buffer&) {})
        .def("sync_ibgda_peers", [](Buffer&, py::object, py::object, py::object, py::object, py::object, py::object,
                                    py::object) {})
        .def("get_mr_info", [](const Buffer&) { return std::make_pair<uint64_t, uint32_t>(0, 0); })
        .def("get_gid", [](const Buffer&) { return std::make_pair<uint64_t, uint64_t>(0, 0); })
        .def("get_local_qpns", [](const Buffer&) { return std::vector<int32_t>(); })
        .def("get_local_lids", [](const Buffer&) { return std::vector<int32_t>(); })
        .def("get_ipc_handle", [](const Buffer&) { return std::vector<int32_t>(); })
        .def("sync_nvlink_ipc_handles", [](Buffer&, py::object, py::object) {})
        .def("pending_calls", &Buffer::pending_calls)
        .def("retained", &Buffer::retained, "(dispatch, combine) keep_alive objects still held")
        // the reference's argument lists (ep_py.cpp:43-44), positional; keep_alive is this module's addition
        .def("dispatch", &Buffer::dispatch, py::arg("x_ptr"), py::arg("topk_idx_ptr"), py::arg("active_ranks_ptr"),
             py::arg("num_tokens"), py::arg("hidden"), py::arg("num_topk"),
             py::arg("num_max_dispatch_tokens_per_rank"), py::arg("num_experts"), py::arg("timeout_us"),
             py::arg("use_fp8"), py::arg("packed_recv_x_ptr"), py::arg("packed_recv_x_scales_ptr"),
             py::arg("packed_recv_count_ptr"), py::arg("packed_recv_src_info_ptr"),
             py::arg("packed_recv_layout_range_ptr"), py::arg("async"), py::arg("return_recv_hook"),
             py::arg("compute_stream_ptr"), py::arg("keep_alive") = py::none())
        .def("combine", &Buffer::combine, py::arg("x_ptr"), py::arg("topk_idx_ptr"), py::arg("topk_weights_ptr"),
             py::arg("src_info_ptr"), py::arg("layout_range_ptr"), py::arg("active_ranks_ptr"),
             py::arg("num_local_experts"), py::arg("num_combined_tokens"), py::arg("hidden"), py::arg("num_topk"),
             py::arg("num_max_dispatch_tokens_per_rank"), py::arg("num_experts"), py::arg("timeout_us"),
             py::arg("zero_copy"), py::arg("combined_x_ptr"), py::arg("async"), py::arg("return_recv_hook"),
             py::arg("compute_stream_ptr"), py::arg("keep_alive") = py::none());

    m.def("_benchmark_legacy_buffer",
          [](const py::object& runtime, const LegacyTensors& t, const LegacyConfig& c) {
              // the reference passes one rank's Buffer; here the loop drives the Buffer's whole world
              if (py::isinstance<Buffer>(runtime)) return benchmark_legacy(runtime.cast<Buffer&>().world, t, c);
              return benchmark_legacy(runtime.cast<WorldPtr>(), t, c);
          },
          py::arg("runtime"), py::arg("tensors"), py::arg("config"));
}
