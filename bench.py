#!/usr/bin/env python3
"""Benchmark of the dispatch + combine hot path on one MI355X.

A step is one whole-world dispatch followed by one whole-world combine of the
DeepSeek-V3 decode configuration (32 logical ranks x 128 tokens, hidden 7168,
256 experts, top-8, fp8 dispatch, bf16 combine), all ranks' tensors resident
in HBM before the timed region.  Prints one JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config NAME]
                    [--no-cpu-baseline] [--opt name=value ...]
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E, published peak
METRIC = "dispatch+combine µs & HBM GB/s (% peak), DSV3 decode 128 tok top-8 fp8"



def measured_traffic(workload, kernel):
    """HBM bytes per launch of a kernel as the profiler's counters saw them: the `traffic_bytes` lines of
    profiles/<workload>_hbm_traffic.txt, which `python -m mooncake_amd.benchmarks.hbm_traffic` writes from two
    `rocprofv3 --pmc` runs of this script (FETCH_SIZE, then WRITE_SIZE), each scaled by what the same counter
    reads for the library's plain copy kernel of known size.  The file records the commit of the library it was
    measured on and a hash of the kernels' sources: (bytes, commit, whether the sources still hash to that).
    A workload or kernel that was not profiled gives (None, None, None)."""
    path = os.path.join(ROOT, "profiles", f"{workload}_hbm_traffic.txt")
    if not os.path.exists(path):
        return None, None, None
    commit, found, sha = None, None, None
    for line in open(path):
        parts = line.split()
        if len(parts) >= 2 and parts[0] == "measured_at_commit":
            commit = parts[1]
        if len(parts) >= 2 and parts[0] == "kernel_sources_sha256":
            sha = parts[1]
        if len(parts) >= 3 and parts[0] == "traffic_bytes" and parts[1] == kernel:
            found = int(parts[2])
    # the figure stands only while the kernels' sources are the ones it was measured on
    from mooncake_amd.benchmarks.hbm_traffic import kernel_sources_sha256
    current = sha is not None and sha == kernel_sources_sha256()
    return found, commit, current


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", default="dsv3_decode")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-flushed", action="store_true", help="skip the cache-flushed timing")
    ap.add_argument("--no-buffer-api", action="store_true", help="skip the per-rank Buffer API timing")
    ap.add_argument("--no-small-world", action="store_true", help="skip the launch-bound small-world shapes")
    ap.add_argument("--small-world", action="store_true",
                    help="instead of the workload, time only the launch-bound small-world shapes and print them as JSON")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU budget for the cpu_baseline sample")
    ap.add_argument("--kernel-iters", type=int, default=30, help="timed launches per kernel for the roofline figures")
    ap.add_argument("--opt", action="append", default=[], help="library tuning option, name=value")
    ap.add_argument("--flush-mb", type=int, default=0,
                    help="write this many MiB before every step of the per-kernel timing loop (cache flush)")
    ap.add_argument("--graph", action="store_true",
                    help="record the step into a HIP graph once and time replays instead of eager launches")
    ap.add_argument("--stream-ceilings", action="store_true",
                    help="instead of the workload, time synthetic streams with the data kernels' read : write mixes "
                         "and byte counts (what the memory system gives each mix), and print them as JSON")
    ap.add_argument("--gather-geometries", action="store_true",
                    help="instead of the workload, time the 8 : 1 gather of whole scattered rows over several layouts "
                         "of the same rows (with and without gaps between the experts' blocks) and the sequential "
                         "gather beside them, and print them as JSON")
    ap.add_argument("--kernel-pass", type=int, default=0, metavar="N",
                    help="instead of timing, run every kernel of the workload (dispatch, cast_back, combine, packed "
                         "combine) and the synthetic streams sized like them N times and exit: the program to put "
                         "under `rocprofv3 --pmc` when comparing hardware counters of the two")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MiB",
                    help="also run the library's plain copy kernel over this many MiB three times (the known-size "
                         "kernel that profiler FETCH_SIZE / WRITE_SIZE readings are scaled against)")
    return ap.parse_args()


def time_pipeline(h, lib, iters, flush=None):
    """Device time of each kernel inside the running dispatch -> combine
    pipeline: events on the launch stream between the phases of every step, no
    host synchronisation inside the loop, so each kernel starts on the cache
    state its predecessor leaves behind (a step moves ~830 MB, far more than L2
    and the 256 MB memory-side cache hold).  The first two steps are dropped."""
    import torch
    phases = [("layout", h.dispatch, lib.PHASE_LAYOUT), ("pack", h.dispatch, lib.PHASE_DATA),
              ("scales", h.dispatch, lib.PHASE_FINISH), ("resolve", h.combine, lib.PHASE_LAYOUT),
              ("reduce", h.combine, lib.PHASE_DATA)]
    if not h.cfg.use_fp8:
        phases = [p for p in phases if p[0] != "scales"]
    if h.world.get_option("combine_direct"):
        # the combine reuses the dispatch's routing state: it has no resolve launch, and an event pair
        # around nothing would only add its own overhead to the combine figure
        phases = [p for p in phases if p[0] != "resolve"]
        phases[-1] = ("reduce", h.combine, lib.PHASE_LAYOUT | lib.PHASE_DATA)
    marks = []
    for _ in range(iters + 2):
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(len(phases) + 1)]
        if flush is not None:
            flush.zero_()       # the reference's cache flush between iterations (ep_test_utils.py:79-104), untimed
        ev[0].record()
        for i, (_, fn, ph) in enumerate(phases):
            fn(phases=ph)
            ev[i + 1].record()
        marks.append(ev)
    torch.cuda.synchronize()
    out = {}
    for i, (name, _, _) in enumerate(phases):
        us = [m[i].elapsed_time(m[i + 1]) * 1e3 for m in marks[2:]]
        out[name] = (sum(us) / len(us), min(us))
    return out


def time_calls(h, iters, flush=None):
    """Device time of a whole dispatch and a whole combine inside the running pipeline: three events per
    step (start, between, end), so each figure carries one marker's overhead instead of one per kernel."""
    import torch
    marks = []
    for _ in range(iters + 2):
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(3)]
        if flush is not None:
            flush.zero_()
        ev[0].record()
        h.dispatch()
        ev[1].record()
        h.combine()
        ev[2].record()
        marks.append(ev)
    torch.cuda.synchronize()
    d = [m[0].elapsed_time(m[1]) * 1e3 for m in marks[2:]]
    c = [m[1].elapsed_time(m[2]) * 1e3 for m in marks[2:]]
    return sum(d) / len(d), sum(c) / len(c)


def time_back_to_back(call, iters):
    """Average launch period of one kernel: `iters` launches of it in a row between one event pair, so the
    markers' own overhead (2-3 us each) is spread over all of them.  This is the figure a profiler's kernel
    duration corresponds to (end of the previous kernel to end of this one)."""
    import torch
    for _ in range(3):
        call()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(iters):
        call()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) * 1e3 / iters


def time_flushed(h, iters, alg):
    """The reference's timing protocol taken to its strict form: the caches are flushed with 512 MiB before
    every timed step (its benchmarks flush 256 MB once, after the warm-up: ep_test_utils.py:79-104), 20 warm-ups
    and `iters` timed steps with an event pair around each call, the first one dropped.  Two kinds of flush,
    because they leave different cache states behind: a written one (the reference's `cache.zero_()`; its dirty
    lines are evicted while the timed kernel runs, which the kernel pays for) and a read-only one (clean lines)."""
    import torch
    flush = torch.empty(512 << 20, dtype=torch.uint8, device=h.device)
    flush.zero_()
    sink = torch.zeros(1, dtype=torch.int64, device=h.device)
    kinds = {"written": lambda: flush.zero_(),
             "read_only": lambda: sink.add_(flush.view(torch.int64).sum())}
    out = {"flush_mib": 512}
    for name, do_flush in kinds.items():
        for _ in range(20):
            h.dispatch()
            h.combine()
        marks = []
        for _ in range(iters + 1):
            ev = [torch.cuda.Event(enable_timing=True) for _ in range(4)]
            do_flush()
            ev[0].record()
            h.dispatch()
            ev[1].record()
            do_flush()
            ev[2].record()
            h.combine()
            ev[3].record()
            marks.append(ev)
        torch.cuda.synchronize()
        d = [m[0].elapsed_time(m[1]) * 1e3 for m in marks[1:]]
        c = [m[2].elapsed_time(m[3]) * 1e3 for m in marks[1:]]
        d_us, c_us = sum(d) / len(d), sum(c) / len(c)
        out[name] = {"dispatch_us": round(d_us, 2), "combine_us": round(c_us, 2),
                     "pct_of_hbm_peak": round((alg["dispatch"] + alg["combine"]) / (d_us + c_us) / 1e3
                                              / HBM_PEAK_GBPS * 100, 2),
                     "dispatch_pct": round(alg["dispatch"] / d_us / 1e3 / HBM_PEAK_GBPS * 100, 2),
                     "combine_pct": round(alg["combine"] / c_us / 1e3 / HBM_PEAK_GBPS * 100, 2)}
    return out


def time_buffer_api(h, steps, warmup):
    """The same step driven the way the reference's callers drive it: one `Buffer.dispatch` and one
    `Buffer.combine` per logical rank (2 x num_ranks calls a step) through the module that replaces
    `mooncake._ep` (ep_py.cpp:26-46), raw addresses in, (event, hook) out.  Wall clock per step like `value`;
    `host_us` is the time the calling thread spends inside the calls of a step (hidden behind the GPU when it is
    below the step time)."""
    import torch
    from mooncake_amd import ep
    cfg = h.cfg
    R, T, H, K, E, L = cfg.num_ranks, cfg.tokens_per_rank, cfg.hidden, cfg.num_topk, cfg.num_experts, \
        cfg.num_local_experts
    nbytes = ep.get_ep_buffer_size_hint(cfg.max_tokens, H, R, E)
    bufs = [ep.Buffer(r, R, nbytes, False, world=h.world) for r in range(R)]
    stream = int(torch.cuda.current_stream().cuda_stream)
    scales = h.recv_scales_phys
    out = {"binding": ep.BINDING, "calls_per_step": 2 * R}
    for mode, (async_, hook) in {"async_finish": (True, False), "default": (False, False),
                                 "return_recv_hook": (False, True)}.items():
        d = [(h.x[r].data_ptr(), h.topk_idx[r].data_ptr(), h.active_ranks[r].data_ptr(), T, H, K, cfg.max_tokens, E,
              -1, cfg.use_fp8, h.recv_x[r].data_ptr(), scales[r].data_ptr() if cfg.use_fp8 else 0,
              h.recv_count[r].data_ptr(), h.src_info[r].data_ptr(), h.layout_range[r].data_ptr(), async_, hook,
              stream) for r in range(R)]
        c = [(h.expert_out[r].data_ptr(), h.topk_idx[r].data_ptr(), h.topk_weights[r].data_ptr(),
              h.src_info[r].data_ptr(), h.layout_range[r].data_ptr(), h.active_ranks[r].data_ptr(), L, T, H, K,
              cfg.max_tokens, E, -1, False, h.combined[r].data_ptr(), async_, hook, stream) for r in range(R)]

        def step():
            for name, args in (("dispatch", d), ("combine", c)):
                res = [getattr(bufs[r], name)(*args[r]) for r in range(R)]
                for ev, fn in res:          # every rank waits for its own result, as a caller of the reference does
                    if ev is not None:
                        ev.current_stream_wait(stream)
                    if fn is not None:
                        fn()
        for _ in range(warmup):
            step()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            step()
        t1 = time.perf_counter()
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        out[mode] = {"us_per_step": round((t2 - t0) / steps * 1e6, 2), "host_us": round((t1 - t0) / steps * 1e6, 2)}
    return out


def time_python_buffer(h, steps, warmup):
    """One level up: the Python `Buffer` with the reference wrapper's signature (mooncake_ep_buffer.py:360-535,
    :538-678), which checks its arguments and allocates the five output tensors of every rank's dispatch with
    torch.empty inside the call (here: unless an earlier call's outputs have been let go of and can be handed out
    again).  In the reference each rank pays that in its own process; here one thread pays it for all ranks, so
    this figure is host-bound and reported for completeness only."""
    import torch
    from mooncake_amd.mooncake_ep_buffer import Buffer, LogicalGroup
    cfg = h.cfg
    R = cfg.num_ranks
    nbytes = Buffer.get_ep_buffer_size_hint(cfg.max_tokens, cfg.hidden, R, cfg.num_experts)
    bufs = [Buffer(LogicalGroup(h.world, r), nbytes) for r in range(R)]
    # each rank's own tensors, as a per-rank caller holds them (slicing the rank-major allocations inside the
    # loop would add seven tensor-indexing operations, about 1.5 us each, to every rank's step)
    xs, idx, wts, act = ([t[r] for r in range(R)] for t in (h.x, h.topk_idx, h.topk_weights, h.active_ranks))
    expert_out, combined = [h.expert_out[r] for r in range(R)], [h.combined[r] for r in range(R)]

    def step():
        res = [bufs[r].dispatch(xs[r], idx[r], act[r], cfg.max_tokens, cfg.num_experts, -1,
                                use_fp8=cfg.use_fp8, async_finish=True) for r in range(R)]
        for r in range(R):
            res[r][3].current_stream_wait()
        outs = [bufs[r].combine(expert_out[r], idx[r], wts[r], act[r], -1, res[r][2],
                                async_finish=True, out=combined[r]) for r in range(R)]
        for r in range(R):
            outs[r][1].current_stream_wait()
    for _ in range(max(2, warmup // 4)):
        step()
    torch.cuda.synchronize()
    n = max(5, steps // 4)
    t0 = time.perf_counter()
    for _ in range(n):
        step()
    torch.cuda.synchronize()
    return {"us_per_step": round((time.perf_counter() - t0) / n * 1e6, 2), "steps": n}


def time_small_world(iters):
    """Launch-bound shapes, reported beside the headline and never part of `value`: the world one deployed
    rank of the DeepSeek-V3 decode configuration sees by itself (1 x 128 tokens, hidden 7168, 256 experts,
    top-8, fp8: 9.4 MB / 16.5 MB of algorithmic traffic, 1.2 / 2.1 us at the HBM peak) and the contract's
    CPU-reference case (4 x 128 tokens, hidden 2048, 16 experts, top-4, bf16).  Each with the one-launch
    dispatch of small worlds on and off: device time per call with calls issued back to back (dispatches in a
    row, combines in a row, whole steps in a row; the best of five such runs) and the kernel launches one call
    makes."""
    import torch
    from mooncake_amd.harness import WorldHarness
    from mooncake_amd.workloads import CONFIGS, EPConfig, algorithmic_bytes, generate
    shapes = {"one_rank_dsv3_decode": EPConfig("one_rank_dsv3_decode", 1, 128, 7168, 256, 8, True),
              "cpu_check": CONFIGS["cpu_check"]}
    out = {}
    for name, cfg in shapes.items():
        data = generate(cfg, seed=0)
        S = int((data["topk_idx"] >= 0).sum())
        alg = algorithmic_bytes(cfg, S)
        rec = {"shape": {"num_ranks": cfg.num_ranks, "tokens_per_rank": cfg.tokens_per_rank, "hidden": cfg.hidden,
                         "num_experts": cfg.num_experts, "num_topk": cfg.num_topk, "use_fp8": cfg.use_fp8},
               "algorithmic_bytes": alg,
               "us_at_hbm_peak": {k: round(v / HBM_PEAK_GBPS / 1e3, 2) for k, v in alg.items()}}
        for label, fused in (("three_launch", 0), ("one_launch", 1)):
            h = WorldHarness(cfg, device="cuda:0")
            h.world.set_option("fused_small", fused)
            h.load(data)
            h.alloc_dispatch_outputs()
            h.alloc_combine_io()
            h.dispatch()
            h.cast_back()
            h.combine()
            torch.cuda.synchronize()

            def step():
                h.dispatch()
                h.combine()
            # calls this short are issued about as fast as they run: the best of five runs is the one the
            # host thread disturbed least
            d_us = min(time_back_to_back(h.dispatch, iters) for _ in range(5))
            c_us = min(time_back_to_back(h.combine, iters) for _ in range(5))
            s_us = min(time_back_to_back(step, iters) for _ in range(5))
            h.dispatch()
            h.combine()
            rec[label] = {"dispatch_us": round(d_us, 2), "combine_us": round(c_us, 2), "step_us": round(s_us, 2),
                          "dispatch_launches": h.world.get_option("last_dispatch_launches"),
                          "combine_launches": h.world.get_option("last_combine_launches"),
                          "pct_of_hbm_peak": round((alg["dispatch"] + alg["combine"]) / s_us / 1e3
                                                   / HBM_PEAK_GBPS * 100, 2)}
            del h
        out[name] = rec
    return out


def stream_ceilings(cfg, S, iters):
    """Synthetic streams (the library's stream_kernel: one 16-byte unit per thread, nothing else) with the read :
    write mix and the byte counts of each data kernel of this workload, launched back to back."""
    import torch
    from mooncake_amd import _lib
    lib = _lib.lib()
    stream = int(torch.cuda.current_stream().cuda_stream)
    H, N = cfg.hidden, cfg.total_tokens
    unit = lambda nbytes: (int(nbytes) + 4095) // 4096 * 4096
    out_rows, exp_rows = unit(N * H * 2), unit(S * H * 2)
    fp8_rows = unit(S * H)
    # name: (kind, unit_bytes, bytes read, bytes written)
    mixes = {
        "copy 1:1 (512 MiB each way)": (0, 512 << 20, 512 << 20, 512 << 20),
        "read only (1 GiB)": (1, 1 << 30, 1 << 30, 0),
        "write only (1 GiB)": (2, 1 << 30, 0, 1 << 30),
        "widen 1:2, cast-back sized": (3, exp_rows, exp_rows // 2, exp_rows),
        "gather 8:1, reduce sized": (4, out_rows, 8 * out_rows, out_rows),
        "scatter 1:4, fp8-pack sized": (5, fp8_rows // 8, fp8_rows // 4, fp8_rows),
    }
    big = max(max(r, w) for _, _, r, w in mixes.values())
    src = torch.empty(big, dtype=torch.uint8, device="cuda:0").fill_(3)
    dst = torch.empty(big, dtype=torch.uint8, device="cuda:0")
    res = {}

    def record(name, us, rd, wr):
        res[name] = {"us": round(us, 2), "read_MB": round(rd / 1e6, 1), "written_MB": round(wr / 1e6, 1),
                     "GBps": round((rd + wr) / us / 1e3, 1), "pct_of_hbm_peak": round((rd + wr) / us / 1e3 / 80, 2)}

    for name, (kind, ub, rd, wr) in mixes.items():
        us = time_back_to_back(lambda: _lib.check(lib.mc_ep_debug_stream(kind, dst.data_ptr(), src.data_ptr(), ub,
                                                                          stream)), iters)
        record(name, us, rd, wr)
    del src
    # the same 8 : 1 gather on the geometry of the packed layout: whole rows at scattered places of
    # [experts, ranks * max_tokens, hidden] bf16, the valid rows at the start of every expert's block
    region_rows = cfg.num_ranks * cfg.max_tokens
    used = max(1, -(-S // cfg.num_experts))
    layout = torch.empty((cfg.num_experts, region_rows, H), dtype=torch.bfloat16, device="cuda:0")
    layout[:, :used].fill_(1.0)
    us = time_back_to_back(lambda: _lib.check(lib.mc_ep_debug_gather_rows(
        dst.data_ptr(), layout.data_ptr(), H * 2, N, cfg.num_experts, region_rows, used, stream)), iters)
    record("gather 8:1 of scattered rows of the packed layout, reduce sized", us, 8 * N * H * 2, N * H * 2)
    # the two gathers once more at the occupancy the combine kernel is launched with from top-7 up
    _lib.check(lib.mc_ep_debug_set_stream_occupancy(20))
    try:
        us = time_back_to_back(lambda: _lib.check(lib.mc_ep_debug_stream(4, dst.data_ptr(), layout.data_ptr(),
                                                                          out_rows, stream)), iters)
        record("gather 8:1, reduce sized, 20 waves per CU", us, 8 * out_rows, out_rows)
        us = time_back_to_back(lambda: _lib.check(lib.mc_ep_debug_gather_rows(
            dst.data_ptr(), layout.data_ptr(), H * 2, N, cfg.num_experts, region_rows, used, stream)), iters)
        record("gather 8:1 of scattered rows of the packed layout, reduce sized, 20 waves per CU", us,
               8 * N * H * 2, N * H * 2)
    finally:
        _lib.check(lib.mc_ep_debug_set_stream_occupancy(0))
    # and the 1 : 4 scatter on the geometry of the fp8 layout: every source row read once, written (at half its
    # size) to 8 whole rows at scattered places of [experts, ranks * max_tokens, hidden] bytes
    layout8 = layout.view(torch.uint8)[: cfg.num_experts * region_rows * H]
    src16 = torch.empty(N * H * 2, dtype=torch.uint8, device="cuda:0").fill_(3)
    us = time_back_to_back(lambda: _lib.check(lib.mc_ep_debug_scatter_rows(
        layout8.data_ptr(), src16.data_ptr(), H, N, cfg.num_experts, region_rows, used, stream)), iters)
    record("scatter 1:4 to scattered rows of the fp8 layout, fp8-pack sized", us, N * H * 2, 8 * N * H)
    return res


def gather_geometries(cfg, S, iters):
    """The scattered-row gather of stream_ceilings over other placements of the same number of rows: is it the
    gaps between the experts' blocks that cost, or reading whole rows in a scattered order?"""
    import torch
    from mooncake_amd import _lib
    lib = _lib.lib()
    stream = int(torch.cuda.current_stream().cuda_stream)
    H, N, E = cfg.hidden, cfg.total_tokens, cfg.num_experts
    region_rows = cfg.num_ranks * cfg.max_tokens
    used = max(1, -(-S // E))
    layout = torch.empty((E, region_rows, H), dtype=torch.bfloat16, device="cuda:0").fill_(1.0)
    dst = torch.empty(N * H * 2, dtype=torch.uint8, device="cuda:0")
    res = {}
    for name, (regions, rows, use) in {
        "the packed layout (a block per expert, valid rows at its start)": (E, region_rows, used),
        "the same rows without gaps (one block)": (1, E * used, E * used),
        "blocks without gaps (experts x valid rows)": (E, used, used),
        "8 blocks": (8, E * used // 8, E * used // 8),
        "16 times the blocks, a 16th of the rows each": (E * 16, max(1, region_rows // 16), max(1, used // 16)),
    }.items():
        us = time_back_to_back(lambda: _lib.check(lib.mc_ep_debug_gather_rows(
            dst.data_ptr(), layout.data_ptr(), H * 2, N, regions, rows, use, stream)), iters)
        res[name] = {"regions": regions, "region_rows": rows, "used": use, "us": round(us, 2)}
    us = time_back_to_back(lambda: _lib.check(lib.mc_ep_debug_stream(4, dst.data_ptr(), layout.data_ptr(),
                                                                      N * H * 2 // 4096 * 4096, stream)), iters)
    res["sequential gather 8:1 (no rows)"] = {"us": round(us, 2)}
    return res


def cpu_baseline(cfg, data, bytes_total, budget_s):
    """The oracle (a scalar C restatement, OpenMP over tokens) timed on this
    host's cores on the same workload: whole steps until the budget is spent."""
    import torch
    from oracle import oracle
    # a one-GPU box's share of its host is 16 cores, whatever os.cpu_count() says there
    threads = min(16, os.cpu_count() or 1)
    oracle.set_threads(threads)
    R = cfg.num_ranks
    nt = [cfg.tokens_per_rank] * R
    eo = torch.empty((R, cfg.num_local_experts, R * cfg.max_tokens, cfg.hidden), dtype=torch.bfloat16)
    times_d, times_c = [], []
    t_begin = time.perf_counter()
    reps = 0
    while reps < 2 or (time.perf_counter() - t_begin < budget_s and reps < 40):
        t0 = time.perf_counter()
        d = oracle.dispatch(data["x"], data["topk_idx"], nt, cfg.max_tokens, cfg.num_experts, cfg.use_fp8, poison=None)
        t1 = time.perf_counter()
        oracle.combine(eo, data["topk_idx"], data["topk_weights"], d["src_info"], d["layout_range"], nt,
                       cfg.max_tokens, cfg.num_experts)
        t2 = time.perf_counter()
        if reps > 0:                                   # first repetition pages the buffers in
            times_d.append(t1 - t0)
            times_c.append(t2 - t1)
        reps += 1
    td, tc = sum(times_d) / len(times_d), sum(times_c) / len(times_c)
    return {
        "value": round(bytes_total / (td + tc) / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "sample": f"{len(times_d)} whole steps of the same workload ({cfg.name}, all {R} logical ranks), "
                  f"first step dropped",
        "dispatch_us": round(td * 1e6, 1),
        "combine_us": round(tc * 1e6, 1),
    }


def main():
    args = parse_args()
    if args.gpus != 1:
        print("bench.py measures the one-GPU path only: the expert-parallel world is emulated as logical ranks "
              "inside one MI355X's HBM; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    from mooncake_amd import _lib
    from mooncake_amd.harness import WorldHarness
    from mooncake_amd.workloads import CONFIGS, algorithmic_bytes, generate

    assert torch.cuda.is_available(), "bench.py needs a GPU"
    torch.cuda.set_device(0)
    cfg = CONFIGS[args.config]
    data = generate(cfg, seed=args.seed)
    S = int((data["topk_idx"] >= 0).sum())
    alg = algorithmic_bytes(cfg, S)

    if args.small_world:
        print(json.dumps({"small_world": time_small_world(max(args.kernel_iters, 100))}))
        return

    if args.stream_ceilings:
        print(json.dumps({"workload": cfg.name, "stream_ceilings": stream_ceilings(cfg, S, args.kernel_iters)}))
        return

    if args.gather_geometries:
        print(json.dumps({"workload": cfg.name, "gather_geometries": gather_geometries(cfg, S, args.kernel_iters)}))
        return

    if args.kernel_pass > 0:
        h = WorldHarness(cfg, device="cuda:0")
        h.load(data)
        h.alloc_dispatch_outputs()
        h.alloc_combine_io()
        lib, stream = _lib.lib(), int(torch.cuda.current_stream().cuda_stream)
        H, N = cfg.hidden, cfg.total_tokens
        big = S * H * 2
        src = torch.empty(big, dtype=torch.uint8, device="cuda:0").fill_(3)
        dst = torch.empty(big, dtype=torch.uint8, device="cuda:0")
        for _ in range(args.kernel_pass):
            h.dispatch()
            h.cast_back()
            h.combine()
            h.combine_packed()
            # gather 8:1 sized like the reduce kernel, scatter 1:4 like the fp8 pack kernel, widen 1:2 like cast_back
            for kind, unit_bytes in ((4, N * H * 2), (5, S * H // 8), (3, S * H * 2)):
                _lib.check(lib.mc_ep_debug_stream(kind, dst.data_ptr(), src.data_ptr(), unit_bytes // 4096 * 4096, stream))
            # the gather again, on scattered rows of the layout the reduce kernel reads (its expert outputs)
            used = max(1, -(-S // cfg.num_experts))
            _lib.check(lib.mc_ep_debug_gather_rows(dst.data_ptr(), h.expert_out.data_ptr(), H * 2, N, cfg.num_experts,
                                                   cfg.num_ranks * cfg.max_tokens, used, stream))
            # and the scatter on scattered rows of a layout shaped like the fp8 payload (the expert outputs' memory,
            # refilled by the next round's cast_back)
            _lib.check(lib.mc_ep_debug_scatter_rows(h.expert_out.data_ptr(), src.data_ptr(), H, N, cfg.num_experts,
                                                    cfg.num_ranks * cfg.max_tokens, used, stream))
        torch.cuda.synchronize()
        print(json.dumps({"workload": cfg.name, "kernel_pass": args.kernel_pass}))
        return

    h = WorldHarness(cfg, device="cuda:0")
    opts = {}
    for o in args.opt:
        k, v = o.split("=")
        h.world.set_option(k, int(v))
        opts[k] = int(v)
    h.load(data)
    h.alloc_dispatch_outputs()
    h.alloc_combine_io()
    h.dispatch()
    h.cast_back()                          # expert outputs = dispatched rows cast back to bf16 (consumer kernel)
    torch.cuda.synchronize()

    def eager_step():
        h.dispatch()
        h.combine()

    step = eager_step
    if args.graph:
        # the step recorded once into a HIP graph and replayed (how serving loops run it)
        eager_step()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            eager_step()
        step = graph.replay

    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    step_gbps = (alg["dispatch"] + alg["combine"]) / (elapsed / args.steps) / 1e9

    # per-kernel device times, measured live inside the pipeline
    flush = torch.empty(args.flush_mb << 20, dtype=torch.uint8, device="cuda:0") if args.flush_mb > 0 else None
    t = time_pipeline(h, _lib, args.kernel_iters, flush)
    d_us, c_us = time_calls(h, args.kernel_iters, flush)
    pack_us, red_us = t["pack"][0], t["reduce"][0]
    kernels = {k: {"us": round(v[0], 2), "min_us": round(v[1], 2)} for k, v in t.items()}
    kernels["pack"].update(bytes=alg["dispatch"], GBps=round(alg["dispatch"] / pack_us / 1e3, 1))
    kernels["reduce"].update(bytes=alg["combine"], GBps=round(alg["combine"] / red_us / 1e3, 1))
    # the two data kernels once more, each launched back to back (see time_back_to_back): reported beside
    # the in-pipeline durations, which carry a marker's overhead each and are the ones the roofline uses
    h.dispatch()
    pack_b2b = time_back_to_back(lambda: h.dispatch(phases=_lib.PHASE_DATA), args.kernel_iters)
    direct = bool(h.world.get_option("combine_direct"))
    red_b2b = time_back_to_back(lambda: h.combine(phases=_lib.PHASE_ALL if direct else _lib.PHASE_DATA),
                                args.kernel_iters)
    kernels["pack"].update(us_back_to_back=round(pack_b2b, 2))
    kernels["reduce"].update(us_back_to_back=round(red_b2b, 2))
    # the consumer of the packed layout (valid rows -> bf16), outside the step: reported, not part of `value`
    H = cfg.hidden
    cast_bytes = S * ((H + H // 128 * 4) if cfg.use_fp8 else 2 * H) + S * 2 * H
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(args.kernel_iters + 1)]
    for _ in range(3):
        h.cast_back()
    for i in range(args.kernel_iters):
        ev[i].record()
        h.cast_back()
    ev[-1].record()
    torch.cuda.synchronize()
    cast_us = ev[0].elapsed_time(ev[-1]) / args.kernel_iters * 1e3
    consumer = {"cast_back_us": round(cast_us, 2), "bytes": cast_bytes, "GBps": round(cast_bytes / cast_us / 1e3, 1)}
    # the combine fused with that consumer (reads dispatch's payload, same result bit for bit): against the two
    # kernels it replaces, both timed back to back
    packed_us = time_back_to_back(h.combine_packed, args.kernel_iters)
    packed_bytes = S * ((H + H // 128 * 4) if cfg.use_fp8 else 2 * H) + alg["combine"] - S * 2 * H
    fused = {"cast_back_plus_reduce_us": round(cast_us + red_b2b, 2), "combine_packed_us": round(packed_us, 2),
             "bytes": packed_bytes, "GBps": round(packed_bytes / packed_us / 1e3, 1),
             "pct_of_hbm_peak": round(packed_bytes / packed_us / 1e3 / HBM_PEAK_GBPS * 100, 2)}
    h.dispatch()
    h.cast_back()
    # the dominant kernel is the one the step spends most time in
    dom = "reduce" if red_us >= pack_us else "pack"
    achieved = kernels[dom]["GBps"]
    if dom == "reduce" and direct:
        # a combine of the last dispatch's handle is the reduce kernel alone: the event pair that time_calls puts
        # around the whole combine brackets exactly that kernel, with fewer host calls between the markers than
        # the per-phase loop has (which otherwise lets the GPU run dry for a microsecond or two)
        kernels["reduce"].update(us_in_step=round(c_us, 2))
        achieved = round(alg["combine"] / c_us / 1e3, 1)
    traffic, traffic_at, traffic_current = measured_traffic(cfg.name, dom)
    if opts or not traffic_current:
        # measured with other options, or on other kernel sources than the ones running now: not this run's figure
        traffic = None
    out = {
        "metric": METRIC,
        "value": round(step_gbps, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "dtype_detail": "bf16 in; fp8 e4m3 payload with f32 scale arithmetic out of dispatch; bf16 rows, f32 "
                        "accumulation, bf16 out of combine",
        "data": "synthetic",
        "config": {"workload": cfg.name, "num_ranks": cfg.num_ranks, "tokens_per_rank": cfg.tokens_per_rank,
                   "hidden": cfg.hidden, "num_experts": cfg.num_experts, "num_topk": cfg.num_topk,
                   "use_fp8": cfg.use_fp8, "valid_selections": S, "seed": args.seed, "options": opts,
                   "launch": "graph replay" if args.graph else "eager"},
        "pct_of_hbm_peak": round(step_gbps / HBM_PEAK_GBPS * 100, 2),
        "dispatch_us": round(d_us, 2),
        "combine_us": round(c_us, 2),
        "tokens_per_s": round(cfg.total_tokens / ((d_us + c_us) * 1e-6), 1),
        "algorithmic_bytes": alg,
        "kernels": kernels,
        "consumer": consumer,
        "fused_combine": fused,
        # `achieved` is priced on the kernel's duration inside the running pipeline (an event pair around it in
        # every step, which carries 2-5 us of marker overhead); the same kernel launched back to back between
        # one event pair, the figure a profiler's average duration corresponds to, is reported beside it
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBPS, 4),
                     "frac_back_to_back": round(kernels[dom]["bytes"] / kernels[dom]["us_back_to_back"] / 1e3
                                                / HBM_PEAK_GBPS, 4),
                     "traffic": traffic, "traffic_measured_at_commit": traffic_at if traffic is not None else None,
                     # true: a summary exists but was measured on other kernel sources; null: no summary for this workload
                     "traffic_summary_stale": (not traffic_current) if traffic_at is not None else None},
    }
    if not args.no_flushed:
        out["flushed"] = time_flushed(h, args.kernel_iters, alg)
    if not args.no_buffer_api:
        out["buffer_api"] = time_buffer_api(h, args.steps, args.warmup)
        out["buffer_api"]["python_buffer_async_finish"] = time_python_buffer(h, args.steps, args.warmup)
    if not args.no_small_world:
        out["small_world"] = time_small_world(max(args.kernel_iters, 100))
    if args.copy_calibration > 0:
        nbytes = args.copy_calibration << 20
        src = torch.empty(nbytes, dtype=torch.uint8, device="cuda:0").fill_(1)
        dst = torch.empty_like(src)
        for _ in range(3):
            _lib.check(_lib.lib().mc_ep_debug_copy(dst.data_ptr(), src.data_ptr(), nbytes,
                                                   int(torch.cuda.current_stream().cuda_stream)))
        torch.cuda.synchronize()
        out["copy_calibration_bytes"] = nbytes
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(cfg, data, alg["dispatch"] + alg["combine"], args.cpu_seconds)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
