/*
 * C ABI of libmooncake_ep_hip.so: mooncake-ep's low-latency MoE dispatch /
 * combine for one AMD MI355X (gfx950), with the expert-parallel world kept as
 * logical ranks inside that GPU's HBM.
 *
 * The entry points are what the reference's Python binding for this path
 * binds (mooncake-ep/src/ep_py.cpp:14-46, class MooncakeEpBuffer in
 * mooncake-ep/include/mooncake_ep_buffer.h:66-194), flattened to plain
 * pointers and integers.  Device addresses and streams travel as uint64_t
 * exactly as in the reference's signatures.  Every function returns 0 on
 * success or an MC_EP_ERR_* code; mc_ep_last_error() returns the message of
 * the calling thread's last failure.  The reference raises EPException
 * ("Failed: Assertion error file:line 'cond'", mooncake_ep_exception.cuh:12-45)
 * where this ABI returns MC_EP_ERR_ASSERT with the same condition text.
 *
 * Threads: the library's host bookkeeping sits behind one process-wide lock,
 * so any thread may call any function; a call holds the lock while it records
 * arguments and enqueues kernels, not while it waits for a collective's peers
 * or results.  What the
 * lock cannot give is order: calls of one rank must come from one thread at a
 * time (the reference's buffer is not thread-safe either,
 * mooncake_ep_buffer.cpp:215-218), and with one driver thread for all ranks a
 * per-rank call returns before its collective is complete (see
 * mc_ep_buffer_dispatch).  A thread per rank, each using its results as soon
 * as its call returns like a process of the reference, sets the option
 * "blocking".  The
 * calls of one world share its scratch (rank tables, routing state, staged
 * scales), so the library serialises them across streams: a call on another
 * stream than the world's previous call first waits for what that stream
 * holds.  A stream that has carried a world's calls must therefore stay valid
 * while later calls of the world may follow on other streams.  Scratch grows
 * by replacement; outgrown allocations are kept until the world is destroyed,
 * because queued kernels and instantiated graphs hold their addresses.
 */
#ifndef MOONCAKE_EP_HIP_H
#define MOONCAKE_EP_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define MC_EP_OK 0
#define MC_EP_ERR_ASSERT 1      /* a host assertion of the reference failed */
#define MC_EP_ERR_HIP 2         /* a HIP runtime call failed */
#define MC_EP_ERR_PENDING 3     /* a collective is waited on before every live rank has called it */
#define MC_EP_ERR_UNSUPPORTED 4 /* zero-copy combine etc. (NotImplementedError in the reference) */
#define MC_EP_ERR_INVALID 5     /* std::invalid_argument in the reference (ValueError through pybind11) */

/* mooncake_ep_configs.cuh:5 */
#define MC_EP_MAX_QP_COUNT 256

/* phases of a whole-world call (the reference's LOW_LATENCY_SEND_PHASE /
 * LOW_LATENCY_RECV_PHASE split, mooncake_ep_configs.cuh:16-17, maps onto the
 * kernels each call is made of; a later phase needs the earlier ones of the
 * same call to have run) */
#define MC_EP_PHASE_LAYOUT 1   /* dispatch: routing counts;  combine: handle -> row resolve */
#define MC_EP_PHASE_DATA 2     /* dispatch: pack (packed_recv_count / src_info / layout_range are complete after
                                  this phase, not before); combine: weighted reduce */
#define MC_EP_PHASE_FINISH 4   /* dispatch: fp8 scales into their column-major layout; combine: nothing */
#define MC_EP_PHASE_ALL 7

typedef struct mc_ep_world mc_ep_world_t;     /* R logical ranks on one device */
typedef struct mc_ep_buffer mc_ep_buffer_t;   /* one rank's MooncakeEpBuffer */
typedef struct mc_ep_event mc_ep_event_t;     /* EventHandle */
typedef struct mc_ep_hook mc_ep_hook_t;       /* the recv hook closure */

const char* mc_ep_last_error(void);

/* get_ep_buffer_size_hint, mooncake_ep_buffer.h:197-203 (BufferPair, :29-63) */
uint64_t mc_ep_get_buffer_size_hint(int num_max_dispatch_tokens_per_rank, int hidden, int num_ranks,
                                    int num_experts);

/* ---- the logical world ------------------------------------------------- */

/* Replaces process-group bootstrap + peer exchange (Buffer.__init__/connect,
 * mooncake-wheel/mooncake/mooncake_ep_buffer.py:93-119,185-304): all ranks
 * share one address space, so there is nothing to exchange.  Uses the
 * calling thread's current HIP device. */
int mc_ep_world_create(int num_ranks, mc_ep_world_t** out);
int mc_ep_world_destroy(mc_ep_world_t* world);
int mc_ep_world_num_ranks(const mc_ep_world_t* world);

/* A silent rank stops calling dispatch/combine (the reference's failed
 * process, mooncake-ep/tests/test_ep_grid.py:121-158); collectives complete
 * without it.  Forces from the host what the reference detects by timeout
 * (mooncake_ep_kernel.cu:417-429, :688-698).  silent == 0 brings the rank back
 * (the reference's restarted process, Buffer.update_ep_member,
 * mooncake_ep_buffer.py:306-307): its next call joins the first round that no
 * rank has opened yet. */
int mc_ep_world_set_rank_silent(mc_ep_world_t* world, int rank, int silent);

/* Options ("pack_waves", "pack_nt", "uniform", "routing_sum", "combine_direct",
 * "combine_chunks", "combine_waves", "combine_nt", "combine_occupancy",
 * "packed_map": tuning knobs
 * for measurement sweeps; "fused_small": 1 (default) dispatches a world of at
 * most 8 ranks and "fused_small_max" (default 4096) selections in one kernel
 * launch - provided the ranks' index lists make at most "fused_small_rounds"
 * rounds of 512 entries, each list counted by itself (default -1: 6 for an
 * fp8 payload, 4 for bf16, which is where the launch stops paying) - and 0
 * always takes the count / pack / scale-transpose launches;
 * "last_dispatch_launches", "last_combine_launches": read them to learn how
 * many kernels the world's last dispatch / combine call enqueued (a rank-table
 * upload counts); "fp8_arith": 0 (default) the fp8 scale arithmetic of the reference's
 * PyTorch statement as CPU PyTorch runs it - 448.0 / amax as reciprocal times
 * 448, amax / 448.0 a true division (mooncake_ep_buffer.py:699-702) - or 1 the
 * reference kernel's own, 448 / amax as one IEEE division and amax * (1 / 448)
 * (mooncake_ep_kernel.cu:184, :252), which differ in the last bit of a scale
 * for about a quarter of all groups; "comm_stream": 1 runs every per-rank
 * collective on the world's communication stream as the reference does, 0
 * (default) on the callers' stream when they all share one; "blocking": 1
 * makes mc_ep_buffer_dispatch / mc_ep_buffer_combine return only when the
 * call's round has been launched - by the thread whose call completed it - so
 * that work the caller enqueues next on its stream is ordered behind the
 * round, which is what a thread per rank needs; a call that has waited
 * "block_timeout_ms" (default 30000) for its peers - the first
 * "block_spin_us" (default 200) of them awake, yielding its core - fails with
 * MC_EP_ERR_PENDING and stays posted; no order is then imposed on its stream). */
int mc_ep_world_set_option(mc_ep_world_t* world, const char* name, int value);
int mc_ep_world_get_option(const mc_ep_world_t* world, const char* name, int* value);

/* Whole-world dispatch: every rank's MooncakeEpBuffer::dispatch
 * (mooncake_ep_buffer.h:116-124, mooncake_ep_buffer.cpp:193-339) in one
 * launch sequence on `stream_ptr`.  Each *_ptrs argument is a host array of
 * num_ranks device addresses (rank r's tensor); num_tokens is a host array.
 * A rank with packed_recv_x_ptrs[r] == 0 receives nothing; a rank with
 * num_tokens[r] == 0 sends nothing.  packed_recv_x_scales_ptrs may be NULL
 * when use_fp8 == 0.  Tensor shapes per rank as in the reference:
 *   x [T_r, hidden] bf16, topk_idx [T_r, num_topk] int64,
 *   packed_recv_x [E/R, R*max, hidden] fp8 e4m3fn | bf16,
 *   packed_recv_x_scales [E/R, hidden/128, R*max] f32 (physical layout),
 *   packed_recv_count [E/R] int32, packed_recv_src_info [E/R, R*max] int32,
 *   packed_recv_layout_range [E/R, R] int64. */
int mc_ep_world_dispatch(mc_ep_world_t* world, const uint64_t* x_ptrs, const uint64_t* topk_idx_ptrs,
                         const int32_t* num_tokens, int hidden, int num_topk,
                         int num_max_dispatch_tokens_per_rank, int num_experts, int use_fp8,
                         const uint64_t* packed_recv_x_ptrs, const uint64_t* packed_recv_x_scales_ptrs,
                         const uint64_t* packed_recv_count_ptrs, const uint64_t* packed_recv_src_info_ptrs,
                         const uint64_t* packed_recv_layout_range_ptrs, int phases, uint64_t stream_ptr);

/* mc_ep_world_dispatch (all phases) for callers that cannot allocate device
 * memory: code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  It has no counterpart in the reference.  The call makes no
 * hipMalloc / hipFree and no other allocating call, whatever the shape: the
 * routing state, the fp8 scale staging rows and the rank table live in a
 * 16 MiB array in static device memory that each GPU the library runs on holds
 * until the process ends.  A shape that needs more (about
 * num_experts * num_ranks * max_tokens * 4 bytes, plus
 * num_ranks * max_tokens * (num_topk * 8 + hidden / 32) bytes) is rejected with
 * MC_EP_ERR_ASSERT and a message that says so; the DeepSeek-V3 decode world
 * (32 x 128 tokens, 256 experts, hidden 7168) needs 5.5 MB.  Same arguments,
 * outputs and errors as mc_ep_world_dispatch otherwise.  Every call on a GPU,
 * from any world, shares that GPU's array and overwrites the last call's
 * contents: calls that overlap on one GPU (different streams without an order
 * between them, or different threads) race.  A combine given this dispatch's
 * handle reads src_info / layout_range as any combine of an older handle does
 * (it does not find the routing state of "the last dispatch"). */
int mc_ep_world_dispatch_noalloc(mc_ep_world_t* world, const uint64_t* x_ptrs, const uint64_t* topk_idx_ptrs,
                                 const int32_t* num_tokens, int hidden, int num_topk,
                                 int num_max_dispatch_tokens_per_rank, int num_experts, int use_fp8,
                                 const uint64_t* packed_recv_x_ptrs, const uint64_t* packed_recv_x_scales_ptrs,
                                 const uint64_t* packed_recv_count_ptrs, const uint64_t* packed_recv_src_info_ptrs,
                                 const uint64_t* packed_recv_layout_range_ptrs, uint64_t stream_ptr);

/* Whole-world combine: every rank's MooncakeEpBuffer::combine
 * (mooncake_ep_buffer.h:126-133, mooncake_ep_buffer.cpp:341-474).
 *   x [E/R, R*max, hidden] bf16 (expert outputs held by the rank; 0: the rank
 *   contributes nothing), topk_idx / topk_weights [T_r, num_topk],
 *   src_info / layout_range: the handle returned by that rank's dispatch,
 *   active_ranks [R] int32 (rank r's own view), combined_x [T_r, hidden] bf16.
 * topk_idx is read as it is when the kernel runs, as in the reference
 * (mooncake_ep_kernel.cu:719-732): a selection that was set to -1 after the
 * dispatch (or no longer names the expert it was dispatched to) contributes
 * nothing, whichever way combine finds its rows. */
int mc_ep_world_combine(mc_ep_world_t* world, const uint64_t* x_ptrs, const uint64_t* topk_idx_ptrs,
                        const uint64_t* topk_weights_ptrs, const uint64_t* src_info_ptrs,
                        const uint64_t* layout_range_ptrs, const uint64_t* active_ranks_ptrs,
                        const int32_t* num_combined_tokens, int hidden, int num_topk,
                        int num_max_dispatch_tokens_per_rank, int num_experts, const uint64_t* combined_x_ptrs,
                        int phases, uint64_t stream_ptr);

/* ---- consumer of the packed layout --------------------------------------- */

/* What the reference's callers do with dispatch's output before the expert
 * GEMMs: per_token_cast_back (mooncake-wheel/tests/ep_test_utils.py:50-53) /
 * dequantize_fp8 (mooncake-ep/tests/test_ep_grid.py:43-48): bf16(f32(fp8) *
 * scale) per 128-element group, reading the scales in the column-major layout
 * dispatch writes (mooncake_ep_buffer.py:479-487) - and, when
 * expert_factor_ptr != 0 (device f32 [num_experts]), the grid test's mock
 * expert on top, bf16(row * factor[expert]) (test_ep_grid.py:168-173).  Only
 * rows below packed_recv_count are read or written.  packed_recv_x_scales_ptrs
 * == NULL means the payload is bf16 (then only the factor applies; out may
 * alias the input).  num_topk bounds the number of valid rows (at most one per
 * selection); 0 if unknown.  Out: [E/R, R*max, hidden] bf16 per rank. */
int mc_ep_world_cast_back(mc_ep_world_t* world, const uint64_t* packed_recv_x_ptrs,
                          const uint64_t* packed_recv_x_scales_ptrs, const uint64_t* packed_recv_count_ptrs,
                          uint64_t expert_factor_ptr, const uint64_t* out_ptrs, int hidden, int num_topk,
                          int num_max_dispatch_tokens_per_rank, int num_experts, uint64_t stream_ptr);

/* Combine fused with that consumer: what mc_ep_world_cast_back (with the same
 * packed_recv_x / scales / expert_factor arguments) followed by
 * mc_ep_world_combine on its output computes, bit for bit, without writing
 * and re-reading the bf16 rows in between: every source row becomes
 * bf16(bf16(f32(fp8) * scale) * factor[expert]) in registers (the grid test's
 * mock expert, mooncake-ep/tests/test_ep_grid.py:160-173, between dispatch and
 * combine) and enters the fp32 sum of mooncake_ep_kernel.cu:711-753.
 * packed_recv_x_scales_ptrs == NULL: bf16 payload; expert_factor_ptr == 0: no
 * factor.  The other arguments are mc_ep_world_combine's. */
int mc_ep_world_combine_packed(mc_ep_world_t* world, const uint64_t* packed_recv_x_ptrs,
                               const uint64_t* packed_recv_x_scales_ptrs, uint64_t expert_factor_ptr,
                               const uint64_t* topk_idx_ptrs, const uint64_t* topk_weights_ptrs,
                               const uint64_t* src_info_ptrs, const uint64_t* layout_range_ptrs,
                               const uint64_t* active_ranks_ptrs, const int32_t* num_combined_tokens, int hidden,
                               int num_topk, int num_max_dispatch_tokens_per_rank, int num_experts,
                               const uint64_t* combined_x_ptrs, int phases, uint64_t stream_ptr);

/* ---- the native benchmark loop ------------------------------------------ */

/* _benchmark_legacy_buffer (bound in mooncake-ep/src/ep_py.cpp:12,26; the loop
 * is mooncake-ep/benchmarks/legacy_buffer_perf.cpp:84-146): clear
 * packed_recv_count, bf16 dispatch, combine, repeated `warmups` times untimed
 * and `iterations` times between a pair of events each; the first timed
 * iteration is dropped.  The structs are LegacyBufferPerfTensors / Config /
 * Result (legacy_buffer_perf.cpp:18-49) with one device address per logical
 * rank where the reference has one address: the loop drives the whole world,
 * every rank with num_tokens tokens.  A null address or a configuration the
 * reference's validate() rejects (:58-82) gives MC_EP_ERR_ASSERT with the
 * reference's message. */
typedef struct {
    const uint64_t* x_ptrs;                          /* [T, H] bf16 */
    const uint64_t* topk_idx_ptrs;                   /* [T, K] int64 */
    const uint64_t* topk_weights_ptrs;               /* [T, K] f32 */
    const uint64_t* active_ranks_ptrs;               /* [R] int32 */
    const uint64_t* expert_x_ptrs;                   /* [E/R, R*max, H] bf16: what combine reads */
    const uint64_t* packed_recv_x_ptrs;              /* [E/R, R*max, H] bf16 */
    const uint64_t* packed_recv_count_ptrs;          /* [E/R] int32 */
    const uint64_t* packed_recv_src_info_ptrs;       /* [E/R, R*max] int32 */
    const uint64_t* packed_recv_layout_range_ptrs;   /* [E/R, R] int64 */
    const uint64_t* combined_x_ptrs;                 /* [T, H] bf16 */
} mc_ep_legacy_perf_tensors_t;

typedef struct {
    int num_tokens;
    int hidden;
    int num_topk;
    int num_local_experts;
    int num_max_dispatch_tokens_per_rank;
    int num_experts;
    int timeout_us;                                  /* -1; kept for the reference's layout, unused */
    int warmups;                                     /* reference default 20 */
    int iterations;                                  /* reference default 30; > 1 */
    uint64_t compute_stream_ptr;
} mc_ep_legacy_perf_config_t;

typedef struct {
    double average_us;
    double min_us;
    double max_us;
} mc_ep_legacy_perf_result_t;

int mc_ep_world_legacy_buffer_perf(mc_ep_world_t* world, const mc_ep_legacy_perf_tensors_t* tensors,
                                   const mc_ep_legacy_perf_config_t* config, mc_ep_legacy_perf_result_t* result);

/* ---- per-rank Buffer: the reference's binding, one object per rank ------ */

/* MooncakeEpBuffer(rank, num_ranks, num_ep_buffer_bytes, disable_p2p),
 * ep_py.cpp:27-30.  num_ranks is the world's. */
int mc_ep_buffer_create(mc_ep_world_t* world, int rank, int64_t num_ep_buffer_bytes, int disable_p2p,
                        mc_ep_buffer_t** out);
int mc_ep_buffer_destroy(mc_ep_buffer_t* buffer);

/* Transport introspection (ep_py.cpp:31-42).  One GPU: no NIC, every peer is
 * in the same address space. */
int mc_ep_buffer_ibgda_disabled(const mc_ep_buffer_t* buffer);   /* 1 */
int mc_ep_buffer_p2p_enabled(const mc_ep_buffer_t* buffer);      /* !disable_p2p */
int mc_ep_buffer_use_fast_path(const mc_ep_buffer_t* buffer);    /* 1 */
int mc_ep_buffer_is_roce(const mc_ep_buffer_t* buffer);          /* 0 */

/* MooncakeEpBuffer::dispatch, argument order of mooncake_ep_buffer.h:116-124.
 * Dispatch is a collective over the world's live ranks: the call records this
 * rank's arguments, and the call that completes the round launches the
 * kernels for all ranks.  *event_out is set when async != 0, *hook_out when
 * return_recv_hook != 0 (else NULL); async together with return_recv_hook is
 * rejected (mooncake_ep_buffer.cpp:226). */
int mc_ep_buffer_dispatch(mc_ep_buffer_t* buffer, uint64_t x_ptr, uint64_t topk_idx_ptr, uint64_t active_ranks_ptr,
                          int num_tokens, int hidden, int num_topk, int num_max_dispatch_tokens_per_rank,
                          int num_experts, int timeout_us, int use_fp8, uint64_t packed_recv_x_ptr,
                          uint64_t packed_recv_x_scales_ptr, uint64_t packed_recv_count_ptr,
                          uint64_t packed_recv_src_info_ptr, uint64_t packed_recv_layout_range_ptr, int async,
                          int return_recv_hook, uint64_t compute_stream_ptr, mc_ep_event_t** event_out,
                          mc_ep_hook_t** hook_out);

/* MooncakeEpBuffer::combine, argument order of mooncake_ep_buffer.h:126-133. */
int mc_ep_buffer_combine(mc_ep_buffer_t* buffer, uint64_t x_ptr, uint64_t topk_idx_ptr, uint64_t topk_weights_ptr,
                         uint64_t src_info_ptr, uint64_t layout_range_ptr, uint64_t active_ranks_ptr,
                         int num_local_experts, int num_combined_tokens, int hidden, int num_topk,
                         int num_max_dispatch_tokens_per_rank, int num_experts, int timeout_us, int zero_copy,
                         uint64_t combined_x_ptr, int async, int return_recv_hook, uint64_t compute_stream_ptr,
                         mc_ep_event_t** event_out, mc_ep_hook_t** hook_out);

/* How many of this rank's dispatch / combine calls still have kernels to be
 * enqueued: their round waits for other live ranks, or (dispatch) for the
 * receive hook that enqueues its second part.  The caller keeps the tensors of
 * that many most recent calls of each kind alive; the reference's callers have
 * no such duty because every process enqueues its own kernels inside the call
 * (mooncake_ep_buffer.cpp:296-316). */
int mc_ep_buffer_pending_calls(const mc_ep_buffer_t* buffer, int* dispatch_pending, int* combine_pending);

/* ---- EventHandle (mooncake_ep_event.h:9-42) and the recv hook ----------- */

/* EventHandle(stream_ptr): an event recorded on that stream now. */
int mc_ep_event_create(uint64_t stream_ptr, mc_ep_event_t** out);
int mc_ep_event_current_stream_wait(mc_ep_event_t* event, uint64_t stream_ptr);
int mc_ep_event_synchronize(mc_ep_event_t* event);
int mc_ep_event_destroy(mc_ep_event_t* event);

/* The closure returned for return_recv_hook (mooncake_ep_buffer.cpp:303-305,
 * :330-335).  A round whose callers all asked for a hook is launched in two
 * parts, as the reference splits SEND and RECV: the call that completes the
 * round enqueues MC_EP_PHASE_LAYOUT | MC_EP_PHASE_DATA, the first hook called
 * enqueues MC_EP_PHASE_FINISH (an fp8 dispatch's scales; nothing for bf16 and
 * for combine), and each hook makes its rank's compute stream wait for the
 * round.  After it returns, work queued on that stream sees the outputs.  The
 * next dispatch of the world enqueues a second part that no hook has asked for
 * yet.  The hook must not outlive its world. */
int mc_ep_hook_call(mc_ep_hook_t* hook);
int mc_ep_hook_destroy(mc_ep_hook_t* hook);

#ifdef __cplusplus
}
#endif

#endif /* MOONCAKE_EP_HIP_H */
