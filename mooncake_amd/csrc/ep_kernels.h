// Launch interface between the host runtime (ep_runtime.hip) and the gfx950
// kernels (ep_kernels.hip).  Internal to the library; the public C ABI is
// include/mooncake_ep_hip.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace mcep {

// The logical EP world lives in one GPU's HBM.  Every rank hands the library
// its own tensors, so kernels find a rank's tensor through a table in device
// memory: tbl[field * R + rank] holds a device address (or a small integer).
enum DispatchField : int {
    DF_X = 0,          // const bf16*  [T_r, H]
    DF_TOPK_IDX,       // const int64* [T_r, K]
    DF_RECV_X,         // fp8|bf16*    [L, R*max, H]      (0: rank takes no part)
    DF_RECV_SCALES,    // float*       [L, H/128, R*max]  (fp8 only)
    DF_RECV_COUNT,     // int32*       [L]
    DF_SRC_INFO,       // int32*       [L, R*max]
    DF_LAYOUT_RANGE,   // int64*       [L, R]
    DF_NUM_TOKENS,     // T_r as an integer (0: rank sends nothing)
    DF_COUNT
};

enum CombineField : int {
    CF_X = 0,          // const bf16*  [L, R*max, H] expert outputs held by the rank
    CF_TOPK_IDX,       // const int64* [T_r, K]
    CF_TOPK_W,         // const float* [T_r, K]
    CF_SRC_INFO,       // const int32* [L, R*max]
    CF_LAYOUT_RANGE,   // const int64* [L, R]
    CF_ACTIVE,         // const int32* [R]  the rank's own view of live ranks
    CF_OUT,            // bf16*        [T_r, H]
    CF_NUM_TOKENS,     // T_r as an integer (0: rank combines nothing)
    CF_SCALES,         // const float* [L, H/128, R*max]: scales of an fp8 payload in CF_X (packed combine only)
    CF_COUNT
};

// table of the packed layout's consumer (cast back to bf16)
enum ConsumerField : int {
    XF_RECV_X = 0,     // const fp8|bf16* [L, R*max, H]   (0: rank takes no part)
    XF_RECV_SCALES,    // const float*    [L, H/128, R*max] (fp8 only)
    XF_RECV_COUNT,     // const int32*    [L]
    XF_OUT,            // bf16*           [L, R*max, H]
    XF_COUNT
};

constexpr int kMaxTopK = 16;          // the reference caps top-k at 11 (mooncake_ep_kernel.cu:487,773)
constexpr int kTableChunk = 384;      // table words one writer launch carries in its kernel arguments
constexpr size_t kZeroRowBytes = 64 * 1024;   // zero row that masked selections read: hidden <= 32768

struct TableChunk {
    uint64_t v[kTableChunk];
};

// The dispatch rank table of a small world, carried in kernel arguments: v[field * R + rank] with the
// call's own R (at most kSmallRanks).
constexpr int kSmallRanks = 8;
constexpr int kSmallListRound = 512;  // index-list entries a wave of dispatch_small_kernel has in flight at a time
struct SmallTable {
    uint64_t v[(int)DF_COUNT * kSmallRanks];
};

// Routing state a dispatch leaves in world-owned device memory.  The world's
// selections are cut into units of kUnitSelections consecutive (token, k)
// entries of one rank (units_per_rank per rank, rank-major).  The count kernel
// produces, per unit and expert, how many of the unit's selections name the
// expert and, per selection, its position among those; an exclusive prefix
// over units turns that into the packed row of every selection:
//     row(sel) = ubegin[unit(sel)][expert(sel)] + selpos[sel]
// which is the deterministic order source rank ascending, token ascending.
constexpr int kUnitSelections = 256;
// With units of 1024 selections and few enough of them, the data kernels add up the counts of the
// earlier units themselves and the prefix pass rides along in the pack launch: one launch less.
constexpr int kBigUnitSelections = 1024;
constexpr int kMaxSummedUnits = 64;

// How the world's selections are cut into units and how packed rows come out of the unit counts.
struct UnitPlan {
    int per_rank = 0;   // units per rank
    int shift = 8;      // log2(selections per unit)
    int total = 0;      // R * per_rank
    int summed = 0;     // 1: the data kernels of dispatch sum earlier units' counts themselves
    int carried = 0;    // 1: the prefix pass rides in the pack launch (needs summed)
    int selections() const { return 1 << shift; }
};

struct RoutingScratch {
    int32_t* ucount;     // [U, E]  selections of unit u that name expert e
    int32_t* ucount_t;   // [E, kMaxSummedUnits]  the same, expert-major (summed plan only)
    int32_t* ubegin;     // [U, E]  exclusive prefix of ucount over units
    int32_t* selpos;     // [R * max_tokens * K]  position inside (unit, expert); -1: no valid expert
    int32_t* selrow;     // [R * max_tokens * K]  expert * R*max + packed row of the selection, -1: none; left by the
                         //                       pack kernel for a combine of the same handle
    int32_t* counts;     // [E]     rows per expert (0 for experts of ranks that take no part)
    int32_t* row_src;    // [E, R * max_tokens]  packed row -> source token slot (rank * max_tokens + token)
};

// One resolved source row of combine's general path (a handle that is not the
// one the last dispatch produced): valid for the launch whose stamp it carries,
// so selections that no routing thread visits need no clearing pass.
struct CombineRoute {       // 16 bytes
    uint64_t src;           // byte address of the expert-output row; packed combine: (expert << 32) | row in its block
    float weight;
    uint32_t stamp;
};

// Address of a per-rank tensor.  When the ranks' tensors are evenly spaced the
// address comes from kernel arguments alone (base + rank * stride); otherwise
// (base == 0) from the rank table, one more dependent load.
struct RankPtr {
    uint64_t base = 0;
    int64_t stride = 0;
};

struct DispatchSource {
    RankPtr x, topk_idx;
    int tokens = -1;        // every rank's token count when they are all equal, else -1 (rank table)
};

struct CombineSource {
    RankPtr topk_idx, topk_weights, out;
    RankPtr x;              // the rows combine reads (expert outputs, or the packed payload)
    RankPtr scales;         // packed combine of an fp8 payload
    int tokens = -1;
};

struct Dims {
    int R;            // logical ranks
    int E;            // experts
    int K;            // top-k
    int H;            // hidden
    int max_tokens;   // num_max_dispatch_tokens_per_rank
    int Tgrid;        // max over ranks of T_r (grid extent in tokens per rank)
    UnitPlan plan;    // set by plan_units()
    int units_per_rank() const { return plan.per_rank; }
    int units() const { return plan.total; }
};

// Tuning knobs, settable at run time for measurement sweeps.
struct Tuning {
    int pack_waves = 4;        // waves per block in the pack kernel
    int pack_nt = -1;          // bit 0: streaming (nontemporal) loads, bit 1: streaming stores; -1: loads by top-k
    int uniform = 1;           // take per-rank addresses from kernel arguments when tensors are evenly spaced
    int fp8_arith = 0;         // fp8 scale arithmetic: 0 = the reference's PyTorch statement as CPU PyTorch runs it,
                               // 1 = the reference kernel's own (see pack_fp8_kernel)
    int combine_direct = 1;    // reuse the last dispatch's routing state when combine gets that dispatch's handle
    int combine_chunks = 0;    // 16-byte chunks per lane in the combine kernel (1 or 2); 0: by top-k
    int combine_waves = 4;     // waves per block in the combine kernel
    int combine_nt = 3;        // bit 0: streaming loads, bit 1: streaming stores
    int combine_occupancy = -1;   // waves of the combine kernel a CU runs at a time; 0: as many as fit, -1: by top-k
    int packed_map = 1;        // packed combine of an fp8 payload: 1 = slabs owned by XCDs, 0 = (rank, slab) groups per XCD
    int routing_sum = 1;       // allow the summed routing plan (see UnitPlan) where the shape permits
    int comm_stream = 0;       // 1: per-rank rounds always run on the world's communication stream
    int fused_small = 1;       // dispatch of a small world (see dispatch_small_kernel) in one launch
    int fused_small_max = 4096;   // ... when the world names at most this many selections
    int fused_small_rounds = -1;  // ... in at most this many rounds of kSmallListRound index-list entries, each rank's
                                  // list counted by itself; -1: 6 for an fp8 payload, 4 for bf16 (measured)
    int last_dispatch_launches = 0;   // read-only in spirit: kernels the world's last dispatch / combine call enqueued
    int last_combine_launches = 0;    // (a rank-table upload counts; launches of other phases' calls do not)
    int blocking = 0;          // 1: a per-rank call returns only when its round has been launched (a thread per rank)
    int block_timeout_ms = 30000;   // how long such a call waits for its peers before it fails
    int block_spin_us = 200;        // ... of which this long awake (yielding the core), before it goes to sleep
};

// Chooses the unit plan for a shape (summed when allowed, the shape permits and there are tokens).
// (plan_units, count_lds_bytes and cast_back_chunks are host arithmetic: ep_plan.cpp.)
void plan_units(Dims& d, const Tuning& t);

hipError_t launch_table_write(uint64_t* d_tbl, const uint64_t* h_tbl, int n_words, hipStream_t stream);

hipError_t launch_count(const uint64_t* d_tbl, const RoutingScratch& sc, const DispatchSource& src, const Dims& d,
                        hipStream_t stream);
hipError_t launch_pack(const uint64_t* d_tbl, const RoutingScratch& sc, const DispatchSource& src, float* scale_stage,
                       const Dims& d, bool use_fp8, const Tuning& t, bool run_pack, bool run_finish,
                       hipStream_t stream);
// The whole dispatch of a small world in one launch (layout, payload, scales, src_info, counts, ranges, and
// selrow for a combine of the same handle).  The caller has checked: R <= kSmallRanks, d.Tgrid > 0.
hipError_t launch_dispatch_small(const SmallTable& tb, int32_t* d_selrow, const Dims& d, bool use_fp8, const Tuning& t,
                                 hipStream_t stream);
// packed: routes carry (expert, row) instead of a row address
hipError_t launch_resolve(const uint64_t* d_tbl, CombineRoute* d_routes, uint32_t stamp, bool packed, const Dims& d,
                          const Tuning& t, hipStream_t stream);
// direct: rows come from the last dispatch's routing state (sc); otherwise from d_routes
hipError_t launch_reduce(const uint64_t* d_tbl, const CombineRoute* d_routes, uint32_t stamp, const RoutingScratch& sc,
                         bool direct, const CombineSource& src, const void* d_zero_row, const Dims& d, const Tuning& t,
                         hipStream_t stream);
// Combine straight from the packed layout: CF_X holds dispatch's payload (fp8 with CF_SCALES, or bf16), every
// row is turned into what the consumer kernel would have made of it (times factor[expert] when d_factor is
// given) on its way into the weighted sum.
hipError_t launch_reduce_packed(const uint64_t* d_tbl, const CombineRoute* d_routes, uint32_t stamp,
                                const RoutingScratch& sc, bool direct, const CombineSource& src, const void* d_zero_row,
                                const float* d_factor, bool use_fp8, const Dims& d, const Tuning& t, hipStream_t stream);
// packed rows below packed_recv_count -> bf16 rows times factor[expert]; max_rows bounds the world's valid rows
// d_chunk_map: 16 bytes x (cast_back_chunks(max_rows, E) + 1) of scratch for the kernel's work list
constexpr int kCastRows = 4;          // packed rows of one expert per work item of the cast-back kernel
long long cast_back_chunks(long long max_rows, int num_experts);
hipError_t launch_cast_back(const uint64_t* d_tbl, void* d_chunk_map, const float* d_factor, bool use_fp8,
                            long long max_rows, const Dims& d, hipStream_t stream);
hipError_t launch_copy(void* dst, const void* src, size_t bytes, hipStream_t stream);
// waves per CU the synthetic streams run at from now on (0: as many as fit)
void set_stream_occupancy(int waves_per_cu);
// a synthetic stream of `unit_bytes / 16` threads with one of the data kernels' read : write mixes (see stream_kernel)
hipError_t launch_stream(int kind, void* dst, const void* src, size_t unit_bytes, hipStream_t stream);
// out_rows rows, each the xor of 8 rows scattered over a [regions, region_rows] layout (see stream_rows_kernel)
hipError_t launch_stream_rows(void* dst, const void* src, int row_bytes, long long out_rows, int regions,
                              long long region_rows, int used, hipStream_t stream);
// in_rows rows of 2 * row_bytes, each folded to row_bytes and written to 8 scattered rows (see stream_rows_scatter_kernel)
hipError_t launch_stream_rows_scatter(void* dst, const void* src, int row_bytes, long long in_rows, int regions,
                                      long long region_rows, int used, hipStream_t stream);
// zero `words` 32-bit words at each of n_ptrs device addresses (host array), one launch per kTableChunk addresses
hipError_t launch_clear_words(const uint64_t* h_ptrs, int n_ptrs, int words, hipStream_t stream);
hipError_t launch_fill_u32(void* dst, uint32_t value, size_t words, hipStream_t stream);

// LDS the count kernel needs (per-wave counts and prefixes for every expert)
constexpr size_t kMaxCountLdsBytes = 144 * 1024;
size_t count_lds_bytes(const Dims& d);
// units the prefix kernel can hold a wave's prefixes for in LDS
constexpr int kMaxUnits = 3500;

}  // namespace mcep
