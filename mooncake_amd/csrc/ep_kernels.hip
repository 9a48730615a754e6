// gfx950 (CDNA4, wave64) kernels for the low-latency MoE dispatch / combine
// path.  Everything here is HBM-bound byte movement: no matrix cores, every
// payload access is a 16-byte vector load or store that a wave issues over a
// contiguous span of a row.
//
//   count_kernel,   routing layout: per-expert histogram of every unit of 1024
//   prefix pass     (or 256) selections, position of each selection inside it,
//                   exclusive prefix over units, per-(expert, source rank)
//                   ranges and per-expert counts.  The prefix pass runs as the
//                   first waves of the pack launch (summed plan) or as
//                   prefix_kernel (table plan).  Restates the count path and
//                   the slot assignment of the reference's dispatch
//                   (mooncake-ep/src/mooncake_ep_kernel.cu:274, :319-356,
//                   :417-437) in a deterministic order: source rank ascending,
//                   token ascending, as the reference's PyTorch statement has
//                   it (mooncake-wheel/mooncake/mooncake_ep_buffer.py:787-817).
//   pack_kernel     one read of each token row, optional bf16 -> fp8 e4m3
//                   quantisation with per-128 amax / 448 scales (the contract
//                   of mooncake_ep_kernel.cu:183-186, :233-264; the scale
//                   arithmetic follows, by default, the reference's PyTorch
//                   statement of it, mooncake_ep_buffer.py:693-703, and the
//                   kernel's own on request - they differ in the last bit of
//                   the scale for about a quarter of all groups), K row stores
//                   straight into [local expert, R*max, hidden]
//                   (the reference needs two hops, :273-306 then :442-466);
//                   scale_transpose_kernel then moves the fp8 scales into
//                   their column-major layout (:457-465).
//   dispatch_small_kernel  all of the above in one launch for a world of a few
//                   thousand selections (one deployed rank's decode step): every
//                   wave rebuilds the routing it needs from the index lists, as
//                   the reference's dispatch is one launch
//                   (mooncake_ep_kernel.cu:138-470).
//   resolve_kernel  combine's handle (src_info, layout_range) -> source row and
//                   weight of each (token, k) (data flow of
//                   mooncake_ep_kernel.cu:611-637); only for a handle that is
//                   not the last dispatch's.
//   reduce_kernel   per token: fp32 fused multiply-add over its top-k expert
//                   rows in k order, round to nearest even bf16
//                   (mooncake_ep_kernel.cu:711-753); a selection counts while
//                   topk_idx, as combine is given it, still names the expert
//                   (:719-732).
//   cast_chunks_kernel,  the consumer of the packed layout: valid rows back to
//   cast_back_kernel     bf16, times a per-expert factor
//                   (per_token_cast_back, mooncake-wheel/tests/ep_test_utils.py:50-53;
//                   the mock expert of mooncake-ep/tests/test_ep_grid.py:168-173).
//   reduce_packed_kernel  combine fused with that consumer: reads dispatch's
//                   payload (fp8 + scales, or bf16) and gives, bit for bit, what
//                   cast_back_kernel followed by reduce_kernel gives.
//   stream_kernel,  measurement only: synthetic streams with the read : write
//   stream_rows_*   mixes and the row geometry of the data kernels, what the
//                   memory system gives them with nothing else in the way; and
//                   copy_kernel, the known-size kernel the profiler's byte
//                   counters are scaled against.
#include "ep_kernels.h"

#include <atomic>

namespace mcep {

namespace {

__device__ __forceinline__ int wave_lane() { return threadIdx.x & 63; }

template <int CTRL>
__device__ __forceinline__ float dpp_move(float v) {
    return __int_as_float(__builtin_amdgcn_mov_dpp(__float_as_int(v), CTRL, 0xF, 0xF, true));
}

// max over aligned groups of 8 (or 16) lanes: two quad permutes, then the
// half-row (and row) mirrors, all in the DPP data path.
template <int GROUP>
__device__ __forceinline__ float group_max(float v) {
    v = fmaxf(v, dpp_move<0xB1>(v));    // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_move<0x4E>(v));    // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_move<0x141>(v));   // row_half_mirror
    if (GROUP == 16) v = fmaxf(v, dpp_move<0x140>(v));   // row_mirror
    return v;
}

// Inclusive prefix sum over the 64 lanes of a wave (all of them active), in the DPP data path: shifts
// by 1, 2, 4, 8 inside each row of 16 lanes (zeros shifted in), then lane 15 of rows 0 and 2 added to
// rows 1 and 3, then lane 31 added to rows 2 and 3.
__device__ __forceinline__ int wave_scan_inclusive(int v) {
    v += __builtin_amdgcn_update_dpp(0, v, 0x111, 0xF, 0xF, true);    // row_shr:1
    v += __builtin_amdgcn_update_dpp(0, v, 0x112, 0xF, 0xF, true);    // row_shr:2
    v += __builtin_amdgcn_update_dpp(0, v, 0x114, 0xF, 0xF, true);    // row_shr:4
    v += __builtin_amdgcn_update_dpp(0, v, 0x118, 0xF, 0xF, true);    // row_shr:8
    v += __builtin_amdgcn_update_dpp(0, v, 0x142, 0xA, 0xF, false);   // row_bcast:15 into rows 1 and 3
    v += __builtin_amdgcn_update_dpp(0, v, 0x143, 0xC, 0xF, false);   // row_bcast:31 into rows 2 and 3
    return v;
}

__device__ __forceinline__ uint64_t read_lane_u64(uint64_t v, int lane) {
    uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, lane);
    uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), lane);
    return ((uint64_t)hi << 32) | lo;
}

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

// Every tensor the kernels touch is device memory, but most addresses reach them as integers (rank tables,
// kernel arguments), which the compiler can only treat as generic pointers: flat loads and stores, which
// also count as LDS / scalar-memory operations when a wave waits.  These helpers say "global" explicitly.
#define MCEP_GLOBAL __attribute__((address_space(1)))
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <bool NT>
__device__ __forceinline__ uint4 load16(const void* p) {
    const MCEP_GLOBAL u32x4* q = (const MCEP_GLOBAL u32x4*)(uintptr_t)p;
    const u32x4 r = NT ? __builtin_nontemporal_load(q) : *q;
    return make_uint4(r.x, r.y, r.z, r.w);
}

template <bool NT>
__device__ __forceinline__ void store16(void* p, uint4 v) {
    MCEP_GLOBAL u32x4* q = (MCEP_GLOBAL u32x4*)(uintptr_t)p;
    const u32x4 r = {v.x, v.y, v.z, v.w};
    if (NT) __builtin_nontemporal_store(r, q);
    else *q = r;
}

template <bool NT>
__device__ __forceinline__ void store8(void* p, uint2 v) {
    MCEP_GLOBAL u32x2* q = (MCEP_GLOBAL u32x2*)(uintptr_t)p;
    const u32x2 r = {v.x, v.y};
    if (NT) __builtin_nontemporal_store(r, q);
    else *q = r;
}

__device__ __forceinline__ float load_f32(uint64_t addr) { return *(const MCEP_GLOBAL float*)(uintptr_t)addr; }
__device__ __forceinline__ int load_i32(uint64_t addr) { return *(const MCEP_GLOBAL int*)(uintptr_t)addr; }

// ---------------------------------------------------------------------------
// table writer: the host's per-rank pointer table travels in kernel arguments
// ---------------------------------------------------------------------------
__global__ void table_write_kernel(uint64_t* dst, TableChunk chunk, int n) {
    const int i = threadIdx.x + blockIdx.x * blockDim.x;
    if (i < n) dst[i] = chunk.v[i];
}

// Clears `words` 32-bit words at each of n addresses carried in kernel
// arguments: one launch where a per-rank hipMemsetAsync would be n launches.
__global__ void clear_words_kernel(TableChunk chunk, int n, int words) {
    const int i = threadIdx.x + blockIdx.x * blockDim.x;
    if (i < n * words) ((uint32_t*)chunk.v[i / words])[i % words] = 0u;
}

// ---------------------------------------------------------------------------
// routing layout
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint64_t rank_ptr(const uint64_t* __restrict__ tbl, const RankPtr& p, int field, int R,
                                             int r) {
    return p.base != 0 ? p.base + (uint64_t)((int64_t)r * p.stride) : tbl[field * R + r];
}

// One block per unit (UNIT consecutive (token, k) selections of one rank), one
// selection per thread.  Each index is read exactly once.
//   1. inside a wave, selections naming the same expert are ranked by lane
//      (a 64-bit lane mask per expert in LDS, filled by LDS atomics);
//   2. the waves' per-expert counts are prefix-summed in LDS, which gives
//      every selection its position inside (unit, expert) and the unit its
//      per-expert histogram;
// prefix_kernel then turns the units' histograms into packed-row offsets.
// (A token is expected to name an expert at most once; if it names one twice,
// each occurrence gets its own row, as in the reference kernel, which sends
// once per k: mooncake_ep_kernel.cu:230,273.)
template <int UNIT>
__global__ __launch_bounds__(UNIT) void count_kernel(const uint64_t* __restrict__ tbl, RoutingScratch sc,
                                                      DispatchSource src, int R, int E, int K, int max_tokens,
                                                      int upr) {
    extern __shared__ unsigned long long lds_count[];
    constexpr int NW = UNIT / 64;
    unsigned long long* wmask = lds_count;                     // [NW][E] lanes of the wave that name e
    uint16_t* wpre = (uint16_t*)(lds_count + (size_t)NW * E);  // [NW][E] selections of e in earlier waves

    const int u = blockIdx.x;
    const int r = u / upr, c = u - r * upr;
    const int tid = threadIdx.x, lane = wave_lane();
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int T = src.tokens >= 0 ? src.tokens : (int)tbl[DF_NUM_TOKENS * R + r];
    const int n = T * K;
    const int sel = c * UNIT + tid;                            // index into the rank's [T, K] list

    int64_t e64 = -1;
    if (sel < n) e64 = ((const int64_t*)rank_ptr(tbl, src.topk_idx, DF_TOPK_IDX, R, r))[sel];
    for (int i = tid; i < NW * E; i += UNIT) wmask[i] = 0;
    const bool valid = e64 >= 0 && e64 < (int64_t)E;
    const int e = valid ? (int)e64 : 0;
    __syncthreads();

    // every lane sets its bit in its expert's mask; the mask then tells a lane
    // how many lower lanes of the wave name the same expert
    if (valid) atomicOr(&wmask[wave * E + e], 1ull << lane);
    __syncthreads();
    const int rank_in_wave = valid ? __popcll(wmask[wave * E + e] & ((1ull << lane) - 1ull)) : 0;

    for (int ee = tid; ee < E; ee += UNIT) {
        int run = 0;
#pragma unroll
        for (int w = 0; w < NW; ++w) {
            wpre[w * E + ee] = (uint16_t)run;
            run += __popcll(wmask[w * E + ee]);
        }
        sc.ucount[(int64_t)u * E + ee] = run;
        // the summed plan (big units) also wants the counts expert-major, for the data kernels' sums
        if (UNIT == kBigUnitSelections) sc.ucount_t[(int64_t)ee * kMaxSummedUnits + u] = run;
    }
    __syncthreads();
    if (sel < n) sc.selpos[(int64_t)r * max_tokens * K + sel] = valid ? (int)wpre[wave * E + e] + rank_in_wave : -1;
}

// Units' histograms -> exclusive prefixes over units (source rank ascending,
// then token ascending), recv_count, layout_range and the per-expert counts.
// One wave per expert, a lane per unit (64 at a time, wave-wide scan); the
// prefixes also go to LDS, from which a lane per source rank then reads its
// rank's begin and end.  (A separate launch rather than "the last block of the
// count kernel": the device-scope release that pattern needs writes back each
// XCD's whole L2, which costs more than a launch.)
constexpr int kPrefixWaves = 4;

// The work of one wave for expert ee; pre is the wave's LDS row of U + 1 ints.
__device__ __forceinline__ void prefix_expert(const uint64_t* __restrict__ tbl, const RoutingScratch& sc, int R, int E,
                                              int max_tokens, int upr, int U, int ee, int* pre) {
    const int lane = wave_lane();
    int carry = 0;
    for (int u0 = 0; u0 < U; u0 += 64) {
        const int u = u0 + lane;
        const int c = (u < U) ? sc.ucount[(int64_t)u * E + ee] : 0;
        const int incl = wave_scan_inclusive(c);
        if (u < U) {
            const int excl = carry + incl - c;
            sc.ubegin[(int64_t)u * E + ee] = excl;
            pre[u] = excl;
        }
        carry += __builtin_amdgcn_readlane(incl, 63);
    }
    if (lane == 0) pre[U] = carry;
    // the same wave wrote pre[] and reads it below: a wave's LDS accesses complete in order
    __builtin_amdgcn_wave_barrier();

    const int L = E / R;
    const int64_t RM = (int64_t)R * max_tokens;
    // A block holds RM rows.  Distinct experts per token can never exceed that;
    // rows past it (possible only with repeated experts) are dropped.
    const int cap = (int)(RM < 0x7fffffff ? RM : 0x7fffffff);
    const int q = ee / L, le = ee - q * L;
    const uint64_t recv_x = tbl[DF_RECV_X * R + q];       // 0: the rank takes no part and receives nothing
    const int kept = carry < cap ? carry : cap;
    if (lane == 0) {
        sc.counts[ee] = recv_x ? kept : 0;
        if (recv_x) ((int32_t*)tbl[DF_RECV_COUNT * R + q])[le] = kept;
    }
    if (recv_x == 0) return;
    int64_t* layout_range = (int64_t*)tbl[DF_LAYOUT_RANGE * R + q] + (int64_t)le * R;
    for (int rr = lane; rr < R; rr += 64) {
        int b = pre[rr * upr], b2 = pre[(rr + 1) * upr];
        b = b < cap ? b : cap;
        b2 = b2 < cap ? b2 : cap;
        // count in the low half, begin in the high half; an empty pair is 0
        layout_range[rr] = (b2 > b) ? (((int64_t)b << 32) | (int64_t)(b2 - b)) : 0;
    }
}

__global__ __launch_bounds__(kPrefixWaves * 64) void prefix_kernel(const uint64_t* __restrict__ tbl,
                                                                    RoutingScratch sc, int R, int E, int max_tokens,
                                                                    int upr, int U) {
    extern __shared__ int lds_prefix[];                     // [kPrefixWaves][U + 1]
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int ee = blockIdx.x * kPrefixWaves + wave;
    if (ee >= E) return;
    prefix_expert(tbl, sc, R, E, max_tokens, upr, U, ee, lds_prefix + (size_t)wave * (U + 1));
}

// The packed row of one (token, k) selection, from the routing state, in two
// steps so that callers can put their own gathers next to the one dependent
// load (ubegin) instead of behind it: every lane works on a valid selection
// index (slots >= K redo slot 0's), nothing is loaded under a branch.  `slot`
// is which of the token's K selections the lane works on.
struct SelKey {
    int e;          // global expert (0 when the selection is not valid)
    int q;          // rank that owns it
    int le;         // its index among that rank's experts
    int pos;        // position inside (unit, expert)
    int unit;
    bool valid;
};

struct SelRow {
    int64_t grow;   // row inside the owner's [L, R*max] layout: le * R*max + slot
    int slot;       // row inside the expert's block
    bool ok;
};

__device__ __forceinline__ SelKey selection_key(const int64_t* __restrict__ idx_row, const RoutingScratch& sc, int R,
                                                int E, int K, int max_tokens, const UnitPlan& up, int r, int t,
                                                int slot) {
    const int li = slot < K ? slot : 0;
    const int i = t * K + li;
    const int64_t e64 = idx_row[li];
    const int pos = sc.selpos[(int64_t)r * max_tokens * K + i];
    SelKey k;
    k.valid = slot < K && e64 >= 0 && e64 < (int64_t)E && pos >= 0;
    k.e = k.valid ? (int)e64 : 0;
    const int L = E / R;
    k.q = k.e / L;
    k.le = k.e - k.q * L;
    k.pos = pos;
    k.unit = r * up.per_rank + (i >> up.shift);
    return k;
}

__device__ __forceinline__ SelRow selection_row(const SelKey& k, int ubegin, int R, int max_tokens) {
    const int64_t RM = (int64_t)R * max_tokens;
    SelRow s;
    s.slot = ubegin + k.pos;
    s.grow = (int64_t)k.le * RM + s.slot;
    s.ok = k.valid && s.slot < RM;
    return s;
}

// Summed plan: the begin of (unit, expert) - the rows that earlier units give the expert - added up
// on the fly from the unit counts.  The wave's lanes split into groups of sel_stride() lanes, one
// group per selection of the token; a group's lanes take the earlier units four at a time and the
// group sums up, so every lane of group k ends with selection k's begin.
__device__ __forceinline__ int sel_stride(const UnitPlan& up, int K) {
    if (!up.summed) return 1;                                  // table plan: lane k works on selection k
    const int kp = K <= 1 ? 1 : (K <= 2 ? 2 : (K <= 4 ? 4 : (K <= 8 ? 8 : 16)));
    return 64 / kp;
}

__device__ __forceinline__ int summed_begin(const RoutingScratch& sc, const SelKey& k, const UnitPlan& up, int r, int t,
                                            int K, int j, int lps) {
    const int unit_max = r * up.per_rank + ((t * K + K - 1) >> up.shift);   // wave-uniform bound
    // a lane takes four consecutive units in one 16-byte load; rows of ucount_t are kMaxSummedUnits long
    const int32_t* row = sc.ucount_t + (int64_t)k.e * kMaxSummedUnits;
    int sum = 0;
    for (int base = 0; base < unit_max; base += 4 * lps) {
        const int u = base + 4 * j;
        int4 v = make_int4(0, 0, 0, 0);
        if (u < k.unit) v = *(const int4*)(row + u);
        sum += (u < k.unit ? v.x : 0) + (u + 1 < k.unit ? v.y : 0) + (u + 2 < k.unit ? v.z : 0) +
               (u + 3 < k.unit ? v.w : 0);
    }
    // sum over the group's lanes (4 to 64 of them): inside rows of 16 lanes in the DPP data path
    sum += __builtin_amdgcn_mov_dpp(sum, 0xB1, 0xF, 0xF, true);                  // quad_perm [1,0,3,2]
    sum += __builtin_amdgcn_mov_dpp(sum, 0x4E, 0xF, 0xF, true);                  // quad_perm [2,3,0,1]
    if (lps >= 8) sum += __builtin_amdgcn_mov_dpp(sum, 0x141, 0xF, 0xF, true);   // row_half_mirror
    if (lps >= 16) sum += __builtin_amdgcn_mov_dpp(sum, 0x140, 0xF, 0xF, true);  // row_mirror
    if (lps >= 32) sum += __shfl_xor(sum, 16);
    if (lps >= 64) sum += __shfl_xor(sum, 32);
    return sum;
}

// ---------------------------------------------------------------------------
// fp8 scales: from the pack waves' staging rows into the column-major output
// ---------------------------------------------------------------------------
// Staged scales -> column-major output.  A work item is 64 packed rows of one
// expert times one part of kTransposeGroups scale groups, and a wave takes one
// item: a lane learns its row's source token slot from row_src (left by the
// pack waves), reads that token's scales as contiguous pieces, all in flight at
// once, and stores them so that the wave writes 64 consecutive floats per scale
// group.
//
// Which expert owns the wave's 64-row chunk follows from the per-expert row
// counts alone: every wave scans ceil(count / 64) over the experts (a DPP scan
// per 64 experts) and finds the expert whose chunk range holds its chunk
// number.  The work list therefore holds no more items than there are chunks
// (at most one partly filled chunk per expert), however uneven the routing is.
constexpr int kTransposeGroups = 32;      // scale groups per wave: 128 bytes of staged scales per lane
constexpr int kTransposeWaves = 4;        // waves per block of scale_transpose_kernel

__device__ __forceinline__ void transpose_task(const uint64_t* __restrict__ tbl, const float* __restrict__ scale_stage,
                                               const RoutingScratch& scratch, int R, int E, int G, int max_tokens,
                                               int parts, int task) {
    const int lane = wave_lane();
    const int target = task / parts, part = task - target * parts;

    // chunk ranges of the experts: expert e owns chunks [begin_e, begin_e + ceil(count_e / 64))
    constexpr int kPre = 4;               // 64-expert pieces whose counts are loaded side by side
    int pre_counts[kPre];
#pragma unroll
    for (int j = 0; j < kPre; ++j) {
        const int ee = j * 64 + lane;
        pre_counts[j] = 0;
        if (ee < E) pre_counts[j] = scratch.counts[ee];
    }
    int carry = 0, e = -1, chunk = 0, count = 0;
    auto piece = [&](int e0, int c) {
        const int n = (c + 63) >> 6;
        const int incl = wave_scan_inclusive(n);
        const int begin = carry + incl - n;
        const unsigned long long owns = __ballot(n > 0 && begin <= target && target < begin + n);
        if (owns) {
            const int l = __builtin_ctzll(owns);
            e = e0 + l;
            chunk = target - __builtin_amdgcn_readlane(begin, l);
            count = __builtin_amdgcn_readlane(c, l);
        }
        carry += __builtin_amdgcn_readlane(incl, 63);
    };
#pragma unroll
    for (int j = 0; j < kPre; ++j)
        if (j * 64 < E) piece(j * 64, pre_counts[j]);
    for (int e0 = kPre * 64; e0 < E; e0 += 64) {
        const int ee = e0 + lane;
        int c = 0;
        if (ee < E) c = scratch.counts[ee];
        piece(e0, c);
    }
    if (e < 0) return;                    // beyond the last chunk
    e = __builtin_amdgcn_readfirstlane(e);
    chunk = __builtin_amdgcn_readfirstlane(chunk);
    count = __builtin_amdgcn_readfirstlane(count);

    const int L = E / R, q = e / L, le = e - q * L;
    const int64_t RM = (int64_t)R * max_tokens;
    const int g0 = part * kTransposeGroups;
    const int n = (g0 + kTransposeGroups < G ? g0 + kTransposeGroups : G) - g0;
    const int row = chunk * 64 + lane;
    const bool valid = row < count;
    // the output address and the row's source slot, side by side
    float* out = (float*)tbl[DF_RECV_SCALES * R + q];
    int slot = 0;
    if (valid) slot = scratch.row_src[(int64_t)e * RM + row];
    const float* sp = scale_stage + (int64_t)slot * G + g0;
    float* dp = out + ((int64_t)le * G + g0) * RM + row;
    if ((G & 3) == 0) {
        // 16-byte loads, all issued before the first store
        constexpr int B = kTransposeGroups / 4;
        float4 v[B];
#pragma unroll
        for (int j = 0; j < B; ++j) v[j] = (4 * j < n) ? *(const float4*)(sp + 4 * j) : make_float4(0, 0, 0, 0);
        if (valid) {
#pragma unroll
            for (int j = 0; j < B; ++j) {
                if (4 * j >= n) break;
                dp[(int64_t)(4 * j + 0) * RM] = v[j].x;
                dp[(int64_t)(4 * j + 1) * RM] = v[j].y;
                dp[(int64_t)(4 * j + 2) * RM] = v[j].z;
                dp[(int64_t)(4 * j + 3) * RM] = v[j].w;
            }
        }
    } else if (valid) {
        for (int g = 0; g < n; ++g) dp[(int64_t)g * RM] = sp[g];
    }
}

__global__ __launch_bounds__(kTransposeWaves * 64) void scale_transpose_kernel(
    const uint64_t* __restrict__ tbl, const float* __restrict__ scale_stage, RoutingScratch scratch, int R, int E,
    int G, int max_tokens, int parts, int total_tasks) {
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * kTransposeWaves + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    transpose_task(tbl, scale_stage, scratch, R, E, G, max_tokens, parts, task);
}

// ---------------------------------------------------------------------------
// dispatch pack
// ---------------------------------------------------------------------------
constexpr int kMaxPackWaves = 8;     // waves per block the launcher may choose

// One wave per (token, 1024-element slab).  Lanes 0..K-1 fetch the K resolved
// destinations; the row slab is read once, quantised in registers and stored
// K times.
struct PackDest {
    uint64_t row;     // byte address of the destination row, 0 = no store
};

// The lanes that work on selection k (lane k, or a group of sel_stride() lanes under the summed
// plan) turn it into destination addresses; callers read them from lane k * sel_stride().  The
// slab-0 wave of a token also records the row's source: src_info for the caller and row_src for the
// scale transposition.
template <bool FP8>
__device__ __forceinline__ PackDest pack_destination(const uint64_t* __restrict__ tbl, const RoutingScratch& sc,
                                                     const int64_t* __restrict__ idx_row, int R, int E, int K,
                                                     int max_tokens, int H, const UnitPlan& up, int r, int t,
                                                     int slab, int lane) {
    const int stride = sel_stride(up, K);
    const int slot = lane / stride, j = lane - slot * stride;
    const SelKey k = selection_key(idx_row, sc, R, E, K, max_tokens, up, r, t, slot);
    // the dependent gathers, side by side; the table's come first because the summed begin waits for
    // its own loads inside, and whatever is issued after that wait is a round trip later
    const uint64_t base = tbl[DF_RECV_X * R + k.q];
    const uint64_t info = (slab == 0) ? tbl[DF_SRC_INFO * R + k.q] : 0;
    const int ub = up.summed ? summed_begin(sc, k, up, r, t, K, j, stride) : sc.ubegin[(int64_t)k.unit * E + k.e];
    const SelRow s = selection_row(k, ub, R, max_tokens);
    PackDest d = {0};
    const int64_t RM = (int64_t)R * max_tokens;
    // where the selection went, for a combine of this dispatch's handle: expert * R*max + row, or -1
    if (slab == 0 && j == 0 && slot < K)
        sc.selrow[((int64_t)r * max_tokens + t) * K + slot] = (s.ok && base != 0) ? (int)((int64_t)k.e * RM + s.slot) : -1;
    if (s.ok && base != 0) {
        d.row = base + (uint64_t)s.grow * (uint64_t)H * (FP8 ? 1 : 2);
        if (slab == 0 && j == 0) {
            ((int32_t*)info)[s.grow] = t;
            sc.row_src[(int64_t)k.e * RM + s.slot] = r * max_tokens + t;
        }
    }
    return d;
}

// token row and top-k row of a wave's token; false when the slot is beyond the rank's token count
__device__ __forceinline__ bool pack_token(const uint64_t* __restrict__ tbl, const DispatchSource& src, int R, int K,
                                           int H, int r, int t, const char** xrow, const int64_t** idx_row) {
    const int T = src.tokens >= 0 ? src.tokens : (int)tbl[DF_NUM_TOKENS * R + r];
    if (t >= T) return false;
    *xrow = (const char*)rank_ptr(tbl, src.x, DF_X, R, r) + (int64_t)t * H * 2;
    *idx_row = (const int64_t*)rank_ptr(tbl, src.topk_idx, DF_TOPK_IDX, R, r) + (int64_t)t * K;
    return true;
}

// Slabs owned by XCDs.  Blocks go round-robin over the 8 XCDs, each with an L2 of its own, so which block
// works on which (token, slab) decides which L2 sees a slab's column-major scales: here every scale of a
// 128-element group passes through one XCD's L2 only, whichever token it belongs to, and all XCDs move
// through the tokens together.  slabs = 8a + b: slab j of the first 8a belongs to XCD j % 8 for every
// token; of the other b, slab 8a + c belongs to m = 8 / b XCDs, which share the tokens of the first
// b * m residues modulo 8 between them, and the 8 - b * m XCDs left over take one of the remaining
// residues each, for all b slabs.  Every XCD then has P = slabs (token residue, slab) pairs per eight
// consecutive tokens, so the work is even.  `w` is the wave's number among those of its XCD (`xcd` =
// block index % 8); false when it is beyond the last token.
__device__ __forceinline__ bool xcd_owned_task(int xcd, int w, int slabs, int tokens, int* n_out, int* s_out) {
    const int P = slabs;
    const int o = w / P, i = w - o * P;
    const int b = slabs & 7, a8 = slabs - b;
    int rho, s;
    if (i < a8) {
        rho = i & 7;
        s = xcd + (i & ~7);
    } else {
        const int ii = i - a8, m = 8 / b, own = b * m;
        if (xcd < own) {
            rho = xcd % m + m * ii;
            s = a8 + xcd / m;
        } else {
            rho = xcd;                  // own + (xcd - own)
            s = a8 + ii;
        }
    }
    const int n = o * 8 + rho;
    *n_out = n;
    *s_out = s;
    return n < tokens;
}

// blocks a launch needs for `tokens` tokens of `slabs` slabs each under that order, wpb waves per block
static long long xcd_owned_blocks(long long tokens, int slabs, int wpb) {
    const long long octets = (tokens + 7) / 8;
    return (octets * slabs + wpb - 1) / wpb * 8;
}

// A lane's 16 consecutive bf16 elements (two 16-byte pieces) -> 16 fp8 e4m3 bytes; a 128-element
// scale group is 8 lanes, whose amax (floor 1e-4, mooncake_ep_kernel.cu:233-264) every lane of
// the group ends up with.  *scale_inv is the group's stored scale.
//   NATIVE  false: the arithmetic of the reference's PyTorch statement as CPU PyTorch runs it,
//           `448.0 / amax` = reciprocal times 448 and `amax / 448.0` a true division
//           (mooncake_ep_buffer.py:699-702); true: the reference kernel's own, an IEEE
//           quotient 448 / amax and amax * (1 / 448) (mooncake_ep_kernel.cu:184, :252).
template <bool NATIVE>
__device__ __forceinline__ uint4 quantise16(uint4 a, uint4 b, float* scale_inv) {
    float f[16];
    const uint32_t u[8] = {a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        f[2 * j] = bf16_lo(u[j]);
        f[2 * j + 1] = bf16_hi(u[j]);
    }
    float amax = 1e-4f;
#pragma unroll
    for (int j = 0; j < 16; ++j) amax = fmaxf(amax, fabsf(f[j]));
    amax = group_max<8>(amax);
    // every division here is the compiler's correctly rounded sequence
    const float scale = NATIVE ? 448.0f / amax : (1.0f / amax) * 448.0f;
    *scale_inv = NATIVE ? amax * (1.0f / 448.0f) : amax / 448.0f;
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j] * scale, f[4 * j + 1] * scale, 0, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j + 2] * scale, f[4 * j + 3] * scale, w, true);
        o[j] = (uint32_t)w;
    }
    return make_uint4(o[0], o[1], o[2], o[3]);
}

// fp8: a lane owns 16 consecutive elements (32 B in, 16 B out), a 128-element
// scale group is 8 lanes.  The group's scales go to the token's row of
// scale_stage (contiguous); scale_transpose_kernel moves them into the
// column-major output with coalesced stores (writing them there from here would
// be 4-byte stores 16 KB apart).
//   NATIVE  which of the reference's two statements of the scale arithmetic (see quantise16)
template <bool NTL, bool NATIVE, bool NTS>
__global__ __launch_bounds__(512) void pack_fp8_kernel(const uint64_t* __restrict__ tbl,
                                                        RoutingScratch sc, DispatchSource src,
                                                        float* __restrict__ scale_stage, int R, int E, int K,
                                                        int max_tokens, int H, UnitPlan up, int slabs, int Tgrid,
                                                        int total_tasks) {
    const int lane = wave_lane();
    int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    if (up.carried) {
        // the first E waves of the launch do the prefix pass (it needs the unit counts only)
        __shared__ int lds_pre[kMaxPackWaves * (kMaxSummedUnits + 1)];
        if (task < E) {
            prefix_expert(tbl, sc, R, E, max_tokens, up.per_rank, up.total, task,
                          lds_pre + (threadIdx.x >> 6) * (kMaxSummedUnits + 1));
            return;
        }
        task -= E;
    }
    const int n = task / slabs, s = task - n * slabs;
    const int r = n / Tgrid, t = n - r * Tgrid;
    const char* xtok;
    const int64_t* idx_row;
    if (!pack_token(tbl, src, R, K, H, r, t, &xtok, &idx_row)) return;

    const int elem0 = s * 1024 + lane * 16;
    const bool active = elem0 < H;
    const char* xrow = xtok + (int64_t)(active ? elem0 : 0) * 2;
    uint4 a = make_uint4(0, 0, 0, 0), b = a;
    if (active) {
        a = load16<NTL>(xrow);
        b = load16<NTL>(xrow + 16);
    }
    const PackDest dst = pack_destination<true>(tbl, sc, idx_row, R, E, K, max_tokens, H, up, r, t, s, lane);
    const int sel_lanes = sel_stride(up, K);   // selection k's destination sits in lane k * sel_lanes

    float scale_inv;
    const uint4 out = quantise16<NATIVE>(a, b, &scale_inv);
    if (active && (lane & 7) == 0)
        scale_stage[((int64_t)r * max_tokens + t) * (H >> 7) + (elem0 >> 7)] = scale_inv;

    for (int k = 0; k < K; ++k) {
        const uint64_t row = read_lane_u64(dst.row, k * sel_lanes);
        if (row == 0) continue;
        if (active) store16<NTS>((void*)(row + elem0), out);
    }
}

// bf16: plain row copy, two unit-stride 16-byte pieces per lane.
template <bool NTL, bool NTS>
__global__ __launch_bounds__(512) void pack_bf16_kernel(const uint64_t* __restrict__ tbl,
                                                         RoutingScratch sc, DispatchSource src,
                                                         float* __restrict__ /*scale_stage*/, int R, int E, int K,
                                                         int max_tokens, int H, UnitPlan up, int slabs, int Tgrid,
                                                         int total_tasks) {
    const int lane = wave_lane();
    int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    if (up.carried) {
        // the first E waves of the launch do the prefix pass (it needs the unit counts only)
        __shared__ int lds_pre[kMaxPackWaves * (kMaxSummedUnits + 1)];
        if (task < E) {
            prefix_expert(tbl, sc, R, E, max_tokens, up.per_rank, up.total, task,
                          lds_pre + (threadIdx.x >> 6) * (kMaxSummedUnits + 1));
            return;
        }
        task -= E;
    }
    const int n = task / slabs, s = task - n * slabs;
    const int r = n / Tgrid, t = n - r * Tgrid;
    const char* xbase;
    const int64_t* idx_row;
    if (!pack_token(tbl, src, R, K, H, r, t, &xbase, &idx_row)) return;

    int64_t off[2];
    bool active[2];
    uint4 v[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int elem = s * 1024 + p * 512 + lane * 8;
        active[p] = elem < H;
        off[p] = (int64_t)elem * 2;
        v[p] = make_uint4(0, 0, 0, 0);
        if (active[p]) v[p] = load16<NTL>(xbase + off[p]);
    }
    const PackDest dst = pack_destination<false>(tbl, sc, idx_row, R, E, K, max_tokens, H, up, r, t, s, lane);
    const int sel_lanes = sel_stride(up, K);   // selection k's destination sits in lane k * sel_lanes

    for (int k = 0; k < K; ++k) {
        const uint64_t row = read_lane_u64(dst.row, k * sel_lanes);
        if (row == 0) continue;
#pragma unroll
        for (int p = 0; p < 2; ++p)
            if (active[p]) store16<NTS>((void*)(row + off[p]), v[p]);
    }
}

// ---------------------------------------------------------------------------
// dispatch of a small world in one launch
// ---------------------------------------------------------------------------
// When the whole world names a few thousand selections (a decode step of one rank, or of a few), the
// three launches above cost more than the bytes they move: each is close to the floor of an empty
// kernel.  Here every wave rebuilds the routing it needs by itself, from the ranks' index lists, so one
// launch does everything - as the reference's dispatch is one launch (mooncake_ep_kernel.cu:138-470).
// The row of a selection is the number of earlier selections (source rank ascending, then token, then
// k) that name the same expert: a data wave reads the lists of the earlier ranks and its own rank's up
// to its token (16-byte loads, two entries per lane, a few KB out of L2) and counts matches for its
// token's K experts at once.  The first E waves count one expert each over the whole lists and write
// recv_count and layout_range.  fp8 scales go straight into the column-major layout (4-byte stores 16 KB
// apart: costly for a large world, nothing next to a launch here).  The rank table travels in the
// kernel's arguments, so there is no table to upload; nothing is shared between waves, no LDS, no atomics.
// The slab-0 wave of a token leaves selrow for a combine of the same handle.
typedef long long i64x2 __attribute__((ext_vector_type(2)));

// counts, per lane, the entries of list[0, n) that equal each of ek[0..KMAX): list and n are wave-uniform;
// entries outside [0, E) equal nothing (targets are in [0, E) or -2)
template <int KMAX>
__device__ __forceinline__ void count_list(uint64_t list, int n, int E, const int (&ek)[KMAX], int (&cnt)[KMAX],
                                           int lane) {
    constexpr int kDepth = 4;             // 16-byte loads in flight per lane
    static_assert(kDepth * 128 == kSmallListRound, "the host prices a world in rounds of this many entries");
    if ((list & 8) != 0 && n > 0) {
        // a list that starts in the middle of a 16-byte unit (rank r's slice of a rank-major tensor with an
        // odd number of entries per rank): its first entry by itself, pairs from there
        if (lane == 0) {
            const int64_t v = *(const MCEP_GLOBAL int64_t*)(uintptr_t)list;
            const int k0 = (uint64_t)v < (uint64_t)E ? (int)v : -1;
#pragma unroll
            for (int k = 0; k < KMAX; ++k) cnt[k] += k0 == ek[k] ? 1 : 0;
        }
        list += 8;
        n -= 1;
    }
    for (int base = 0; base < n; base += kDepth * 128) {
        i64x2 v[kDepth];
#pragma unroll
        for (int j = 0; j < kDepth; ++j) {
            const int i = base + j * 128 + 2 * lane;
            v[j] = i64x2{-1, -1};
            if (i + 1 < n) v[j] = *(const MCEP_GLOBAL i64x2*)(uintptr_t)(list + (uint64_t)i * 8);
            else if (i < n) v[j].x = *(const MCEP_GLOBAL int64_t*)(uintptr_t)(list + (uint64_t)i * 8);
        }
#pragma unroll
        for (int j = 0; j < kDepth; ++j) {
            const int k0 = (uint64_t)v[j].x < (uint64_t)E ? (int)v[j].x : -1;
            const int k1 = (uint64_t)v[j].y < (uint64_t)E ? (int)v[j].y : -1;
#pragma unroll
            for (int k = 0; k < KMAX; ++k) cnt[k] += (k0 == ek[k] ? 1 : 0) + (k1 == ek[k] ? 1 : 0);
        }
    }
}

__device__ __forceinline__ int wave_total(int v) { return __builtin_amdgcn_readlane(wave_scan_inclusive(v), 63); }

// recv_count and layout_range of expert ee, by one wave: its selections in every rank's list
__device__ __forceinline__ void small_expert(const SmallTable& tb, int R, int E, int K, int max_tokens, int ee) {
    const int lane = wave_lane();
    const int L = E / R, q = ee / L, le = ee - q * L;
    const int64_t RM = (int64_t)R * max_tokens;
    const int cap = (int)(RM < 0x7fffffff ? RM : 0x7fffffff);   // rows past a block's capacity are dropped
    const int target[1] = {ee};
    int run = 0, mine_b = 0, mine_e = 0;
    for (int rr = 0; rr < R; ++rr) {
        int c[1] = {0};
        count_list<1>(tb.v[DF_TOPK_IDX * R + rr], (int)tb.v[DF_NUM_TOKENS * R + rr] * K, E, target, c, lane);
        const int total = wave_total(c[0]);
        if (lane == rr) {
            mine_b = run;
            mine_e = run + total;
        }
        run += total;
    }
    const uint64_t recv_x = tb.v[DF_RECV_X * R + q];              // 0: the rank takes no part and receives nothing
    if (recv_x == 0) return;
    if (lane == 0) ((int32_t*)tb.v[DF_RECV_COUNT * R + q])[le] = run < cap ? run : cap;
    if (lane < R) {
        const int b = mine_b < cap ? mine_b : cap, b2 = mine_e < cap ? mine_e : cap;
        // count in the low half, begin in the high half; an empty pair is 0
        ((int64_t*)tb.v[DF_LAYOUT_RANGE * R + q])[(int64_t)le * R + lane] =
            (b2 > b) ? (((int64_t)b << 32) | (int64_t)(b2 - b)) : 0;
    }
}

template <int KMAX, bool FP8, bool NATIVE>
__global__ __launch_bounds__(256) void dispatch_small_kernel(SmallTable tb, int32_t* __restrict__ selrow, int R, int E,
                                                              int K, int max_tokens, int H, int slabs, int Tgrid,
                                                              int total_tasks) {
    const int lane = wave_lane();
    int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    if (task < E) {
        small_expert(tb, R, E, K, max_tokens, task);
        return;
    }
    task -= E;
    const int n = task / slabs, s = task - n * slabs;
    const int r = n / Tgrid, t = n - r * Tgrid;
    if (t >= (int)tb.v[DF_NUM_TOKENS * R + r]) return;
    const char* xtok = (const char*)tb.v[DF_X * R + r] + (int64_t)t * H * 2;
    const uint64_t own_list = tb.v[DF_TOPK_IDX * R + r];

    // the payload loads first: everything below hides behind them
    constexpr int kSlabBytes = 2048;
    const int elem0 = s * 1024 + lane * (FP8 ? 16 : 8);          // bf16: the first of two 512-element halves
    uint4 a = make_uint4(0, 0, 0, 0), b = a;
    bool act_a, act_b;
    if (FP8) {
        act_a = act_b = elem0 < H;
        if (act_a) {
            a = load16<false>(xtok + (int64_t)elem0 * 2);
            b = load16<false>(xtok + (int64_t)elem0 * 2 + 16);
        }
    } else {
        act_a = elem0 < H;
        act_b = elem0 + 512 < H;
        if (act_a) a = load16<false>(xtok + (int64_t)elem0 * 2);
        if (act_b) b = load16<false>(xtok + (int64_t)elem0 * 2 + kSlabBytes / 2);
    }

    // the token's K experts, one per lane, and each as a wave-uniform target
    const int li = lane < K ? lane : 0;
    const int64_t e64 = *(const MCEP_GLOBAL int64_t*)(uintptr_t)(own_list + (uint64_t)((int64_t)t * K + li) * 8);
    const bool valid = lane < K && (uint64_t)e64 < (uint64_t)E;
    const int e = valid ? (int)e64 : 0;
    const int L = E / R, q = e / L, le = e - q * L;
    // the owner's tensors: asked for as soon as the expert is known, needed after the count
    const uint64_t base = tb.v[DF_RECV_X * R + q];
    const uint64_t info = tb.v[DF_SRC_INFO * R + q];
    const uint64_t sbase = FP8 ? tb.v[DF_RECV_SCALES * R + q] : 0;
    const int target = valid ? e : -2;
    int ek[KMAX], cnt[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        ek[k] = __builtin_amdgcn_readlane(target, k);
        cnt[k] = 0;
    }
    // selections of earlier ranks, then of this rank's earlier tokens
    for (int rr = 0; rr < r; ++rr)
        count_list<KMAX>(tb.v[DF_TOPK_IDX * R + rr], (int)tb.v[DF_NUM_TOKENS * R + rr] * K, E, ek, cnt, lane);
    count_list<KMAX>(own_list, t * K, E, ek, cnt, lane);
    int slot = 0;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        const int total = wave_total(cnt[k]);
        // plus the token's own earlier selections of the same expert (a repeated expert gets a row per occurrence)
        if (lane == k) slot += total;
        if (lane > k && ek[k] == target) slot += 1;
    }
    const int64_t RM = (int64_t)R * max_tokens;
    const bool ok = valid && slot < RM && base != 0;
    const int64_t grow = (int64_t)le * RM + slot;
    uint64_t row = 0, srow = 0;
    if (ok) {
        row = base + (uint64_t)grow * (uint64_t)H * (FP8 ? 1 : 2);
        if (FP8) srow = sbase + (uint64_t)((int64_t)le * (H >> 7) * RM + slot) * 4;
    }
    if (s == 0 && lane < K) {
        // where the selection went, for a combine of this dispatch's handle: expert * R*max + row, or -1
        selrow[((int64_t)r * max_tokens + t) * K + lane] = ok ? (int)((int64_t)e * RM + slot) : -1;
        if (ok) ((int32_t*)info)[grow] = t;
    }

    if (FP8) {
        float scale_inv;
        const uint4 out = quantise16<NATIVE>(a, b, &scale_inv);
        const uint64_t goff = (uint64_t)((int64_t)(elem0 >> 7) * RM) * 4;
        for (int k = 0; k < K; ++k) {
            const uint64_t dst = read_lane_u64(row, k);
            if (dst == 0) continue;
            if (act_a) store16<false>((void*)(dst + elem0), out);
            if (act_a && (lane & 7) == 0) *(MCEP_GLOBAL float*)(uintptr_t)(read_lane_u64(srow, k) + goff) = scale_inv;
        }
    } else {
        for (int k = 0; k < K; ++k) {
            const uint64_t dst = read_lane_u64(row, k);
            if (dst == 0) continue;
            if (act_a) store16<false>((void*)(dst + (int64_t)elem0 * 2), a);
            if (act_b) store16<false>((void*)(dst + (int64_t)elem0 * 2 + kSlabBytes / 2), b);
        }
    }
}

// ---------------------------------------------------------------------------
// combine
// ---------------------------------------------------------------------------
// Handle -> routes.  One wave per (expert, token-owner rank) pair: the packed
// rows [begin, begin + count) of that pair carry the owner's token indices in
// src_info; each row finds its k in the token's top-k list and leaves the
// row's address and weight there.  Experts on ranks the owner sees as
// inactive, and rows of ranks that take no part, leave no route.
template <bool PACKED>
__global__ __launch_bounds__(256) void resolve_kernel(const uint64_t* __restrict__ tbl,
                                                       CombineRoute* __restrict__ routes, uint32_t stamp, int R,
                                                       int E, int K, int H, int max_tokens, int total_tasks) {
    const int lane = wave_lane();
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    const int e = task / R, r = task - e * R;
    const int L = E / R, q = e / L, le = e - q * L;
    const int T = (int)tbl[CF_NUM_TOKENS * R + r];
    if (T == 0) return;
    const uint64_t base = tbl[CF_X * R + q];
    const int64_t* lrp = (const int64_t*)tbl[CF_LAYOUT_RANGE * R + q];
    const int32_t* sip = (const int32_t*)tbl[CF_SRC_INFO * R + q];
    if (base == 0 || lrp == nullptr || sip == nullptr) return;
    if (((const int32_t*)tbl[CF_ACTIVE * R + r])[q] == 0) return;   // skip experts on inactive ranks
    const int64_t RM = (int64_t)R * max_tokens;
    const int64_t lr = lrp[(int64_t)le * R + r];
    const int count = (int)(lr & 0xffffffffll), begin = (int)(lr >> 32);
    if (begin < 0 || count <= 0 || (int64_t)begin + count > RM) return;   // empty or malformed
    sip += (int64_t)le * RM + begin;
    const int64_t* idx = (const int64_t*)tbl[CF_TOPK_IDX * R + r];
    const float* wts = (const float*)tbl[CF_TOPK_W * R + r];
    CombineRoute* rts = routes + (int64_t)r * max_tokens * K;
    const uint64_t row0 = base + (uint64_t)((int64_t)le * RM + begin) * H * 2;
    for (int i = lane; i < count; i += 64) {
        const int t = sip[i];
        if (t < 0 || t >= T) continue;
        for (int k0 = 0; k0 < K; k0 += 4) {
            int64_t cand[4];
            float wt[4];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const bool in = k0 + j < K;
                cand[j] = in ? idx[(int64_t)t * K + k0 + j] : -1;
                wt[j] = in ? wts[(int64_t)t * K + k0 + j] : 0.0f;
            }
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                if (cand[j] == (int64_t)e) {
                    CombineRoute rt;
                    rt.src = PACKED ? (((uint64_t)e << 32) | (uint32_t)(begin + i)) : row0 + (uint64_t)i * H * 2;
                    rt.weight = wt[j];
                    rt.stamp = stamp;
                    rts[(int64_t)t * K + k0 + j] = rt;
                }
            }
        }
    }
}

// Where combine finds the row of selection `lane` of token (r, t) when the handle is the last
// dispatch's: the pack kernel left expert * R*max + row in selrow (-1: the selection went nowhere);
// the row counts only while topk_idx still names that expert.
// One load away from the payload when the ranks' row tensors are evenly spaced (the address then comes
// from kernel arguments), two otherwise (rank table).  `live` is loaded but not waited for: whether
// the owner is active only decides the weight, so the caller issues its payload loads first.
struct DirectRow {
    uint64_t base;      // the owner's row tensor, 0: none
    int64_t grow;       // row inside the owner's [L, R*max] layout
    int e, q, le, slot;
    int live;           // the token owner's active_ranks entry for the expert's rank
    bool has;
};

__device__ __forceinline__ DirectRow direct_row(const uint64_t* __restrict__ tbl, const RoutingScratch& sc,
                                                const RankPtr& x, const RankPtr& topk_idx, int R, int E, int K,
                                                int max_tokens, int r, int t, int lane) {
    const int RM = R * max_tokens;
    const int L = E / R;
    const uint64_t active = tbl[CF_ACTIVE * R + r];
    const int li = lane < K ? lane : 0;
    // The selection as combine is given it, next to the row the dispatch left (two independent loads):
    // combine reads topk_idx itself and skips what is negative there (mooncake_ep_kernel.cu:719-732), so
    // a selection masked - or pointed elsewhere - after the dispatch has no row.
    const int64_t now = ((const MCEP_GLOBAL int64_t*)(uintptr_t)rank_ptr(tbl, topk_idx, CF_TOPK_IDX, R, r))[(int64_t)t * K + li];
    const int sr = sc.selrow[((int64_t)r * max_tokens + t) * K + li];
    DirectRow d;
    d.has = lane < K && sr >= 0 && now == (int64_t)(sr / RM);
    d.e = d.has ? sr / RM : 0;
    d.slot = d.has ? sr - d.e * RM : 0;
    d.q = d.e / L;
    d.le = d.e - d.q * L;
    d.base = rank_ptr(tbl, x, CF_X, R, d.q);
    d.grow = (int64_t)d.le * RM + d.slot;
    // `live` is asked for last, behind whatever the base address had to wait for (a table entry when the
    // ranks' tensors are not evenly spaced): loads complete in order for a waiting wave, so a load issued
    // before that wait would be waited for as well, ahead of the payload
    int q_late = d.q;
    asm volatile("" : "+v"(q_late) : "v"((uint32_t)d.base), "v"((uint32_t)(d.base >> 32)));
    d.live = load_i32(active + (uint64_t)q_late * 4);
    return d;
}

// One wave per (token, slab of CH * 512 elements).  Lanes 0..K-1 find the K
// source rows (a masked, inactive or unknown selection reads a zero row with
// weight 0, which leaves the fp32 accumulator unchanged), then every lane
// issues all KMAX * CH 16-byte loads before the first multiply-add.
//   DIRECT   the handle is the one the last dispatch produced: rows come from
//            that dispatch's routing state, no resolve kernel has run;
//   !DIRECT  rows come from the routes the resolve kernel left.
template <int KMAX, int CH, bool NTL, bool NTS, bool DIRECT>
__global__ __launch_bounds__(512) void reduce_kernel(const uint64_t* __restrict__ tbl,
                                                      const CombineRoute* __restrict__ routes, uint32_t stamp,
                                                      RoutingScratch sc, CombineSource cs,
                                                      const void* __restrict__ zero_row, int R, int E, int K,
                                                      int max_tokens, int H, int slabs, int Tgrid,
                                                      int total_tasks) {
    const int lane = wave_lane();
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    const int n = task / slabs, s = task - n * slabs;
    const int r = n / Tgrid, t = n - r * Tgrid;
    const int T = cs.tokens >= 0 ? cs.tokens : (int)tbl[CF_NUM_TOKENS * R + r];
    char* orow = (char*)rank_ptr(tbl, cs.out, CF_OUT, R, r) + (int64_t)t * H * 2;

    uint64_t src = (uint64_t)zero_row;
    float w = 0.0f;
    int live = 1;
    if (DIRECT) {
        // the caller's top-k rows exist only for t < T
        if (t >= T) return;
        const uint64_t w_row = rank_ptr(tbl, cs.topk_weights, CF_TOPK_W, R, r) + (uint64_t)((int64_t)t * K) * 4;
        const float wl = load_f32(w_row + (uint64_t)(lane < K ? lane : 0) * 4);
        const DirectRow d = direct_row(tbl, sc, cs.x, cs.topk_idx, R, E, K, max_tokens, r, t, lane);
        if (d.has && d.base != 0) {
            src = d.base + (uint64_t)d.grow * (uint64_t)H * 2;
            w = wl;
        }
        live = d.live;         // not looked at before the payload loads are on their way
    } else {
        // A token slot beyond the rank's count has only stale routes (zero
        // rows); it is computed like any other and dropped at the store, so
        // that no wave waits for the rank's token count before its loads.
        uint4 rt = make_uint4(0, 0, 0, 0);
        if (lane < K) rt = *(const uint4*)(routes + ((int64_t)r * max_tokens + t) * K + lane);
        asm volatile("" : "+v"(rt.x), "+v"(rt.y), "+v"(rt.z), "+v"(rt.w));   // one 16-byte load, no branch on the stamp
        const bool ok = (lane < K) && (rt.w == stamp);
        src = ok ? (((uint64_t)rt.y << 32) | rt.x) : (uint64_t)zero_row;
        w = ok ? __uint_as_float(rt.z) : 0.0f;
    }

    int64_t off[CH];
    bool active[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        const int elem = (s * CH + c) * 512 + lane * 8;
        active[c] = elem < H;
        off[c] = active[c] ? (int64_t)elem * 2 : 0;
    }

    uint4 v[KMAX][CH];
    float wk[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        const uint64_t p = read_lane_u64(src, k);
#pragma unroll
        for (int c = 0; c < CH; ++c) v[k][c] = load16<NTL>((const void*)(p + off[c]));
    }
    // An expert on a rank the token's owner sees as inactive is skipped (mooncake_ep_kernel.cu:729-732):
    // its row was fetched before that was known, so the row is dropped here (it may hold anything) and
    // the weight is zero, as for a selection that went nowhere.
    if (DIRECT && live == 0) w = 0.0f;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        wk[k] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w), k));
        if (DIRECT && __builtin_amdgcn_readlane(live, k) == 0) {
#pragma unroll
            for (int c = 0; c < CH; ++c) v[k][c] = make_uint4(0, 0, 0, 0);
        }
    }

    if (t >= T) return;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        float acc[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
#pragma unroll
        for (int k = 0; k < KMAX; ++k) {
            const uint32_t u[4] = {v[k][c].x, v[k][c].y, v[k][c].z, v[k][c].w};
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[2 * j] = __builtin_fmaf(bf16_lo(u[j]), wk[k], acc[2 * j]);
                acc[2 * j + 1] = __builtin_fmaf(bf16_hi(u[j]), wk[k], acc[2 * j + 1]);
            }
        }
        uint32_t o[4];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
            typedef float f2 __attribute__((ext_vector_type(2)));
            const f2 pr = {acc[2 * j], acc[2 * j + 1]};
            const bf2 cv = __builtin_convertvector(pr, bf2);   // v_cvt_pk_bf16_f32: round to nearest even
            o[j] = __builtin_bit_cast(uint32_t, cv);
        }
        if (active[c]) store16<NTS>(orow + off[c], make_uint4(o[0], o[1], o[2], o[3]));
    }
}

// ---------------------------------------------------------------------------
// consumer of the packed layout: cast back to bf16 (+ per-expert factor)
// ---------------------------------------------------------------------------
__device__ __forceinline__ uint32_t pack_bf16_rne(float a, float b) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    const f2 pr = {a, b};
    return __builtin_bit_cast(uint32_t, __builtin_convertvector(pr, bf2));   // v_cvt_pk_bf16_f32
}

// x rounded to bf16 (nearest even) and kept as an f32: the conversion of the pair (0, x) leaves bf16(x) in
// the upper half of the register, which is that value's f32 encoding - one instruction where packing two
// values and unpacking them again takes three for two
__device__ __forceinline__ float round_bf16(float x) {
    return __uint_as_float(pack_bf16_rne(0.0f, x));
}

// out = bf16(bf16(a * s) * f), both roundings to nearest even, for a pair
__device__ __forceinline__ uint32_t scale_round_twice(float a, float b, float s, float f) {
    return pack_bf16_rne(round_bf16(a * s) * f, round_bf16(b * s) * f);
}

// Combine straight from the packed layout dispatch wrote: what cast_back_kernel followed by
// reduce_kernel computes, without the bf16 expert rows in between.  Every source row is turned, in
// registers, into exactly what the consumer would have stored -
//     bf16( bf16( f32(fp8) * scale ) * factor[expert] ),  both roundings to nearest even
// (per_token_cast_back, mooncake-wheel/tests/ep_test_utils.py:50-53, and the mock expert of
// mooncake-ep/tests/test_ep_grid.py:168-173; a bf16 payload takes the factor alone) - and then
// enters the fp32 fused multiply-add chain in k order (mooncake_ep_kernel.cu:711-753), so the result
// is bit for bit that of the two-kernel path.
//
// One wave per (token, slab): 1024 elements of an fp8 payload (16 payload bytes and one scale per lane
// and row; a 128-element scale group is 8 lanes, and the scales of a row sit R*max floats apart in the
// column-major layout), 512 elements of a bf16 payload.  Lanes 0..K-1 find the K rows as reduce_kernel
// does; a masked, inactive or unknown selection reads the zero row with weight 0.
//
// Up to top-8 the register budget is that of eight waves per SIMD: left to itself the compiler spends
// twice as many on the variant without a factor (to hoist every load), and at four waves per SIMD that
// variant ran 5 % slower.  (Sixteen rows in flight do not fit that budget.)
//   CH  bf16 payloads only: 16-byte chunks per lane and row, 512 elements apart (two when there are few
//       rows per token, as in reduce_kernel: half as many waves, each with as many loads in flight)
template <int KMAX, bool FP8, bool FACTOR, bool DIRECT, int CH = 1>
__global__ __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(KMAX <= 8 ? 8 : 4, 8))) void reduce_packed_kernel(const uint64_t* __restrict__ tbl,
                                                             const CombineRoute* __restrict__ routes, uint32_t stamp,
                                                             RoutingScratch sc, CombineSource cs,
                                                             const void* __restrict__ zero_row,
                                                             const float* __restrict__ factor, int R, int E, int K,
                                                             int max_tokens, int H, int slabs, int Tgrid,
                                                             int group_blocks) {
    static_assert(!FP8 || CH == 1, "an fp8 payload is one 16-byte chunk of 16 elements per lane");
    constexpr int kSlab = FP8 ? 1024 : 512 * CH;
    constexpr int kChunkElems = FP8 ? 16 : 8;          // elements in a lane's 16-byte chunk
    const int lane = wave_lane();
    // Blocks go round-robin over the 8 XCDs, each with an L2 of its own.  The rows that the source ranks
    // sent to an expert are neighbours in the expert's block, so their scales of one group share 64-byte
    // sectors.  group_blocks > 0 (bf16 payloads, which have no scales; option packed_map = 0): all the waves
    // of a (rank, slab) pair are given to one XCD, next to each other in launch order (group_blocks
    // consecutive blocks of that XCD).  group_blocks < 0 (fp8): slabs are owned by XCDs (xcd_owned_task).
    const int wpb = blockDim.x >> 6;
    const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
    int r, s, t;
    if (group_blocks > 0) {
        const int gl = seq / group_blocks, tb = seq - gl * group_blocks;
        const int gid = gl * 8 + xcd;
        if (gid >= R * slabs) return;
        r = gid / slabs;
        s = gid - r * slabs;
        t = __builtin_amdgcn_readfirstlane(tb * wpb + (threadIdx.x >> 6));
        if (t >= Tgrid) return;
    } else {
        // slabs owned by XCDs (see xcd_owned_task): a slab's scales are read through one XCD's L2
        const int w = __builtin_amdgcn_readfirstlane(seq * wpb + (threadIdx.x >> 6));
        int n;
        if (!xcd_owned_task(xcd, w, slabs, R * Tgrid, &n, &s)) return;
        r = n / Tgrid;
        t = n - r * Tgrid;
    }
    const int T = cs.tokens >= 0 ? cs.tokens : (int)tbl[CF_NUM_TOKENS * R + r];
    if (t >= T) return;
    char* orow = (char*)rank_ptr(tbl, cs.out, CF_OUT, R, r) + (int64_t)t * H * 2;
    const int64_t RM = (int64_t)R * max_tokens;
    const int G = H >> 7, L = E / R;

    // lanes 0..K-1: where the selection's row, its scales and its factor are
    uint64_t src = (uint64_t)zero_row, ssrc = (uint64_t)zero_row;
    float w = 0.0f, f = 1.0f;
    int sstride = 0;                     // bytes between a row's consecutive scale groups (0: the zero row)
    int live = 1;                        // DIRECT: loaded here, looked at after the payload loads are issued
    {
        int e = 0, slot = 0;
        bool ok = false;
        float wl = 0.0f;
        if (DIRECT) {
            const uint64_t w_row = rank_ptr(tbl, cs.topk_weights, CF_TOPK_W, R, r) + (uint64_t)((int64_t)t * K) * 4;
            wl = load_f32(w_row + (uint64_t)(lane < K ? lane : 0) * 4);
            const DirectRow d = direct_row(tbl, sc, cs.x, cs.topk_idx, R, E, K, max_tokens, r, t, lane);
            ok = d.has;
            e = d.e;
            slot = d.slot;
            live = d.live;
        } else {
            uint4 rt = make_uint4(0, 0, 0, 0);
            if (lane < K) rt = *(const uint4*)(routes + ((int64_t)r * max_tokens + t) * K + lane);
            ok = (lane < K) && (rt.w == stamp) && (int)rt.y < E && (int64_t)rt.x < RM;
            e = ok ? (int)rt.y : 0;
            slot = ok ? (int)rt.x : 0;
            wl = __uint_as_float(rt.z);
        }
        const int q = e / L, le = e - q * L;
        const uint64_t base = rank_ptr(tbl, cs.x, CF_X, R, q);
        const uint64_t sbase = FP8 ? rank_ptr(tbl, cs.scales, CF_SCALES, R, q) : 0;
        const float fe = FACTOR ? factor[e] : 1.0f;
        if (ok && base != 0 && (!FP8 || sbase != 0)) {
            const int64_t grow = (int64_t)le * RM + slot;
            src = base + (uint64_t)grow * (uint64_t)H * (FP8 ? 1 : 2);
            if (FP8) {
                ssrc = sbase + (uint64_t)((int64_t)le * G * RM + slot) * 4;
                sstride = (int)(RM * 4);
            }
            w = wl;
            f = fe;
        }
    }

    int elem[CH];
    bool on[CH];
    int64_t poff[CH];
#pragma unroll
    for (int c = 0; c < CH; ++c) {
        elem[c] = s * kSlab + c * 512 + lane * kChunkElems;
        on[c] = elem[c] < H;
        poff[c] = on[c] ? (int64_t)elem[c] * (FP8 ? 1 : 2) : 0;
    }
    const int group = on[0] ? (elem[0] >> 7) : 0;

    uint4 v[KMAX][CH];
    float sv[KMAX], wk[KMAX], fk[KMAX];
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        const uint64_t p = read_lane_u64(src, k);
#pragma unroll
        for (int c = 0; c < CH; ++c) v[k][c] = load16<true>((const void*)(p + poff[c]));
        if (FP8) {
            const uint64_t sp = read_lane_u64(ssrc, k);
            const int st = __builtin_amdgcn_readlane(sstride, k);
            sv[k] = load_f32(sp + (uint64_t)((int64_t)group * st));
        } else {
            sv[k] = 1.0f;
        }
    }

    // a row of a rank the token's owner sees as inactive was fetched before that was known: drop it
    if (DIRECT && live == 0) w = 0.0f;
    // the expert's factor was loaded behind the row table, like `live`: looked at only now, when the payload
    // loads are on their way
    asm volatile("" : "+v"(f));
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        fk[k] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(f), k));
        wk[k] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w), k));
        if (DIRECT && __builtin_amdgcn_readlane(live, k) == 0) {
#pragma unroll
            for (int c = 0; c < CH; ++c) v[k][c] = make_uint4(0, 0, 0, 0);
            sv[k] = 0.0f;
        }
    }
#pragma unroll
    for (int c = 0; c < CH; ++c) {
    float acc[kChunkElems];
#pragma unroll
    for (int j = 0; j < kChunkElems; ++j) acc[j] = 0.0f;
#pragma unroll
    for (int k = 0; k < KMAX; ++k) {
        const uint32_t u[4] = {v[k][c].x, v[k][c].y, v[k][c].z, v[k][c].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (FP8) {
                typedef float f2 __attribute__((ext_vector_type(2)));
                const f2 a = __builtin_amdgcn_cvt_pk_f32_fp8((int)u[j], false);
                const f2 b = __builtin_amdgcn_cvt_pk_f32_fp8((int)u[j], true);
                float e[4] = {round_bf16(a.x * sv[k]), round_bf16(a.y * sv[k]), round_bf16(b.x * sv[k]),
                              round_bf16(b.y * sv[k])};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    if (FACTOR) e[i] = round_bf16(e[i] * fk[k]);
                    acc[4 * j + i] = __builtin_fmaf(e[i], wk[k], acc[4 * j + i]);
                }
            } else {
                float e[2] = {bf16_lo(u[j]), bf16_hi(u[j])};
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    if (FACTOR) e[i] = round_bf16(e[i] * fk[k]);
                    acc[2 * j + i] = __builtin_fmaf(e[i], wk[k], acc[2 * j + i]);
                }
            }
        }
    }
    if (!on[c]) continue;
    uint32_t o[kChunkElems / 2];
#pragma unroll
    for (int j = 0; j < kChunkElems / 2; ++j) o[j] = pack_bf16_rne(acc[2 * j], acc[2 * j + 1]);
    store16<true>(orow + (int64_t)elem[c] * 2, make_uint4(o[0], o[1], o[2], o[3]));
    if constexpr (FP8) store16<true>(orow + (int64_t)elem[c] * 2 + 16, make_uint4(o[4], o[5], o[6], o[7]));
    }
}

// Work list of the cast-back kernel: which (expert, row chunk) each chunk
// number is, from the packed_recv_count tensors alone; map[0].x is the number
// of chunks.  Per block: a thread per expert fetches the count, one wave scans
// ceil(count / kCastRows) over the experts in LDS, then a thread per chunk
// finds its expert by bisection of the scanned begins.  It costs a launch, and
// saves every block of the main kernel the same scan (a chain of dependent
// loads) in front of its first row.
constexpr int kCastWaves = 4;        // waves per block of the main kernel: kCastRows / kCastWaves rows each
constexpr int kCastCols = 1024;
constexpr int kCastMaxExperts = 4096;
constexpr int kCastMapBlocks = 8;      // each repeats the scan (cheap) and writes an eighth of the entries

__global__ __launch_bounds__(1024) void cast_chunks_kernel(const uint64_t* __restrict__ tbl, int4* __restrict__ map,
                                                           int R, int E, int max_tokens, int max_chunks) {
    __shared__ int lds_count[kCastMaxExperts];
    __shared__ int lds_begin[kCastMaxExperts + 1];
    const int lane = wave_lane();
    const int L = E / R;
    const int64_t RM = (int64_t)R * max_tokens;
    for (int ee = threadIdx.x; ee < E; ee += blockDim.x) {
        const int qq = ee / L;
        const int32_t* cnt = (const int32_t*)tbl[XF_RECV_COUNT * R + qq];
        int c = 0;
        // a rank without tensors takes no part
        if (cnt != nullptr && tbl[XF_RECV_X * R + qq] != 0 && tbl[XF_OUT * R + qq] != 0) c = cnt[ee - qq * L];
        lds_count[ee] = c < 0 ? 0 : (c > RM ? (int)RM : c);
    }
    __syncthreads();
    if (threadIdx.x < 64) {
        int carry = 0;
        for (int e0 = 0; e0 < E; e0 += 64) {
            const int ee = e0 + lane;
            const int n = (ee < E) ? (lds_count[ee] + kCastRows - 1) / kCastRows : 0;
            const int incl = wave_scan_inclusive(n);
            if (ee < E) lds_begin[ee] = carry + incl - n;
            carry += __builtin_amdgcn_readlane(incl, 63);
        }
        if (lane == 0) {
            lds_begin[E] = carry;
            if (blockIdx.x == 0) map[0] = make_int4(carry < max_chunks ? carry : max_chunks, 0, 0, 0);
        }
    }
    __syncthreads();
    const int total = lds_begin[E] < max_chunks ? lds_begin[E] : max_chunks;
    for (int i = blockIdx.x * blockDim.x + threadIdx.x; i < total; i += gridDim.x * blockDim.x) {
        // the last expert whose first chunk number is <= i (experts without rows share their successor's begin)
        int lo = 0, hi = E;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (lds_begin[mid] <= i) lo = mid; else hi = mid;
        }
        map[1 + i] = make_int4(lo, i - lds_begin[lo], lds_count[lo], 0);
    }
}

// A block takes one chunk (kCastRows consecutive packed rows of one expert)
// times kCastCols columns, so only rows below packed_recv_count cost anything;
// each of its kCastWaves waves converts one row of the chunk.  A lane owns two
// pieces of 8 elements half the block's width apart: per piece 8 payload bytes
// and one scale (fp8; the scales of a row sit R*max floats apart in the
// column-major layout, and the four chunks that share their 64-byte sectors
// run next to each other on one XCD) or 16 payload bytes (bf16), and one
// 16-byte store that is contiguous across the wave.  No LDS.
template <bool FP8>
__global__ __launch_bounds__(kCastWaves * 64) void cast_back_kernel(const uint64_t* __restrict__ tbl,
                                                         const int4* __restrict__ map,
                                                         const float* __restrict__ factor, int R, int E, int H,
                                                         int max_tokens, int parts, int max_chunks) {
    const int lane = wave_lane();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // Blocks go round-robin over the 8 XCDs, each with an L2 of its own.  The four chunks that share
    // 64-byte sectors of scales (16 consecutive rows of one group) are therefore given to four blocks
    // of the same XCD, next to each other in launch order: block = (set / 8 * 4 + chunk % 4) * 8 + set % 8,
    // with set = (chunk / 4) * parts + part.
    const int xcd = blockIdx.x & 7, seq = blockIdx.x >> 3;
    const int set = (seq >> 2) * 8 + xcd;
    const int part = set % parts;
    const int target = (set / parts) * 4 + (seq & 3);
    const int L = E / R;
    const int64_t RM = (int64_t)R * max_tokens;
    const int total = map[0].x;
    const int4 item = map[1 + (target < max_chunks ? target : 0)];
    if (target >= total) return;            // block-uniform
    const int e = __builtin_amdgcn_readfirstlane(item.x);
    const int chunk = __builtin_amdgcn_readfirstlane(item.y);
    const int count = __builtin_amdgcn_readfirstlane(item.z);

    const int q = e / L, le = e - q * L;
    const int G = H / 128;
    const int col0 = part * kCastCols;
    const int ncols = (H - col0 < kCastCols) ? (H - col0) : kCastCols;
    const int row0 = chunk * kCastRows;
    const float f = factor != nullptr ? factor[e] : 1.0f;
    const uint8_t* in = (const uint8_t*)tbl[XF_RECV_X * R + q];
    uint8_t* out = (uint8_t*)tbl[XF_OUT * R + q];

    // A lane owns two pieces of 8 elements, half a block's width apart, so that each
    // of its two 16-byte stores lands in a run of 1 KB written by the wave as a whole.
    // Piece p covers columns col0 + p * 512 + lane * 8 .. + 7; 16 lanes share a scale group.
    constexpr int kHalf = kCastCols / 2;
    bool on[2];
    int64_t in_off[2], out_off[2];
    const float* scale_col[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const int col = p * kHalf + lane * 8;
        on[p] = col < ncols;
        const int c = on[p] ? col : 0;
        in_off[p] = (int64_t)(col0 + c) * (FP8 ? 1 : 2);
        out_off[p] = (int64_t)(col0 + c) * 2;
        scale_col[p] = FP8 ? (const float*)tbl[XF_RECV_SCALES * R + q] + ((int64_t)le * G + (col0 + c) / 128) * RM
                           : nullptr;
    }

    constexpr int kWaveRows = kCastRows / kCastWaves;
    constexpr int kBatch = kWaveRows < 8 ? kWaveRows : 8;   // rows whose loads are in flight together
    const int64_t row_base = (int64_t)le * RM;
    for (int b = 0; b < kWaveRows; b += kBatch) {
        const int r_first = row0 + wave * kWaveRows + b;
        if (r_first >= count) break;
        uint4 v[kBatch][2];
        float sv[kBatch][2];
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            const int row = r_first + i < count ? r_first + i : r_first;
            const uint8_t* src = in + (row_base + row) * H * (FP8 ? 1 : 2);
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                if (FP8) {
                    const uint2 w = *(const uint2*)(src + in_off[p]);
                    v[i][p] = make_uint4(w.x, w.y, 0u, 0u);
                    sv[i][p] = scale_col[p][row];
                } else {
                    v[i][p] = load16<true>(src + in_off[p]);
                }
            }
        }
#pragma unroll
        for (int i = 0; i < kBatch; ++i) {
            if (r_first + i >= count) break;       // wave-uniform
            uint8_t* dst = out + (row_base + r_first + i) * H * 2;
#pragma unroll
            for (int p = 0; p < 2; ++p) {
                uint32_t o[4];
                if (FP8) {
                    typedef float f2 __attribute__((ext_vector_type(2)));
                    const f2 a0 = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[i][p].x, false);
                    const f2 a1 = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[i][p].x, true);
                    const f2 a2 = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[i][p].y, false);
                    const f2 a3 = __builtin_amdgcn_cvt_pk_f32_fp8((int)v[i][p].y, true);
                    const float sc = sv[i][p];
                    o[0] = scale_round_twice(a0.x, a0.y, sc, f);
                    o[1] = scale_round_twice(a1.x, a1.y, sc, f);
                    o[2] = scale_round_twice(a2.x, a2.y, sc, f);
                    o[3] = scale_round_twice(a3.x, a3.y, sc, f);
                } else {
                    const uint32_t w[4] = {v[i][p].x, v[i][p].y, v[i][p].z, v[i][p].w};
#pragma unroll
                    for (int j = 0; j < 4; ++j) o[j] = pack_bf16_rne(bf16_lo(w[j]) * f, bf16_hi(w[j]) * f);
                }
                if (on[p]) store16<false>(dst + out_off[p], make_uint4(o[0], o[1], o[2], o[3]));
            }
        }
    }
}

__global__ __launch_bounds__(256) void copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = src[i];
}

// Synthetic streams with the read : write mixes of the data kernels, one 16-byte unit per thread and
// nothing else: what this GPU's memory system gives each mix when no routing, arithmetic or row
// structure is in the way (the ceilings the data kernels are compared with).
//   0 copy      read n, write n units                         (1 : 1)
//   1 read      read n units, write nothing
//   2 write     write n units
//   3 widen     read n half units (8 bytes), write n units    (1 : 2, the cast-back kernel's mix)
//   4 gather8   read 8 streams of n units, write n            (8 : 1, the reduce kernel's mix)
//   5 scatter8  read 2n units, write 8 streams of n           (1 : 4, the fp8 pack kernel's mix)
template <int KIND>
__global__ __launch_bounds__(256) void stream_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src,
                                                      size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    if (KIND == 0) {
        dst[i] = src[i];
    } else if (KIND == 1) {
        const uint4 v = load16<true>(src + i);
        if (v.x == 0x12345678u && v.y == 0x9abcdef0u && v.z == 1u && v.w == 2u) dst[0] = v;   // never, in practice
    } else if (KIND == 2) {
        dst[i] = make_uint4((uint32_t)i, 1u, 2u, 3u);
    } else if (KIND == 3) {
        const uint2 v = ((const uint2*)src)[i];
        dst[i] = make_uint4(v.x, v.y, v.x ^ v.y, v.x + v.y);
    } else if (KIND == 4) {
        uint4 v[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) v[k] = load16<true>(src + (size_t)k * n + i);
        uint4 a = v[0];
#pragma unroll
        for (int k = 1; k < 8; ++k) {
            a.x ^= v[k].x; a.y ^= v[k].y; a.z ^= v[k].z; a.w ^= v[k].w;
        }
        store16<true>(dst + i, a);
    } else {
        const uint4 a = load16<true>(src + 2 * i), b = load16<true>(src + 2 * i + 1);
        const uint4 o = make_uint4(a.x ^ b.x, a.y ^ b.y, a.z ^ b.z, a.w ^ b.w);
#pragma unroll
        for (int k = 0; k < 8; ++k) dst[(size_t)k * n + i] = o;
    }
}

// The reduce kernel's address pattern without its index loads and arithmetic: every output row of
// row_units 16-byte units is the xor of 8 whole source rows, and each source row sits at a computed,
// scattered place of a [regions, region_rows] layout of which the first `used` rows per region are
// touched, each once (the packed receive layout: a region per expert, valid rows at its start).
__global__ __launch_bounds__(256) void stream_rows_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src,
                                                           int row_units, size_t n, int regions, size_t region_rows,
                                                           int used) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    // a row is a whole number of waves (row_units % 64 == 0), so the row arithmetic is the wave's, not the lane's
    const uint32_t ro = __builtin_amdgcn_readfirstlane((uint32_t)(i / (size_t)row_units));
    const size_t c = i - (size_t)ro * (size_t)row_units;
    const uint32_t total = (uint32_t)regions * (uint32_t)used;
    uint4 v[8];
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        // a permutation of the regions * used rows (the multiplier is prime), so every row is read once
        const uint32_t p = (uint32_t)(((uint64_t)(ro * 8u + (uint32_t)k) * 2654435761ull) % total);
        const uint32_t region = p % (uint32_t)regions, rr = p / (uint32_t)regions;
        v[k] = load16<true>(src + ((size_t)region * region_rows + rr) * (size_t)row_units + c);
    }
    uint4 a = v[0];
#pragma unroll
    for (int k = 1; k < 8; ++k) {
        a.x ^= v[k].x; a.y ^= v[k].y; a.z ^= v[k].z; a.w ^= v[k].w;
    }
    store16<true>(dst + i, a);
}

// The fp8 pack kernel's address pattern alone: every source row of 2 * row_units units is read once,
// folded to row_units units and written to 8 whole rows at computed, scattered places of a
// [regions, region_rows] layout (the first `used` rows of every region, each written once).
__global__ __launch_bounds__(256) void stream_rows_scatter_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src,
                                                                   int row_units, size_t n, int regions,
                                                                   size_t region_rows, int used) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    const uint32_t ri = __builtin_amdgcn_readfirstlane((uint32_t)(i / (size_t)row_units));
    const size_t c = i - (size_t)ri * (size_t)row_units;
    const uint32_t total = (uint32_t)regions * (uint32_t)used;
    const uint4 a = load16<true>(src + 2 * i), b = load16<true>(src + 2 * i + 1);
    const uint4 o = make_uint4(a.x ^ b.x, a.y ^ b.y, a.z ^ b.z, a.w ^ b.w);
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const uint32_t p = (uint32_t)(((uint64_t)(ri * 8u + (uint32_t)k) * 2654435761ull) % total);
        const uint32_t region = p % (uint32_t)regions, rr = p / (uint32_t)regions;
        store16<false>(dst + ((size_t)region * region_rows + rr) * (size_t)row_units + c, o);
    }
}

__global__ __launch_bounds__(256) void fill_kernel(uint32_t* __restrict__ dst, uint32_t value, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = value;
}

}  // namespace

// ---------------------------------------------------------------------------
// launchers
// ---------------------------------------------------------------------------

hipError_t launch_table_write(uint64_t* d_tbl, const uint64_t* h_tbl, int n_words, hipStream_t stream) {
    for (int base = 0; base < n_words; base += kTableChunk) {
        TableChunk chunk;
        const int n = (n_words - base < kTableChunk) ? (n_words - base) : kTableChunk;
        for (int i = 0; i < n; ++i) chunk.v[i] = h_tbl[base + i];
        for (int i = n; i < kTableChunk; ++i) chunk.v[i] = 0;
        hipLaunchKernelGGL(table_write_kernel, dim3((n + 127) / 128), dim3(128), 0, stream, d_tbl + base, chunk, n);
        hipError_t err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    return hipSuccess;
}

hipError_t launch_clear_words(const uint64_t* h_ptrs, int n_ptrs, int words, hipStream_t stream) {
    if (words <= 0) return hipSuccess;
    TableChunk chunk;
    for (int base = 0; base < n_ptrs; base += kTableChunk) {
        const int n = (n_ptrs - base < kTableChunk) ? (n_ptrs - base) : kTableChunk;
        for (int i = 0; i < kTableChunk; ++i) chunk.v[i] = i < n ? h_ptrs[base + i] : 0;
        const long long total = (long long)n * words;
        if (total > 0x7fffffffll) return hipErrorInvalidValue;
        hipLaunchKernelGGL(clear_words_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream, chunk, n,
                           words);
        hipError_t err = hipGetLastError();
        if (err != hipSuccess) return err;
    }
    return hipSuccess;
}

hipError_t launch_count(const uint64_t* d_tbl, const RoutingScratch& sc, const DispatchSource& src, const Dims& d,
                        hipStream_t stream) {
    const size_t lds = count_lds_bytes(d);
    if (lds > kMaxCountLdsBytes) return hipErrorInvalidValue;
    const void* kern = d.plan.shift == 10 ? (const void*)count_kernel<kBigUnitSelections>
                                          : (const void*)count_kernel<kUnitSelections>;
    if (lds > 48 * 1024) {
        hipError_t err = hipFuncSetAttribute(kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
    }
    if (d.plan.shift == 10)
        hipLaunchKernelGGL(count_kernel<kBigUnitSelections>, dim3(d.units()), dim3(kBigUnitSelections), lds, stream,
                           d_tbl, sc, src, d.R, d.E, d.K, d.max_tokens, d.units_per_rank());
    else
        hipLaunchKernelGGL(count_kernel<kUnitSelections>, dim3(d.units()), dim3(kUnitSelections), lds, stream, d_tbl,
                           sc, src, d.R, d.E, d.K, d.max_tokens, d.units_per_rank());
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
    if (d.plan.carried) return hipSuccess;   // the prefix pass rides in the pack launch
    const size_t plds = (size_t)kPrefixWaves * (d.units() + 1) * sizeof(int);
    if (plds > 60 * 1024) return hipErrorInvalidValue;
    hipLaunchKernelGGL(prefix_kernel, dim3((d.E + kPrefixWaves - 1) / kPrefixWaves), dim3(kPrefixWaves * 64), plds,
                       stream, d_tbl, sc, d.R, d.E, d.max_tokens, d.units_per_rank(), d.units());
    return hipGetLastError();
}

static int clamp_waves(int w) { return w < 1 ? 1 : (w > kMaxPackWaves ? kMaxPackWaves : w); }

// Dynamic LDS a launch of wpb-wave blocks asks for (and never touches) so that a CU runs at most
// `waves_per_cu` waves of it: floor(waves_per_cu / wpb) blocks fill the CU's LDS, at least one, at most what
// 64 KiB per block allow without raising the kernel's limit.  0: no limit.
static size_t occupancy_pad_bytes(int waves_per_cu, int wpb) {
    constexpr size_t kCuLdsBytes = 160 * 1024, kMaxPad = 64 * 1024;
    if (waves_per_cu <= 0) return 0;
    const size_t blocks = waves_per_cu / wpb > 0 ? (size_t)(waves_per_cu / wpb) : 1;
    const size_t pad = kCuLdsBytes / blocks / 1024 * 1024;
    return pad > kMaxPad ? kMaxPad : pad;
}

static long long transpose_items(const Dims& d, int* parts_out) {
    const int G = d.H / 128;
    const int parts = (G + kTransposeGroups - 1) / kTransposeGroups;
    // every selection is at most one row, and each expert has at most one partly filled chunk
    const long long chunks = ((long long)d.R * d.Tgrid * d.K + 63) / 64 + d.E;
    *parts_out = parts;
    return chunks * parts;
}

template <typename Kern>
static hipError_t launch_pack_t(Kern kern, const uint64_t* d_tbl, const RoutingScratch& sc, const DispatchSource& src,
                                float* stage, const Dims& d, const Tuning& t, hipStream_t stream) {
    const int slabs = (d.H + 1023) / 1024;
    long long total = (long long)d.R * d.Tgrid * slabs;
    if (total <= 0) return hipSuccess;
    if (d.plan.carried) total += d.E;   // the prefix pass: a wave per expert in front of the data waves
    if (total > 0x7fffffffll) return hipErrorInvalidValue;
    const int wpb = clamp_waves(t.pack_waves);
    const int blocks = (int)((total + wpb - 1) / wpb);
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(wpb * 64), 0, stream, d_tbl, sc, src, stage, d.R, d.E, d.K,
                       d.max_tokens, d.H, d.plan, slabs, d.Tgrid, (int)total);
    return hipGetLastError();
}

hipError_t launch_pack(const uint64_t* d_tbl, const RoutingScratch& sc, const DispatchSource& src, float* scale_stage,
                       const Dims& d, bool use_fp8, const Tuning& t, bool run_pack, bool run_finish,
                       hipStream_t stream) {
    // Streaming hints (bit 0: loads, bit 1: stores).  Default: streaming loads when a token's row goes to many
    // experts, ordinary stores.  Both hints together always lose (+6 to +9 us on the decode workloads).
    // Streaming stores with ordinary loads win in the steady state - 2 % of the DeepSeek-V3 decode step, 5 to
    // 13 % of a dispatch whose payload is several times the 256 MB memory-side cache - but lose under the
    // reference's timing protocol, a written cache flush before every timed call (8 x 1024 tokens, hidden 7168,
    // top-8, bf16: 218 against 180 us), and a consumer that reads a cacheable payload next finds it in memory
    // instead of that cache.  They are an option (pack_nt = 2), not the default.
    const int nt = t.pack_nt >= 0 ? t.pack_nt : (d.K > 4 ? 1 : 0);
    const bool ntl = (nt & 1) != 0, nts = (nt & 2) != 0;
    if (use_fp8 && scale_stage == nullptr) return hipErrorInvalidValue;
    hipError_t err = hipSuccess;
    if (run_pack) {
#define MCEP_PF(A, B)                                                                                   \
    (nts ? launch_pack_t(pack_fp8_kernel<A, B, true>, d_tbl, sc, src, scale_stage, d, t, stream)        \
         : launch_pack_t(pack_fp8_kernel<A, B, false>, d_tbl, sc, src, scale_stage, d, t, stream))
#define MCEP_PB(A)                                                                                      \
    (nts ? launch_pack_t(pack_bf16_kernel<A, true>, d_tbl, sc, src, scale_stage, d, t, stream)          \
         : launch_pack_t(pack_bf16_kernel<A, false>, d_tbl, sc, src, scale_stage, d, t, stream))
        if (!use_fp8)
            err = ntl ? MCEP_PB(true) : MCEP_PB(false);
        else
            err = ntl ? (t.fp8_arith == 1 ? MCEP_PF(true, true) : MCEP_PF(true, false))
                      : (t.fp8_arith == 1 ? MCEP_PF(false, true) : MCEP_PF(false, false));
#undef MCEP_PB
#undef MCEP_PF
    }
    if (err != hipSuccess || !use_fp8 || !run_finish) return err;
    int parts = 1;
    const long long items = transpose_items(d, &parts);
    if (items > 0x7fffffffll) return hipErrorInvalidValue;
    hipLaunchKernelGGL(scale_transpose_kernel, dim3((unsigned)((items + kTransposeWaves - 1) / kTransposeWaves)),
                       dim3(kTransposeWaves * 64), 0, stream, d_tbl, scale_stage, sc, d.R, d.E, d.H / 128, d.max_tokens,
                       parts, (int)items);
    return hipGetLastError();
}

template <int KMAX>
static hipError_t launch_dispatch_small_t(const SmallTable& tb, int32_t* d_selrow, const Dims& d, bool use_fp8,
                                          const Tuning& t, hipStream_t stream) {
    const int slabs = (d.H + 1023) / 1024;
    const long long total = (long long)d.E + (long long)d.R * d.Tgrid * slabs;
    if (total > 0x7fffffffll) return hipErrorInvalidValue;
    constexpr int wpb = 4;
    const dim3 grid((unsigned)((total + wpb - 1) / wpb)), block(wpb * 64);
#define MCEP_SMALL(FP8, NATIVE)                                                                              \
    hipLaunchKernelGGL((dispatch_small_kernel<KMAX, FP8, NATIVE>), grid, block, 0, stream, tb, d_selrow, d.R, \
                       d.E, d.K, d.max_tokens, d.H, slabs, d.Tgrid, (int)total)
    if (!use_fp8) MCEP_SMALL(false, false);
    else if (t.fp8_arith == 1) MCEP_SMALL(true, true);
    else MCEP_SMALL(true, false);
#undef MCEP_SMALL
    return hipGetLastError();
}

hipError_t launch_dispatch_small(const SmallTable& tb, int32_t* d_selrow, const Dims& d, bool use_fp8, const Tuning& t,
                                 hipStream_t stream) {
    if (d.R > kSmallRanks || d.Tgrid <= 0 || d_selrow == nullptr) return hipErrorInvalidValue;
    if (d.K <= 2) return launch_dispatch_small_t<2>(tb, d_selrow, d, use_fp8, t, stream);
    if (d.K <= 4) return launch_dispatch_small_t<4>(tb, d_selrow, d, use_fp8, t, stream);
    if (d.K <= 8) return launch_dispatch_small_t<8>(tb, d_selrow, d, use_fp8, t, stream);
    return launch_dispatch_small_t<16>(tb, d_selrow, d, use_fp8, t, stream);
}

hipError_t launch_resolve(const uint64_t* d_tbl, CombineRoute* d_routes, uint32_t stamp, bool packed, const Dims& d,
                          const Tuning& /*t*/, hipStream_t stream) {
    const long long total = (long long)d.E * d.R;
    if (total <= 0) return hipSuccess;
    if (total > 0x7fffffffll) return hipErrorInvalidValue;
    const int wpb = 4;
    const int blocks = (int)((total + wpb - 1) / wpb);
    if (packed)
        hipLaunchKernelGGL(resolve_kernel<true>, dim3(blocks), dim3(wpb * 64), 0, stream, d_tbl, d_routes, stamp, d.R,
                           d.E, d.K, d.H, d.max_tokens, (int)total);
    else
        hipLaunchKernelGGL(resolve_kernel<false>, dim3(blocks), dim3(wpb * 64), 0, stream, d_tbl, d_routes, stamp, d.R,
                           d.E, d.K, d.H, d.max_tokens, (int)total);
    return hipGetLastError();
}

namespace {
struct ReduceLaunch {
    const uint64_t* d_tbl;
    const CombineRoute* d_routes;
    uint32_t stamp;
    RoutingScratch sc;
    CombineSource src;
    const void* d_zero_row;
};
}  // namespace

template <int KMAX, int CH, bool DIRECT>
static hipError_t launch_reduce_t(const ReduceLaunch& rl, const Dims& d, const Tuning& t, hipStream_t stream) {
    const int slabs = (d.H + CH * 512 - 1) / (CH * 512);
    const long long total = (long long)d.R * d.Tgrid * slabs;
    if (total <= 0) return hipSuccess;
    if (total > 0x7fffffffll) return hipErrorInvalidValue;
    const int wpb = clamp_waves(t.combine_waves);
    const int blocks = (int)((total + wpb - 1) / wpb);
    const bool ntl = t.combine_nt & 1, nts = t.combine_nt & 2;
    // Waves per CU.  With seven or more rows per token - 7 KB and more of loads in flight per wave - the
    // kernel is fastest at 16 to 20 waves per CU: 1.5 to 4 % faster at top-8, depending on the machine, than at
    // the 32 the hardware would run (fewer rows being walked at once), a little at top-11 and top-16; 12
    // waves no longer cover the latency.  With fewer rows per wave it wants all 32 (top-3: 39.6 us against
    // 41.1 at 20).  The limit is imposed with unused dynamic LDS: a CU's 160 KiB hold so many blocks and no more.
    const int occupancy = t.combine_occupancy >= 0 ? t.combine_occupancy : (d.K >= 7 ? 20 : 0);
    const size_t pad = occupancy_pad_bytes(occupancy, wpb);
#define MCEP_REDUCE(A, B)                                                                                        \
    hipLaunchKernelGGL((reduce_kernel<KMAX, CH, A, B, DIRECT>), dim3(blocks), dim3(wpb * 64), pad, stream, rl.d_tbl, \
                       rl.d_routes, rl.stamp, rl.sc, rl.src, rl.d_zero_row, d.R, d.E, d.K, d.max_tokens, d.H,    \
                       slabs, d.Tgrid, (int)total)
    if (ntl && nts) MCEP_REDUCE(true, true);
    else if (ntl) MCEP_REDUCE(true, false);
    else if (nts) MCEP_REDUCE(false, true);
    else MCEP_REDUCE(false, false);
#undef MCEP_REDUCE
    return hipGetLastError();
}

hipError_t launch_reduce(const uint64_t* d_tbl, const CombineRoute* d_routes, uint32_t stamp, const RoutingScratch& sc,
                         bool direct, const CombineSource& src, const void* d_zero_row, const Dims& d, const Tuning& t,
                         hipStream_t stream) {
    const ReduceLaunch rl{d_tbl, d_routes, stamp, sc, src, d_zero_row};
    // measured: with few rows per token a lane needs two chunks to keep enough loads in flight
    const int ch = t.combine_chunks > 0 ? (t.combine_chunks >= 2 ? 2 : 1) : (d.K <= 4 ? 2 : 1);
#define MCEP_K(KMAX)                                                                                   \
    do {                                                                                               \
        if (direct) return ch == 2 ? launch_reduce_t<KMAX, 2, true>(rl, d, t, stream)                  \
                                   : launch_reduce_t<KMAX, 1, true>(rl, d, t, stream);                 \
        return ch == 2 ? launch_reduce_t<KMAX, 2, false>(rl, d, t, stream)                             \
                       : launch_reduce_t<KMAX, 1, false>(rl, d, t, stream);                            \
    } while (0)
    if (d.K <= 1) MCEP_K(1);
    if (d.K <= 2) MCEP_K(2);
    if (d.K <= 4) MCEP_K(4);
    if (d.K <= 6) MCEP_K(6);
    if (d.K <= 8) MCEP_K(8);
    if (d.K <= 12) MCEP_K(12);
    MCEP_K(16);
#undef MCEP_K
}

template <int KMAX, bool FP8, bool FACTOR, bool DIRECT, int CH = 1>
static hipError_t launch_reduce_packed_t(const ReduceLaunch& rl, const float* d_factor, const Dims& d, const Tuning& t,
                                         hipStream_t stream) {
    const int slab = FP8 ? 1024 : 512 * CH;
    const int slabs = (d.H + slab - 1) / slab;
    if (d.Tgrid <= 0) return hipSuccess;
    const int wpb = clamp_waves(t.combine_waves);
    int group_blocks;
    long long blocks;
    if (FP8 && t.packed_map != 0) {
        blocks = xcd_owned_blocks((long long)d.R * d.Tgrid, slabs, wpb);
        group_blocks = -1;
    } else {
        // (rank, slab) groups, eight at a time (one per XCD), each a run of group_blocks blocks
        group_blocks = (d.Tgrid + wpb - 1) / wpb;
        const long long rounds = ((long long)d.R * slabs + 7) / 8;
        blocks = rounds * 8 * group_blocks;
    }
    if (blocks > 0x7fffffffll) return hipErrorInvalidValue;
    hipLaunchKernelGGL((reduce_packed_kernel<KMAX, FP8, FACTOR, DIRECT, CH>), dim3((unsigned)blocks), dim3(wpb * 64), 0,
                       stream, rl.d_tbl, rl.d_routes, rl.stamp, rl.sc, rl.src, rl.d_zero_row, d_factor, d.R, d.E, d.K,
                       d.max_tokens, d.H, slabs, d.Tgrid, group_blocks);
    return hipGetLastError();
}

hipError_t launch_reduce_packed(const uint64_t* d_tbl, const CombineRoute* d_routes, uint32_t stamp,
                                const RoutingScratch& sc, bool direct, const CombineSource& src, const void* d_zero_row,
                                const float* d_factor, bool use_fp8, const Dims& d, const Tuning& t, hipStream_t stream) {
    const ReduceLaunch rl{d_tbl, d_routes, stamp, sc, src, d_zero_row};
    const bool fac = d_factor != nullptr;
#define MCEP_P4(KMAX, FP8, FACTOR)                                                                   \
    (direct ? launch_reduce_packed_t<KMAX, FP8, FACTOR, true>(rl, d_factor, d, t, stream)            \
            : launch_reduce_packed_t<KMAX, FP8, FACTOR, false>(rl, d_factor, d, t, stream))
#define MCEP_PK(KMAX)                                                                                \
    do {                                                                                             \
        if (use_fp8) return fac ? MCEP_P4(KMAX, true, true) : MCEP_P4(KMAX, true, false);            \
        return fac ? MCEP_P4(KMAX, false, true) : MCEP_P4(KMAX, false, false);                       \
    } while (0)
    // a bf16 payload with few rows per token: two chunks per lane, as in the combine kernel
#define MCEP_P2(KMAX, FACTOR)                                                                        \
    (direct ? launch_reduce_packed_t<KMAX, false, FACTOR, true, 2>(rl, d_factor, d, t, stream)       \
            : launch_reduce_packed_t<KMAX, false, FACTOR, false, 2>(rl, d_factor, d, t, stream))
    const int ch = t.combine_chunks > 0 ? (t.combine_chunks >= 2 ? 2 : 1) : (d.K <= 4 ? 2 : 1);
    if (!use_fp8 && ch == 2 && d.K <= 2) return fac ? MCEP_P2(2, true) : MCEP_P2(2, false);
    if (!use_fp8 && ch == 2 && d.K <= 4) return fac ? MCEP_P2(4, true) : MCEP_P2(4, false);
#undef MCEP_P2
    if (d.K <= 2) MCEP_PK(2);
    if (d.K <= 4) MCEP_PK(4);
    if (d.K <= 8) MCEP_PK(8);
    MCEP_PK(16);
#undef MCEP_PK
#undef MCEP_P4
}

hipError_t launch_cast_back(const uint64_t* d_tbl, void* d_chunk_map, const float* d_factor, bool use_fp8,
                            long long max_rows, const Dims& d, hipStream_t stream) {
    const int parts = (d.H + kCastCols - 1) / kCastCols;
    const long long chunks = cast_back_chunks(max_rows, d.E);
    const long long total = chunks * parts;
    if (total <= 0) return hipSuccess;
    if (total > 0x7fffffffll || d.E > kCastMaxExperts) return hipErrorInvalidValue;
    int4* map = (int4*)d_chunk_map;
    hipLaunchKernelGGL(cast_chunks_kernel, dim3(kCastMapBlocks), dim3(1024), 0, stream, d_tbl, map, d.R, d.E, d.max_tokens,
                       (int)chunks);
    // sets of four chunks times parts, rounded up to whole rounds over the 8 XCDs
    const long long sets = (chunks + 3) / 4 * parts;
    const long long blocks = (sets + 7) / 8 * 8 * 4;
    if (blocks > 0x7fffffffll) return hipErrorInvalidValue;
    if (use_fp8)
        hipLaunchKernelGGL(cast_back_kernel<true>, dim3((unsigned)blocks), dim3(kCastWaves * 64), 0, stream, d_tbl, map,
                           d_factor, d.R, d.E, d.H, d.max_tokens, parts, (int)chunks);
    else
        hipLaunchKernelGGL(cast_back_kernel<false>, dim3((unsigned)blocks), dim3(kCastWaves * 64), 0, stream, d_tbl,
                           map, d_factor, d.R, d.E, d.H, d.max_tokens, parts, (int)chunks);
    return hipGetLastError();
}

hipError_t launch_copy(void* dst, const void* src, size_t bytes, hipStream_t stream) {
    const size_t n = bytes / 16;
    if (n == 0) return hipSuccess;
    size_t blocks = (n + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (uint4*)dst, (const uint4*)src, n);
    return hipGetLastError();
}

// waves per CU the synthetic streams below are held to (0: as many as fit), so that a stream can be measured
// at the occupancy its kernel runs at
static std::atomic<int> g_stream_occupancy{0};
void set_stream_occupancy(int waves_per_cu) {
    g_stream_occupancy.store(waves_per_cu > 0 ? waves_per_cu : 0, std::memory_order_relaxed);
}
static size_t stream_pad_bytes() { return occupancy_pad_bytes(g_stream_occupancy.load(std::memory_order_relaxed), 4); }

hipError_t launch_stream(int kind, void* dst, const void* src, size_t unit_bytes, hipStream_t stream) {
    const size_t pad = stream_pad_bytes();
    const size_t n = unit_bytes / 16;
    if (n == 0) return hipSuccess;
    const size_t blocks = (n + 255) / 256;
    if (blocks > 0x7fffffffull || kind < 0 || kind > 5) return hipErrorInvalidValue;
    const dim3 grid((unsigned)blocks), block(256);
    uint4* d = (uint4*)dst;
    const uint4* s = (const uint4*)src;
    switch (kind) {
        case 0: hipLaunchKernelGGL(stream_kernel<0>, grid, block, pad, stream, d, s, n); break;
        case 1: hipLaunchKernelGGL(stream_kernel<1>, grid, block, pad, stream, d, s, n); break;
        case 2: hipLaunchKernelGGL(stream_kernel<2>, grid, block, pad, stream, d, s, n); break;
        case 3: hipLaunchKernelGGL(stream_kernel<3>, grid, block, pad, stream, d, s, n); break;
        case 4: hipLaunchKernelGGL(stream_kernel<4>, grid, block, pad, stream, d, s, n); break;
        default: hipLaunchKernelGGL(stream_kernel<5>, grid, block, pad, stream, d, s, n); break;
    }
    return hipGetLastError();
}

hipError_t launch_stream_rows(void* dst, const void* src, int row_bytes, long long out_rows, int regions,
                              long long region_rows, int used, hipStream_t stream) {
    const int row_units = row_bytes / 16;
    const size_t n = (size_t)out_rows * row_units;
    if (n == 0) return hipSuccess;
    if (row_units % 64 != 0 || (long long)regions * used > 0x7fffffffll) return hipErrorInvalidValue;
    const size_t blocks = (n + 255) / 256;
    if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
    hipLaunchKernelGGL(stream_rows_kernel, dim3((unsigned)blocks), dim3(256), stream_pad_bytes(),
                       stream, (uint4*)dst, (const uint4*)src,
                       row_units, n, regions, (size_t)region_rows, used);
    return hipGetLastError();
}

hipError_t launch_stream_rows_scatter(void* dst, const void* src, int row_bytes, long long in_rows, int regions,
                                      long long region_rows, int used, hipStream_t stream) {
    const int row_units = row_bytes / 16;
    const size_t n = (size_t)in_rows * row_units;
    if (n == 0) return hipSuccess;
    if (row_units % 64 != 0 || (long long)regions * used > 0x7fffffffll) return hipErrorInvalidValue;
    const size_t blocks = (n + 255) / 256;
    if (blocks > 0x7fffffffull) return hipErrorInvalidValue;
    hipLaunchKernelGGL(stream_rows_scatter_kernel, dim3((unsigned)blocks), dim3(256),
                       stream_pad_bytes(), stream, (uint4*)dst,
                       (const uint4*)src, row_units, n, regions, (size_t)region_rows, used);
    return hipGetLastError();
}

hipError_t launch_fill_u32(void* dst, uint32_t value, size_t words, hipStream_t stream) {
    if (words == 0) return hipSuccess;
    size_t blocks = (words + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    hipLaunchKernelGGL(fill_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (uint32_t*)dst, value, words);
    return hipGetLastError();
}

}  // namespace mcep
