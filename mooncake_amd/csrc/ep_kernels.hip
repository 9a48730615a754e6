// gfx950 (CDNA4, wave64) kernels for the low-latency MoE dispatch / combine
// path.  Everything here is HBM-bound byte movement: no matrix cores, every
// payload access is a 16-byte vector load or store that a wave issues over a
// contiguous span of a row.
//
//   layout_kernel   routing layout: per-expert histogram, per-(expert, source
//                   rank) ranges by prefix sum, source-index map and the
//                   resolved destination of every (rank, token, k) selection.  Restates the count
//                   path and the slot assignment of the reference's dispatch
//                   (mooncake-ep/src/mooncake_ep_kernel.cu:274, :319-356,
//                   :417-437) in a deterministic order: source rank ascending,
//                   token ascending, as the reference's PyTorch statement has
//                   it (mooncake-wheel/mooncake/mooncake_ep_buffer.py:787-817).
//   pack_kernel     one read of each token row, optional bf16 -> fp8 e4m3
//                   quantisation with per-128 amax / 448 scales
//                   (mooncake_ep_kernel.cu:183-186, :233-264), K row stores
//                   straight into [local expert, R*max, hidden]
//                   (the reference needs two hops, :273-306 then :442-466).
//   resolve_kernel  combine's handle (src_info, layout_range) -> source row and
//                   weight of each (token, k) (data flow of
//                   mooncake_ep_kernel.cu:611-637).
//   reduce_kernel   per token: fp32 fused multiply-add over its top-k expert
//                   rows in k order, round to nearest even bf16
//                   (mooncake_ep_kernel.cu:711-753).
#include "ep_kernels.h"

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

__device__ __forceinline__ uint64_t read_lane_u64(uint64_t v, int lane) {
    uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, lane);
    uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), lane);
    return ((uint64_t)hi << 32) | lo;
}

__device__ __forceinline__ float bf16_lo(uint32_t u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(uint32_t u) { return __uint_as_float(u & 0xffff0000u); }

template <bool NT>
__device__ __forceinline__ uint4 load16(const void* p) {
    if (NT) {
        const uint32_t* q = (const uint32_t*)p;
        typedef uint32_t v4 __attribute__((ext_vector_type(4)));
        v4 r = __builtin_nontemporal_load((const v4*)q);
        return make_uint4(r.x, r.y, r.z, r.w);
    }
    return *(const uint4*)p;
}

template <bool NT>
__device__ __forceinline__ void store16(void* p, uint4 v) {
    if (NT) {
        typedef uint32_t v4 __attribute__((ext_vector_type(4)));
        v4 r = {v.x, v.y, v.z, v.w};
        __builtin_nontemporal_store(r, (v4*)p);
    } else {
        *(uint4*)p = v;
    }
}

template <bool NT>
__device__ __forceinline__ void store8(void* p, uint2 v) {
    if (NT) {
        typedef uint32_t v2 __attribute__((ext_vector_type(2)));
        v2 r = {v.x, v.y};
        __builtin_nontemporal_store(r, (v2*)p);
    } else {
        *(uint2*)p = v;
    }
}

// ---------------------------------------------------------------------------
// table writer: the host's per-rank pointer table travels in kernel arguments
// ---------------------------------------------------------------------------
__global__ void table_write_kernel(uint64_t* dst, TableChunk chunk, int n) {
    const int i = threadIdx.x + blockIdx.x * blockDim.x;
    if (i < n) dst[i] = chunk.v[i];
}

// ---------------------------------------------------------------------------
// routing layout
// ---------------------------------------------------------------------------
// One block per global expert e.  The world's selections form a flat list of
// 64-entry words, rank-major with a fixed number of words per rank, so that a
// wave's ballot of "selects e" over one word lists tokens of one source rank in
// ascending order.  (A token is expected to name an expert at most once; if it
// names one twice, each occurrence gets its own row, as in the reference
// kernel, which sends once per k: mooncake_ep_kernel.cu:230,273.)
//   pass 1  ballots of every word -> LDS.  Each block starts at its own offset
//           into the list: all E blocks read the same R*T*K indices, and
//           without the rotation they would all ask the same L2 channel for
//           the same line at the same time.
//   scan    exclusive prefix of the per-word popcounts = packed row of the
//           first hit of each word; rank boundaries give (begin, count).
//   pass 2  ballot bits -> src_info entries and resolved destination routes.
struct LayoutScratch {
    int32_t* row_src;    // [E, R*max]  packed row -> source token slot (rank * max_tokens + token)
    int32_t* counts;     // [E]         recv_count of every global expert
};

template <bool FP8>
__global__ __launch_bounds__(1024) void layout_kernel(const uint64_t* __restrict__ tbl,
                                                       DispatchRoute* __restrict__ routes, LayoutScratch scratch,
                                                       uint32_t stamp, int R, int E, int K, int H, int max_tokens,
                                                       int words_per_rank, int rotate) {
    extern __shared__ unsigned long long lds[];
    const int W = R * words_per_rank;
    unsigned long long* masks = lds;                       // [W]   ballots
    unsigned long long* rank_idx = lds + W;                // [R]   topk_idx address of each rank
    int* wbeg = (int*)(rank_idx + R);                      // [W+1] packed row of each word's first hit
    int* rank_n = wbeg + W + 1;                            // [R]   selections (tokens * K) of each rank
    int* wave_tot = rank_n + R;                            // [16]

    const int e = blockIdx.x;
    const int L = E / R, q = e / L, le = e - q * L;
    // the wave index is wave-uniform: keep it (and all word / rank arithmetic
    // that follows from it) in scalar registers
    const int lane = wave_lane(), wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), nwaves = blockDim.x >> 6;
    const int64_t RM = (int64_t)R * max_tokens;

    // a rank that takes no part in this dispatch receives nothing; routes
    // towards it keep an old stamp and are skipped by the pack kernel
    const uint64_t recv_x = tbl[DF_RECV_X * R + q];
    if (recv_x == 0) {
        if (threadIdx.x == 0) scratch.counts[e] = 0;
        return;
    }
    // the rank table is read once per block, not once per word
    for (int r = threadIdx.x; r < R; r += blockDim.x) {
        rank_n[r] = (int)tbl[DF_NUM_TOKENS * R + r] * K;
        rank_idx[r] = tbl[DF_TOPK_IDX * R + r];
    }
    int32_t* recv_count = (int32_t*)tbl[DF_RECV_COUNT * R + q];
    int32_t* src_info = (int32_t*)tbl[DF_SRC_INFO * R + q] + (int64_t)le * RM;
    int64_t* layout_range = (int64_t*)tbl[DF_LAYOUT_RANGE * R + q] + (int64_t)le * R;
    __syncthreads();

    // An item is a run of up to U consecutive words of one rank; a wave takes
    // IPR items per round and has all their loads in flight before the first ballot.
    constexpr int U = 8, IPR = 4;
    const int items_per_rank = (words_per_rank + U - 1) / U;
    const int items = R * items_per_rank;
    const int start = rotate ? (int)(((long long)e * items) / E) : 0;
    for (int it0 = wave * IPR; it0 < items; it0 += nwaves * IPR) {
        int64_t v[IPR][U];
        int word0[IPR];
#pragma unroll
        for (int a = 0; a < IPR; ++a) {
            word0[a] = -1;
            int item = it0 + a;
            if (item < items) {
                item += start;
                if (item >= items) item -= items;
                const int r = item / items_per_rank, w0 = (item - r * items_per_rank) * U;
                const int n = rank_n[r];
                const int64_t* idx = (const int64_t*)rank_idx[r];
                word0[a] = r * words_per_rank + w0;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int i = (w0 + u) * 64 + lane;
                    v[a][u] = (w0 + u < words_per_rank && i < n) ? idx[i] : -1;
                }
            } else {
#pragma unroll
                for (int u = 0; u < U; ++u) v[a][u] = -1;
            }
        }
#pragma unroll
        for (int a = 0; a < IPR; ++a) {
            if (word0[a] < 0) continue;
            const int w0 = word0[a] % words_per_rank;
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if (w0 + u >= words_per_rank) break;
                const unsigned long long m = __ballot(v[a][u] == (int64_t)e);
                if (lane == 0) masks[word0[a] + u] = m;
            }
        }
    }
    __syncthreads();

    // block-wide exclusive scan of the per-word hit counts
    int carry = 0;
    for (int base = 0; base < W; base += blockDim.x) {
        const int gi = base + threadIdx.x;
        const int c = (gi < W) ? __popcll(masks[gi]) : 0;
        int incl = c;
#pragma unroll
        for (int d = 1; d < 64; d <<= 1) {
            const int up = __shfl_up(incl, d);
            if (lane >= d) incl += up;
        }
        if (lane == 63) wave_tot[wave] = incl;
        __syncthreads();
        int before = carry;
        for (int w2 = 0; w2 < wave; ++w2) before += wave_tot[w2];
        if (gi < W) wbeg[gi] = before + incl - c;
        int total = 0;
        for (int w2 = 0; w2 < nwaves; ++w2) total += wave_tot[w2];
        carry += total;
        __syncthreads();
    }
    // A block holds RM rows.  Distinct experts per token can never exceed that;
    // rows past it (possible only with repeated experts) are dropped.
    const int cap = (int)(RM < 0x7fffffff ? RM : 0x7fffffff);
    if (threadIdx.x == 0) {
        wbeg[W] = carry;
        const int kept = carry < cap ? carry : cap;
        recv_count[le] = kept;
        scratch.counts[e] = kept;
    }
    __syncthreads();
    for (int r = threadIdx.x; r < R; r += blockDim.x) {
        int b = wbeg[r * words_per_rank], b2 = wbeg[(r + 1) * words_per_rank];
        b = b < cap ? b : cap;
        b2 = b2 < cap ? b2 : cap;
        const int c = b2 - b;
        // count in the low half, begin in the high half; an empty pair is 0
        layout_range[r] = c ? (((int64_t)b << 32) | (int64_t)c) : 0;
    }

    // Ballot bits -> rows.  32 words per wave step, one per lane; only words
    // with hits (about one in five for 256 experts) are walked.
    const uint64_t row_bytes = (uint64_t)H * (FP8 ? 1 : 2);
    const uint64_t row0 = recv_x + (uint64_t)le * RM * row_bytes;
    const uint64_t scale0 = FP8 ? tbl[DF_RECV_SCALES * R + q] + (uint64_t)le * (H / 128) * RM * 4 : 0;
    int32_t* row_src = scratch.row_src + (int64_t)e * RM;
    for (int base = wave * 32; base < W; base += nwaves * 32) {
        const int mine = base + (lane & 31);
        const unsigned long long mword = (mine < W) ? masks[mine] : 0;
        const int mbeg = (mine < W) ? wbeg[mine] : 0;
        unsigned int nz = (unsigned int)__ballot(mword != 0);      // lanes 32..63 mirror lanes 0..31
        while (nz) {
            const int j = __builtin_ctz(nz);
            nz &= nz - 1;
            const unsigned long long m = read_lane_u64(mword, j);
            const int wb = __builtin_amdgcn_readlane(mbeg, j);
            if ((m >> lane) & 1ull) {
                const int pos = wb + __popcll(m & ((1ull << lane) - 1ull));
                if (pos < cap) {
                    const int gi = base + j;
                    const int r = gi / words_per_rank, w = gi - r * words_per_rank;
                    const int i = w * 64 + lane;
                    const int t = i / K, k = i - t * K;
                    src_info[pos] = t;
                    row_src[pos] = r * max_tokens + t;
                    DispatchRoute rt;
                    rt.row = row0 + (uint64_t)pos * row_bytes;
                    rt.scale = FP8 ? scale0 + (uint64_t)pos * 4 : 0;
                    rt.stamp = stamp;
                    rt.pad[0] = rt.pad[1] = rt.pad[2] = 0;
                    routes[((int64_t)r * max_tokens + t) * K + k] = rt;
                }
            }
        }
    }
}

// ---------------------------------------------------------------------------
// dispatch pack
// ---------------------------------------------------------------------------
// One wave per (token, 1024-element slab).  Lanes 0..K-1 fetch the K resolved
// destinations; the row slab is read once, quantised in registers and stored
// K times.
struct PackDest {
    uint64_t row;     // byte address of the destination row, 0 = no store
    uint64_t scale;   // byte address of scales[le][0][slot] (fp8)
};

// Where a wave finds its token row.  When every rank's x is the same distance
// from the previous rank's and all ranks hold the same number of tokens, the
// address comes from kernel arguments alone; otherwise from the rank table
// (one more dependent scalar load before the row loads can be issued).
struct PackSource {
    uint64_t x_base;      // rank 0's x when uniform, else 0
    int64_t x_stride;     // bytes between consecutive ranks' x
    int tokens;           // every rank's token count when uniform
};

__device__ __forceinline__ const char* pack_source_row(const uint64_t* __restrict__ tbl, const PackSource& src, int R,
                                                       int H, int r, int t, bool* in_range) {
    if (src.x_base != 0) {
        *in_range = t < src.tokens;
        return (const char*)(src.x_base + (uint64_t)((int64_t)r * src.x_stride)) + (int64_t)t * H * 2;
    }
    *in_range = t < (int)tbl[DF_NUM_TOKENS * R + r];
    return (const char*)tbl[DF_X * R + r] + (int64_t)t * H * 2;
}

struct PackRouteRaw {
    uint4 a, b;
};

// issue the route loads (no dependency on anything but the task index) ...
__device__ __forceinline__ PackRouteRaw pack_route_issue(const DispatchRoute* __restrict__ routes, int K,
                                                         int max_tokens, int r, int t, int lane) {
    PackRouteRaw raw = {make_uint4(0, 0, 0, 0), make_uint4(0, 0, 0, 0)};
    if (lane < K) {
        const uint4* p = (const uint4*)(routes + ((int64_t)r * max_tokens + t) * K + lane);
        raw.a = p[0];
        raw.b = p[1];
    }
    return raw;
}

// ... and consume them after the row loads are in flight.  The empty asm keeps
// the compiler from fetching the stamp first and the rest behind a branch.
__device__ __forceinline__ PackDest pack_route_finish(PackRouteRaw raw, uint32_t stamp, int K, int lane) {
    asm volatile("" : "+v"(raw.a.x), "+v"(raw.a.y), "+v"(raw.a.z), "+v"(raw.a.w), "+v"(raw.b.x));
    const bool ok = (lane < K) && (raw.b.x == stamp);
    PackDest d;
    d.row = ok ? (((uint64_t)raw.a.y << 32) | raw.a.x) : 0;
    d.scale = ok ? (((uint64_t)raw.a.w << 32) | raw.a.z) : 0;
    return d;
}

// fp8, variant 0: a lane owns 16 consecutive elements (32 B in, 16 B out),
// a 128-element scale group is 8 lanes.
template <bool NTL, bool NTS>
__global__ __launch_bounds__(512) void pack_fp8_kernel(const uint64_t* __restrict__ tbl,
                                                        const DispatchRoute* __restrict__ routes, uint32_t stamp,
                                                        PackSource src, float* __restrict__ scale_stage, int R,
                                                        int K, int max_tokens, int H, int slabs, int Tgrid,
                                                        int total_tasks) {
    const int lane = wave_lane();
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    const int n = task / slabs, s = task - n * slabs;
    const int r = n / Tgrid, t = n - r * Tgrid;
    const PackRouteRaw raw = pack_route_issue(routes, K, max_tokens, r, t, lane);
    bool in_range;
    const char* xtok = pack_source_row(tbl, src, R, H, r, t, &in_range);
    if (!in_range) return;

    const int elem0 = s * 1024 + lane * 16;
    const bool active = elem0 < H;
    const char* xrow = xtok + (int64_t)(active ? elem0 : 0) * 2;
    uint4 a = make_uint4(0, 0, 0, 0), b = a;
    if (active) {
        a = load16<NTL>(xrow);
        b = load16<NTL>(xrow + 16);
    }
    const PackDest dst = pack_route_finish(raw, stamp, K, lane);

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
    // the arithmetic of CPU PyTorch for `448.0 / amax` (reciprocal, then times
    // 448) and `amax / 448.0` (true division), both correctly rounded
    const float scale = (1.0f / amax) * 448.0f;
    const float scale_inv = amax / 448.0f;
    uint32_t o[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        int w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j] * scale, f[4 * j + 1] * scale, 0, false);
        w = __builtin_amdgcn_cvt_pk_fp8_f32(f[4 * j + 2] * scale, f[4 * j + 3] * scale, w, true);
        o[j] = (uint32_t)w;
    }
    const uint4 out = make_uint4(o[0], o[1], o[2], o[3]);
    const int64_t scale_off = (int64_t)(elem0 >> 7) * ((int64_t)R * max_tokens) * 4;
    const bool scale_lane = active && ((lane & 7) == 0);
    // staged: the token's scales go to one contiguous row, a second kernel
    // moves them into the column-major output with coalesced stores
    if (scale_stage != nullptr && scale_lane)
        scale_stage[((int64_t)r * max_tokens + t) * (H >> 7) + (elem0 >> 7)] = scale_inv;
    const bool scatter_scales = scale_lane && scale_stage == nullptr;

    for (int k = 0; k < K; ++k) {
        const uint64_t row = read_lane_u64(dst.row, k);
        const uint64_t sc = read_lane_u64(dst.scale, k);
        if (row == 0) continue;
        if (active) store16<NTS>((void*)(row + elem0), out);
        if (scatter_scales) *(float*)(sc + scale_off) = scale_inv;
    }
}

// fp8, variant 1: a lane owns two 8-element pieces 512 elements apart, so both
// 16-byte loads of a wave are unit-stride; a scale group is 16 lanes and the
// stores are 8 bytes per lane.
template <bool NTL, bool NTS>
__global__ __launch_bounds__(512) void pack_fp8_split_kernel(const uint64_t* __restrict__ tbl,
                                                              const DispatchRoute* __restrict__ routes,
                                                              uint32_t stamp, PackSource src,
                                                              float* __restrict__ scale_stage, int R, int K,
                                                              int max_tokens, int H, int slabs, int Tgrid,
                                                              int total_tasks) {
    const int lane = wave_lane();
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    const int n = task / slabs, s = task - n * slabs;
    const int r = n / Tgrid, t = n - r * Tgrid;
    const PackRouteRaw raw = pack_route_issue(routes, K, max_tokens, r, t, lane);
    bool in_range;
    const char* xbase = pack_source_row(tbl, src, R, H, r, t, &in_range);
    if (!in_range) return;

    int elem[2];
    bool active[2];
    uint4 v[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        elem[p] = s * 1024 + p * 512 + lane * 8;
        active[p] = elem[p] < H;
        v[p] = make_uint4(0, 0, 0, 0);
        if (active[p]) v[p] = load16<NTL>(xbase + (int64_t)elem[p] * 2);
    }
    const PackDest dst = pack_route_finish(raw, stamp, K, lane);

    uint2 out[2];
    float scale_inv[2];
#pragma unroll
    for (int p = 0; p < 2; ++p) {
        const uint32_t u[4] = {v[p].x, v[p].y, v[p].z, v[p].w};
        float f[8];
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            f[2 * j] = bf16_lo(u[j]);
            f[2 * j + 1] = bf16_hi(u[j]);
        }
        float amax = 1e-4f;
#pragma unroll
        for (int j = 0; j < 8; ++j) amax = fmaxf(amax, fabsf(f[j]));
        amax = group_max<16>(amax);
        const float scale = (1.0f / amax) * 448.0f;
        scale_inv[p] = amax / 448.0f;
        int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[0] * scale, f[1] * scale, 0, false);
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(f[2] * scale, f[3] * scale, w0, true);
        int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[4] * scale, f[5] * scale, 0, false);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(f[6] * scale, f[7] * scale, w1, true);
        out[p] = make_uint2((uint32_t)w0, (uint32_t)w1);
    }
    const int64_t RM4 = (int64_t)R * max_tokens * 4;
    const bool scale_lane = (lane & 15) == 0;
    if (scale_stage != nullptr && scale_lane) {
#pragma unroll
        for (int p = 0; p < 2; ++p)
            if (active[p]) scale_stage[((int64_t)r * max_tokens + t) * (H >> 7) + (elem[p] >> 7)] = scale_inv[p];
    }
    const bool scatter_scales = scale_lane && scale_stage == nullptr;

    for (int k = 0; k < K; ++k) {
        const uint64_t row = read_lane_u64(dst.row, k);
        const uint64_t sc = read_lane_u64(dst.scale, k);
        if (row == 0) continue;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            if (active[p]) {
                store8<NTS>((void*)(row + elem[p]), out[p]);
                if (scatter_scales) *(float*)(sc + (int64_t)(elem[p] >> 7) * RM4) = scale_inv[p];
            }
        }
    }
}

// bf16: plain row copy, two unit-stride 16-byte pieces per lane.
template <bool NTL, bool NTS>
__global__ __launch_bounds__(512) void pack_bf16_kernel(const uint64_t* __restrict__ tbl,
                                                         const DispatchRoute* __restrict__ routes, uint32_t stamp,
                                                         PackSource src, float* __restrict__ /*scale_stage*/, int R,
                                                         int K, int max_tokens, int H, int slabs, int Tgrid,
                                                         int total_tasks) {
    const int lane = wave_lane();
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    const int n = task / slabs, s = task - n * slabs;
    const int r = n / Tgrid, t = n - r * Tgrid;
    const PackRouteRaw raw = pack_route_issue(routes, K, max_tokens, r, t, lane);
    bool in_range;
    const char* xbase = pack_source_row(tbl, src, R, H, r, t, &in_range);
    if (!in_range) return;

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
    const PackDest dst = pack_route_finish(raw, stamp, K, lane);

    for (int k = 0; k < K; ++k) {
        const uint64_t row = read_lane_u64(dst.row, k);
        if (row == 0) continue;
#pragma unroll
        for (int p = 0; p < 2; ++p)
            if (active[p]) store16<NTS>((void*)(row + off[p]), v[p]);
    }
}

// Staged scales -> column-major output.  kTransposeWaves waves per expert,
// each taking 64 packed rows at a time: a lane learns its row's source token
// slot from the layout kernel's row_src, reads that token's H/128 scales as
// contiguous 16-byte pieces - a batch of them in flight at once - and stores
// them so that the wave writes 64 consecutive floats per scale group.
constexpr int kTransposeWaves = 8;

__global__ __launch_bounds__(256) void scale_transpose_kernel(const uint64_t* __restrict__ tbl,
                                                               const float* __restrict__ scale_stage,
                                                               LayoutScratch scratch, int R, int E, int G,
                                                               int max_tokens, int total_tasks) {
    const int lane = wave_lane();
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    const int e = task / kTransposeWaves, wi = task - e * kTransposeWaves;
    const int L = E / R, q = e / L, le = e - q * L;
    const int64_t RM = (int64_t)R * max_tokens;
    // issued together: the expert's row count, this wave's first source slots
    // (in bounds whatever the count turns out to be) and the output address
    const int32_t* row_src = scratch.row_src + (int64_t)e * RM;
    int row = wi * 64 + lane;
    int slot = (row < RM) ? row_src[row] : 0;
    const int count = scratch.counts[e];
    float* out = (float*)tbl[DF_RECV_SCALES * R + q];
    if (wi * 64 >= count) return;
    out += (int64_t)le * G * RM;

    for (int row0 = wi * 64; row0 < count; row0 += kTransposeWaves * 64) {
        row = row0 + lane;
        const bool valid = row < count;
        if (row0 != wi * 64) slot = valid ? row_src[row] : 0;
        const float* sp = scale_stage + (int64_t)(valid ? slot : 0) * G;
        float* dp = out + row;
        int g = 0;
        if ((G & 3) == 0) {
            constexpr int B = 8;   // 16-byte loads in flight per lane
            for (; g + 4 * B <= G; g += 4 * B) {
                float4 v[B];
#pragma unroll
                for (int j = 0; j < B; ++j) v[j] = *(const float4*)(sp + g + 4 * j);
                if (valid) {
#pragma unroll
                    for (int j = 0; j < B; ++j) {
                        dp[(int64_t)(g + 4 * j + 0) * RM] = v[j].x;
                        dp[(int64_t)(g + 4 * j + 1) * RM] = v[j].y;
                        dp[(int64_t)(g + 4 * j + 2) * RM] = v[j].z;
                        dp[(int64_t)(g + 4 * j + 3) * RM] = v[j].w;
                    }
                }
            }
            for (; g < G; g += 4) {
                const float4 v = *(const float4*)(sp + g);
                if (valid) {
                    dp[(int64_t)(g + 0) * RM] = v.x;
                    dp[(int64_t)(g + 1) * RM] = v.y;
                    dp[(int64_t)(g + 2) * RM] = v.z;
                    dp[(int64_t)(g + 3) * RM] = v.w;
                }
            }
        }
        if (valid)
            for (; g < G; ++g) dp[(int64_t)g * RM] = sp[g];
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
                    rt.src = row0 + (uint64_t)i * H * 2;
                    rt.weight = wt[j];
                    rt.stamp = stamp;
                    rts[(int64_t)t * K + k0 + j] = rt;
                }
            }
        }
    }
}

// One wave per (token, slab of CH * 512 elements).  Lanes 0..K-1 fetch the K
// routes (a masked, inactive or unknown selection reads a zero row with
// weight 0, which leaves the fp32 accumulator unchanged), then every lane
// issues all KMAX * CH 16-byte loads before the first multiply-add.
template <int KMAX, int CH, bool NTL, bool NTS>
__global__ __launch_bounds__(512) void reduce_kernel(const uint64_t* __restrict__ tbl,
                                                      const CombineRoute* __restrict__ routes, uint32_t stamp,
                                                      const void* __restrict__ zero_row, int R, int K,
                                                      int max_tokens, int H, int slabs, int Tgrid, int total_tasks) {
    const int lane = wave_lane();
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    const int n = task / slabs, s = task - n * slabs;
    const int r = n / Tgrid, t = n - r * Tgrid;
    // A token slot beyond the rank's count has only stale routes (zero rows);
    // it is computed like any other and dropped at the store, so that no wave
    // waits for the rank's token count before it can issue its loads.
    const int T = (int)tbl[CF_NUM_TOKENS * R + r];
    char* orow = (char*)tbl[CF_OUT * R + r] + (int64_t)t * H * 2;

    uint4 rt = make_uint4(0, 0, 0, 0);
    if (lane < K) rt = *(const uint4*)(routes + ((int64_t)r * max_tokens + t) * K + lane);
    asm volatile("" : "+v"(rt.x), "+v"(rt.y), "+v"(rt.z), "+v"(rt.w));   // one 16-byte load, no branch on the stamp
    const bool ok = (lane < K) && (rt.w == stamp);
    const uint64_t src = ok ? (((uint64_t)rt.y << 32) | rt.x) : (uint64_t)zero_row;
    const float w = ok ? __uint_as_float(rt.z) : 0.0f;

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
        wk[k] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w), k));
#pragma unroll
        for (int c = 0; c < CH; ++c) v[k][c] = load16<NTL>((const void*)(p + off[c]));
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

__global__ __launch_bounds__(256) void copy_kernel(uint4* __restrict__ dst, const uint4* __restrict__ src, size_t n) {
    size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t stride = (size_t)gridDim.x * blockDim.x;
    for (; i < n; i += stride) dst[i] = src[i];
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

size_t layout_lds_bytes(const Dims& d) {
    const size_t words_per_rank = ((size_t)d.max_tokens * d.K + 63) / 64;
    const size_t W = (size_t)d.R * words_per_rank;
    return W * 8 + (size_t)d.R * 8 + (W + 1) * 4 + (size_t)d.R * 4 + 16 * 4 + 16;
}

hipError_t launch_layout(const uint64_t* d_tbl, DispatchRoute* d_routes, int32_t* d_row_src, int32_t* d_counts,
                         uint32_t stamp, const Dims& d, bool use_fp8, const Tuning& t, hipStream_t stream) {
    const size_t lds = layout_lds_bytes(d);
    if (lds > kMaxLayoutLdsBytes) return hipErrorInvalidValue;
    const int words_per_rank = (int)(((size_t)d.max_tokens * d.K + 63) / 64);
    int block = t.layout_block;
    if (block < 64) block = 64;
    if (block > 1024) block = 1024;
    block &= ~63;
    auto kern = use_fp8 ? layout_kernel<true> : layout_kernel<false>;
    if (lds > 48 * 1024) {
        hipError_t err = hipFuncSetAttribute((const void*)kern, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (err != hipSuccess) return err;
    }
    LayoutScratch scratch{d_row_src, d_counts};
    hipLaunchKernelGGL(kern, dim3(d.E), dim3(block), lds, stream, d_tbl, d_routes, scratch, stamp, d.R, d.E, d.K,
                       d.H, d.max_tokens, words_per_rank, t.layout_rotate);
    return hipGetLastError();
}

static int clamp_waves(int w) { return w < 1 ? 1 : (w > 8 ? 8 : w); }

template <typename Kern>
static hipError_t launch_pack_t(Kern kern, const uint64_t* d_tbl, const DispatchRoute* d_routes, uint32_t stamp,
                                const PackLaunch& pl, float* stage, const Dims& d, const Tuning& t,
                                hipStream_t stream) {
    const int slabs = (d.H + 1023) / 1024;
    const long long total = (long long)d.R * d.Tgrid * slabs;
    if (total <= 0) return hipSuccess;
    if (total > 0x7fffffffll) return hipErrorInvalidValue;
    const int wpb = clamp_waves(t.pack_waves);
    const int blocks = (int)((total + wpb - 1) / wpb);
    PackSource src;
    src.x_base = pl.x_base;
    src.x_stride = pl.x_stride;
    src.tokens = pl.uniform_tokens;
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(wpb * 64), 0, stream, d_tbl, d_routes, stamp, src, stage, d.R, d.K,
                       d.max_tokens, d.H, slabs, d.Tgrid, (int)total);
    return hipGetLastError();
}

hipError_t launch_pack(const uint64_t* d_tbl, const DispatchRoute* d_routes, uint32_t stamp, const PackLaunch& pl,
                       const Dims& d, bool use_fp8, const Tuning& t, bool run_pack, bool run_finish,
                       hipStream_t stream) {
    const bool ntl = t.pack_nt & 1, nts = t.pack_nt & 2;
    float* stage = (use_fp8 && t.scale_mode == 1) ? pl.scale_stage : nullptr;
    hipError_t err = hipSuccess;
    if (run_pack) {
#define MCEP_PACK(KERN)                                                                                \
    (ntl ? (nts ? launch_pack_t(KERN<true, true>, d_tbl, d_routes, stamp, pl, stage, d, t, stream)     \
                : launch_pack_t(KERN<true, false>, d_tbl, d_routes, stamp, pl, stage, d, t, stream))   \
         : (nts ? launch_pack_t(KERN<false, true>, d_tbl, d_routes, stamp, pl, stage, d, t, stream)    \
                : launch_pack_t(KERN<false, false>, d_tbl, d_routes, stamp, pl, stage, d, t, stream)))
    if (!use_fp8) err = MCEP_PACK(pack_bf16_kernel);
    else if (t.pack_variant == 1) err = MCEP_PACK(pack_fp8_split_kernel);
    else err = MCEP_PACK(pack_fp8_kernel);
#undef MCEP_PACK
    }
    if (err != hipSuccess || stage == nullptr || !run_finish) return err;
    const long long total = (long long)d.E * kTransposeWaves;
    const int wpb = 4;
    LayoutScratch scratch{pl.row_src, pl.counts};
    hipLaunchKernelGGL(scale_transpose_kernel, dim3((unsigned)((total + wpb - 1) / wpb)), dim3(wpb * 64), 0, stream,
                       d_tbl, stage, scratch, d.R, d.E, d.H / 128, d.max_tokens, (int)total);
    return hipGetLastError();
}

hipError_t launch_resolve(const uint64_t* d_tbl, CombineRoute* d_routes, uint32_t stamp, const Dims& d,
                          const Tuning& /*t*/, hipStream_t stream) {
    const long long total = (long long)d.E * d.R;
    if (total <= 0) return hipSuccess;
    if (total > 0x7fffffffll) return hipErrorInvalidValue;
    const int wpb = 4;
    const int blocks = (int)((total + wpb - 1) / wpb);
    hipLaunchKernelGGL(resolve_kernel, dim3(blocks), dim3(wpb * 64), 0, stream, d_tbl, d_routes, stamp, d.R, d.E, d.K,
                       d.H, d.max_tokens, (int)total);
    return hipGetLastError();
}

template <int KMAX, int CH>
static hipError_t launch_reduce_t(const uint64_t* d_tbl, const CombineRoute* d_routes, uint32_t stamp,
                                  const void* d_zero_row, const Dims& d, const Tuning& t, hipStream_t stream) {
    const int slabs = (d.H + CH * 512 - 1) / (CH * 512);
    const long long total = (long long)d.R * d.Tgrid * slabs;
    if (total <= 0) return hipSuccess;
    if (total > 0x7fffffffll) return hipErrorInvalidValue;
    const int wpb = clamp_waves(t.combine_waves);
    const int blocks = (int)((total + wpb - 1) / wpb);
    const bool ntl = t.combine_nt & 1, nts = t.combine_nt & 2;
#define MCEP_REDUCE(A, B)                                                                                       \
    hipLaunchKernelGGL((reduce_kernel<KMAX, CH, A, B>), dim3(blocks), dim3(wpb * 64), 0, stream, d_tbl, d_routes, \
                       stamp, d_zero_row, d.R, d.K, d.max_tokens, d.H, slabs, d.Tgrid, (int)total)
    if (ntl && nts) MCEP_REDUCE(true, true);
    else if (ntl) MCEP_REDUCE(true, false);
    else if (nts) MCEP_REDUCE(false, true);
    else MCEP_REDUCE(false, false);
#undef MCEP_REDUCE
    return hipGetLastError();
}

hipError_t launch_reduce(const uint64_t* d_tbl, const CombineRoute* d_routes, uint32_t stamp, const void* d_zero_row,
                         const Dims& d, const Tuning& t, hipStream_t stream) {
    const int ch = t.combine_chunks >= 2 ? 2 : 1;
#define MCEP_K(KMAX)                                                                                    \
    return ch == 2 ? launch_reduce_t<KMAX, 2>(d_tbl, d_routes, stamp, d_zero_row, d, t, stream)         \
                   : launch_reduce_t<KMAX, 1>(d_tbl, d_routes, stamp, d_zero_row, d, t, stream)
    if (d.K <= 1) { MCEP_K(1); }
    if (d.K <= 2) { MCEP_K(2); }
    if (d.K <= 4) { MCEP_K(4); }
    if (d.K <= 6) { MCEP_K(6); }
    if (d.K <= 8) { MCEP_K(8); }
    if (d.K <= 12) { MCEP_K(12); }
    MCEP_K(16);
#undef MCEP_K
}

hipError_t launch_copy(void* dst, const void* src, size_t bytes, hipStream_t stream) {
    const size_t n = bytes / 16;
    if (n == 0) return hipSuccess;
    size_t blocks = (n + 255) / 256;
    if (blocks > 256 * 64) blocks = 256 * 64;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)blocks), dim3(256), 0, stream, (uint4*)dst, (const uint4*)src, n);
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
