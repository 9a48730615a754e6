// gfx950 (CDNA4, wave64) kernels for the low-latency MoE dispatch / combine
// path.  Everything here is HBM-bound byte movement: no matrix cores, every
// payload access is a 16-byte vector load or store that a wave issues over a
// contiguous span of a row.
//
//   layout_kernel   routing layout: per-expert histogram, per-(expert, source
//                   rank) ranges by prefix sum, source-index map and the
//                   (rank, token, k) -> packed-row map.  Restates the count
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
//   resolve_kernel  combine's handle (src_info, layout_range) -> packed row of
//                   each (token, k) (data flow of mooncake_ep_kernel.cu:611-637).
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
// One block per global expert e.  Selections of a source rank are scanned in
// flat (token, k) order, 64 per wave step, so a wave's ballot of "selects e"
// lists that rank's tokens in ascending order (a token names an expert at most
// once; a repeated expert is counted at its first k only).  Pass 1 keeps the
// ballots in LDS and counts per source rank; wave 0 turns the counts into
// begins by prefix sum; pass 2 turns ballot bits into packed rows.
__device__ __forceinline__ unsigned long long select_mask(const int64_t* idx, int n, int K, int e, int word,
                                                          int lane) {
    const int i = word * 64 + lane;
    const int64_t v = (i < n) ? idx[i] : -1;
    bool hit = (v == (int64_t)e);
    if (hit) {
        const int t = i / K, k = i - t * K;
        for (int k2 = 0; k2 < k; ++k2)
            if (idx[t * K + k2] == (int64_t)e) hit = false;
    }
    return __ballot(hit);
}

__global__ __launch_bounds__(1024) void layout_kernel(const uint64_t* __restrict__ tbl,
                                                       int32_t* __restrict__ slot_map, int R, int E, int K,
                                                       int max_tokens, int words_per_rank, int masks_in_lds) {
    extern __shared__ unsigned long long lds[];
    unsigned long long* masks = lds;
    int* cnt = (int*)(lds + (masks_in_lds ? (size_t)R * words_per_rank : 0));
    int* beg = cnt + R;

    const int e = blockIdx.x;
    const int L = E / R, q = e / L, le = e - q * L;
    const int lane = wave_lane(), wave = threadIdx.x >> 6, nwaves = blockDim.x >> 6;
    const int64_t RM = (int64_t)R * max_tokens;

    // a rank that takes no part in this dispatch receives nothing
    if (tbl[DF_RECV_X * R + q] == 0) return;
    int32_t* recv_count = (int32_t*)tbl[DF_RECV_COUNT * R + q];
    int32_t* src_info = (int32_t*)tbl[DF_SRC_INFO * R + q] + (int64_t)le * RM;
    int64_t* layout_range = (int64_t*)tbl[DF_LAYOUT_RANGE * R + q] + (int64_t)le * R;

    for (int r = wave; r < R; r += nwaves) {
        const int n = (int)tbl[DF_NUM_TOKENS * R + r] * K;
        const int64_t* idx = (const int64_t*)tbl[DF_TOPK_IDX * R + r];
        int c = 0;
        const int nwords = (n + 63) >> 6;
        int w = 0;
        for (; w + 4 <= nwords; w += 4) {
            // four independent loads in flight per lane
            unsigned long long m0 = select_mask(idx, n, K, e, w + 0, lane);
            unsigned long long m1 = select_mask(idx, n, K, e, w + 1, lane);
            unsigned long long m2 = select_mask(idx, n, K, e, w + 2, lane);
            unsigned long long m3 = select_mask(idx, n, K, e, w + 3, lane);
            if (masks_in_lds && lane == 0) {
                unsigned long long* mw = masks + (size_t)r * words_per_rank + w;
                mw[0] = m0; mw[1] = m1; mw[2] = m2; mw[3] = m3;
            }
            c += __popcll(m0) + __popcll(m1) + __popcll(m2) + __popcll(m3);
        }
        for (; w < nwords; ++w) {
            unsigned long long m = select_mask(idx, n, K, e, w, lane);
            if (masks_in_lds && lane == 0) masks[(size_t)r * words_per_rank + w] = m;
            c += __popcll(m);
        }
        if (lane == 0) cnt[r] = c;
    }
    __syncthreads();

    if (wave == 0) {
        int running = 0;
        for (int r0 = 0; r0 < R; r0 += 64) {
            const int r = r0 + lane;
            const int v = (r < R) ? cnt[r] : 0;
            int incl = v;
#pragma unroll
            for (int d = 1; d < 64; d <<= 1) {
                const int u = __shfl_up(incl, d);
                if (lane >= d) incl += u;
            }
            const int b = running + incl - v;
            if (r < R) {
                beg[r] = b;
                // count in the low half, begin in the high half; an empty pair is 0
                layout_range[r] = v ? (((int64_t)b << 32) | (int64_t)v) : 0;
            }
            running += __shfl(incl, 63);
        }
        if (lane == 0) recv_count[le] = running;
    }
    __syncthreads();

    for (int r = wave; r < R; r += nwaves) {
        const int n = (int)tbl[DF_NUM_TOKENS * R + r] * K;
        const int64_t* idx = (const int64_t*)tbl[DF_TOPK_IDX * R + r];
        int32_t* smap = slot_map + (int64_t)r * max_tokens * K;
        int run = beg[r];
        const int nwords = (n + 63) >> 6;
        for (int w = 0; w < nwords; ++w) {
            const unsigned long long m =
                masks_in_lds ? masks[(size_t)r * words_per_rank + w] : select_mask(idx, n, K, e, w, lane);
            if (m == 0) continue;
            if ((m >> lane) & 1ull) {
                const int pos = run + __popcll(m & ((1ull << lane) - 1ull));
                const int i = w * 64 + lane;
                const int t = i / K, k = i - t * K;
                src_info[pos] = t;
                smap[i] = pos;
                for (int k2 = k + 1; k2 < K; ++k2)
                    if (idx[t * K + k2] == (int64_t)e) smap[t * K + k2] = pos;
            }
            run += __popcll(m);
        }
    }
}

// ---------------------------------------------------------------------------
// dispatch pack
// ---------------------------------------------------------------------------
// One wave per (token, 1024-element slab).  Lanes 0..K-1 resolve the K
// destination rows; the row slab is read once, quantised in registers and
// stored K times.
struct PackDest {
    uint64_t row;     // byte address of the destination row, 0 = no store
    uint64_t scale;   // byte address of scales[le][0][slot] (fp8)
};

template <bool FP8>
__device__ __forceinline__ PackDest pack_resolve(const uint64_t* __restrict__ tbl,
                                                 const int32_t* __restrict__ slot_map, int R, int E, int K,
                                                 int max_tokens, int H, int r, int t, int lane) {
    PackDest d = {0, 0};
    if (lane < K) {
        const int64_t e64 = ((const int64_t*)tbl[DF_TOPK_IDX * R + r])[t * K + lane];
        if (e64 >= 0 && e64 < (int64_t)E) {
            const int e = (int)e64, L = E / R, q = e / L, le = e - q * L;
            const int slot = slot_map[((int64_t)r * max_tokens + t) * K + lane];
            const int64_t RM = (int64_t)R * max_tokens;
            const uint64_t base = tbl[DF_RECV_X * R + q];
            if (base != 0) {
                d.row = base + (uint64_t)(((int64_t)le * RM + slot) * H) * (FP8 ? 1 : 2);
                if (FP8) d.scale = tbl[DF_RECV_SCALES * R + q] + (uint64_t)((int64_t)le * (H / 128) * RM + slot) * 4;
            }
        }
    }
    return d;
}

// fp8, variant 0: a lane owns 16 consecutive elements (32 B in, 16 B out),
// a 128-element scale group is 8 lanes.
template <bool NTL, bool NTS>
__global__ __launch_bounds__(512) void pack_fp8_kernel(const uint64_t* __restrict__ tbl,
                                                        const int32_t* __restrict__ slot_map, int R, int E, int K,
                                                        int max_tokens, int H, int slabs, int Tgrid,
                                                        int total_tasks) {
    const int lane = wave_lane();
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    const int n = task / slabs, s = task - n * slabs;
    const int r = n / Tgrid, t = n - r * Tgrid;
    if (t >= (int)tbl[DF_NUM_TOKENS * R + r]) return;

    const int elem0 = s * 1024 + lane * 16;
    const bool active = elem0 < H;
    const char* xrow = (const char*)tbl[DF_X * R + r] + ((int64_t)t * H + (active ? elem0 : 0)) * 2;
    uint4 a = make_uint4(0, 0, 0, 0), b = a;
    if (active) {
        a = load16<NTL>(xrow);
        b = load16<NTL>(xrow + 16);
    }
    const PackDest dst = pack_resolve<true>(tbl, slot_map, R, E, K, max_tokens, H, r, t, lane);

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

    for (int k = 0; k < K; ++k) {
        const uint64_t row = read_lane_u64(dst.row, k);
        const uint64_t sc = read_lane_u64(dst.scale, k);
        if (row == 0) continue;
        if (active) store16<NTS>((void*)(row + elem0), out);
        if (scale_lane) *(float*)(sc + scale_off) = scale_inv;
    }
}

// fp8, variant 1: a lane owns two 8-element pieces 512 elements apart, so both
// 16-byte loads of a wave are unit-stride; a scale group is 16 lanes and the
// stores are 8 bytes per lane.
template <bool NTL, bool NTS>
__global__ __launch_bounds__(512) void pack_fp8_split_kernel(const uint64_t* __restrict__ tbl,
                                                              const int32_t* __restrict__ slot_map, int R, int E,
                                                              int K, int max_tokens, int H, int slabs, int Tgrid,
                                                              int total_tasks) {
    const int lane = wave_lane();
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    const int n = task / slabs, s = task - n * slabs;
    const int r = n / Tgrid, t = n - r * Tgrid;
    if (t >= (int)tbl[DF_NUM_TOKENS * R + r]) return;

    const char* xbase = (const char*)tbl[DF_X * R + r] + (int64_t)t * H * 2;
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
    const PackDest dst = pack_resolve<true>(tbl, slot_map, R, E, K, max_tokens, H, r, t, lane);

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

    for (int k = 0; k < K; ++k) {
        const uint64_t row = read_lane_u64(dst.row, k);
        const uint64_t sc = read_lane_u64(dst.scale, k);
        if (row == 0) continue;
#pragma unroll
        for (int p = 0; p < 2; ++p) {
            if (active[p]) {
                store8<NTS>((void*)(row + elem[p]), out[p]);
                if ((lane & 15) == 0) *(float*)(sc + (int64_t)(elem[p] >> 7) * RM4) = scale_inv[p];
            }
        }
    }
}

// bf16: plain row copy, two unit-stride 16-byte pieces per lane.
template <bool NTL, bool NTS>
__global__ __launch_bounds__(512) void pack_bf16_kernel(const uint64_t* __restrict__ tbl,
                                                         const int32_t* __restrict__ slot_map, int R, int E, int K,
                                                         int max_tokens, int H, int slabs, int Tgrid,
                                                         int total_tasks) {
    const int lane = wave_lane();
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    const int n = task / slabs, s = task - n * slabs;
    const int r = n / Tgrid, t = n - r * Tgrid;
    if (t >= (int)tbl[DF_NUM_TOKENS * R + r]) return;

    const char* xbase = (const char*)tbl[DF_X * R + r] + (int64_t)t * H * 2;
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
    const PackDest dst = pack_resolve<false>(tbl, slot_map, R, E, K, max_tokens, H, r, t, lane);

    for (int k = 0; k < K; ++k) {
        const uint64_t row = read_lane_u64(dst.row, k);
        if (row == 0) continue;
#pragma unroll
        for (int p = 0; p < 2; ++p)
            if (active[p]) store16<NTS>((void*)(row + off[p]), v[p]);
    }
}

// ---------------------------------------------------------------------------
// combine
// ---------------------------------------------------------------------------
// One wave per token: for each k, the (expert, source rank) block named by
// layout_range is searched for the token index, 64 src_info entries per step.
__global__ __launch_bounds__(256) void resolve_kernel(const uint64_t* __restrict__ tbl,
                                                       int32_t* __restrict__ slot_map, int R, int E, int K,
                                                       int max_tokens, int Tgrid, int total_tasks) {
    const int lane = wave_lane();
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    const int r = task / Tgrid, t = task - r * Tgrid;
    if (t >= (int)tbl[CF_NUM_TOKENS * R + r]) return;
    const int L = E / R;
    const int64_t RM = (int64_t)R * max_tokens;
    const int64_t* idx = (const int64_t*)tbl[CF_TOPK_IDX * R + r] + (int64_t)t * K;
    int32_t* smap = slot_map + ((int64_t)r * max_tokens + t) * K;

    for (int k = 0; k < K; ++k) {
        const int64_t e64 = idx[k];
        int found = -1;
        if (e64 >= 0 && e64 < (int64_t)E) {
            const int e = (int)e64, q = e / L, le = e - q * L;
            const int64_t* lrp = (const int64_t*)tbl[CF_LAYOUT_RANGE * R + q];
            const int32_t* sip = (const int32_t*)tbl[CF_SRC_INFO * R + q];
            if (lrp != nullptr && sip != nullptr) {
                const int64_t lr = lrp[(int64_t)le * R + r];
                int count = (int)(lr & 0xffffffffll);
                int begin = (int)(lr >> 32);
                if (begin < 0 || count < 0 || (int64_t)begin + count > RM) count = 0;   // malformed handle
                sip += (int64_t)le * RM + begin;
                for (int i0 = 0; i0 < count; i0 += 64) {
                    const int i = i0 + lane;
                    const bool hit = (i < count) && (sip[i] == t);
                    const unsigned long long m = __ballot(hit);
                    if (m) {
                        found = begin + i0 + (__ffsll((long long)m) - 1);
                        break;
                    }
                }
            }
        }
        if (lane == 0) smap[k] = found;
    }
}

// One wave per (token, slab of CH * 512 elements).  Lanes 0..KMAX-1 resolve
// the K source rows (a masked, inactive or unknown selection reads a zero row
// with weight 0, which leaves the fp32 accumulator unchanged), then every
// lane issues all KMAX * CH 16-byte loads before the first multiply-add.
template <int KMAX, int CH, bool NTL, bool NTS>
__global__ __launch_bounds__(512) void reduce_kernel(const uint64_t* __restrict__ tbl,
                                                      const int32_t* __restrict__ slot_map,
                                                      const void* __restrict__ zero_row, int R, int E, int K,
                                                      int max_tokens, int H, int slabs, int Tgrid, int total_tasks) {
    const int lane = wave_lane();
    const int task = __builtin_amdgcn_readfirstlane(blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6));
    if (task >= total_tasks) return;
    const int n = task / slabs, s = task - n * slabs;
    const int r = n / Tgrid, t = n - r * Tgrid;
    if (t >= (int)tbl[CF_NUM_TOKENS * R + r]) return;

    uint64_t src = (uint64_t)zero_row;
    float w = 0.0f;
    if (lane < K) {
        const int64_t e64 = ((const int64_t*)tbl[CF_TOPK_IDX * R + r])[(int64_t)t * K + lane];
        if (e64 >= 0 && e64 < (int64_t)E) {
            const int e = (int)e64, L = E / R, q = e / L, le = e - q * L;
            const int slot = slot_map[((int64_t)r * max_tokens + t) * K + lane];
            const int live = ((const int32_t*)tbl[CF_ACTIVE * R + r])[q];   // skip experts on inactive ranks
            const uint64_t base = tbl[CF_X * R + q];
            if (slot >= 0 && live != 0 && base != 0) {
                src = base + (uint64_t)(((int64_t)le * R * max_tokens + slot) * H) * 2;
                w = ((const float*)tbl[CF_TOPK_W * R + r])[(int64_t)t * K + lane];
            }
        }
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
        wk[k] = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w), k));
#pragma unroll
        for (int c = 0; c < CH; ++c) v[k][c] = load16<NTL>((const void*)(p + off[c]));
    }

    char* orow = (char*)tbl[CF_OUT * R + r] + (int64_t)t * H * 2;
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

size_t layout_lds_bytes(const Dims& d, bool* masks_in_lds) {
    const size_t words_per_rank = ((size_t)d.max_tokens * d.K + 63) / 64;
    const size_t fixed = (size_t)d.R * 2 * sizeof(int);
    const size_t with_masks = (size_t)d.R * words_per_rank * 8 + fixed;
    const bool fits = with_masks <= 60 * 1024;
    if (masks_in_lds) *masks_in_lds = fits;
    return fits ? with_masks : fixed;
}

hipError_t launch_layout(const uint64_t* d_tbl, int32_t* d_slot_map, const Dims& d, const Tuning& t,
                         hipStream_t stream) {
    bool in_lds = false;
    const size_t lds = layout_lds_bytes(d, &in_lds);
    const int words_per_rank = (int)(((size_t)d.max_tokens * d.K + 63) / 64);
    int block = t.layout_block;
    if (block < 64) block = 64;
    if (block > 1024) block = 1024;
    block &= ~63;
    hipLaunchKernelGGL(layout_kernel, dim3(d.E), dim3(block), lds, stream, d_tbl, d_slot_map, d.R, d.E, d.K,
                       d.max_tokens, words_per_rank, in_lds ? 1 : 0);
    return hipGetLastError();
}

template <typename Kern>
static hipError_t launch_wave_tasks(Kern kern, int waves_per_block, long long total_tasks, hipStream_t stream,
                                    const uint64_t* d_tbl, const int32_t* d_slot_map, const Dims& d, int slabs) {
    if (total_tasks <= 0) return hipSuccess;
    if (total_tasks > 0x7fffffffll) return hipErrorInvalidValue;
    const int blocks = (int)((total_tasks + waves_per_block - 1) / waves_per_block);
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(waves_per_block * 64), 0, stream, d_tbl, d_slot_map, d.R, d.E, d.K,
                       d.max_tokens, d.H, slabs, d.Tgrid, (int)total_tasks);
    return hipGetLastError();
}

static int clamp_waves(int w) { return w < 1 ? 1 : (w > 8 ? 8 : w); }

hipError_t launch_pack(const uint64_t* d_tbl, const int32_t* d_slot_map, float* /*d_scale_stage*/, const Dims& d,
                       bool use_fp8, const Tuning& t, hipStream_t stream) {
    const int slabs = (d.H + 1023) / 1024;
    const long long total = (long long)d.R * d.Tgrid * slabs;
    const int wpb = clamp_waves(t.pack_waves);
    const bool ntl = t.nontemporal & 1, nts = t.nontemporal & 2;
#define MCEP_PACK(KERN)                                                                                      \
    (ntl ? (nts ? launch_wave_tasks(KERN<true, true>, wpb, total, stream, d_tbl, d_slot_map, d, slabs)       \
                : launch_wave_tasks(KERN<true, false>, wpb, total, stream, d_tbl, d_slot_map, d, slabs))     \
         : (nts ? launch_wave_tasks(KERN<false, true>, wpb, total, stream, d_tbl, d_slot_map, d, slabs)      \
                : launch_wave_tasks(KERN<false, false>, wpb, total, stream, d_tbl, d_slot_map, d, slabs)))
    if (!use_fp8) return MCEP_PACK(pack_bf16_kernel);
    if (t.pack_variant == 1) return MCEP_PACK(pack_fp8_split_kernel);
    return MCEP_PACK(pack_fp8_kernel);
#undef MCEP_PACK
}

hipError_t launch_resolve(const uint64_t* d_tbl, int32_t* d_slot_map, const Dims& d, const Tuning& /*t*/,
                          hipStream_t stream) {
    const long long total = (long long)d.R * d.Tgrid;
    if (total <= 0) return hipSuccess;
    const int wpb = 4;
    const int blocks = (int)((total + wpb - 1) / wpb);
    hipLaunchKernelGGL(resolve_kernel, dim3(blocks), dim3(wpb * 64), 0, stream, d_tbl, d_slot_map, d.R, d.E, d.K,
                       d.max_tokens, d.Tgrid, (int)total);
    return hipGetLastError();
}

template <int KMAX, int CH>
static hipError_t launch_reduce_t(const uint64_t* d_tbl, const int32_t* d_slot_map, const void* d_zero_row,
                                  const Dims& d, const Tuning& t, hipStream_t stream) {
    const int slabs = (d.H + CH * 512 - 1) / (CH * 512);
    const long long total = (long long)d.R * d.Tgrid * slabs;
    if (total <= 0) return hipSuccess;
    if (total > 0x7fffffffll) return hipErrorInvalidValue;
    const int wpb = clamp_waves(t.combine_waves);
    const int blocks = (int)((total + wpb - 1) / wpb);
    const bool ntl = t.nontemporal & 1, nts = t.nontemporal & 2;
#define MCEP_REDUCE(A, B)                                                                                       \
    hipLaunchKernelGGL((reduce_kernel<KMAX, CH, A, B>), dim3(blocks), dim3(wpb * 64), 0, stream, d_tbl, d_slot_map, \
                       d_zero_row, d.R, d.E, d.K, d.max_tokens, d.H, slabs, d.Tgrid, (int)total)
    if (ntl && nts) MCEP_REDUCE(true, true);
    else if (ntl) MCEP_REDUCE(true, false);
    else if (nts) MCEP_REDUCE(false, true);
    else MCEP_REDUCE(false, false);
#undef MCEP_REDUCE
    return hipGetLastError();
}

hipError_t launch_reduce(const uint64_t* d_tbl, const int32_t* d_slot_map, const void* d_zero_row, const Dims& d,
                         const Tuning& t, hipStream_t stream) {
    const int ch = t.combine_chunks >= 2 ? 2 : 1;
#define MCEP_K(KMAX)                                                                             \
    return ch == 2 ? launch_reduce_t<KMAX, 2>(d_tbl, d_slot_map, d_zero_row, d, t, stream)       \
                   : launch_reduce_t<KMAX, 1>(d_tbl, d_slot_map, d_zero_row, d, t, stream)
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
