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
    CF_COUNT
};

constexpr int kMaxTopK = 16;          // the reference caps top-k at 11 (mooncake_ep_kernel.cu:487,773)
constexpr int kTableChunk = 384;      // table words one writer launch carries in its kernel arguments
constexpr size_t kZeroRowBytes = 64 * 1024;   // zero row that masked selections read: hidden <= 32768

struct TableChunk {
    uint64_t v[kTableChunk];
};

// What the routing kernels hand to the data kernels: one fully resolved entry
// per (rank, token, k) selection.  An entry is valid for the launch whose
// stamp it carries, so entries that no routing thread visits (masked or
// out-of-range experts, selections absent from a handle) need no clearing pass.
struct DispatchRoute {      // 32 bytes
    uint64_t row;           // byte address of the destination payload row
    uint64_t scale;         // byte address of scales[le][0][row] (fp8)
    uint32_t stamp;
    uint32_t pad[3];
};

struct CombineRoute {       // 16 bytes
    uint64_t src;           // byte address of the expert-output row
    float weight;
    uint32_t stamp;
};

struct Dims {
    int R;            // logical ranks
    int E;            // experts
    int K;            // top-k
    int H;            // hidden
    int max_tokens;   // num_max_dispatch_tokens_per_rank
    int Tgrid;        // max over ranks of T_r (grid extent in tokens per rank)
};

// Tuning knobs, settable at run time for measurement sweeps.
struct Tuning {
    int layout_block = 1024;   // threads per expert block in the layout kernel
    int layout_rotate = 1;     // start each expert block at its own offset into the selection list
    int pack_variant = 0;      // 0: 32 B/lane loads, 16 B stores; 1: two coalesced 16 B loads, 8 B stores
    int pack_waves = 4;        // waves per block in the pack kernel
    int pack_nt = 1;           // bit 0: streaming (nontemporal) loads, bit 1: streaming stores
    int pack_uniform = 1;      // take x addresses from kernel arguments when the ranks' x are evenly spaced
    int scale_mode = 1;        // 0: scatter scales from the pack kernel; 1: staged + transposing pass
    int combine_chunks = 1;    // 16-byte chunks per lane in the combine kernel
    int combine_waves = 4;     // waves per block in the combine kernel
    int combine_nt = 3;        // bit 0: streaming loads, bit 1: streaming stores
};

// Per-launch inputs of the pack kernel beyond the rank table.
struct PackLaunch {
    uint64_t x_base = 0;        // nonzero: rank r's x is x_base + r * x_stride and every rank has uniform_tokens
    int64_t x_stride = 0;
    int uniform_tokens = 0;
    float* scale_stage = nullptr;   // [R * max_tokens, H / 128] staging rows for fp8 scales
    int32_t* row_src = nullptr;     // [E, R * max_tokens] packed row -> source token slot, from the layout kernel
    int32_t* counts = nullptr;      // [E] rows per expert, from the layout kernel
};

hipError_t launch_table_write(uint64_t* d_tbl, const uint64_t* h_tbl, int n_words, hipStream_t stream);

hipError_t launch_layout(const uint64_t* d_tbl, DispatchRoute* d_routes, int32_t* d_row_src, int32_t* d_counts,
                         uint32_t stamp, const Dims& d, bool use_fp8, const Tuning& t, hipStream_t stream);
hipError_t launch_pack(const uint64_t* d_tbl, const DispatchRoute* d_routes, uint32_t stamp, const PackLaunch& pl,
                       const Dims& d, bool use_fp8, const Tuning& t, bool run_pack, bool run_finish,
                       hipStream_t stream);
hipError_t launch_resolve(const uint64_t* d_tbl, CombineRoute* d_routes, uint32_t stamp, const Dims& d,
                          const Tuning& t, hipStream_t stream);
hipError_t launch_reduce(const uint64_t* d_tbl, const CombineRoute* d_routes, uint32_t stamp, const void* d_zero_row,
                         const Dims& d, const Tuning& t, hipStream_t stream);
hipError_t launch_copy(void* dst, const void* src, size_t bytes, hipStream_t stream);
hipError_t launch_fill_u32(void* dst, uint32_t value, size_t words, hipStream_t stream);

// selections (R * max_tokens * K) the layout kernel can hold ballots for in LDS
constexpr size_t kMaxLayoutLdsBytes = 144 * 1024;
size_t layout_lds_bytes(const Dims& d);

}  // namespace mcep
