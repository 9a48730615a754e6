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
    int pack_variant = 0;      // 0: 32 B/lane loads, 16 B stores; 1: two coalesced 16 B loads, 8 B stores
    int pack_waves = 4;        // waves per block in the pack kernel
    int scale_mode = 0;        // 0: scatter scales from the pack kernel; 1: staged + transposing pass
    int combine_chunks = 1;    // 16-byte chunks per lane in the combine kernel
    int combine_waves = 4;     // waves per block in the combine kernel
    int nontemporal = 0;       // bit 0: streaming loads, bit 1: streaming stores
};

hipError_t launch_table_write(uint64_t* d_tbl, const uint64_t* h_tbl, int n_words, hipStream_t stream);

hipError_t launch_layout(const uint64_t* d_tbl, int32_t* d_slot_map, const Dims& d, const Tuning& t, hipStream_t stream);
hipError_t launch_pack(const uint64_t* d_tbl, const int32_t* d_slot_map, float* d_scale_stage, const Dims& d,
                       bool use_fp8, const Tuning& t, hipStream_t stream);
hipError_t launch_resolve(const uint64_t* d_tbl, int32_t* d_slot_map, const Dims& d, const Tuning& t,
                          hipStream_t stream);
hipError_t launch_reduce(const uint64_t* d_tbl, const int32_t* d_slot_map, const void* d_zero_row, const Dims& d,
                         const Tuning& t, hipStream_t stream);
hipError_t launch_copy(void* dst, const void* src, size_t bytes, hipStream_t stream);
hipError_t launch_fill_u32(void* dst, uint32_t value, size_t words, hipStream_t stream);

size_t layout_lds_bytes(const Dims& d, bool* masks_in_lds);

}  // namespace mcep
