/*
 * CPU oracle for mooncake-ep's low-latency dispatch / combine contract.
 *
 * TEST INFRASTRUCTURE ONLY.  Nothing that ships (the HIP library, the Python
 * package) may link, import or call this file.  It exists so that the parity
 * tests, the smoke check and the bench's cpu_baseline leg have an independent
 * scalar restatement of the algorithm to compare against and to time.
 *
 * Every function cites the reference lines it restates (paths relative to the
 * reference checkout):
 *   K  = mooncake-ep/src/mooncake_ep_kernel.cu
 *   U  = mooncake-ep/include/mooncake_ep_utils.cuh
 *   PY = mooncake-wheel/mooncake/mooncake_ep_buffer.py
 *   TU = mooncake-wheel/tests/ep_test_utils.py
 *
 * Where the CUDA kernel and the PyTorch statements of the contract disagree,
 * this oracle follows the PyTorch statements (deterministic order, `/ 448`
 * scales, zero for an empty layout entry), except for the combine
 * accumulation, which follows the kernel (fp32, fused multiply-add, k order).
 *
 * World layout used by every entry point (all arrays contiguous, rank-major):
 *   R ranks, E experts, L = E / R local experts per rank, RM = R * max_tokens
 *   topk_idx   int64  [R, Tmax, K]     rows >= num_tokens[r] are ignored
 *   x          bf16   [R, Tmax, H]     (as uint16 bit patterns)
 *   recv_x     fp8/bf16 [R, L, RM, H]
 *   scales     f32    [R, L, H/128, RM]   (the physical, column-major layout
 *                                          behind PY:479-487's transpose)
 *   recv_count i32    [R, L]
 *   src_info   i32    [R, L, RM]
 *   layout_range i64  [R, L, R]
 *
 * What pins each function (independently of this file's own formulas); no
 * function here is "parity unpinned":
 *   oracle_f32_to_e4m3fn / e4m3fn_to_f32   torch's float8_e4m3fn cast on all 65 536 bf16 values and all 256
 *                                          codes, OCP known answers            tests/test_oracle_fp8.py
 *   oracle_f32_to_bf16                     torch's bf16 cast, ties and NaN     tests/test_oracle_fp8.py
 *   oracle_quantise_rows                   the reference's per_token_cast_to_fp8 (TU:42-47) run by torch,
 *                                          amax floor, round trip bound        tests/test_oracle_fp8.py
 *   oracle_layout / oracle_dispatch        brute-force triple loop, bincount closed form, the structured-row
 *                                          checks of the reference's tests, per-rank torch statement of
 *                                          PY:787-869, committed fixtures      tests/test_oracle_contract.py,
 *                                                                              tests/test_golden.py
 *   oracle_invert_handle / oracle_combine  closed forms x * sum(w) and x * sum(factor * w), float64 gather-sum
 *                                          within one bf16 ulp, linearity      tests/test_oracle_contract.py
 *   oracle_cast_back                       per_token_cast_back (TU:50-53) and the grid test's mock expert run
 *                                          by torch, every fp8 code            tests/test_oracle_cast_back.py
 *   oracle_buffer_size_hint                the value the reference's layout arithmetic gives for its own
 *                                          test shapes                         tests/test_oracle_contract.py
 *
 * Build: see oracle/Makefile (gcc -O2 -ffp-contract=off -fopenmp).
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

#define ORACLE_API __attribute__((visibility("default")))

/* ------------------------------------------------------------------------ */
/* scalar conversions                                                        */
/* ------------------------------------------------------------------------ */

static inline uint32_t f32_bits(float f) { uint32_t u; memcpy(&u, &f, 4); return u; }
static inline float bits_f32(uint32_t u) { float f; memcpy(&f, &u, 4); return f; }

/* bf16 -> f32 is exact: the 16 bits are the top half of the f32. */
static inline float bf16_to_f32(uint16_t h) { return bits_f32((uint32_t)h << 16); }

/* f32 -> bf16, round to nearest even; NaN maps to the quiet NaN 0x7FC0
 * (the convention of torch's bfloat16 cast; K:750 uses __float2bfloat16,
 * which is RNE as well). */
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u = f32_bits(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return 0x7fc0;
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

/* shift right by s with round-to-nearest-even */
static inline uint32_t rne_shift(uint32_t m, int s) {
    if (s <= 0) return m << (-s);
    if (s > 31) return 0;
    uint32_t q = m >> s;
    uint32_t rem = m & ((1u << s) - 1u);
    uint32_t half = 1u << (s - 1);
    if (rem > half || (rem == half && (q & 1u))) q++;
    return q;
}

/* f32 -> OCP fp8 e4m3fn (1-4-3, bias 7, no infinities, 0x7F/0xFF = NaN),
 * round to nearest even.  A magnitude that rounds above 448 becomes NaN, as
 * in torch's float8_e4m3fn cast, which PY:699-701 and TU:47 call.  (The CUDA
 * kernel saturates instead, mooncake_ep_device.h:98-100; the two agree on
 * every value the amax scaling can produce.)  Written from the format's
 * definition with integer arithmetic, independent of any library routine. */
static inline uint8_t f32_to_e4m3fn(float f) {
    uint32_t b = f32_bits(f);
    uint8_t sign = (uint8_t)((b >> 24) & 0x80u);
    uint32_t a = b & 0x7fffffffu;
    if (a > 0x7f800000u) return sign | 0x7f;        /* NaN */
    if (a == 0x7f800000u) return sign | 0x7f;       /* Inf: no encoding */
    int e = (int)(a >> 23) - 127;                   /* unbiased exponent */
    if (e < -11) return sign;                       /* < 2^-11: rounds to 0 */
    uint32_t mant = (a & 0x7fffffu) | 0x800000u;    /* 1.23 fixed point */
    uint32_t enc;
    if (e < -6) {
        /* subnormal: quantum 2^-9, value = mant * 2^(e-23) */
        uint32_t q = rne_shift(mant, 14 - e);       /* 0..8; 8 == 2^-6 */
        enc = q;
    } else {
        uint32_t q = rne_shift(mant, 20);           /* 8..16 */
        if (q == 16) { q = 8; e += 1; }
        if (e > 8) return sign | 0x7f;
        enc = ((uint32_t)(e + 7) << 3) | (q & 7u);
        if (enc > 0x7e) return sign | 0x7f;
    }
    return sign | (uint8_t)enc;
}

static inline float e4m3fn_to_f32(uint8_t v) {
    uint32_t sign = (uint32_t)(v & 0x80u) << 24;
    uint32_t ex = (v >> 3) & 0xfu, m = v & 7u;
    float mag;
    if (ex == 0xf && m == 7) return bits_f32(sign | 0x7fc00000u);
    if (ex == 0) mag = ldexpf((float)m, -9);
    else mag = ldexpf(1.0f + (float)m / 8.0f, (int)ex - 7);
    return bits_f32(f32_bits(mag) | sign);
}

/* exported scalar/array forms so the tests can sweep them against torch */
ORACLE_API void oracle_f32_to_e4m3fn(const float* in, uint8_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = f32_to_e4m3fn(in[i]);
}
ORACLE_API void oracle_e4m3fn_to_f32(const uint8_t* in, float* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = e4m3fn_to_f32(in[i]);
}
ORACLE_API void oracle_f32_to_bf16(const float* in, uint16_t* out, int64_t n) {
    for (int64_t i = 0; i < n; ++i) out[i] = f32_to_bf16(in[i]);
}

/* ------------------------------------------------------------------------ */
/* per-128 quantisation of one row                                           */
/* ------------------------------------------------------------------------ */

/* PY:694-703 == TU:42-47 (amax clamp 1e-4, payload f32(x) * (448.0 / amax)
 * cast to e4m3fn, stored scale amax / 448.0) with the kernel's group size and
 * amax floor (K:183-186, K:243-252).  The arithmetic is the one CPU PyTorch
 * performs for those two expressions: `448.0 / tensor` is Tensor.__rtruediv__,
 * i.e. reciprocal() * 448.0 - two roundings, different from the IEEE quotient
 * 448 / amax (which K:252 computes) in about a quarter of all groups - while
 * `tensor / 448.0` is a true IEEE division (K:252 multiplies by 1/448
 * instead).  tests/test_oracle_fp8.py pins both against torch itself.
 * NaN elements do not raise amax (fmaxf, K:247); they encode as fp8 NaN. */
/* Which of the reference's two statements of the scale arithmetic is restated: 0 (default) the PyTorch
 * one above, 1 the CUDA kernel's own - scale = 448 / amax as one IEEE division (K:252; nvcc divides
 * correctly rounded unless told otherwise, and the reference's build does not tell it) and the stored
 * scale amax * (1 / 448) with the constant folded at compile time (K:184, K:252).  The two differ in
 * the last bit of either scale for about a quarter of all amax values.
 * tests/test_oracle_fp8.py pins mode 1 against numpy's float32 division and product. */
static int g_fp8_arith = 0;

ORACLE_API void oracle_set_fp8_arith(int mode) { g_fp8_arith = mode ? 1 : 0; }

static void quantise_row(const uint16_t* x, int H, uint8_t* q, float* scales, int64_t scale_stride) {
    const int native = g_fp8_arith;
    for (int g = 0; g < H / 128; ++g) {
        float amax = 1e-4f;
        for (int j = 0; j < 128; ++j) amax = fmaxf(amax, fabsf(bf16_to_f32(x[g * 128 + j])));
        const float scale = native ? 448.0f / amax : (1.0f / amax) * 448.0f;
        const float scale_inv = native ? amax * (1.0f / 448.0f) : amax / 448.0f;
        for (int j = 0; j < 128; ++j) q[g * 128 + j] = f32_to_e4m3fn(bf16_to_f32(x[g * 128 + j]) * scale);
        scales[(int64_t)g * scale_stride] = scale_inv;
    }
}

ORACLE_API void oracle_quantise_rows(const uint16_t* x, int64_t rows, int H, uint8_t* q, float* scales) {
    /* scales come back row-major [rows, H/128] */
    for (int64_t i = 0; i < rows; ++i) quantise_row(x + i * H, H, q + i * H, scales + i * (H / 128), 1);
}

/* ------------------------------------------------------------------------ */
/* routing layout                                                            */
/* ------------------------------------------------------------------------ */

/* Order and ranges as PY:787-817: for each local expert, source ranks in
 * ascending order, within a rank tokens in ascending order.  The contract has
 * a token name an expert at most once; should it name one twice, each
 * occurrence gets its own row in k order, as the kernel sends once per k
 * (K:230, K:273) - PY:797-802 would count such a token once.
 * layout_range = (begin << 32) |
 * count with count in the low half (U:160-169, PY:1023-1024) and 0 for an
 * empty pair (PY:817); src_info[row] = token index at the source (K:231,
 * K:446, PY:838).  recv_count = sum of counts (K:430, PY:831).  Rows at and
 * beyond recv_count are not written.  A source rank with src_present[r] == 0
 * sends nothing (K:424-429: an inactive, silent rank yields zero tokens).
 * slot_map[r,t,k] = row of that selection in its expert's packed block, or -1
 * for topk_idx == -1: the inverse map a one-hop combine needs. */
ORACLE_API void oracle_layout(int R, int E, int K, int Tmax, int max_tokens, const int32_t* num_tokens,
                              const int64_t* topk_idx, const int32_t* src_present, int32_t* recv_count,
                              int64_t* layout_range, int32_t* src_info, int32_t* slot_map) {
    const int L = E / R;
    const int64_t RM = (int64_t)R * max_tokens;
    if (slot_map)
        for (int64_t i = 0; i < (int64_t)R * Tmax * K; ++i) slot_map[i] = -1;
    for (int e = 0; e < E; ++e) {
        const int q = e / L, le = e % L;   /* K:276-277 */
        int begin = 0;
        for (int r = 0; r < R; ++r) {
            int count = 0;
            const int T = (src_present && !src_present[r]) ? 0 : num_tokens[r];
            for (int t = 0; t < T; ++t) {
                const int64_t* row = topk_idx + ((int64_t)r * Tmax + t) * K;
                for (int k = 0; k < K; ++k) {
                    if (row[k] != e) continue;
                    if ((int64_t)begin + count >= RM) continue;   /* only duplicates can overflow: dropped */
                    const int slot = begin + count;
                    src_info[((int64_t)q * L + le) * RM + slot] = t;
                    if (slot_map) slot_map[((int64_t)r * Tmax + t) * K + k] = slot;
                    ++count;
                }
            }
            layout_range[((int64_t)q * L + le) * R + r] = count ? (((int64_t)begin << 32) | (int64_t)count) : 0;
            begin += count;
        }
        recv_count[q * L + le] = begin;
    }
}

/* ------------------------------------------------------------------------ */
/* dispatch                                                                  */
/* ------------------------------------------------------------------------ */

/* Whole-world dispatch: layout (above) + payload.  bf16 mode is a row gather
 * (K:267, PY:835-837); fp8 mode quantises each source row once (K:233-264)
 * and places payload and scales at the packed row (K:452-465; scales
 * column-major with stride RM between groups, K:460-464, PY:479-487). */
ORACLE_API void oracle_dispatch(int R, int E, int K, int Tmax, int max_tokens, int H, int use_fp8,
                                const int32_t* num_tokens, const uint16_t* x, const int64_t* topk_idx,
                                const int32_t* src_present, void* recv_x, float* scales, int32_t* recv_count,
                                int64_t* layout_range, int32_t* src_info, int32_t* slot_map_out) {
    const int G = H / 128;
    const int64_t RM = (int64_t)R * max_tokens;
    int32_t* slot_map = slot_map_out ? slot_map_out : (int32_t*)malloc(sizeof(int32_t) * (size_t)R * Tmax * K);
    oracle_layout(R, E, K, Tmax, max_tokens, num_tokens, topk_idx, src_present, recv_count, layout_range, src_info,
                  slot_map);
#pragma omp parallel
    {
        uint8_t* qrow = (uint8_t*)malloc((size_t)H);
        float* srow = (float*)malloc(sizeof(float) * (size_t)G);
#pragma omp for schedule(static)
        for (int64_t n = 0; n < (int64_t)R * Tmax; ++n) {
            const int r = (int)(n / Tmax), t = (int)(n % Tmax);
            const int T = (src_present && !src_present[r]) ? 0 : num_tokens[r];
            if (t >= T) continue;
            const uint16_t* xr = x + n * H;
            if (use_fp8) quantise_row(xr, H, qrow, srow, 1);
            for (int k = 0; k < K; ++k) {
                const int64_t e = topk_idx[n * K + k];
                const int slot = slot_map[n * K + k];
                if (e < 0 || slot < 0) continue;
                const int64_t row = (int64_t)e * RM + slot;   /* == (q*L + le)*RM + slot */
                if (use_fp8) {
                    memcpy((uint8_t*)recv_x + row * H, qrow, (size_t)H);
                    float* sc = scales + (int64_t)e * G * RM + slot;
                    for (int g = 0; g < G; ++g) sc[(int64_t)g * RM] = srow[g];
                } else {
                    memcpy((uint16_t*)recv_x + row * H, xr, (size_t)H * 2);
                }
            }
        }
        free(qrow);
        free(srow);
    }
    if (!slot_map_out) free(slot_map);
}

/* ------------------------------------------------------------------------ */
/* combine                                                                   */
/* ------------------------------------------------------------------------ */

/* Inverse of the handle: for every packed row named by (layout_range,
 * src_info) find the (rank, token, k) it serves.  This is the data flow of
 * the kernel's combine SEND (K:611-637: rows [offset, offset+count) of local
 * expert le go to rank dst at position global_expert * max + src_info[row]),
 * turned into a lookup table. */
ORACLE_API void oracle_invert_handle(int R, int E, int K, int Tmax, int max_tokens, const int32_t* num_tokens,
                                     const int64_t* topk_idx, const int32_t* src_info, const int64_t* layout_range,
                                     int32_t* slot_map) {
    const int64_t RM = (int64_t)R * max_tokens;
    for (int64_t i = 0; i < (int64_t)R * Tmax * K; ++i) slot_map[i] = -1;
    for (int e = 0; e < E; ++e) {
        for (int r = 0; r < R; ++r) {
            const int64_t lr = layout_range[(int64_t)e * R + r];
            const int count = (int)(lr & 0xffffffffLL), begin = (int)(lr >> 32);   /* U:171-178, PY:1023-1024 */
            for (int i = begin; i < begin + count; ++i) {
                const int t = src_info[(int64_t)e * RM + i];
                if (t < 0 || t >= num_tokens[r]) continue;   /* PY:1031-1032 */
                const int64_t* row = topk_idx + ((int64_t)r * Tmax + t) * K;
                for (int k = 0; k < K; ++k)
                    if (row[k] == e) slot_map[((int64_t)r * Tmax + t) * K + k] = i;
            }
        }
    }
}

/* K:711-753: per token, for k = 0..K-1 with topk_idx >= 0 and the expert's
 * owner rank active (K:728-732), acc += f32(expert_out_row) * w[t,k] in fp32,
 * then RNE to bf16 (K:750).  nvcc contracts the multiply-add at K:742 into a
 * fused multiply-add; use_fma = 1 restates that, use_fma = 0 rounds the
 * product first (the two differ by at most one bf16 ulp after rounding in
 * the cases tested).  active is [R(owner view), R]; NULL means all ones.
 * A selection whose row cannot be found in the handle contributes nothing. */
ORACLE_API void oracle_combine(int R, int E, int K, int Tmax, int max_tokens, int H, int use_fma,
                               const int32_t* num_tokens, const uint16_t* expert_out, const int64_t* topk_idx,
                               const float* topk_weights, const int32_t* src_info, const int64_t* layout_range,
                               const int32_t* active, uint16_t* out) {
    const int L = E / R;
    const int64_t RM = (int64_t)R * max_tokens;
    int32_t* slot_map = (int32_t*)malloc(sizeof(int32_t) * (size_t)R * Tmax * K);
    oracle_invert_handle(R, E, K, Tmax, max_tokens, num_tokens, topk_idx, src_info, layout_range, slot_map);
#pragma omp parallel
    {
        float* acc = (float*)malloc(sizeof(float) * (size_t)H);
#pragma omp for schedule(static)
        for (int64_t n = 0; n < (int64_t)R * Tmax; ++n) {
            const int r = (int)(n / Tmax), t = (int)(n % Tmax);
            if (t >= num_tokens[r]) continue;
            for (int j = 0; j < H; ++j) acc[j] = 0.0f;
            for (int k = 0; k < K; ++k) {
                const int64_t e = topk_idx[n * K + k];
                if (e < 0 || e >= E) continue;   /* ids outside [0, E) name no expert */
                if (active && !active[(int64_t)r * R + e / L]) continue;
                const int slot = slot_map[n * K + k];
                if (slot < 0) continue;
                const uint16_t* src = expert_out + ((int64_t)e * RM + slot) * H;
                const float w = topk_weights[n * K + k];
                if (use_fma)
                    for (int j = 0; j < H; ++j) acc[j] = fmaf(bf16_to_f32(src[j]), w, acc[j]);
                else
                    for (int j = 0; j < H; ++j) acc[j] = acc[j] + bf16_to_f32(src[j]) * w;
            }
            uint16_t* o = out + n * H;
            for (int j = 0; j < H; ++j) o[j] = f32_to_bf16(acc[j]);
        }
        free(acc);
    }
    free(slot_map);
}

/* Size hint: BufferPair in mooncake_ep_buffer.h:29-63 sums, over two buffers,
 * two signalling areas of E ints and two data areas of E * max * (2*16 + 2H)
 * bytes; get_ep_buffer_size_hint (:197-203) returns that total. */
ORACLE_API uint64_t oracle_buffer_size_hint(int max_tokens, int hidden, int num_ranks, int num_experts) {
    (void)num_ranks;
    uint64_t signaling = (uint64_t)num_experts * 4u;
    uint64_t data = (uint64_t)num_experts * (uint64_t)max_tokens * (2u * 16u + (uint64_t)hidden * 2u);
    return 4u * signaling + 4u * data;
}

/* The consumer of the packed layout.  per_token_cast_back
 * (mooncake-wheel/tests/ep_test_utils.py:50-53) and dequantize_fp8
 * (mooncake-ep/tests/test_ep_grid.py:43-48): f32(fp8) * scale per 128-element
 * group, rounded to bf16; then, when factor != NULL, the grid test's mock
 * expert (test_ep_grid.py:168-173): f32(that bf16) * factor[expert], rounded to
 * bf16 again (a bf16 tensor times a scalar is computed in fp32 and rounded
 * once).  recv_x is [E, RM, H] bytes (fp8) or bf16 when scales == NULL; scales
 * is the physical column-major [E, H/128, RM]; only rows below count[e] are
 * read or written. */
ORACLE_API void oracle_cast_back(int E, int RM, int H, const void* recv_x, const float* scales,
                                 const int32_t* count, const float* factor, uint16_t* out) {
    const int G = H / 128;
#pragma omp parallel for schedule(dynamic)
    for (int e = 0; e < E; ++e) {
        const int64_t rows = count[e] < 0 ? 0 : (count[e] > RM ? RM : count[e]);
        for (int64_t row = 0; row < rows; ++row) {
            const int64_t base = ((int64_t)e * RM + row) * H;
            for (int j = 0; j < H; ++j) {
                uint16_t v;
                if (scales) {
                    const float s = scales[((int64_t)e * G + j / 128) * RM + row];
                    v = f32_to_bf16(e4m3fn_to_f32(((const uint8_t*)recv_x)[base + j]) * s);
                } else {
                    v = ((const uint16_t*)recv_x)[base + j];
                }
                if (factor) v = f32_to_bf16(bf16_to_f32(v) * factor[e]);
                out[base + j] = v;
            }
        }
    }
}
