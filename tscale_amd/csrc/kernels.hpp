// Parameter blocks and host-side launchers shared between the kernel files and the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "wg_map.h"

namespace tsattn {

struct DecodeParams {
    const uint8_t *q;
    int64_t q_pitch;
    const float *q_scale;
    float q_scale_const;
    const uint8_t *k, *v;
    int64_t seq_stride, head_stride, tok_stride;
    const float *ks, *vs;
    int64_t s_seq_stride, s_head_stride;
    float ks_const, vs_const;
    const int32_t *cache_len;
    int64_t window;
    float slope;
    int n_heads;
    int n_splits;
    float *part_acc; // [seq][head][split][d]
    float *part_ml;  // [seq][head][split][2] = running max, sum
    void *dbg;
    int64_t dbg_pitch;
    float *out;           // final output; written by the split kernel itself when there is one split and no append
    // fused append (all null/0 when not used): the new token's row goes to row cache_len[seq] of the cache, the
    // token attends as if cache_len were one more, and the merge kernel bumps cache_len afterwards
    const uint8_t *k_new, *v_new;
    int64_t new_pitch;
    const float *ks_new, *vs_new;
    int32_t *cache_len_rw;
    int max_len;
    int32_t *seq_done; // [n_seqs] arrival counters of the single-split fused append, zero between launches
    // fused KVProduct of the output (kv_out null = off)
    const uint8_t *kv_k;
    int64_t kv_k_pitch;
    uint8_t *kv_out;
    int64_t kv_out_pitch;
    int kv_rep;
    float kv_mult;
};

hipError_t launch_decode(const DecodeParams &p, int dtype, int head_dim, bool qbf16, int n_seqs, float *out, hipStream_t st);

struct PrefillParams {
    const uint8_t *q, *k, *v;
    int64_t q_pitch, k_pitch, v_pitch;
    const float *qs, *ks, *vs;
    int64_t scale_pitch;
    float qs_const, ks_const, vs_const;
    const float *k_global_scale;
    const int32_t *span_start, *span_finish; // n_parts arrays, span_part_stride entries apart (part i: every row's i-th span)
    const int32_t *span_tiles; // optional per-128-row summary (SPAN_TILE_* layout below), one after the other for the parts
    int n_parts;
    int64_t span_part_stride;
    float slope;
    void *out;
    int64_t out_pitch;
    float *sum_weight_log;
    void *dbg;
    int64_t dbg_pitch;
    int n_tokens;
    int n_heads;
    int period_tiles; // query tiles per period of equal span structure, 0 = unknown (launch order only)
    // optional fused consumer (kv_out != nullptr): KVProduct of the f32 result with the rows of kv_k; out may then be null
    const uint8_t *kv_k;
    int64_t kv_k_pitch;
    uint8_t *kv_out;
    int64_t kv_out_pitch;
    int kv_rep;
    float kv_mult;
    // optional scratch of the long-range kernel (vt != nullptr selects it): room for V as f16, transposed
    void *vt;
    int64_t vt_pitch; // halves per (head, x) row
    int64_t ks_pitch; // long-range kernel only: floats between the heads of ks (set by its launcher)
    WgMap map;        // set by the launcher: how workgroup ids map to (head, query tile)
};

hipError_t launch_prefill(const PrefillParams &p, int dtype, int head_dim, int out_dtype, hipStream_t st);

// The long-range kernel (head width 128, no ALiBi slope) and its scratch: V as f16 [head][x][vt_pitch], the column of
// token t at VT_PAD + t (tokens of every 16 reordered), every other column zero.
constexpr int VT_PAD = 32;
inline int64_t prefill_long_vt_pitch(int64_t n_tokens) { return (n_tokens + 63) / 64 * 64 + 256; }
size_t prefill_long_workspace_bytes(int64_t n_tokens, int n_heads, int head_dim);
hipError_t launch_prefill_long(const PrefillParams &p, int dtype, int out_dtype, hipStream_t st);
hipError_t prepare_prefill_long(); // once per device, at handle creation: lets the kernels ask for their LDS

hipError_t launch_quantize_rows(int src_dtype, int dst_dtype, const void *src, int64_t src_pitch, int64_t n_rows,
                                int n_heads, int head_dim, void *dst, int64_t dst_pitch, float *scale,
                                int64_t scale_pitch, hipStream_t st);

// Layout of one entry of the span summary (32 int32 per 128 query rows): the workgroup's key range, then for each
// of its four 32-row waves the extremes of the rows' spans and whether every row has keys.
constexpr int SPAN_TILE_INTS = 32;
constexpr int SPAN_TILE_MIN_A = 0, SPAN_TILE_MAX_B = 1; // over rows that have keys; MIN_A > MAX_B if none has
constexpr int SPAN_TILE_WAVE0 = 4, SPAN_TILE_WAVE_INTS = 5; // per wave: min_a, max_a, min_b, max_b, all_have_keys
// Combines attention results over disjoint (or repeated) key sets of the same rows, each with the zero vector in it
struct MergeParams {
    int n_parts;
    int64_t n_tokens;
    int n_heads, head_dim;
    const float *part_out;   // part i: part_out + i * part_out_stride, rows of part_out_pitch floats
    int64_t part_out_pitch, part_out_stride;
    const float *part_swl;   // part i: part_swl + i * part_swl_stride, [head][scale_pitch]
    int64_t scale_pitch, part_swl_stride;
    void *out;               // f32 or f16 rows of out_pitch bytes
    int64_t out_pitch;
    float *swl;              // optional [head][scale_pitch]
};
hipError_t launch_merge_lookups(const MergeParams &p, bool out_f16, hipStream_t st);

hipError_t launch_build_span_tiles(int64_t n_tokens, const int32_t *span_start, const int32_t *span_finish, int32_t *tiles, hipStream_t st);

hipError_t launch_build_spans(int n_seqs, const int32_t *seq_offset, int64_t n_tokens, const uint8_t *doc_start_flag,
                              int64_t window, int32_t *span_start, int32_t *span_finish, hipStream_t st);

struct AppendParams {
    const uint8_t *k_new, *v_new;
    int64_t new_pitch;
    const float *ks_new, *vs_new;
    uint8_t *k, *v;
    int64_t seq_stride, head_stride, tok_stride;
    float *ks, *vs;
    int64_t s_seq_stride, s_head_stride;
    int32_t *cache_len;
    int max_len;
    int n_heads;
    int head_dim;
};

hipError_t launch_cache_append(const AppendParams &p, int n_seqs, hipStream_t st);

// n int32 at p become zero (a kernel: memset nodes are avoided in code a caller may capture into a graph)
hipError_t launch_zero_i32(int32_t *p, int n, hipStream_t st);

struct ProduceParams {
    const void *src;
    int64_t src_pitch; // elements per row
    int64_t n_rows;
    int n_heads;
    const int32_t *pos;
    const float *rope;
    int64_t rope_len;
    float rotate_dir, vec_scale, scale_mult;
    uint8_t *dst;
    int64_t dst_pitch;
    float *scale;
    int64_t scale_pitch, scale_row_stride;
    int relu;
    int src_planes;
    int64_t src_plane_stride;
    int rope_heads;       // heads below it are rotated (set to n_heads when all are)
    int scale_head_begin, scale_head_count;
    float *resid;
    int64_t resid_pitch;
    float resid_scale;
};

hipError_t launch_rope_normalize(const ProduceParams &p, int dst_dtype, int head_dim, bool src_i32, hipStream_t st);
void fill_rope_table(int width, int64_t max_len, float *table);

struct KvProductParams {
    const uint8_t *k;
    int64_t k_pitch;   // bytes
    const void *val;
    int64_t val_pitch; // elements
    int64_t n_rows;
    int n_heads, head_dim, rep;
    float mult;
    uint8_t *kv;
    int64_t kv_pitch;  // bytes
};

hipError_t launch_kv_product(const KvProductParams &p, bool val_f16, hipStream_t st);

struct GemmParams {
    const uint8_t *a, *w;
    int64_t a_pitch, w_pitch; // bytes
    int64_t m, n, k;
    int mode;                 // tsattn_mm_mode
    float scale;
    void *out;
    int64_t out_pitch;        // elements
    void *workspace;          // optional room for split-K partial sums (few rows)
    int64_t workspace_bytes;
    int64_t split_stride;     // set by the launcher: elements between the parts' planes
    // optional last step (ep_head_dim != 0): the producer applied to the int32 result, as launch_rope_normalize would
    // be with src = the result; src, src_pitch, n_rows, n_heads and the planes are filled in by the launcher
    ProduceParams ep;
    int ep_head_dim, ep_dst_dtype;
};

hipError_t launch_matmul_i8(const GemmParams &p, hipStream_t st, int *planes_out);
hipError_t prepare_matmul_i8(); // once per device, before the first product

struct HeadParams {
    int64_t n_rows;
    // embedding
    int dim;
    const int32_t *labels;
    int labels_per_row;
    const uint8_t *embed;
    int64_t embed_pitch, n_labels;
    float embed_scale;
    float *state;
    int64_t state_pitch;
    // softmax
    int64_t n;
    const int32_t *src;
    int src_planes;
    int64_t src_plane_stride, src_pitch;
    float scale;
    const float *bias;
    float *prob;
    int64_t prob_pitch;
    int32_t *argmax;
    // sampling
    float temperature;
    const uint32_t *rnd;
    int64_t rnd_pitch;
    uint64_t seed, offset;
};

hipError_t launch_embed_rows(const HeadParams &p, hipStream_t st);
hipError_t launch_softmax_rows(const HeadParams &p, hipStream_t st);
hipError_t launch_sample_rows(const HeadParams &p, hipStream_t st);

struct FillParams {
    const int32_t *seq_offset;
    const uint8_t *k_src, *v_src;
    int64_t pitch;
    const float *ks_src, *vs_src;
    int64_t scale_pitch;
    uint8_t *k, *v;
    int64_t seq_stride, head_stride, tok_stride;
    float *ks, *vs;
    int64_t s_seq_stride, s_head_stride;
    int32_t *cache_len;
    int max_len;
    int n_seqs;
    int n_heads;
    int head_dim;
    int64_t n_tokens;
};

hipError_t launch_cache_fill(const FillParams &p, hipStream_t st);

} // namespace tsattn
