/*
 * tsattn.h -- C ABI of the MI355X (gfx950) implementation of TScale's quantized attention.
 *
 * Plain C: pointers, sizes and a stream handle; no C++ or framework types cross this boundary.
 * All data pointers are DEVICE pointers unless stated otherwise.  Every call that takes a stream is
 * asynchronous on that stream (pass the hipStream_t as void*, NULL = the default stream), never
 * synchronises, never allocates and never reads device data on the host, so it can be captured
 * into a HIP graph.  A handle belongs to one device and one host thread at a time, and calls on one handle must not
 * overlap on the device (one stream, or ordered streams): decode keeps split partials and arrival counters in it.
 *
 * Reference lines are given relative to the reference's code/ directory.
 *
 * Attention definition (per sequence, head, query row `from`):
 *     keys   to in [span_start[from], span_finish[from]]   (inclusive; finish < start = no keys)
 *     acc    = sum_x q[from][x] * k[to][x]                 (int8: exact int32; e4m3: fp32 MFMA sum)
 *     dp     = acc * ks[to] * sqrtf(1/d)*(0.5f/0.693147f) * qs[from] - slope * (from - to)
 *     m      = max(0, max_to dp)                           (a zero vector of logit 0 always takes part)
 *     l      = exp2(-m) + sum_to exp2(dp - m)
 *     out[x] = sum_to exp2(dp - m) * vs[to] * v[to][x] / l
 *     sum_weight_log = m + log2(l)
 */
#ifndef TSATTN_H
#define TSATTN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef struct tsattn_ctx *tsattn_handle_t;

enum tsattn_status {
    TSATTN_OK = 0,
    TSATTN_ERR_BAD_ARG = 1,     /* null pointer, negative size, misaligned pitch */
    TSATTN_ERR_UNSUPPORTED = 2, /* head_dim other than 64/128, unknown dtype */
    TSATTN_ERR_HIP = 3,         /* the HIP runtime reported an error; see tsattn_last_error */
    TSATTN_ERR_SCRATCH = 4      /* sizes exceed what the handle was created for */
};

enum tsattn_dtype { TSATTN_I8 = 0, TSATTN_E4M3 = 1 };               /* Q/K/V element type */
enum tsattn_out_dtype { TSATTN_OUT_F32 = 0, TSATTN_OUT_F16 = 1 };   /* prefill output type */
enum tsattn_src_dtype { TSATTN_SRC_F32 = 0, TSATTN_SRC_BF16 = 1, TSATTN_SRC_I32 = 2 };  /* producer input types */
enum tsattn_q_dtype { TSATTN_Q_8BIT = 0, TSATTN_Q_BF16 = 1 };       /* decode query type */

/* Sizes the handle's one-time scratch is provisioned for (decode split partials). */
typedef struct tsattn_config {
    int device;            /* HIP device ordinal */
    int max_seqs;          /* decode: sequences per call */
    int max_heads;
    int max_head_dim;      /* 64 or 128 */
    int max_splits;        /* decode: KV splits per (sequence, head); 0 = library default */
} tsattn_config;

/* Context lifetime.  Replaces the per-context arena of the reference
 * (TAttentionComputeCtx::AllocateCuda, gpt/compute/gpt_cuda.cu:231-302): the only allocation the
 * library ever makes happens in tsattn_create. */
size_t tsattn_scratch_bytes(const tsattn_config *cfg);
int tsattn_create(const tsattn_config *cfg, tsattn_handle_t *out);
int tsattn_destroy(tsattn_handle_t h);
/* Text of the last error on the calling thread (never NULL).  The reference aborts instead
 * (Y_VERIFY, util/eden_core.h:111). */
const char *tsattn_last_error(void);

/* ---------------------------------------------------------------------------------------------
 * Prefill.  Replaces
 *   GPU: CudaCall(c, Fp8Att)...(scaleQV, QK, QV, QVscale)(VT)(AttSpans, AttSpanPtr, AlibiSlope)
 *        .Write(&ValLookup, &SumWeightLog)              gpt/compute/gpt_cuda.cu:503-507
 *        and the Fp16Att int8 variant                    gpt/compute/gpt_cuda.cu:511-515
 *        (kernels gpt/compute/gpt_att_fp8.cuh:43-248, gpt_att_fp16.cuh:120-318)
 *   CPU: TAttentionComputer::ComputeValLookup            gpt/compute/gpt_cpu.cpp:391-441, call :633
 * Unlike Fp8Att, V is taken in the same [token][head*d] layout as Q and K: no transposed copy
 * (gpt_cuda.cu:501) is needed.
 */
#define TSATTN_PREFILL_MAX_KV_PITCH ((int64_t)8 << 20)
#define TSATTN_PREFILL_LONG_SPAN 6144   /* span_len_hint from which a workspace is used: measured equal to the standard kernel at 4096 keys per row, 7-10 % faster from 8192 on */
typedef struct tsattn_prefill_args {
    int dtype;                 /* tsattn_dtype of q, k, v */
    int out_dtype;             /* tsattn_out_dtype */
    int64_t n_tokens;          /* all sequences of the batch concatenated */
    int n_heads;
    int head_dim;              /* 64 or 128 */
    const void *q, *k, *v;     /* [n_tokens][n_heads*head_dim] 8-bit */
    int64_t q_pitch, k_pitch, v_pitch;   /* row pitch in bytes, multiple of 16; k_pitch and v_pitch at most
                                            TSATTN_PREFILL_MAX_KV_PITCH */
    const float *q_scale, *k_scale, *v_scale; /* [n_heads][n_tokens] or NULL = the constant below */
    int64_t scale_pitch;       /* floats between heads */
    float q_scale_const, k_scale_const, v_scale_const;
    const float *k_global_scale; /* optional device float multiplied into every key scale
                                    (the QV matrix scale, gpt_cuda.cu:476) */
    const int32_t *span_start;   /* [n_tokens] inclusive first key of each row */
    const int32_t *span_finish;  /* [n_tokens] inclusive last key; < start = row sees no key */
    float alibi_slope;
    void *out;                   /* [n_tokens][n_heads*head_dim] f32 or f16 */
    int64_t out_pitch;           /* bytes */
    float *sum_weight_log;       /* optional [n_heads][n_tokens] (pitch scale_pitch) */
    void *debug_qk_acc;          /* optional raw QK^T accumulators, [n_heads][n_tokens][debug_pitch]
                                    int32 (int8 inputs) or f32 (e4m3); only in-span pairs are written */
    int64_t debug_pitch;         /* elements per (head, from) row of debug_qk_acc */
    const int32_t *span_tiles;   /* optional: what tsattn_build_span_tiles made from THESE span arrays (per 128 query
                                    rows the key range the rows need, per 32 rows the extremes of their spans); the
                                    kernel then starts loading K and V without first reducing the spans itself.
                                    NULL = derive it in the kernel.  Same result either way. */
    int64_t causal_period;       /* scheduling hint, 0 = none: rows t and t + causal_period have spans of equal
                                    length and spans grow with t inside a period (a batch of equal-length
                                    sequences under a wide causal window, as the reference's fixed-length
                                    fragments are).  Only the order in which work is launched depends on it,
                                    never the result; a value the kernel cannot use is ignored. */
    /* Optional fused consumer (kv_out == NULL = off): KVProduct of the result with each token's K vector, as
     * tsattn_kv_product(k = kv_k, value = out, mult = kv_mult) would make it from an f32 `out` afterwards, bit for
     * bit (the batch form of cpu_infer.cpp:511, :320-337; on the GPU the reference does it in its own kernel,
     * gpt/compute/gpt_combiner.cuh:13-37).  dtype must be int8 and out_dtype f32 (TSATTN_ERR_UNSUPPORTED otherwise:
     * make the two calls); `out` may then be NULL (the result itself is not written) and debug_qk_acc must be. */
    const void *kv_k;          /* int8 [n_tokens][n_heads*head_dim], row pitch kv_k_pitch bytes, 4-byte aligned */
    int64_t kv_k_pitch;
    void *kv_out;              /* int8 [n_tokens][n_heads*kv_rep*head_dim], row pitch kv_out_pitch bytes, 16-byte aligned */
    int64_t kv_out_pitch;
    int kv_rep;                /* 1..4 */
    float kv_mult;
    /* Optional scratch for rows with long spans (NULL = none).  With at least tsattn_prefill_workspace_bytes(n_tokens,
     * n_heads, head_dim) bytes here (16-byte aligned) and span_len_hint >= TSATTN_PREFILL_LONG_SPAN, head_dim 128 and no
     * ALiBi slope (nor debug_qk_acc, nor the fused KVProduct), the
     * call first writes V once as f16 with the value scales folded in, transposed, into the workspace, and the attention
     * kernel streams K and that copy through LDS without touching them in registers (the reference keeps such a
     * transposed copy of V too: Transpose, gpt_cuda.cu:501, VT of TAttentionComputeCtx).  Same result within the
     * output tolerance; the workspace holds nothing between calls.  span_len_hint: the typical number of keys of a
     * row -- the layer's attention width clipped to the sequence length (gpt/model_params/model_dim.h:83-91); 0 =
     * unknown.  Only the choice of kernel depends on it. */
    void *workspace;
    int64_t workspace_bytes;
    int64_t span_len_hint;
    /* Rows with several spans (TAttentionInfo allows any number per row, gpt/att/att.h:24-47; the reference's kernels walk
     * a list of key ranges per query block, att.h:95-181): n_span_parts > 1 says that span_start and span_finish hold that
     * many arrays of n_tokens entries, span_part_stride entries apart -- part i is every row's i-th span, finish < start
     * where a row has fewer -- and span_tiles (if given) one summary after the other, tsattn_span_tiles_count(n_tokens)
     * entries each.  One launch, one softmax over all keys of all of a row's spans, a key that lies in c of them counted c
     * times, as the CPU loop over the spans counts it (gpt_cpu.cpp:405-436).  0 or 1: one span per row.  At most 64. */
    int n_span_parts;
    int64_t span_part_stride;
} tsattn_prefill_args;

int tsattn_prefill(tsattn_handle_t h, const tsattn_prefill_args *a, void *stream);
/* Bytes of tsattn_prefill_args.workspace that let a call of this size take the long-span kernel (0: that kernel does
 * not serve this head_dim). */
size_t tsattn_prefill_workspace_bytes(int64_t n_tokens, int n_heads, int head_dim);

/* ---------------------------------------------------------------------------------------------
 * Decode of one new token per sequence over a KV cache.  Replaces
 *   ComputeValLookup(att.AttentionWidth, att.AlibiSlope, dims, kvCache, qk, &valLookup)
 *                                                        gpt/train/cpu_infer.cpp:413-460, call :509
 * The cache is planar: element (seq, head, to, x) lives at
 *   cache + seq*seq_stride + head*head_stride + to*tok_stride + x      (bytes)
 * and its row scale at  scale + seq*s_seq_stride + head*s_head_stride + to   (floats).
 * cache_len[seq] counts valid rows INCLUDING the current token, which the caller appended first
 * (cpu_infer.cpp:506); the token attends to rows cache_len-2 ... cache_len-1-min(cache_len-1, window),
 * or to itself only when window == 0 (cpu_infer.cpp:423-431).
 */
typedef struct tsattn_decode_args {
    int dtype;                 /* tsattn_dtype of the cache (and of q when q_dtype == TSATTN_Q_8BIT) */
    int q_dtype;               /* tsattn_q_dtype; BF16 queries are quantised per head with the absmax
                                  rule (scale = absmax/127 or /256) before the dot products */
    int n_seqs, n_heads, head_dim;
    const void *q;             /* [n_seqs][n_heads*head_dim] */
    int64_t q_pitch;           /* bytes per sequence */
    const float *q_scale;      /* [n_seqs][n_heads] or NULL = constant; ignored for BF16 queries */
    float q_scale_const;
    const void *k_cache, *v_cache;
    int64_t seq_stride, head_stride, tok_stride; /* bytes; tok_stride multiple of 16 */
    const float *k_scale, *v_scale;              /* NULL = constant */
    int64_t s_seq_stride, s_head_stride;         /* floats */
    float k_scale_const, v_scale_const;
    const int32_t *cache_len;  /* device [n_seqs] */
    int max_len;               /* host-side upper bound of cache_len (sizes the grid) */
    int64_t window;
    float alibi_slope;
    float *out;                /* [n_seqs][n_heads*head_dim] f32 */
    int n_splits;              /* KV splits per (seq, head); 0 = choose from max_len */
    void *debug_qk_acc;        /* optional [n_seqs][n_heads][debug_pitch] int32 / f32 */
    int64_t debug_pitch;
    /* Optional fused append.  With k_new non-NULL the call does what tsattn_cache_append followed by tsattn_decode
     * would do with the same arguments (kvCache.AddVectors then ComputeValLookup, cpu_infer.cpp:506-509), in one
     * launch (one split: short windows) or two instead of three or four: cache_len is then the length BEFORE the
     * append and is updated by the call, and the caches, scale planes and cache_len must be writable.  Such calls
     * use counters in the handle: calls on one handle must not overlap on the device (one stream, or ordered).  Not available with window == 0 (the token would
     * attend to the row being written): make the two calls then. */
    const void *k_new, *v_new; /* [n_seqs][n_heads*head_dim] 8-bit */
    int64_t new_pitch;         /* bytes per sequence, multiple of 16 */
    const float *k_scale_new, *v_scale_new; /* [n_seqs][n_heads]; NULL = leave the scale planes untouched */
    /* Optional fused consumer (kv_out == NULL = off): KVProduct of the result with the token's K vector, as
     * tsattn_kv_product(k = kv_k, value = out, mult = kv_mult) would make it from `out` afterwards (cpu_infer.cpp:511,
     * :320-337); `out` is written as well. */
    const void *kv_k;          /* int8 [n_seqs][n_heads*head_dim], row pitch kv_k_pitch bytes, 4-byte aligned */
    int64_t kv_k_pitch;
    void *kv_out;              /* int8 [n_seqs][n_heads*kv_rep*head_dim], row pitch kv_out_pitch bytes */
    int64_t kv_out_pitch;
    int kv_rep;                /* 1..4 */
    float kv_mult;
} tsattn_decode_args;

int tsattn_decode(tsattn_handle_t h, const tsattn_decode_args *a, void *stream);

/* tsattn_decode for callers that cannot allocate device memory: code under HIP graph capture that has no handle yet,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference.  Same arguments, same
 * kernels and the same results as tsattn_decode, but no handle: the split partials and arrival counters live in an array
 * that is part of the library's device image (about 8.1 MiB per GPU the library runs on, held until the process ends),
 * and the call -- the first one on a device included -- makes no hipMalloc / hipFree or other allocating call.  It runs
 * on the calling thread's current device; `stream` must belong to it.
 * Limits (TSATTN_ERR_SCRATCH beyond them): n_seqs <= TSATTN_STATIC_MAX_SEQS and n_seqs * n_heads * splits <=
 * TSATTN_STATIC_MAX_PARTS, where splits is n_splits, or with n_splits == 0 what the library chooses (never more than
 * fits).  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two threads) race;
 * order them. */
#define TSATTN_STATIC_MAX_PARTS 16384
#define TSATTN_STATIC_MAX_SEQS 1024
int tsattn_decode_static(const tsattn_decode_args *a, void *stream);

/* Append one token per sequence to the cache at row cache_len[seq], then increment cache_len[seq]
 * on the device.  Replaces TAttentionVecHistory::AddVectors, gpt/train/cpu_infer.cpp:403-408
 * (call :506).  k_new, v_new: [n_seqs][n_heads*head_dim] 8-bit; *_scale_new: [n_seqs][n_heads]. */
typedef struct tsattn_append_args {
    int n_seqs, n_heads, head_dim;
    const void *k_new, *v_new;
    int64_t new_pitch;         /* bytes per sequence */
    const float *k_scale_new, *v_scale_new; /* NULL = leave the scale planes untouched */
    void *k_cache, *v_cache;
    int64_t seq_stride, head_stride, tok_stride;
    float *k_scale, *v_scale;
    int64_t s_seq_stride, s_head_stride;
    int32_t *cache_len;        /* device [n_seqs], updated in place */
    int max_len;               /* rows per (seq, head) plane; a full cache is left unchanged */
} tsattn_append_args;

int tsattn_cache_append(tsattn_handle_t h, const tsattn_append_args *a, void *stream);

/* Append a whole prefill batch to the cache: sequence s owns tokens [seq_offset[s], seq_offset[s+1])
 * of the [n_tokens][n_heads*head_dim] K and V arrays (the layout tsattn_prefill reads); they are
 * written to cache rows cache_len[s], cache_len[s]+1, ... and cache_len[s] grows by their count.
 * Same result as TAttentionVecHistory::AddVectors once per token, which is how the reference feeds a
 * prompt to its cache (gpt/train/cpu_infer.cpp:403-408, token loop :586-600).  Rows that would land
 * at or beyond max_len are dropped. */
typedef struct tsattn_fill_args {
    int n_seqs, n_heads, head_dim;
    int64_t n_tokens;
    const int32_t *seq_offset; /* device [n_seqs+1], ascending, seq_offset[n_seqs] <= n_tokens */
    const void *k, *v;         /* [n_tokens][n_heads*head_dim] 8-bit */
    int64_t pitch;             /* bytes per token row */
    const float *k_scale, *v_scale; /* [n_heads][scale_pitch] planes; NULL = leave the cache's scale planes untouched */
    int64_t scale_pitch;       /* floats */
    void *k_cache, *v_cache;
    int64_t seq_stride, head_stride, tok_stride;
    float *k_scale_cache, *v_scale_cache;
    int64_t s_seq_stride, s_head_stride;
    int32_t *cache_len;        /* device [n_seqs], updated in place */
    int max_len;
} tsattn_fill_args;

int tsattn_cache_fill(tsattn_handle_t h, const tsattn_fill_args *a, void *stream);

/* Summary of a span list for tsattn_prefill (its span_tiles argument), built once per batch and mask and shared
 * by every layer and head that uses the same spans: TSATTN_SPAN_TILE_INTS int32 per 128 query rows.
 * The reference builds its per-64-row tile-skip list on the host for the same purpose
 * (TAttentionSpanGroup / GroupAttention, gpt/att/att.h:56-64,95-181).  tiles: device array of
 * tsattn_span_tiles_count(n_tokens) * TSATTN_SPAN_TILE_INTS int32. */
#define TSATTN_SPAN_TILE_INTS 32
int64_t tsattn_span_tiles_count(int64_t n_tokens);
int tsattn_build_span_tiles(tsattn_handle_t h, int64_t n_tokens, const int32_t *span_start, const int32_t *span_finish,
                            int32_t *tiles, void *stream);

/* Rows with more than one span.  TAttentionInfo holds any number of spans per row (gpt/att/att.h:24-47); the
 * reference's CPU path loops over a row's spans inside one softmax (gpt/compute/gpt_cpu.cpp:405-436), its GPU kernels
 * walk them as span groups (att.h:95-181).  Here: call tsattn_prefill once per span of the rows -- part i with every
 * row's i-th span, an empty span (finish < start) for rows that have fewer -- each into its own f32 result and
 * sum_weight_log, then combine the parts with this call.  Every part has the zero vector among its keys; the weights
 * of the parts add up and the zero vector counts once: with W_i = 2^swl_i,
 *   out = sum_i out_i W_i / (sum_i W_i - (n_parts - 1)),   sum_weight_log = log2 of that denominator,
 * the result of one softmax over all the spans (keys that lie in two spans of a row count twice, as in the reference).
 * part_out: n_parts results [n_tokens][n_heads*head_dim] f32, part_out_stride floats apart, rows part_out_pitch floats
 * (a multiple of 4), 16-byte aligned; part_swl: n_parts planes [n_heads][scale_pitch], part_swl_stride floats apart.
 * out must not overlap the parts. */
typedef struct tsattn_merge_args {
    int n_parts;               /* 1..64 */
    int64_t n_tokens;
    int n_heads, head_dim;     /* head_dim a multiple of 4 */
    const float *part_out;
    int64_t part_out_pitch, part_out_stride;
    const float *part_swl;
    int64_t scale_pitch, part_swl_stride;
    int out_dtype;             /* tsattn_out_dtype */
    void *out;                 /* [n_tokens][n_heads*head_dim], 16-byte aligned */
    int64_t out_pitch;         /* bytes, multiple of 16 */
    float *sum_weight_log;     /* optional [n_heads][scale_pitch] */
} tsattn_merge_args;

int tsattn_merge_lookups(tsattn_handle_t h, const tsattn_merge_args *a, void *stream);

/* Producer of Q, K or V for the calls above from a projection result: optional RoPE at each row's position, then per
 * head sko = sqrt(mean x^2), scale = sko * vec_scale, values / scale converted to int8 (round to nearest even,
 * clamped to +-127) or e4m3, and scale * scale_mult written to scale[head * scale_pitch + row].  Replaces
 * ApplyRope + NormalizeState of the reference's inference path (gpt/train/cpu_infer.cpp:486-499, :358-391,
 * gpt/att/rope.cpp:28-46; the GPU epilogue TStoreRowTileNormalizeRope, gpt/compute/gpt_rope.cuh:4-66, computes the
 * same per 128-wide head), in the CPU path's operation order: results are identical to it bit for bit.
 * scale_mult is how the reference folds QVScale * VEC_SCALE * CalcDotScale(dim) into the cached key scale
 * (cpu_infer.cpp:502-504). */
typedef struct tsattn_produce_args {
    int src_dtype;             /* TSATTN_SRC_F32 or TSATTN_SRC_I32 */
    int dst_dtype;             /* tsattn_dtype */
    int64_t n_rows;
    int n_heads, head_dim;     /* head_dim 64 or 128; also 256, 384, 512 (the feed-forward groups of 128 * ReluMult,
                                  gpt/model_params/model_dim.h:66) with an int8 result and no rotation */
    const void *src;           /* [n_rows][n_heads*head_dim], 16-byte aligned */
    int64_t src_pitch;         /* elements per row, multiple of 4 */
    const int32_t *pos;        /* device [n_rows]: position of each row in its sequence; NULL = no rotation */
    const float *rope;         /* device [rope_len][head_dim] table, see tsattn_fill_rope_table; NULL only with pos == NULL */
    int64_t rope_len;          /* positions are clamped into [0, rope_len) */
    float rotate_dir;          /* +1 (the forward direction) or -1 */
    float vec_scale;           /* the reference's VEC_SCALE = 1/24 */
    float scale_mult;
    void *dst;                 /* [n_rows][n_heads*head_dim] 8-bit */
    int64_t dst_pitch;         /* bytes per row, multiple of 16 */
    float *scale;              /* [n_heads][scale_pitch] or NULL */
    int64_t scale_pitch;
    /* Element (head, row) of scale is scale[head * scale_pitch + row * scale_row_stride]; 0 means 1 (planes
     * [n_heads][scale_pitch], what tsattn_prefill reads).  scale_pitch = 1 with scale_row_stride = n_heads gives
     * [n_rows][n_heads], what tsattn_cache_append and the fused append of tsattn_decode read. */
    int64_t scale_row_stride;
    /* Non-zero: negative results become 0 after the conversion, the ReLU of the reference's int8 feed-forward
     * block (gpt/train/cpu_infer.cpp:520-524).  int8 only. */
    int relu;
    /* Options that let one call take the place of several (all 0 / NULL = not used):
     * src_planes > 1 (int32 source only): the source is the sum of that many int32 arrays src_plane_stride elements
     *   apart: the parts of a matrix product whose K was split (tsattn_matmul_i8, TSATTN_MM_I32_PLANES);
     * rope_heads > 0: only heads below it are rotated (a row that holds the qk and qv heads first, then k and v);
     * scale_head_count > 0: scales are written only for heads scale_head_begin .. +scale_head_count, at index
     *   head - scale_head_begin, with scale_row_stride >= scale_head_count in the [row][head] layout;
     * resid (f32 [n_rows][resid_pitch], n_heads*head_dim wide): the residual update that precedes the normalisation,
     *   resid += source * resid_scale (AddScaled, cpu_infer.cpp:308-316, calls :514, :526), written back, and
     *   the updated rows are what is normalised. */
    int src_planes;
    int64_t src_plane_stride;
    int rope_heads;
    int scale_head_begin, scale_head_count;
    float *resid;
    int64_t resid_pitch;
    float resid_scale;
} tsattn_produce_args;

int tsattn_rope_normalize_rows(tsattn_handle_t h, const tsattn_produce_args *a, void *stream);

/* Consumer of the attention output: kv[row][(head*rep + blk)*head_dim + z] = int8(k[row][head*head_dim + (z ^ blk)] *
 * value[row][head*head_dim + z] * mult), blk < rep (the reference's COMBINER_REP = 4), int8 = round to nearest even
 * clamped to +-127.  Replaces KVProduct, gpt/train/cpu_infer.cpp:320-337 (call :511; GPU form
 * gpt/compute/gpt_combiner.cuh:13-37, whose kvMult is `mult`).  k: int8 [n_rows][n_heads*head_dim]; value: the
 * attention output, f32 or f16 (tsattn_out_dtype); pitches of k and kv in bytes, of value in elements; all 16-byte
 * aligned. */
int tsattn_kv_product(tsattn_handle_t h, int64_t n_rows, int n_heads, int head_dim, int rep, const void *k, int64_t k_pitch,
                      int value_dtype, const void *value, int64_t value_pitch, float mult, void *kv, int64_t kv_pitch,
                      void *stream);

/* int8 matrix product of the reference's int8 inference path: out[m][n] (op)= sum_k a[m][k] * w[n][k], exact in
 * int32.  Replaces MulForward, gpt/train/cpu_infer.cpp:294-305 (one weight row per output; calls :481-488, :513,
 * :519, :525, :558: the four projections, the combiner, the two FFN matrices, the final layer) and, with
 * TSATTN_MM_ADD_SCALED, the AddScaled that follows the combiner and the FFN (:308-316, calls :514, :526).
 * a: int8 [m][k], w: int8 [n][k], pitches in bytes; k a positive multiple of 64 (DotInt8 asks the same, :184-210);
 * out: [m][n], pitch in elements; pointers and byte pitches multiples of 16, out 4-byte aligned. */
enum tsattn_mm_mode {
    TSATTN_MM_I32 = 0,        /* out (int32) = sum */
    TSATTN_MM_F32 = 1,        /* out (f32) = (float)sum * scale   (MulForward into TVector<float>: scale 1) */
    TSATTN_MM_ADD_SCALED = 2, /* out (f32) += (float)sum * scale  (AddScaled) */
    /* out (int32 [planes][m][n], n = out_pitch) = partial sums whose total over the planes is the product; *planes_out
     * (host memory) receives their number: 1 with more than 128 rows (out holds m * n ints), up to 16 with fewer (K may
     * be split; out holds 16 * m * n ints).
     * For a consumer that adds the planes up itself (tsattn_rope_normalize_rows with src_planes) and so saves the
     * launch that would. */
    TSATTN_MM_I32_PLANES = 3,
};

typedef struct tsattn_matmul_args {
    int64_t m, n, k;
    const void *a;             /* int8 [m][k], 16-byte aligned */
    int64_t a_pitch;           /* bytes, multiple of 16, at most 8 MiB */
    const void *w;             /* int8 [n][k], 16-byte aligned */
    int64_t w_pitch;           /* bytes, multiple of 16, at most 8 MiB */
    int mode;                  /* tsattn_mm_mode */
    float scale;
    void *out;
    int64_t out_pitch;
    /* Optional scratch of the caller's (16-byte aligned): with at most 128 rows the weights are streamed once and K
     * is split over more workgroups if there is room for the parts' sums (2 x 4 x m x n bytes or more; 16 x 4 x m x n
     * is never exceeded).  The result is the same with and without it. */
    void *workspace;
    int64_t workspace_bytes;
    int *planes_out;           /* TSATTN_MM_I32_PLANES: host int that receives the number of planes */
    const struct tsattn_produce_args *epilogue; /* optional, TSATTN_MM_I32_PLANES only (host pointer, read during the call):
                                  tsattn_rope_normalize_rows applied to the product, as that call would be afterwards with
                                  src = out (its src, src_dtype, src_pitch, src_planes, src_plane_stride, n_rows and n_heads
                                  are taken from the product: n_heads = n / head_dim, which must divide n).  This is the
                                  reference's projection with its normalising epilogue (TStoreRowTileNormalizeRope,
                                  gpt/compute/gpt_rope.cuh:4-66, lib/cuda/cuda_matmul.cuh:146-204).  Large products with an
                                  int8 result do it in the product's own kernel and never write the int32 sums; otherwise
                                  the library makes the two launches.  Either way `out` is scratch: what it holds after the
                                  call is unspecified. */
} tsattn_matmul_args;

int tsattn_matmul_i8(tsattn_handle_t h, const tsattn_matmul_args *a, void *stream);

/* The two ends of ComputePrediction (gpt/train/cpu_infer.cpp:552-582) around the layers.
 *
 * tsattn_embed_rows: state[row][x] = sum over the row's labels of embed[label][x] * embed_scale, added in label order
 * (:559-565).  labels: int32 [n_rows][labels_per_row], entries outside [0, n_labels) are empty slots; embed: int8
 * [n_labels][embed_pitch bytes]; dim a multiple of 16; state f32 [n_rows][state_pitch], 16-byte aligned.
 *
 * tsattn_softmax_rows: the final SoftMax (:340-355 with TSoftMaxBuf :220-281, base 2): w[k] = vec[k] * scale + bias[k],
 * prob[k] = 2^(w[k] - M) / sum, M = max(0, max w); argmax[row] = the first k of the largest w (the greedy choice).
 * vec: int32 [n_rows][src_pitch], optionally the sum of src_planes arrays src_plane_stride elements apart
 * (TSATTN_MM_I32_PLANES); bias f32 [n] or NULL; prob f32 [n_rows][prob_pitch] or NULL; argmax int32 [n_rows] or NULL. */
int tsattn_embed_rows(tsattn_handle_t h, int64_t n_rows, int dim, const int32_t *labels, int labels_per_row, const void *embed,
                      int64_t embed_pitch, int64_t n_labels, float embed_scale, float *state, int64_t state_pitch, void *stream);
int tsattn_softmax_rows(tsattn_handle_t h, int64_t n_rows, int64_t n, const int32_t *src, int src_planes, int64_t src_plane_stride,
                        int64_t src_pitch, float scale, const float *bias, float *prob, int64_t prob_pitch, int32_t *argmax,
                        void *stream);

/* SampleFromDistr (gpt/train/cpu_infer.cpp:585-599), the Gumbel-max choice from a distribution:
 * choice[row] = the first k of the largest score[k] = (float)(logf(prob[k]) / temperature - log(-log(u[k]))), with
 * u[k] = (r[k] + 0.5) / 2^32 in double, which is GenRandReal3 of the reference's 32-bit generator
 * (lib/random/mersenne.h:233-235, TXRng = TMersenne<ui32>, gpt/rng/xrng.h:4).  rnd: device uint32 [n_rows][rnd_pitch],
 * the words r supplied by the caller (for instance that generator's stream), or NULL: the word of (row, k) is then
 * the upper half of splitmix64's output function applied to seed + (offset + row * n + k + 1) * 0x9E3779B97F4A7C15 --
 * a counter-based generator: same seed and offset, same choices; advance offset by n_rows * n per call.  This is not
 * the reference's MT19937 stream; the distribution of the choices is the same.  temperature > 0.
 * prob f32 [n_rows][prob_pitch] (tsattn_softmax_rows' output); choice int32 [n_rows]. */
int tsattn_sample_rows(tsattn_handle_t h, int64_t n_rows, int64_t n, const float *prob, int64_t prob_pitch, float temperature,
                       const uint32_t *rnd, int64_t rnd_pitch, uint64_t seed, uint64_t offset, int32_t *choice, void *stream);

/* The table ApplyRope reads: FillRopeBuf, gpt/att/rope.cpp:4-24.  Host function, host memory:
 * table[t * head_dim + x], t < max_len; copy it to the device once. */
void tsattn_fill_rope_table(int head_dim, int64_t max_len, float *table);

/* Per-(row, head) absmax quantiser: scale = absmax/127 (int8) or absmax/256 (e4m3), values
 * round-to-nearest-even, int8 clamped to [-127,127].  Replaces NormalizeVecsRowTileMax /
 * TStoreRowTileMaxNormalize (gpt/compute/row_tile_scale.cuh:59-81, lib/cuda/cuda_matmul.cuh:207-260,
 * lib/cuda/cuda_util.cuh:286-297).  src: [n_rows][n_heads*head_dim] f32 or bf16;
 * scale written to scale[head*scale_pitch + row]. */
int tsattn_quantize_rows(tsattn_handle_t h, int src_dtype, int dst_dtype, const void *src,
                         int64_t src_pitch, int64_t n_rows, int n_heads, int head_dim, void *dst,
                         int64_t dst_pitch, float *scale, int64_t scale_pitch, void *stream);

/* Window metadata on the device: one inclusive key span per token from the window width, the
 * sequence boundaries and optional in-sequence document starts.  Replaces the host-side span
 * emission of GenerateAttentionGraph / AddAttSpans (gpt/att/sliding_window.cpp:80-87,150-154,
 * 205-223) and the fragment shift of InitLabelData (:253-290).  seq_offset: device int32
 * [n_seqs+1] first token of each sequence; doc_start_flag: optional device uint8 [n_tokens]. */
int tsattn_build_spans(tsattn_handle_t h, int n_seqs, const int32_t *seq_offset, int64_t n_tokens,
                       const uint8_t *doc_start_flag, int64_t window, int32_t *span_start,
                       int32_t *span_finish, void *stream);

/* Library build identification (kernel set and target), for logs. */
const char *tsattn_version(void);

#ifdef __cplusplus
}
#endif
#endif
