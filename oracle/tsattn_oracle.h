/*
 * tsattn_oracle.h -- CPU restatement of TScale's attention arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY.  This library is the checker for the HIP kernels: it may be
 * called from tests/, from __graft_entry__.smoke() and from the cpu_baseline leg of
 * bench.py, and from nowhere else.  The product library (libtsattn.so) never links,
 * loads or falls back to anything in this directory.
 *
 * Every function names the reference lines (paths relative to the reference's code/
 * directory) whose arithmetic it restates.  Pinning status is listed per function in
 * tsattn_oracle.c's header comment.
 */
#ifndef TSATTN_ORACLE_H
#define TSATTN_ORACLE_H

#include <stdint.h>
#include <stddef.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { TSO_I8 = 0, TSO_E4M3 = 1 };

/* ---- element formats (util/fp8.h:4-21, 48-60; train/cpu_infer.cpp:88-92) ---- */
float   tso_e4m3_to_float(uint8_t x);
uint8_t tso_float_to_e4m3(float x);            /* round-nearest-even, saturate to +-448 */
int8_t  tso_float_to_i8(float x);              /* round-nearest-even, clamp to [-127,127] */
float   tso_bf16_to_float(uint16_t x);
uint16_t tso_float_to_bf16(float x);           /* round-nearest-even */
float   tso_att_dot_scale(int head_dim);       /* sqrtf(1/d) * (0.5f/0.693147f), model_dim.h:19-31 */

/* ---- absmax row quantiser (lib/cuda/cuda_matmul.cuh:237-249, cuda_util.cuh:290-297) ----
 * x: [n_rows][n_heads*head_dim] fp32 (row pitch x_pitch floats); one scale per (row, head)
 * written to scale[head*scale_pitch + row].  q has row pitch q_pitch bytes. */
void tso_quantize_rows(int dtype, const float *x, int64_t x_pitch, int64_t n_rows, int n_heads,
                       int head_dim, uint8_t *q, int64_t q_pitch, float *scale, int64_t scale_pitch);
/* same for bf16 source rows (decode query prologue) */
void tso_fill_rope(int width, int64_t max_len, float *rope);
void tso_apply_rope(const float *rope_row, float rotate_dir, int dim, int head_size, float *vec);
void tso_normalize_heads(int dtype, const float *state, int dim, int n_heads, float vec_scale, uint8_t *res,
                         float *head_scale);
void tso_rope_normalize_rows(int dtype, const void *src, int src_is_i32, int64_t src_pitch, int64_t n_rows,
                             const int32_t *pos, const float *rope, float rotate_dir, int n_heads, int head_dim,
                             float vec_scale, float scale_mult, uint8_t *q, int64_t q_pitch, float *scale,
                             int64_t scale_pitch);
void tso_kv_product(const int8_t *k, int64_t k_pitch, const float *val, int64_t val_pitch, int64_t n_rows, int n_heads,
                    int head_dim, int rep, float mult, int8_t *kv, int64_t kv_pitch);
void tso_matmul_i8(const int8_t *a, int64_t a_pitch, const int8_t *w, int64_t w_pitch, int64_t m, int64_t n, int64_t k, int mode,
                   float scale, void *out, int64_t out_pitch);
void tso_quantize_rows_bf16(int dtype, const uint16_t *x, int64_t x_pitch, int64_t n_rows,
                            int n_heads, int head_dim, uint8_t *q, int64_t q_pitch, float *scale,
                            int64_t scale_pitch);

/* ---- attention spans (att/sliding_window.cpp:80-87,205-223,253-290) ----
 * Tokens of all sequences are concatenated; seq_offset[n_seq+1] gives each sequence's first
 * token.  doc_start_flag (nullable) marks tokens at which a new document starts inside a
 * sequence (the reference's DocStartToken test, :150-154, position 0 of a sequence never
 * resets).  Writes inclusive [start, finish] per token, finish < start meaning "no keys". */
void tso_make_spans(int64_t n_seq, const int64_t *seq_offset, const uint8_t *doc_start_flag,
                    int64_t window, int32_t *span_start, int32_t *span_finish);

/* ---- layer schedule (model_params/model_dim.cpp:55-97, ALIBI_V3 branch and depth==1) ----
 * Returns the number of layers written (>= depth, the reference emits layer pairs). */
int tso_init_alibi(int depth, int64_t wide_window, int max_layers, int64_t *width, float *slope);

/* ---- integer / exact dot products (train/cpu_infer.cpp:184-210) ---- */
int32_t tso_dot_i8(const int8_t *a, const int8_t *b, int n);          /* exact, scalar */
int32_t tso_dot_i8_simd(const int8_t *a, const int8_t *b, int n);     /* sign trick + vpdpbusd / maddubs */
float   tso_dot_e4m3(const uint8_t *a, const uint8_t *b, int n);      /* exact sum, rounded once */

/* raw QK^T accumulators for a block of (from, to) pairs of one head: acc[(from-from0)*n_to + (to-to0)]
 * int32 for TSO_I8 (bit-exact target), float for TSO_E4M3 (exact sum rounded once). */
void tso_qk_accum(int dtype, const uint8_t *q, int64_t q_pitch, const uint8_t *k, int64_t k_pitch,
                  int head, int head_dim, int64_t from0, int64_t n_from, int64_t to0, int64_t n_to,
                  void *acc);

/* ---- prefill, fp32 inputs: compute/gpt_cpu.cpp:374-441 verbatim semantics ----
 * qk, qv: [len][n_heads*q_dim]; v: [len][n_heads*tt_dim]; one inclusive span list per row in CSR
 * form (span_ptr[len+1], spans as start/finish pairs).  out: [len][n_heads*tt_dim];
 * sum_weight, max_dp: [n_heads][len] (nullable). */
void tso_prefill_f32(int64_t len, int n_heads, int q_dim, int tt_dim, const float *qk,
                     const float *qv, const float *v, const int32_t *span_ptr,
                     const int32_t *spans, float alibi_slope, float *out, float *sum_weight,
                     float *max_dp);

/* ---- prefill, quantised inputs with per-row scales (generalisation of gpt_cpu.cpp:391-441 with
 * the logit product order of train/cpu_infer.cpp:448 and value order of :454) ----
 * q,k,v: [n_tokens][n_heads*head_dim] 8-bit; scales [n_heads][n_tokens] (pitch scale_pitch) or
 * NULL = the constant given.  span_start/finish: one inclusive span per row.
 * out fp32 [n_tokens][n_heads*head_dim] (pitch out_pitch floats); sum_weight_log [n_heads][n_tokens]
 * nullable (= max + log2(sum), gpt_att_fp16.cuh:249).  n_threads<=1: single thread. */
void tso_prefill_q8(int dtype, int64_t n_tokens, int n_heads, int head_dim, const uint8_t *q,
                    const uint8_t *k, const uint8_t *v, int64_t pitch, const float *q_scale,
                    const float *k_scale, const float *v_scale, int64_t scale_pitch,
                    float q_scale_const, float k_scale_const, float v_scale_const,
                    const int32_t *span_start, const int32_t *span_finish, float alibi_slope,
                    float *out, int64_t out_pitch, float *sum_weight_log, int n_threads);

/* ---- decode over a KV cache: train/cpu_infer.cpp:413-460 (+220-281 softmax buffer) ----
 * One call handles n_seq sequences.  Cache planes are addressed with explicit strides so both the
 * reference's token-major rows and a planar [seq][head][L][d] layout can be fed:
 *   K byte address = k + seq*k_seq_stride + head*k_head_stride + to*k_tok_stride   (same for v)
 *   scale address  = ks + seq*s_seq_stride + head*s_head_stride + to               (floats)
 * q: [n_seq][n_heads*head_dim] 8-bit, q_scale [n_seq][n_heads] (nullable = constant).
 * cache_len[seq] counts valid rows INCLUDING the current token (appended before the call,
 * cpu_infer.cpp:506-509).  window==0 means "self only".  exp2_mode 0: libm exp2f; 1: the
 * reference's AVX2 polynomial (cpu_infer.cpp:247-280) evaluated lane-faithfully.
 * qk_acc (nullable): raw accumulators [n_seq][n_heads][max_len] (int32 / float), max_len = qk_acc_pitch.
 * use_simd: 1 = vpdpbusd/AVX2 dot (timed baseline), 0 = scalar. */
void tso_decode(int dtype, int64_t n_seq, int n_heads, int head_dim, const uint8_t *q,
                const float *q_scale, float q_scale_const, const uint8_t *k, const uint8_t *v,
                int64_t seq_stride, int64_t head_stride, int64_t tok_stride, const float *k_scale,
                const float *v_scale, int64_t s_seq_stride, int64_t s_head_stride,
                float k_scale_const, float v_scale_const, const int32_t *cache_len, int64_t window,
                float alibi_slope, int exp2_mode, int use_simd, float *out, void *qk_acc,
                int64_t qk_acc_pitch, int n_threads);

/* ---- one layer of the int8 inference path for one new token per sequence: AddLookupProduct,
 * train/cpu_infer.cpp:465-527 ----
 * Matrices are int8 with one row per output (MulForward's kqv[k]); *_scale are the matrix scales ConvertMatrix
 * returned (:94-121).  head_dim is QDim == TTDim.  state: [n_seq][dim] f32, updated in place.  t[seq]: the token's
 * position (rope row).  The KV cache is addressed as in tso_decode (key scales only; queries and values carry the
 * constant VEC_SCALE, :16); cache_len[seq] is the length before the call and is incremented (a full cache drops the
 * row).  val_lookup (nullable): the attention output [n_seq][head_count*head_dim]. */
typedef struct tso_layer_params {
    int dim, head_count, head_dim, relu_dim;
    const int8_t *qk, *qv, *k, *v;   /* [head_count*head_dim][dim] */
    const int8_t *combiner;          /* [dim][head_count*head_dim*4] */
    const int8_t *expand;            /* [relu_dim][dim] */
    const int8_t *contract;          /* [dim][relu_dim] */
    float qv_scale, combiner_scale, contract_scale;
    int64_t attention_width;
    float alibi_slope;
} tso_layer_params;

void tso_add_lookup_product(const tso_layer_params *L, int64_t n_seq, const int32_t *t, const float *rope, float *state,
                            uint8_t *k_cache, uint8_t *v_cache, int64_t seq_stride, int64_t head_stride, int64_t tok_stride,
                            float *k_scale_cache, int64_t s_seq_stride, int64_t s_head_stride, int32_t *cache_len, int max_len,
                            float *val_lookup, int n_threads);

/* ---- the two ends of ComputePrediction around the layers (train/cpu_infer.cpp:552-582) ----
 * tso_embed_rows: state[row][x] = sum over the row's labels of embed[label][x] * scale, in label order (:559-565);
 * labels outside [0, n_labels) are empty slots.
 * tso_softmax_rows: SoftMax (:340-355): w[k] = vec[k] * scale + bias[k] through the softmax buffer (exp2_mode as in
 * tso_decode), prob[k] = Buf[k] * Scale; argmax = the first index of the largest w.  bias, prob, argmax nullable. */
void tso_embed_rows(int64_t n_rows, int dim, const int32_t *labels, int labels_per_row, const int8_t *embed, int64_t n_labels,
                    float scale, float *state);
void tso_softmax_rows(int64_t n_rows, int64_t n, const int32_t *vec, float scale, const float *bias, int exp2_mode, float *prob,
                      int32_t *argmax);

/* ---- SampleFromDistr (train/cpu_infer.cpp:585-599): the Gumbel-max choice ----
 * score[k] = (float)(logf(prob[k]) / temperature - log(-log(u[k]))), u[k] = (r[k] + 0.5) / 2^32 in double (GenRandReal3 of the
 * reference's 32-bit generator, lib/random/mersenne.h:233-235); choice = the first k of the largest score above -1e38, else 0.
 * rnd: the words r, [n_rows][rnd_pitch], or NULL: r[k] of row `row` = tso_mix32(seed, offset + row * n + k) (a counter-based
 * generator, not the reference's MT19937 stream). */
uint32_t tso_mix32(uint64_t seed, uint64_t index);
void tso_sample_rows(int64_t n_rows, int64_t n, const float *prob, int64_t prob_pitch, float temperature, const uint32_t *rnd,
                     int64_t rnd_pitch, uint64_t seed, uint64_t offset, int32_t *choice);

/* softmax buffer of cpu_infer.cpp:220-281 on its own (for bounding the polynomial):
 * in: n logits (the caller includes the leading 0 if wanted); out: n weights already multiplied by
 * Scale.  Returns Scale. */
float tso_softmax_buf(const float *logits, int n, int exp2_mode, float *weights);

int tso_simd_level(void); /* 0 scalar, 1 avx2 maddubs, 2 avx-vnni / avx512-vnni(vl) */
int tso_max_threads(void);

#ifdef __cplusplus
}
#endif
#endif
