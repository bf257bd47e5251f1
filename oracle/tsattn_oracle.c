/*
 * tsattn_oracle.c -- CPU restatement of TScale's attention arithmetic.
 *
 * TEST INFRASTRUCTURE ONLY (see tsattn_oracle.h).  Nothing in the product library depends on
 * this file; it exists so that the HIP kernels can be compared with the reference algorithm on
 * identical inputs, and so that the same algorithm can be timed on host cores.
 *
 * Reference lines restated (paths relative to the reference's code/ directory) and how each
 * function is pinned by tests/test_oracle_*.py:
 *
 *   tso_e4m3_to_float      util/fp8.h:4-21               pinned: all 256 codes against the OCP e4m3fn
 *                                                         table built from first principles and
 *                                                         against torch.float8_e4m3fn
 *   tso_float_to_e4m3      util/fp8.h:48-60 (cvt.rn.satfinite)  pinned: round trip of all codes, ties
 *                                                         between neighbours go to even, saturation,
 *                                                         and torch's float8_e4m3fn cast on a dense sweep
 *   tso_float_to_i8        train/cpu_infer.cpp:88-92     pinned: ties-to-even and clamp cases
 *   tso_quantize_rows      lib/cuda/cuda_matmul.cuh:237-249, cuda_util.cuh:290-297
 *                                                         pinned: numpy restatement + absmax row maps
 *                                                         to +-127 / +-256
 *   tso_make_spans         att/sliding_window.cpp:80-87,150-154,205-223,253-290
 *                                                         pinned: brute-force enumeration of allowed
 *                                                         (from,to) pairs
 *   tso_init_alibi         model_params/model_dim.cpp:55-97   pinned: doc/model.md layer pattern
 *   tso_dot_i8(_simd)      train/cpu_infer.cpp:184-210   pinned: int64 brute force, extreme values
 *   tso_dot_e4m3           (exact-sum definition)        pinned: Fraction arithmetic in Python
 *   tso_prefill_f32        compute/gpt_cpu.cpp:374-441   pinned: closed forms (equal logits, single
 *                                                         key, empty row, ALiBi geometric series),
 *                                                         textbook softmax with an extra zero key
 *   tso_prefill_q8         same + cpu_infer.cpp:448,454  pinned: equals tso_prefill_f32 on dequantised
 *                                                         inputs; scale-shift invariance
 *   tso_decode             train/cpu_infer.cpp:413-460   pinned: equals prefill row t on cache [0..t]
 *   tso_softmax_buf        train/cpu_infer.cpp:220-281   pinned: against exp2 in double, |rel| < 1e-5
 *   tso_fill_rope, tso_apply_rope   att/rope.cpp:4-46     pinned: the reference's own FillRopeBuf / ApplyRope built
 *                                                         into oracle/_ref (bit-identical tables and rotations);
 *                                                         rotation preserves each pair's norm
 *   tso_normalize_heads    train/cpu_infer.cpp:358-391 (e4m3 target: compute/gpt_rope.cuh:41-46,61)
 *                                                         pinned: constant vector -> 24, zero vector, scale
 *                                                         invariance, numpy restatement with the same
 *                                                         sequential float sum
 *   tso_rope_normalize_rows  train/cpu_infer.cpp:486-499  composition of the two above
 *   tso_kv_product         train/cpu_infer.cpp:320-337   pinned: numpy restatement (index shuffle z ^ blk, products,
 *                                                         rounding), blk 0 = plain product, the four blocks are
 *                                                         permutations of each other when value is constant
 *   tso_matmul_i8          train/cpu_infer.cpp:294-316   pinned: numpy int64 matrix product (a library routine), +-127
 *                                                         extremes; the scaled forms against the same product in
 *                                                         float64
 *   tso_add_lookup_product train/cpu_infer.cpp:465-527   pinned: the same layer in float64 with nothing rounded to
 *                                                         int8 (division by rms * VEC_SCALE, complex rotation, an
 *                                                         ordinary softmax with one zero key, real-valued KV cache;
 *                                                         what the reference's own Check does, :625-685) agrees over
 *                                                         several tokens to within the int8 rounding, and does not
 *                                                         with k and v exchanged in KVProduct, the key scale's
 *                                                         CalcDotScale taken of the head width, a VEC_SCALE dropped,
 *                                                         or the ReLU in front of the normalisation; plus invariants
 *                                                         (state scale, zero matrices, first token, linearity)
 *   tso_embed_rows         train/cpu_infer.cpp:559-565   pinned: numpy gather and sum
 *   tso_softmax_rows       train/cpu_infer.cpp:340-355   pinned: scipy's softmax on ln 2 * w (a library routine), rows
 *                                                         sum to 1, adding a constant to the bias changes nothing
 *                                                         while the largest w stays above 0
 *   tso_sample_rows        train/cpu_infer.cpp:585-599   pinned: frequencies of the choices follow prob^(1/T) normalised
 *                                                         (the Gumbel-max identity; temperatures 1 and 2), a tiny
 *                                                         temperature gives the largest probability, words handed in
 *                                                         and words from the counter generator agree
 *
 * The reference holds no golden vectors or known-answer tests for this path, and the two files
 * that contain it (gpt_cpu.cpp, cpu_infer.cpp) cannot be compiled without the CUDA SDK, so the
 * pins above are mathematical ones.
 */
#include "tsattn_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#if defined(__x86_64__)
#include <immintrin.h>
#endif
#ifdef _OPENMP
#include <omp.h>
#endif

/* model_params/model_dim.h:19-31 */
#define TS_LOG2 0.693147f
#define TS_ATT_DOTPRODUCT_SCALE 0.5f

float tso_att_dot_scale(int head_dim)
{
    float dot_scale = sqrtf(1.0f / (float)head_dim);          /* CalcDotScale */
    float att_mult = TS_ATT_DOTPRODUCT_SCALE / TS_LOG2;       /* CalcAttentionMult */
    return dot_scale * att_mult;                              /* gpt_cpu.cpp:376 */
}

/* ------------------------------------------------------------------------------------------ */
/* element formats                                                                            */

float tso_e4m3_to_float(uint8_t x)
{
    /* util/fp8.h:4-21: bias 7, 3 mantissa bits, subnormals at e==0, no infinities.  The reference
     * decodes 0x7f/0xff as 480; OCP calls them NaN.  Quantised data never holds them. */
    int e = (x >> 3) & 15;
    int m = x & 7;
    float sign = (x & 0x80) ? -1.0f : 1.0f;
    if (e == 0) {
        return sign * ldexpf((float)m, -9);
    }
    return sign * ldexpf(1.0f + (float)m * 0.125f, e - 7);
}

uint8_t tso_float_to_e4m3(float x)
{
    uint8_t sign = signbit(x) ? 0x80 : 0;
    float a = fabsf(x);
    if (isnan(x)) {
        return (uint8_t)(sign | 0x7f);
    }
    if (a >= 448.0f) {
        return (uint8_t)(sign | 0x7e); /* satfinite */
    }
    if (a < ldexpf(1.0f, -6)) {
        /* subnormal range: step 2^-9, 8 steps reach the first normal */
        int q = (int)nearbyintf(ldexpf(a, 9)); /* default rounding mode = nearest even */
        return (uint8_t)(sign | q);             /* q == 8 encodes as e=1,m=0 automatically */
    }
    int e;
    (void)frexpf(a, &e); /* a = f * 2^e, f in [0.5,1) -> floor(log2 a) = e-1 */
    e -= 1;
    int q = (int)nearbyintf(ldexpf(a, 3 - e)); /* in [8,16] */
    if (q == 16) {
        q = 8;
        e += 1;
    }
    int code = ((e + 7) << 3) | (q - 8);
    if (code > 0x7e) {
        code = 0x7e;
    }
    return (uint8_t)(sign | code);
}

int8_t tso_float_to_i8(float x)
{
    /* cpu_infer.cpp:88-92: _mm_cvtss_si32 (nearest even) then clamp to [-127,127] */
    float r = nearbyintf(x);
    if (!(r <= 127.0f)) {
        r = (r != r) ? 0.0f : 127.0f;
    }
    if (r < -127.0f) {
        r = -127.0f;
    }
    return (int8_t)(int)r;
}

float tso_bf16_to_float(uint16_t x)
{
    uint32_t u = (uint32_t)x << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

uint16_t tso_float_to_bf16(float x)
{
    uint32_t u;
    memcpy(&u, &x, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) {
        return (uint16_t)((u >> 16) | 0x40);
    }
    uint32_t lsb = (u >> 16) & 1;
    u += 0x7fffu + lsb;
    return (uint16_t)(u >> 16);
}

/* ------------------------------------------------------------------------------------------ */
/* absmax row quantiser                                                                       */

static void quantize_head_row(int dtype, const float *x, int head_dim, uint8_t *q, float *scale)
{
    /* cuda_matmul.cuh:237-249: maxVal = max |x|; discrScale = maxVal/127 (i8) or /256 (e4m3);
     * values multiplied by 1/discrScale and converted round-to-nearest.  All-zero row: scale 0. */
    float max_val = 0;
    for (int i = 0; i < head_dim; ++i) {
        max_val = fmaxf(max_val, fabsf(x[i]));
    }
    float discr = 0;
    float mult = 0;
    if (max_val > 0) {
        discr = (dtype == TSO_I8) ? max_val / 127 : max_val / 256;
        mult = 1 / discr;
    }
    for (int i = 0; i < head_dim; ++i) {
        float y = x[i] * mult;
        q[i] = (dtype == TSO_I8) ? (uint8_t)tso_float_to_i8(y) : tso_float_to_e4m3(y);
    }
    *scale = discr;
}

void tso_quantize_rows(int dtype, const float *x, int64_t x_pitch, int64_t n_rows, int n_heads,
                       int head_dim, uint8_t *q, int64_t q_pitch, float *scale, int64_t scale_pitch)
{
    for (int64_t t = 0; t < n_rows; ++t) {
        for (int h = 0; h < n_heads; ++h) {
            quantize_head_row(dtype, x + t * x_pitch + (int64_t)h * head_dim, head_dim,
                              q + t * q_pitch + (int64_t)h * head_dim, scale + h * scale_pitch + t);
        }
    }
}

void tso_quantize_rows_bf16(int dtype, const uint16_t *x, int64_t x_pitch, int64_t n_rows,
                            int n_heads, int head_dim, uint8_t *q, int64_t q_pitch, float *scale,
                            int64_t scale_pitch)
{
    float *tmp = (float *)malloc(sizeof(float) * (size_t)head_dim);
    for (int64_t t = 0; t < n_rows; ++t) {
        for (int h = 0; h < n_heads; ++h) {
            const uint16_t *src = x + t * x_pitch + (int64_t)h * head_dim;
            for (int i = 0; i < head_dim; ++i) {
                tmp[i] = tso_bf16_to_float(src[i]);
            }
            quantize_head_row(dtype, tmp, head_dim, q + t * q_pitch + (int64_t)h * head_dim,
                              scale + h * scale_pitch + t);
        }
    }
    free(tmp);
}

/* ------------------------------------------------------------------------------------------ */
/* producer of the attention operands: RoPE, per-head RMS normalisation, 8-bit conversion       */

/* FillRopeBuf, att/rope.cpp:4-24: rope[t][base + k] = cos(t * f), rope[t][base + k + 32] = sin(t * f),
 * f = theta^-(2 * (base/2 + k) / width), theta = 500000; blocks of 64 columns. */
void tso_fill_rope(int width, int64_t max_len, float *rope)
{
    float theta = 500000;
    float *freq = (float *)malloc(sizeof(float) * (size_t)(width / 2 + 1));
    for (int k = 0; k < width / 2; ++k) {
        /* C++ overload resolution in the reference: log(float) is the float function, its product with the
         * double (k * 2. / width) and exp of it are double; cos(float) and sin(float) below are float */
        freq[k] = (float)exp((double)(-logf(theta)) * (k * 2. / width));
    }
    for (int64_t t = 0; t < max_len; ++t) {
        for (int base = 0; base < width; base += 2 * 32) {
            for (int k = 0; k < 32; ++k) {
                float angle = t * freq[base / 2 + k];
                rope[t * width + base + k] = cosf(angle);
                rope[t * width + base + k + 32] = sinf(angle);
            }
        }
    }
    free(freq);
}

/* ReferenceApplyRope, att/rope.cpp:28-46, on one vector of dim/head_size heads; rope_row = ropeBuf[t]. */
void tso_apply_rope(const float *rope_row, float rotate_dir, int dim, int head_size, float *vec)
{
    for (int offset = 0; offset < dim; offset += head_size) {
        for (int blk = 0; blk < head_size; blk += 64) {
            for (int k = 0; k < 32; ++k) {
                float v0 = vec[offset + blk + k];
                float v1 = vec[offset + blk + k + 32];
                float cos_value = rope_row[blk + k];
                float sin_value = rope_row[blk + k + 32] * rotate_dir;
                float r0 = v0 * cos_value - v1 * sin_value;
                float r1 = v0 * sin_value + v1 * cos_value;
                vec[offset + blk + k] = r0;
                vec[offset + blk + k + 32] = r1;
            }
        }
    }
}

/* NormalizeState, train/cpu_infer.cpp:358-391: per head sko = sqrt(sum x^2 / headDim) (float, summed in index
 * order), discrScale = sko * vec_scale, values multiplied by 1/discrScale and converted (int8: cpu_infer.cpp:88-92;
 * e4m3: the conversion of the GPU epilogue, gpt_rope.cuh:41-46,61).  A zero head gives zeros and scale 0. */
void tso_normalize_heads(int dtype, const float *state, int dim, int n_heads, float vec_scale, uint8_t *res,
                         float *head_scale)
{
    int head_dim = dim / n_heads;
    for (int h = 0; h < n_heads; ++h) {
        int offset = h * head_dim;
        float sum2 = 0;
        for (int x = 0; x < head_dim; ++x) {
            sum2 += state[offset + x] * state[offset + x];
        }
        if (sum2 == 0) {
            for (int x = 0; x < head_dim; ++x) {
                res[offset + x] = 0;
            }
            if (head_scale) head_scale[h] = 0;
        } else {
            float sko = sqrtf(sum2 / head_dim);
            float discr_scale = sko * vec_scale;
            float mult = 1 / discr_scale;
            for (int x = 0; x < head_dim; ++x) {
                float y = state[offset + x] * mult;
                res[offset + x] = (dtype == TSO_I8) ? (uint8_t)tso_float_to_i8(y) : tso_float_to_e4m3(y);
            }
            if (head_scale) head_scale[h] = discr_scale;
        }
    }
}

/* AddLookupProduct's operand preparation, train/cpu_infer.cpp:486-499: ApplyRope(ropeBuf, dir, t, &src) then
 * NormalizeState(&dst, src, headCount, &headScale), per row; the written scale is headScale * scale_mult
 * (cpu_infer.cpp:502-504 folds the matrix scale into the key scale that way).  pos == NULL: no rotation
 * (the K and V projections, :496-499).  src_is_i32: the projection results that are int32 (:479-482). */
void tso_rope_normalize_rows(int dtype, const void *src, int src_is_i32, int64_t src_pitch, int64_t n_rows,
                             const int32_t *pos, const float *rope, float rotate_dir, int n_heads, int head_dim,
                             float vec_scale, float scale_mult, uint8_t *q, int64_t q_pitch, float *scale,
                             int64_t scale_pitch)
{
    int dim = n_heads * head_dim;
    float *tmp = (float *)malloc(sizeof(float) * (size_t)dim);
    float *hs = (float *)malloc(sizeof(float) * (size_t)n_heads);
    for (int64_t t = 0; t < n_rows; ++t) {
        for (int i = 0; i < dim; ++i) {
            tmp[i] = src_is_i32 ? (float)((const int32_t *)src)[t * src_pitch + i] : ((const float *)src)[t * src_pitch + i];
        }
        if (pos) {
            tso_apply_rope(rope + (int64_t)pos[t] * head_dim, rotate_dir, dim, head_dim, tmp);
        }
        tso_normalize_heads(dtype, tmp, dim, n_heads, vec_scale, q + t * q_pitch, hs);
        if (scale) {
            for (int h = 0; h < n_heads; ++h) {
                scale[h * scale_pitch + t] = hs[h] * scale_mult;
            }
        }
    }
    free(tmp);
    free(hs);
}

/* KVProduct, train/cpu_infer.cpp:320-337: the step after attention.  Per head and block blk < rep (COMBINER_REP = 4,
 * model_params/model_dim.h:12): kv[head*d*rep + blk*d + z] = int8(k[head*d + (z ^ blk)] * valLookup[head*d + z]),
 * int8 = round to nearest even clamped to +-127 (:88-92).  mult multiplies the product before the conversion (1 in
 * the CPU path; the GPU kernel's kvMult, compute/gpt_combiner.cuh:13-37). */
void tso_kv_product(const int8_t *k, int64_t k_pitch, const float *val, int64_t val_pitch, int64_t n_rows, int n_heads,
                    int head_dim, int rep, float mult, int8_t *kv, int64_t kv_pitch)
{
    for (int64_t t = 0; t < n_rows; ++t) {
        for (int head = 0; head < n_heads; ++head) {
            int head_offset = head * head_dim;
            for (int blk = 0; blk < rep; ++blk) {
                int64_t base = (int64_t)head * head_dim * rep + (int64_t)blk * head_dim;
                for (int z = 0; z < head_dim; ++z) {
                    int8_t key_shfl = k[t * k_pitch + head_offset + (z ^ blk)];
                    float value = val[t * val_pitch + head_offset + z];
                    kv[t * kv_pitch + base + z] = tso_float_to_i8((key_shfl * value) * mult);
                }
            }
        }
    }
}

/* MulForward, train/cpu_infer.cpp:294-305: res[n] = DotInt8(vec, w[n]) for every weight row n (exact int32), kept as
 * int32 (mode 0) or converted to float (mode 1: the TVector<float> instantiation, times `scale`, 1 in the
 * reference); mode 2 is the AddScaled that follows it (:308-316): out[n] += delta[n] * scale.  One activation row
 * per token. */
void tso_matmul_i8(const int8_t *a, int64_t a_pitch, const int8_t *w, int64_t w_pitch, int64_t m, int64_t n, int64_t k, int mode,
                   float scale, void *out, int64_t out_pitch)
{
#ifdef _OPENMP
#pragma omp parallel for schedule(static)
#endif
    for (int64_t i = 0; i < m; ++i) {
        for (int64_t j = 0; j < n; ++j) {
            int32_t sum = tso_dot_i8_simd(a + i * a_pitch, w + j * w_pitch, (int)k);
            if (mode == 0) {
                ((int32_t *)out)[i * out_pitch + j] = sum;
            } else if (mode == 1) {
                ((float *)out)[i * out_pitch + j] = (float)sum * scale;
            } else {
                ((float *)out)[i * out_pitch + j] += (float)sum * scale; /* (*pRes)[k] += delta[k] * scale */
            }
        }
    }
}

/* ------------------------------------------------------------------------------------------ */
/* spans and layer schedule                                                                   */

void tso_make_spans(int64_t n_seq, const int64_t *seq_offset, const uint8_t *doc_start_flag,
                    int64_t window, int32_t *span_start, int32_t *span_finish)
{
    for (int64_t s = 0; s < n_seq; ++s) {
        int64_t ptr = seq_offset[s];                 /* sliding_window.cpp:260, span.Shift(ptr) :279 */
        int64_t len = seq_offset[s + 1] - ptr;
        int64_t doc_start = 0;                       /* :142 */
        for (int64_t t = 0; t < len; ++t) {
            if (doc_start_flag && t > 0 && doc_start_flag[ptr + t]) {
                doc_start = t;                       /* :150-154 */
            }
            int64_t a, b;
            if (window == 0) {
                a = t;                               /* :213-216 self attention */
                b = t;
            } else {
                a = (doc_start > t - window) ? doc_start : t - window; /* :82 */
                b = t - 1;                                             /* :83, finishOffset = 1 */
                if (b < a) {                                           /* :84 span omitted */
                    a = t;
                    b = t - 1;
                }
            }
            span_start[ptr + t] = (int32_t)(a + ptr);
            span_finish[ptr + t] = (int32_t)(b + ptr);
        }
    }
}

int tso_init_alibi(int depth, int64_t wide_window, int max_layers, int64_t *width, float *slope)
{
    int n = 0;
    if (depth == 1) {                                /* model_dim.cpp:60-64 */
        if (max_layers < 1) return 0;
        width[0] = wide_window;
        slope[0] = 0.1f;
        return 1;
    }
    if (depth <= 0) {
        return 0;
    }
    /* ALIBI_V3, model_dim.cpp:73-92: widths {0,1,64,wide}; ids 1,1 then alternating 2(0.5),3(0) */
    int group_count = (depth + 1) / 2;
    int w1count = group_count / 6;
    if (w1count < 1) w1count = 1;
    for (int k = 0; k < w1count && n + 2 <= max_layers; ++k) {
        width[n] = 1; slope[n] = 0; ++n;
        width[n] = 1; slope[n] = 0; ++n;
    }
    for (int k = w1count; k < group_count && n + 2 <= max_layers; ++k) {
        width[n] = 64; slope[n] = 0.5f; ++n;
        width[n] = wide_window; slope[n] = 0; ++n;
    }
    return n;
}

/* ------------------------------------------------------------------------------------------ */
/* dot products                                                                               */

int32_t tso_dot_i8(const int8_t *a, const int8_t *b, int n)
{
    int32_t sum = 0;
    for (int i = 0; i < n; ++i) {
        sum += (int32_t)a[i] * (int32_t)b[i];
    }
    return sum;
}

#if defined(__x86_64__)
static inline int32_t hsum_epi32(__m256i v)
{
    /* cpu_infer.cpp:164-182 */
    __m128i lo = _mm256_castsi256_si128(v);
    __m128i hi = _mm256_extracti128_si256(v, 1);
    lo = _mm_add_epi32(lo, hi);
    __m128i sh = _mm_shuffle_epi32(lo, _MM_SHUFFLE(0, 3, 2, 1));
    lo = _mm_add_epi32(lo, sh);
    sh = _mm_shuffle_epi32(lo, _MM_SHUFFLE(1, 0, 3, 2));
    lo = _mm_add_epi32(lo, sh);
    return _mm_extract_epi32(lo, 0);
}

__attribute__((target("avx2"))) static int32_t dot_i8_avx2(const int8_t *a, const int8_t *b, int n)
{
    /* the sign trick of cpu_infer.cpp:184-196 (|x| as the unsigned operand, y*sign(x) as the
     * signed one); vpmaddubsw + vpmaddwd stand in for vpdpbusd.  |x|,|y| <= 127 keeps the
     * 16-bit pair sums below saturation (2*127*127 = 32258). */
    __m256i sum = _mm256_setzero_si256();
    const __m256i ones = _mm256_set1_epi16(1);
    for (int i = 0; i < n; i += 32) {
        __m256i x = _mm256_loadu_si256((const __m256i *)(a + i));
        __m256i y = _mm256_loadu_si256((const __m256i *)(b + i));
        __m256i ax = _mm256_sign_epi8(x, x);
        __m256i sy = _mm256_sign_epi8(y, x);
        __m256i p16 = _mm256_maddubs_epi16(ax, sy);
        sum = _mm256_add_epi32(sum, _mm256_madd_epi16(p16, ones));
    }
    return hsum_epi32(sum);
}

__attribute__((target("avx2,avxvnni"))) static int32_t dot_i8_avxvnni(const int8_t *a, const int8_t *b, int n)
{
    /* cpu_infer.cpp:184-210 with the same instruction (vpdpbusd, VEX form) */
    __m256i sum = _mm256_setzero_si256();
    for (int i = 0; i < n; i += 32) {
        __m256i x = _mm256_loadu_si256((const __m256i *)(a + i));
        __m256i y = _mm256_loadu_si256((const __m256i *)(b + i));
        __m256i ax = _mm256_sign_epi8(x, x);
        __m256i sy = _mm256_sign_epi8(y, x);
        sum = _mm256_dpbusd_avx_epi32(sum, ax, sy);
    }
    return hsum_epi32(sum);
}

__attribute__((target("avx2,avx512f,avx512vl,avx512vnni"))) static int32_t dot_i8_avx512vnni(const int8_t *a, const int8_t *b, int n)
{
    /* same, EVEX-encoded vpdpbusd on 256-bit registers */
    __m256i sum = _mm256_setzero_si256();
    for (int i = 0; i < n; i += 32) {
        __m256i x = _mm256_loadu_si256((const __m256i *)(a + i));
        __m256i y = _mm256_loadu_si256((const __m256i *)(b + i));
        __m256i ax = _mm256_sign_epi8(x, x);
        __m256i sy = _mm256_sign_epi8(y, x);
        sum = _mm256_dpbusd_epi32(sum, ax, sy);
    }
    return hsum_epi32(sum);
}
#endif

static int g_simd_level = -1;

int tso_simd_level(void)
{
    if (g_simd_level < 0) {
        int lvl = 0;
#if defined(__x86_64__)
        __builtin_cpu_init();
        if (__builtin_cpu_supports("avx2")) {
            lvl = 1;
            if (__builtin_cpu_supports("avx512vnni") && __builtin_cpu_supports("avx512vl")) {
                lvl = 3;
            } else if (__builtin_cpu_supports("avxvnni")) {
                lvl = 2;
            }
        }
#endif
        g_simd_level = lvl;
    }
    return g_simd_level;
}

int32_t tso_dot_i8_simd(const int8_t *a, const int8_t *b, int n)
{
#if defined(__x86_64__)
    if ((n & 31) == 0) {
        switch (tso_simd_level()) {
        case 3: return dot_i8_avx512vnni(a, b, n);
        case 2: return dot_i8_avxvnni(a, b, n);
        case 1: return dot_i8_avx2(a, b, n);
        default: break;
        }
    }
#endif
    return tso_dot_i8(a, b, n);
}

static int32_t g_e4m3_fix[256]; /* value * 2^9 as an integer; every e4m3 value is a multiple of 2^-9 */
static float g_e4m3_f32[256];
static int g_e4m3_ready = 0;

static void e4m3_tables(void)
{
    if (!g_e4m3_ready) {
        for (int i = 0; i < 256; ++i) {
            float f = tso_e4m3_to_float((uint8_t)i);
            g_e4m3_f32[i] = f;
            g_e4m3_fix[i] = (int32_t)ldexpf(f, 9);
        }
        g_e4m3_ready = 1;
    }
}

float tso_dot_e4m3(const uint8_t *a, const uint8_t *b, int n)
{
    e4m3_tables();
    int64_t sum = 0; /* products are multiples of 2^-18, |sum| < 2^43 for n <= 4096: exact */
    for (int i = 0; i < n; ++i) {
        sum += (int64_t)g_e4m3_fix[a[i]] * (int64_t)g_e4m3_fix[b[i]];
    }
    return (float)ldexp((double)sum, -18); /* one rounding, to nearest even */
}

void tso_qk_accum(int dtype, const uint8_t *q, int64_t q_pitch, const uint8_t *k, int64_t k_pitch,
                  int head, int head_dim, int64_t from0, int64_t n_from, int64_t to0, int64_t n_to,
                  void *acc)
{
    int64_t off = (int64_t)head * head_dim;
    for (int64_t i = 0; i < n_from; ++i) {
        for (int64_t j = 0; j < n_to; ++j) {
            const uint8_t *qa = q + (from0 + i) * q_pitch + off;
            const uint8_t *kb = k + (to0 + j) * k_pitch + off;
            if (dtype == TSO_I8) {
                ((int32_t *)acc)[i * n_to + j] = tso_dot_i8((const int8_t *)qa, (const int8_t *)kb, head_dim);
            } else {
                ((float *)acc)[i * n_to + j] = tso_dot_e4m3(qa, kb, head_dim);
            }
        }
    }
}

/* ------------------------------------------------------------------------------------------ */
/* prefill, fp32 inputs (compute/gpt_cpu.cpp:374-441)                                         */

static float calc_dp_f32(const float *qk, const float *qv, int64_t pitch, int head_q_dim, int64_t q_offset,
                         int64_t from, int64_t to, float att_dot_scale, float alibi_slope)
{
    /* gpt_cpu.cpp:379-389 */
    float sum = 0;
    for (int x = 0; x < head_q_dim; ++x) {
        sum += qk[from * pitch + q_offset + x] * qv[to * pitch + q_offset + x];
    }
    float dp = sum * att_dot_scale;
    dp += -(alibi_slope) * (float)(from - to); /* GetAttentionDecay, model_dim.h:33 */
    return dp;
}

void tso_prefill_f32(int64_t len, int n_heads, int q_dim, int tt_dim, const float *qk,
                     const float *qv, const float *v, const int32_t *span_ptr,
                     const int32_t *spans, float alibi_slope, float *out, float *sum_weight,
                     float *max_dp_out)
{
    float att_dot_scale = tso_att_dot_scale(q_dim);
    int64_t q_pitch = (int64_t)n_heads * q_dim;
    int64_t tt_pitch = (int64_t)n_heads * tt_dim;
    float *val = (float *)malloc(sizeof(float) * (size_t)tt_dim);
    for (int head = 0; head < n_heads; ++head) {
        int64_t q_offset = (int64_t)head * q_dim;
        int64_t tt_offset = (int64_t)head * tt_dim;
        for (int64_t from = 0; from < len; ++from) {
            float max_dp = 0; /* :410 the zero vector's logit takes part in the max */
            for (int32_t ai = span_ptr[from]; ai < span_ptr[from + 1]; ++ai) {
                for (int64_t to = spans[2 * ai]; to <= spans[2 * ai + 1]; ++to) {
                    float dp = calc_dp_f32(qk, qv, q_pitch, q_dim, q_offset, from, to, att_dot_scale, alibi_slope);
                    max_dp = fmaxf(max_dp, dp);
                }
            }
            float sw = exp2f(-max_dp); /* :419 zero vector of weight 1 */
            memset(val, 0, sizeof(float) * (size_t)tt_dim);
            for (int32_t ai = span_ptr[from]; ai < span_ptr[from + 1]; ++ai) {
                for (int64_t to = spans[2 * ai]; to <= spans[2 * ai + 1]; ++to) {
                    float dp = calc_dp_f32(qk, qv, q_pitch, q_dim, q_offset, from, to, att_dot_scale, alibi_slope);
                    float w = exp2f(dp - max_dp);
                    sw += w;
                    for (int x = 0; x < tt_dim; ++x) {
                        val[x] += w * v[to * tt_pitch + tt_offset + x];
                    }
                }
            }
            if (sum_weight) sum_weight[(int64_t)head * len + from] = sw;
            if (max_dp_out) max_dp_out[(int64_t)head * len + from] = max_dp;
            float inv = 1 / sw;
            for (int x = 0; x < tt_dim; ++x) {
                out[from * tt_pitch + tt_offset + x] = val[x] * inv;
            }
        }
    }
    free(val);
}

/* ------------------------------------------------------------------------------------------ */
/* prefill, 8-bit inputs with per-row scales                                                  */

static inline float acc_to_float(int dtype, const uint8_t *a, const uint8_t *b, int d)
{
    if (dtype == TSO_I8) {
        return (float)tso_dot_i8((const int8_t *)a, (const int8_t *)b, d);
    }
    return tso_dot_e4m3(a, b, d);
}

void tso_prefill_q8(int dtype, int64_t n_tokens, int n_heads, int head_dim, const uint8_t *q,
                    const uint8_t *k, const uint8_t *v, int64_t pitch, const float *q_scale,
                    const float *k_scale, const float *v_scale, int64_t scale_pitch,
                    float q_scale_const, float k_scale_const, float v_scale_const,
                    const int32_t *span_start, const int32_t *span_finish, float alibi_slope,
                    float *out, int64_t out_pitch, float *sum_weight_log, int n_threads)
{
    e4m3_tables();
    float att_dot_scale = tso_att_dot_scale(head_dim);
    if (n_threads < 1) n_threads = 1;
    int64_t n_jobs = (int64_t)n_heads * n_tokens;
#pragma omp parallel num_threads(n_threads)
    {
        float *val = (float *)malloc(sizeof(float) * (size_t)head_dim);
#pragma omp for schedule(dynamic, 16)
        for (int64_t job = 0; job < n_jobs; ++job) {
            int head = (int)(job / n_tokens);
            int64_t from = job % n_tokens;
            int64_t off = (int64_t)head * head_dim;
            const uint8_t *qrow = q + from * pitch + off;
            float qs = q_scale ? q_scale[head * scale_pitch + from] : q_scale_const;
            int64_t lo = span_start[from], hi = span_finish[from];
            /* pass 1: maximum, the zero vector's logit 0 included (gpt_cpu.cpp:410-417) */
            float max_dp = 0;
            for (int64_t to = lo; to <= hi; ++to) {
                float ks = k_scale ? k_scale[head * scale_pitch + to] : k_scale_const;
                float acc = acc_to_float(dtype, qrow, k + to * pitch + off, head_dim);
                float dp = acc * ks * att_dot_scale * qs - alibi_slope * (float)(from - to); /* cpu_infer.cpp:448 */
                max_dp = fmaxf(max_dp, dp);
            }
            /* pass 2: weights and weighted values (gpt_cpu.cpp:419-431) */
            float sw = exp2f(-max_dp);
            memset(val, 0, sizeof(float) * (size_t)head_dim);
            for (int64_t to = lo; to <= hi; ++to) {
                float ks = k_scale ? k_scale[head * scale_pitch + to] : k_scale_const;
                float vs = v_scale ? v_scale[head * scale_pitch + to] : v_scale_const;
                float acc = acc_to_float(dtype, qrow, k + to * pitch + off, head_dim);
                float dp = acc * ks * att_dot_scale * qs - alibi_slope * (float)(from - to);
                float w = exp2f(dp - max_dp);
                sw += w;
                float wv = w * vs; /* cpu_infer.cpp:454: weight times value scale, then times the 8-bit value */
                const uint8_t *vrow = v + to * pitch + off;
                if (dtype == TSO_I8) {
                    for (int x = 0; x < head_dim; ++x) {
                        val[x] += wv * (float)(int8_t)vrow[x];
                    }
                } else {
                    for (int x = 0; x < head_dim; ++x) {
                        val[x] += wv * g_e4m3_f32[vrow[x]];
                    }
                }
            }
            float inv = 1 / sw;
            for (int x = 0; x < head_dim; ++x) {
                out[from * out_pitch + off + x] = val[x] * inv;
            }
            if (sum_weight_log) {
                sum_weight_log[head * scale_pitch + from] = max_dp + log2f(sw); /* gpt_att_fp16.cuh:249 */
            }
        }
        free(val);
    }
}

/* ------------------------------------------------------------------------------------------ */
/* softmax buffer (train/cpu_infer.cpp:220-281)                                               */

static float exp2_poly_lane(float x_minus_max)
{
    /* one lane of cpu_infer.cpp:254-275 */
    float x = x_minus_max;
    x = (x > -127.0f) ? x : -127.0f; /* _mm256_max_ps(x, -127): NaN in x yields -127 as well */
    float xf = floorf(x);
    x = x - xf;
    int32_t xfi = (int32_t)nearbyintf(xf); /* cvtps_epi32 */
    float x2 = x * x;
    const float c0 = -3.069678791803394491901405992213472390777e-1f;
    const float c1 = -6.558811624324781017147952441210509604385e-2f;
    const float c2 = -1.355574723481491770403079319055785445381e-2f;
    float res = fmaf(fmaf(c2, x, c1), x, c0);
    float x_by_1_minus_x = x - x2;
    res = fmaf(res, x_by_1_minus_x, x);
    res = res + 1.0f;
    int32_t bits;
    memcpy(&bits, &res, 4);
    bits += (int32_t)((uint32_t)xfi << 23);
    memcpy(&res, &bits, 4);
    return res;
}

static float hsum8(const float *x)
{
    /* sse_utils.h:208-230: (x0+x4)+(x2+x6) then + ((x1+x5)+(x3+x7)) */
    float s0 = x[0] + x[4], s1 = x[1] + x[5], s2 = x[2] + x[6], s3 = x[3] + x[7];
    float d0 = s0 + s2, d1 = s1 + s3;
    return d0 + d1;
}

/* buf must hold ceil(n/8)*8 floats; entries beyond n are the -1e38 padding of TSoftMaxBuf.
 * Overwrites buf with the un-normalised weights and returns Scale = 1/sum. */
static float softmax_buf_inplace(float *buf, int n, float max_value, int exp2_mode)
{
    int groups = (n + 7) / 8;
    if (exp2_mode == 1) {
        float lane_sum[8] = {0, 0, 0, 0, 0, 0, 0, 0};
        for (int i = 0; i < groups; ++i) {
            for (int j = 0; j < 8; ++j) {
                float r = exp2_poly_lane(buf[i * 8 + j] - max_value);
                buf[i * 8 + j] = r;
                lane_sum[j] += r;
            }
        }
        return 1 / hsum8(lane_sum);
    }
    float sum = 0;
    for (int i = 0; i < n; ++i) {
        float r = exp2f(buf[i] - max_value);
        buf[i] = r;
        sum += r;
    }
    return 1 / sum;
}

float tso_softmax_buf(const float *logits, int n, int exp2_mode, float *weights)
{
    int cap = ((n + 7) / 8) * 8;
    if (cap < 8) cap = 8;
    float *buf = (float *)malloc(sizeof(float) * (size_t)cap);
    float max_value = 0; /* TSoftMaxBuf::Clear: MaxValue = 0 */
    for (int i = 0; i < cap; ++i) buf[i] = -1e38f;
    for (int i = 0; i < n; ++i) {
        buf[i] = logits[i];
        max_value = (max_value > logits[i]) ? max_value : logits[i];
    }
    float scale = softmax_buf_inplace(buf, n, max_value, exp2_mode);
    for (int i = 0; i < n; ++i) weights[i] = buf[i] * scale;
    free(buf);
    return scale;
}

/* ------------------------------------------------------------------------------------------ */
/* decode over a KV cache (train/cpu_infer.cpp:413-460)                                       */

void tso_decode(int dtype, int64_t n_seq, int n_heads, int head_dim, const uint8_t *q,
                const float *q_scale, float q_scale_const, const uint8_t *k, const uint8_t *v,
                int64_t seq_stride, int64_t head_stride, int64_t tok_stride, const float *k_scale,
                const float *v_scale, int64_t s_seq_stride, int64_t s_head_stride,
                float k_scale_const, float v_scale_const, const int32_t *cache_len, int64_t window,
                float alibi_slope, int exp2_mode, int use_simd, float *out, void *qk_acc,
                int64_t qk_acc_pitch, int n_threads)
{
    e4m3_tables();
    float att_dot_scale = tso_att_dot_scale(head_dim);
    if (n_threads < 1) n_threads = 1;
    int64_t n_jobs = n_seq * n_heads;
#pragma omp parallel for schedule(dynamic, 1) num_threads(n_threads)
    for (int64_t job = 0; job < n_jobs; ++job) {
        int64_t s = job / n_heads;
        int head = (int)(job % n_heads);
        int64_t cur = (int64_t)cache_len[s] - 1; /* :422 */
        float *o = out + (s * n_heads + head) * head_dim;
        for (int x = 0; x < head_dim; ++x) o[x] = 0;
        if (cur < 0) {
            continue;
        }
        /* :423-431 the key list: self only for width 0, else cur-1 ... cur-min(cur,width) */
        int64_t to_count, to_first, to_step;
        if (window == 0) {
            to_count = 1; to_first = cur; to_step = 0;
        } else {
            to_count = (cur < window) ? cur : window; to_first = cur - 1; to_step = -1;
        }
        int cap = (int)(((to_count + 1 + 7) / 8) * 8);
        float *buf = (float *)malloc(sizeof(float) * (size_t)cap);
        for (int i = 0; i < cap; ++i) buf[i] = -1e38f;
        const uint8_t *qrow = q + (s * n_heads + head) * head_dim;
        float qs = q_scale ? q_scale[s * n_heads + head] : q_scale_const;
        const uint8_t *kbase = k + s * seq_stride + head * head_stride;
        const uint8_t *vbase = v + s * seq_stride + head * head_stride;
        const float *ksb = k_scale ? k_scale + s * s_seq_stride + head * s_head_stride : NULL;
        const float *vsb = v_scale ? v_scale + s * s_seq_stride + head * s_head_stride : NULL;
        float max_value = 0;
        buf[0] = 0; /* :444 softMax.Add(0) */
        for (int64_t z = 0; z < to_count; ++z) {
            int64_t to = to_first + z * to_step;
            const uint8_t *krow = kbase + to * tok_stride;
            float accf;
            if (dtype == TSO_I8) {
                int32_t acc = use_simd ? tso_dot_i8_simd((const int8_t *)qrow, (const int8_t *)krow, head_dim)
                                       : tso_dot_i8((const int8_t *)qrow, (const int8_t *)krow, head_dim);
                if (qk_acc) ((int32_t *)qk_acc)[(s * n_heads + head) * qk_acc_pitch + to] = acc;
                accf = (float)acc;
            } else {
                accf = tso_dot_e4m3(qrow, krow, head_dim);
                if (qk_acc) ((float *)qk_acc)[(s * n_heads + head) * qk_acc_pitch + to] = accf;
            }
            float ks = ksb ? ksb[to] : k_scale_const;
            float logit = accf * ks * att_dot_scale * qs - alibi_slope * (float)(cur - to); /* :448 */
            buf[z + 1] = logit;
            max_value = (max_value > logit) ? max_value : logit;
        }
        float scale = softmax_buf_inplace(buf, (int)to_count + 1, max_value, exp2_mode); /* :450 */
        for (int64_t z = 0; z < to_count; ++z) {
            int64_t to = to_first + z * to_step;
            float vs = vsb ? vsb[to] : v_scale_const;
            float w = buf[z + 1] * scale * vs; /* :454 */
            const uint8_t *vrow = vbase + to * tok_stride;
            if (dtype == TSO_I8) {
                for (int x = 0; x < head_dim; ++x) o[x] += w * (float)(int8_t)vrow[x];
            } else {
                for (int x = 0; x < head_dim; ++x) o[x] += w * g_e4m3_f32[vrow[x]];
            }
        }
        free(buf);
    }
}

int tso_max_threads(void)
{
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}

/* ------------------------------------------------------------------------------------------ */
/* one layer, one token per sequence                                                          */

static const float TSO_VEC_SCALE = 1.0f / 24; /* train/cpu_infer.cpp:16 */
#define TSO_STATE_NORM_TILE 128               /* model_params/model_dim.h:22 */
#define TSO_COMBINER_REP 4                    /* model_params/model_dim.h:12 */

void tso_add_lookup_product(const tso_layer_params *L, int64_t n_seq, const int32_t *t, const float *rope, float *state,
                            uint8_t *k_cache, uint8_t *v_cache, int64_t seq_stride, int64_t head_stride, int64_t tok_stride,
                            float *k_scale_cache, int64_t s_seq_stride, int64_t s_head_stride, int32_t *cache_len, int max_len,
                            float *val_lookup, int n_threads)
{
    const int dim = L->dim, H = L->head_count, d = L->head_dim, qsum = H * d, kvdim = qsum * TSO_COMBINER_REP, rdim = L->relu_dim;
    uint8_t *norm = (uint8_t *)malloc((size_t)n_seq * dim);
    float *qk_src = (float *)malloc(sizeof(float) * (size_t)n_seq * qsum), *qv_src = (float *)malloc(sizeof(float) * (size_t)n_seq * qsum);
    int32_t *k_src = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_seq * qsum), *v_src = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_seq * qsum);
    uint8_t *qk = (uint8_t *)malloc((size_t)n_seq * qsum), *qv = (uint8_t *)malloc((size_t)n_seq * qsum);
    uint8_t *k = (uint8_t *)malloc((size_t)n_seq * qsum), *v = (uint8_t *)malloc((size_t)n_seq * qsum);
    float *qv_head_scale = (float *)malloc(sizeof(float) * (size_t)n_seq * H); /* [H][n_seq] */
    float *val = (float *)malloc(sizeof(float) * (size_t)n_seq * qsum);
    int8_t *kv = (int8_t *)malloc((size_t)n_seq * kvdim);
    int32_t *relu_src = (int32_t *)malloc(sizeof(int32_t) * (size_t)n_seq * rdim);
    uint8_t *relu = (uint8_t *)malloc((size_t)n_seq * rdim);

    /* :476-477  NormalizeState(&normState, *pState, dim / STATE_NORM_TILE, nullptr) */
    tso_rope_normalize_rows(TSO_I8, state, 0, dim, n_seq, NULL, NULL, 1.0f, dim / TSO_STATE_NORM_TILE, TSO_STATE_NORM_TILE, TSO_VEC_SCALE, 1.0f,
                            norm, dim, NULL, 0);
    /* :479-486  the four projections: qk and qv into float vectors, k and v into int32 */
    tso_matmul_i8((const int8_t *)norm, dim, L->qk, dim, n_seq, qsum, dim, 1, 1.0f, qk_src, qsum);
    tso_matmul_i8((const int8_t *)norm, dim, L->qv, dim, n_seq, qsum, dim, 1, 1.0f, qv_src, qsum);
    tso_matmul_i8((const int8_t *)norm, dim, L->k, dim, n_seq, qsum, dim, 0, 1.0f, k_src, qsum);
    tso_matmul_i8((const int8_t *)norm, dim, L->v, dim, n_seq, qsum, dim, 0, 1.0f, v_src, qsum);
    /* :487-499  rope on qk and qv, per-head normalisation of all four; :501-503 the key scale takes the matrix scale */
    tso_rope_normalize_rows(TSO_I8, qk_src, 0, qsum, n_seq, t, rope, 1.0f, H, d, TSO_VEC_SCALE, 1.0f, qk, qsum, NULL, 0);
    const float key_mult = L->qv_scale * TSO_VEC_SCALE * sqrtf(1.0f / (float)dim);
    tso_rope_normalize_rows(TSO_I8, qv_src, 0, qsum, n_seq, t, rope, 1.0f, H, d, TSO_VEC_SCALE, key_mult, qv, qsum, qv_head_scale, n_seq);
    tso_rope_normalize_rows(TSO_I8, k_src, 1, qsum, n_seq, NULL, NULL, 1.0f, H, d, TSO_VEC_SCALE, 1.0f, k, qsum, NULL, 0);
    tso_rope_normalize_rows(TSO_I8, v_src, 1, qsum, n_seq, NULL, NULL, 1.0f, H, d, TSO_VEC_SCALE, 1.0f, v, qsum, NULL, 0);
    /* :504  kvCache.AddVectors(qv, qvHeadScale, v) */
    for (int64_t s = 0; s < n_seq; ++s) {
        int len = cache_len[s];
        if (len < 0 || len >= max_len) continue;
        for (int h = 0; h < H; ++h) {
            memcpy(k_cache + s * seq_stride + h * head_stride + (int64_t)len * tok_stride, qv + s * qsum + h * d, (size_t)d);
            memcpy(v_cache + s * seq_stride + h * head_stride + (int64_t)len * tok_stride, v + s * qsum + h * d, (size_t)d);
            k_scale_cache[s * s_seq_stride + h * s_head_stride + len] = qv_head_scale[(int64_t)h * n_seq + s];
        }
        cache_len[s] = len + 1;
    }
    /* :506-507  ComputeValLookup(att.AttentionWidth, att.AlibiSlope, dims, kvCache, qk, &valLookup) */
    tso_decode(TSO_I8, n_seq, H, d, qk, NULL, TSO_VEC_SCALE, k_cache, v_cache, seq_stride, head_stride, tok_stride, k_scale_cache, NULL,
               s_seq_stride, s_head_stride, 0.0f, TSO_VEC_SCALE, cache_len, L->attention_width, L->alibi_slope, 0, 1, val, NULL, 0, n_threads);
    if (val_lookup) memcpy(val_lookup, val, sizeof(float) * (size_t)n_seq * qsum);
    /* :509-514  KVProduct, combiner, AddScaled */
    tso_kv_product((const int8_t *)k, qsum, val, qsum, n_seq, H, d, TSO_COMBINER_REP, 1.0f, kv, kvdim);
    tso_matmul_i8(kv, kvdim, L->combiner, kvdim, n_seq, dim, kvdim, 2, L->combiner_scale * TSO_VEC_SCALE * sqrtf(1.0f / (float)kvdim), state, dim);
    /* :516-526  feed-forward: normalise, expand, normalise per head, ReLU, contract, AddScaled */
    tso_rope_normalize_rows(TSO_I8, state, 0, dim, n_seq, NULL, NULL, 1.0f, dim / TSO_STATE_NORM_TILE, TSO_STATE_NORM_TILE, TSO_VEC_SCALE, 1.0f,
                            norm, dim, NULL, 0);
    tso_matmul_i8((const int8_t *)norm, dim, L->expand, dim, n_seq, rdim, dim, 0, 1.0f, relu_src, rdim);
    tso_rope_normalize_rows(TSO_I8, relu_src, 1, rdim, n_seq, NULL, NULL, 1.0f, H, rdim / H, TSO_VEC_SCALE, 1.0f, relu, rdim, NULL, 0);
    for (int64_t i = 0; i < n_seq * rdim; ++i) {
        if ((int8_t)relu[i] < 0) relu[i] = 0; /* x = Max<i8>(0, x) */
    }
    tso_matmul_i8((const int8_t *)relu, rdim, L->contract, rdim, n_seq, dim, rdim, 2, L->contract_scale * TSO_VEC_SCALE * sqrtf(1.0f / (float)rdim), state, dim);

    free(norm); free(qk_src); free(qv_src); free(k_src); free(v_src); free(qk); free(qv); free(k); free(v);
    free(qv_head_scale); free(val); free(kv); free(relu_src); free(relu);
}

/* ------------------------------------------------------------------------------------------ */
/* embedding and final softmax (train/cpu_infer.cpp:552-582)                                  */

void tso_embed_rows(int64_t n_rows, int dim, const int32_t *labels, int labels_per_row, const int8_t *embed, int64_t n_labels,
                    float scale, float *state)
{
    for (int64_t r = 0; r < n_rows; ++r) {
        float *st = state + r * dim;
        for (int x = 0; x < dim; ++x) st[x] = 0; /* ClearPodArray(&state, dim) */
        for (int l = 0; l < labels_per_row; ++l) {
            int32_t label = labels[r * labels_per_row + l];
            if (label < 0 || label >= n_labels) continue;
            for (int x = 0; x < dim; ++x) {
                st[x] += embed[(int64_t)label * dim + x] * scale; /* state[x] += LabelEmbed[label][x] * LabelEmbedScale */
            }
        }
    }
}

void tso_softmax_rows(int64_t n_rows, int64_t n, const int32_t *vec, float scale, const float *bias, int exp2_mode, float *prob,
                      int32_t *argmax)
{
    int64_t cap = ((n + 7) / 8) * 8;
    if (cap < 8) cap = 8;
    float *buf = (float *)malloc(sizeof(float) * (size_t)cap);
    for (int64_t r = 0; r < n_rows; ++r) {
        float max_value = 0; /* a fresh TSoftMaxBuf: MaxValue = 0 */
        float best = -INFINITY;
        int32_t arg = 0;
        for (int64_t i = n; i < cap; ++i) buf[i] = -1e38f;
        for (int64_t k = 0; k < n; ++k) {
            float w = vec[r * n + k] * scale + (bias ? bias[k] : 0.0f); /* vec[k] * vecScale + bias[k] */
            buf[k] = w;
            max_value = (max_value > w) ? max_value : w;
            if (w > best) { best = w; arg = (int32_t)k; }
        }
        if (argmax) argmax[r] = arg;
        if (prob) {
            float sc = softmax_buf_inplace(buf, (int)n, max_value, exp2_mode);
            for (int64_t k = 0; k < n; ++k) prob[r * n + k] = buf[k] * sc;
        }
    }
    free(buf);
}

/* ------------------------------------------------------------------------------------------ */
/* SampleFromDistr: train/cpu_infer.cpp:585-599                                               */

uint32_t tso_mix32(uint64_t seed, uint64_t index)
{
    uint64_t z = seed + (index + 1) * 0x9E3779B97F4A7C15ull; /* splitmix64's output function on a counter */
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (uint32_t)(z >> 32);
}

void tso_sample_rows(int64_t n_rows, int64_t n, const float *prob, int64_t prob_pitch, float temperature, const uint32_t *rnd,
                     int64_t rnd_pitch, uint64_t seed, uint64_t offset, int32_t *choice)
{
    for (int64_t row = 0; row < n_rows; ++row) {
        float best = -1e38f;
        int64_t res = 0;
        for (int64_t k = 0; k < n; ++k) {
            const uint32_t r = rnd ? rnd[row * rnd_pitch + k] : tso_mix32(seed, offset + (uint64_t)(row * n + k));
            const double u = ((double)r + 0.5) * (1.0 / 4294967296.0);
            const float score = (float)((double)(logf(prob[row * prob_pitch + k]) / temperature) - log(-log(u)));
            if (score > best) {
                best = score;
                res = k;
            }
        }
        choice[row] = (int32_t)res;
    }
}
