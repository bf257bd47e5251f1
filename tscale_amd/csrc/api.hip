// C ABI of the library (declared in include/tsattn.h): argument checks, the handle and the
// launches.  Nothing here allocates, frees or synchronises except tsattn_create / tsattn_destroy.
#include <hip/hip_runtime.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include <algorithm>
#include <mutex>

#include "../../include/tsattn.h"
#include "../../include/tsattn_test_hooks.h"
#include "kernels.hpp"

struct tsattn_ctx {
    int device;
    int max_seqs, max_heads, max_head_dim, max_splits;
    float *part_acc;
    float *part_ml;
    int32_t *seq_done;
};

// Scratch of the entry point that allocates nothing (tsattn_decode_static): split partials [pair][split][d] f32, their
// (max, sum) pairs, per-sequence arrival counters.  One copy per GPU the library runs on, held until the process ends.
constexpr int64_t STATIC_ACC_BYTES = (int64_t)TSATTN_STATIC_MAX_PARTS * 128 * sizeof(float);
constexpr int64_t STATIC_ML_BYTES = (int64_t)TSATTN_STATIC_MAX_PARTS * 2 * sizeof(float);
constexpr int64_t STATIC_CNT_BYTES = (int64_t)TSATTN_STATIC_MAX_SEQS * sizeof(int32_t);
static __device__ __align__(256) uint8_t g_decode_scratch[STATIC_ACC_BYTES + STATIC_ML_BYTES + STATIC_CNT_BYTES];
constexpr int STATIC_MAX_DEVICES = 64;
static uint8_t *g_static_ptr[STATIC_MAX_DEVICES]; // this device's copy of the array, from hipGetSymbolAddress
static std::mutex g_static_mutex;

struct DecodeScratch {
    int max_seqs, max_head_dim, max_splits;
    int64_t max_pairs, max_parts; // (sequence, head) pairs; pairs x splits
    float *part_acc, *part_ml;
    int32_t *seq_done;
    bool clear_counters;
};

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char *fmt, ...)
{
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

int hip_fail(hipError_t e, const char *what)
{
    return fail(TSATTN_ERR_HIP, "%s: %s", what, hipGetErrorString(e));
}

constexpr int DEFAULT_MAX_SPLITS = 32;

int cfg_splits(const tsattn_config *cfg) { return cfg->max_splits > 0 ? cfg->max_splits : DEFAULT_MAX_SPLITS; }

bool head_dim_ok(int d) { return d == 64 || d == 128; }
bool dtype_ok(int t) { return t == TSATTN_I8 || t == TSATTN_E4M3; }
bool aligned16(const void *p) { return (((uintptr_t)p) & 15) == 0; }

} // namespace

// The body of both decode entry points; `lim` says what the scratch behind part_acc / part_ml / seq_done was sized for.
static int decode_with_scratch(const DecodeScratch &lim, const tsattn_decode_args *a, void *stream)
{
    if (!dtype_ok(a->dtype)) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_decode: dtype %d", a->dtype);
    if (a->q_dtype != TSATTN_Q_8BIT && a->q_dtype != TSATTN_Q_BF16) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_decode: q_dtype %d", a->q_dtype);
    if (!head_dim_ok(a->head_dim)) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_decode: head_dim %d (64 or 128 supported)", a->head_dim);
    if (a->n_seqs < 0 || a->n_heads <= 0 || a->max_len < 0 || a->window < 0) return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: negative size");
    if (a->n_seqs == 0) return TSATTN_OK;
    if (!a->q || !a->k_cache || !a->v_cache || !a->cache_len || !a->out) return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: null data pointer");
    const int qbytes = a->q_dtype == TSATTN_Q_BF16 ? 2 : 1;
    if (a->q_pitch < (int64_t)a->n_heads * a->head_dim * qbytes || a->q_pitch % 16) return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: q_pitch");
    if (a->tok_stride < a->head_dim || a->tok_stride % 16 || a->head_stride % 16 || a->seq_stride % 16)
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: cache strides must be multiples of 16 bytes, tok_stride >= head_dim");
    if (!aligned16(a->q) || !aligned16(a->k_cache) || !aligned16(a->v_cache)) return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: q and caches must be 16-byte aligned");
    if (a->debug_qk_acc && a->debug_pitch < a->max_len) return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: debug_pitch < max_len");
    if (a->n_seqs > lim.max_seqs || a->head_dim > lim.max_head_dim || (int64_t)a->n_seqs * a->n_heads > lim.max_pairs)
        return fail(TSATTN_ERR_SCRATCH, "tsattn_decode: %d seqs x %d heads x d%d exceeds the scratch's %d seqs, %lld (seq, head) pairs, d%d", a->n_seqs,
                    a->n_heads, a->head_dim, lim.max_seqs, (long long)lim.max_pairs, lim.max_head_dim);
    const int max_splits = (int)std::min<int64_t>(lim.max_splits, lim.max_parts / ((int64_t)a->n_seqs * a->n_heads));
    int splits = a->n_splits;
    if (splits < 0 || splits > max_splits) return fail(TSATTN_ERR_SCRATCH, "tsattn_decode: n_splits %d exceeds the scratch's %d for this batch", splits, max_splits);
    if (splits == 0) {
        // One workgroup streams its rows fast enough that one or two per compute unit reach the memory's rate, and every
        // split beyond that only adds to the merge: about 384 workgroups in all (measured best at 4096 rows: 1 split from
        // 256 (sequence, head) pairs up, 4 at 128, 8 at 32 and below), and at least 512 cache rows per split
        const int64_t pairs = (int64_t)a->n_seqs * a->n_heads;
        int64_t want = 384 / pairs;
        int64_t rows = a->max_len;   // rows one query can see
        if (a->window < rows) rows = a->window > 0 ? a->window : 1;
        int64_t by_len = (rows + 511) / 512;
        if (want > by_len) want = by_len;
        if (want < 1) want = 1;
        if (want > max_splits) want = max_splits;
        splits = (int)want;
    }
    tsattn::DecodeParams p = {};
    p.q = (const uint8_t *)a->q; p.q_pitch = a->q_pitch; p.q_scale = a->q_scale; p.q_scale_const = a->q_scale_const;
    p.k = (const uint8_t *)a->k_cache; p.v = (const uint8_t *)a->v_cache;
    p.seq_stride = a->seq_stride; p.head_stride = a->head_stride; p.tok_stride = a->tok_stride;
    p.ks = a->k_scale; p.vs = a->v_scale; p.s_seq_stride = a->s_seq_stride; p.s_head_stride = a->s_head_stride;
    p.ks_const = a->k_scale_const; p.vs_const = a->v_scale_const;
    p.cache_len = a->cache_len; p.window = a->window; p.slope = a->alibi_slope;
    p.n_heads = a->n_heads; p.n_splits = splits;
    p.part_acc = lim.part_acc; p.part_ml = lim.part_ml;
    p.dbg = a->debug_qk_acc; p.dbg_pitch = a->debug_pitch;
    p.out = a->out;
    p.k_new = (const uint8_t *)a->k_new; p.v_new = (const uint8_t *)a->v_new; p.new_pitch = a->new_pitch;
    p.ks_new = a->k_scale_new; p.vs_new = a->v_scale_new;
    p.cache_len_rw = const_cast<int32_t *>(a->cache_len); p.max_len = a->max_len;
    p.seq_done = lim.seq_done;
    if (a->kv_out) {
        if (!a->kv_k) return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: the fused KVProduct needs kv_k");
        if (a->dtype != TSATTN_I8) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_decode: the fused KVProduct is defined for int8 keys");
        if (a->kv_rep < 1 || a->kv_rep > 4) return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: kv_rep %d (1..4)", a->kv_rep);
        if (((uintptr_t)a->kv_k & 3) || a->kv_k_pitch % 4 || a->kv_k_pitch < (int64_t)a->n_heads * a->head_dim ||
            a->kv_out_pitch < (int64_t)a->n_heads * a->head_dim * a->kv_rep)
            return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: kv_k must be 4-byte aligned and the kv pitches must cover a row");
        p.kv_k = (const uint8_t *)a->kv_k; p.kv_k_pitch = a->kv_k_pitch; p.kv_out = (uint8_t *)a->kv_out; p.kv_out_pitch = a->kv_out_pitch;
        p.kv_rep = a->kv_rep; p.kv_mult = a->kv_mult;
    }
    if (a->k_new || a->v_new) {
        if (!a->k_new || !a->v_new) return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: fused append needs both k_new and v_new");
        if (a->window == 0) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_decode: fused append is not available with window 0; call tsattn_cache_append first");
        if (a->new_pitch % 16 || a->new_pitch < (int64_t)a->n_heads * a->head_dim || !aligned16(a->k_new) || !aligned16(a->v_new))
            return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: k_new/v_new must be 16-byte aligned with a pitch that covers a row");
        if ((a->k_scale_new && !a->k_scale) || (a->v_scale_new && !a->v_scale)) return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: new scales given without scale planes");
    }
    if (lim.clear_counters && a->k_new) {
        // the arrival counters of the single-split fused append start at zero: a launch leaves them so, but this scratch is
        // shared by every caller on the device (a fill kernel, not a memset: callers may be capturing a graph)
        hipError_t ez = tsattn::launch_zero_i32(lim.seq_done, a->n_seqs, (hipStream_t)stream);
        if (ez != hipSuccess) return hip_fail(ez, "counter clear launch");
    }
    hipError_t e = tsattn::launch_decode(p, a->dtype, a->head_dim, a->q_dtype == TSATTN_Q_BF16, a->n_seqs, a->out, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "decode launch");
    return TSATTN_OK;
}


extern "C" {

const char *tsattn_last_error(void) { return g_err; }

const char *tsattn_version(void) { return "tsattn 0.1 gfx950 (hip; mfma f8f6f4/i8 prefill, split-kv decode)"; }

size_t tsattn_scratch_bytes(const tsattn_config *cfg)
{
    if (!cfg || cfg->max_seqs < 0 || cfg->max_heads < 0 || cfg->max_head_dim < 0) return 0;
    size_t parts = (size_t)cfg->max_seqs * cfg->max_heads * cfg_splits(cfg);
    return parts * ((size_t)cfg->max_head_dim + 2) * sizeof(float) + (size_t)cfg->max_seqs * sizeof(int32_t);
}

int tsattn_create(const tsattn_config *cfg, tsattn_handle_t *out)
{
    if (!cfg || !out) return fail(TSATTN_ERR_BAD_ARG, "tsattn_create: null argument");
    if (cfg->max_seqs < 0 || cfg->max_heads < 0 || cfg->max_head_dim < 0 || cfg->max_splits < 0)
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_create: negative size");
    if (cfg->max_head_dim != 0 && !head_dim_ok(cfg->max_head_dim))
        return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_create: head_dim %d (64 or 128 supported)", cfg->max_head_dim);
    int n_dev = 0;
    hipError_t e = hipGetDeviceCount(&n_dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDeviceCount");
    if (cfg->device < 0 || cfg->device >= n_dev) return fail(TSATTN_ERR_BAD_ARG, "tsattn_create: device %d of %d", cfg->device, n_dev);
    e = hipSetDevice(cfg->device);
    if (e != hipSuccess) return hip_fail(e, "hipSetDevice");
    e = tsattn::prepare_matmul_i8();
    if (e == hipSuccess) e = tsattn::prepare_prefill_long();
    if (e != hipSuccess) return hip_fail(e, "hipFuncSetAttribute");
    tsattn_ctx *c = new tsattn_ctx();
    c->device = cfg->device;
    c->max_seqs = cfg->max_seqs;
    c->max_heads = cfg->max_heads;
    c->max_head_dim = cfg->max_head_dim;
    c->max_splits = cfg_splits(cfg);
    c->part_acc = nullptr;
    c->part_ml = nullptr;
    c->seq_done = nullptr;
    size_t parts = (size_t)c->max_seqs * c->max_heads * c->max_splits;
    if (parts > 0 && c->max_head_dim > 0) {
        e = hipMalloc((void **)&c->part_acc, parts * c->max_head_dim * sizeof(float));
        if (e != hipSuccess) { delete c; return hip_fail(e, "hipMalloc(split partials)"); }
        e = hipMalloc((void **)&c->part_ml, parts * 2 * sizeof(float));
        if (e != hipSuccess) { (void)hipFree(c->part_acc); delete c; return hip_fail(e, "hipMalloc(split max/sum)"); }
    }
    if (c->max_seqs > 0) {
        // arrival counters of the single-split fused append: zero here, and left at zero by every launch
        e = hipMalloc((void **)&c->seq_done, (size_t)c->max_seqs * sizeof(int32_t));
        if (e == hipSuccess) e = hipMemset(c->seq_done, 0, (size_t)c->max_seqs * sizeof(int32_t));
        if (e != hipSuccess) {
            if (c->seq_done) (void)hipFree(c->seq_done);
            if (c->part_acc) (void)hipFree(c->part_acc);
            if (c->part_ml) (void)hipFree(c->part_ml);
            delete c;
            return hip_fail(e, "hipMalloc(arrival counters)");
        }
    }
    *out = c;
    return TSATTN_OK;
}

int tsattn_destroy(tsattn_handle_t h)
{
    if (!h) return TSATTN_OK;
    if (h->part_acc) (void)hipFree(h->part_acc);
    if (h->part_ml) (void)hipFree(h->part_ml);
    if (h->seq_done) (void)hipFree(h->seq_done);
    delete h;
    return TSATTN_OK;
}

int tsattn_prefill(tsattn_handle_t h, const tsattn_prefill_args *a, void *stream)
{
    if (!h || !a) return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: null argument");
    if (!dtype_ok(a->dtype)) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_prefill: dtype %d", a->dtype);
    if (a->out_dtype != TSATTN_OUT_F32 && a->out_dtype != TSATTN_OUT_F16)
        return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_prefill: out_dtype %d", a->out_dtype);
    if (!head_dim_ok(a->head_dim)) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_prefill: head_dim %d (64 or 128 supported)", a->head_dim);
    if (a->n_tokens < 0 || a->n_heads <= 0) return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: n_tokens %lld n_heads %d", (long long)a->n_tokens, a->n_heads);
    if (a->n_tokens > 0x7fffffff - 256) return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: n_tokens too large");
    if (a->n_tokens == 0) return TSATTN_OK;
    if (!a->q || !a->k || !a->v || (!a->out && !a->kv_out) || !a->span_start || !a->span_finish)
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: null data pointer");
    const int64_t row = (int64_t)a->n_heads * a->head_dim;
    if (a->q_pitch < row || a->k_pitch < row || a->v_pitch < row || (a->q_pitch | a->k_pitch | a->v_pitch) % 16)
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: input pitch must be >= %lld and a multiple of 16", (long long)row);
    // (the kernel addresses the rows of a key tile with 32-bit offsets from the tile's first row)
    if (a->k_pitch > TSATTN_PREFILL_MAX_KV_PITCH || a->v_pitch > TSATTN_PREFILL_MAX_KV_PITCH)
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: k_pitch and v_pitch may be at most %lld bytes", (long long)TSATTN_PREFILL_MAX_KV_PITCH);
    const int64_t out_row = row * (a->out_dtype == TSATTN_OUT_F16 ? 2 : 4);
    if (a->out && (a->out_pitch < out_row || a->out_pitch % 16)) return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: out_pitch must be >= %lld and a multiple of 16", (long long)out_row);
    if (!aligned16(a->q) || !aligned16(a->k) || !aligned16(a->v) || !aligned16(a->out))
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: q, k, v, out must be 16-byte aligned");
    if ((a->q_scale || a->k_scale || a->v_scale || a->sum_weight_log) && a->scale_pitch < a->n_tokens)
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: scale_pitch %lld < n_tokens", (long long)a->scale_pitch);
    if (a->debug_qk_acc && a->debug_pitch < a->n_tokens) return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: debug_pitch < n_tokens");

    if (a->n_span_parts > 1 && (a->n_span_parts > 64 || a->span_part_stride < a->n_tokens))
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: n_span_parts %d (at most 64) with span_part_stride %lld (at least n_tokens)", a->n_span_parts, (long long)a->span_part_stride);
    if (a->kv_out) {
        if (!a->kv_k) return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: the fused KVProduct needs kv_k");
        if (a->out_dtype != TSATTN_OUT_F32 || a->dtype != TSATTN_I8)
            return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_prefill: the fused KVProduct goes with int8 attention and takes the f32 result (out_dtype f32)");
        if (a->debug_qk_acc) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_prefill: no fused KVProduct together with debug_qk_acc");
        if (a->kv_rep < 1 || a->kv_rep > 4) return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: kv_rep %d (1..4)", a->kv_rep);
        if (((uintptr_t)a->kv_k & 3) || a->kv_k_pitch % 4 || a->kv_k_pitch < row || !aligned16(a->kv_out) || a->kv_out_pitch % 16 ||
            a->kv_out_pitch < row * a->kv_rep)
            return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: kv_k must be 4-byte aligned, kv_out 16-byte aligned (pitches too) and the kv pitches must cover a row");
    }

    tsattn::PrefillParams p = {};
    if (a->kv_out) {
        p.kv_k = (const uint8_t *)a->kv_k; p.kv_k_pitch = a->kv_k_pitch; p.kv_out = (uint8_t *)a->kv_out; p.kv_out_pitch = a->kv_out_pitch;
        p.kv_rep = a->kv_rep; p.kv_mult = a->kv_mult;
    }
    p.q = (const uint8_t *)a->q; p.k = (const uint8_t *)a->k; p.v = (const uint8_t *)a->v;
    p.q_pitch = a->q_pitch; p.k_pitch = a->k_pitch; p.v_pitch = a->v_pitch;
    p.qs = a->q_scale; p.ks = a->k_scale; p.vs = a->v_scale;
    p.scale_pitch = a->scale_pitch;
    p.qs_const = a->q_scale_const; p.ks_const = a->k_scale_const; p.vs_const = a->v_scale_const;
    p.k_global_scale = a->k_global_scale;
    p.span_start = a->span_start; p.span_finish = a->span_finish;
    p.span_tiles = a->span_tiles;
    p.n_parts = a->n_span_parts > 1 ? a->n_span_parts : 1;
    p.span_part_stride = p.n_parts > 1 ? a->span_part_stride : 0;
    p.slope = a->alibi_slope;
    p.out = a->out; p.out_pitch = a->out_pitch;
    p.sum_weight_log = a->sum_weight_log;
    p.dbg = a->debug_qk_acc; p.dbg_pitch = a->debug_pitch;
    p.n_tokens = (int)a->n_tokens; p.n_heads = a->n_heads;
    p.period_tiles = (a->causal_period > 0 && a->causal_period % 128 == 0 && a->n_tokens % a->causal_period == 0) ? (int)(a->causal_period / 128) : 0;
    // Long spans with room for the f16 copy of V: the kernel that streams K and that copy through LDS.  (It addresses
    // K and the copy with 31-bit byte offsets.)
    if (a->workspace && a->span_len_hint >= TSATTN_PREFILL_LONG_SPAN && a->head_dim == 128 && a->alibi_slope == 0.0f && !a->debug_qk_acc && !a->kv_out && a->n_span_parts <= 1) {
        const size_t need = tsattn::prefill_long_workspace_bytes(a->n_tokens, a->n_heads, a->head_dim);
        const int64_t vt_pitch = tsattn::prefill_long_vt_pitch(a->n_tokens);
        if (!aligned16(a->workspace)) return fail(TSATTN_ERR_BAD_ARG, "tsattn_prefill: workspace must be 16-byte aligned");
        if (need != 0 && a->workspace_bytes >= (int64_t)need && a->n_tokens * a->k_pitch < ((int64_t)1 << 31) && 128 * vt_pitch * 2 < ((int64_t)1 << 31)) {
            p.vt = a->workspace;
            p.vt_pitch = vt_pitch;
        }
    }
    hipError_t e = tsattn::launch_prefill(p, a->dtype, a->head_dim, a->out_dtype, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "prefill launch");
    return TSATTN_OK;
}

size_t tsattn_prefill_workspace_bytes(int64_t n_tokens, int n_heads, int head_dim)
{
    if (n_tokens <= 0 || n_heads <= 0) return 0;
    return tsattn::prefill_long_workspace_bytes(n_tokens, n_heads, head_dim);
}

int tsattn_decode(tsattn_handle_t h, const tsattn_decode_args *a, void *stream)
{
    if (!h || !a) return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode: null argument");
    DecodeScratch lim;
    lim.max_seqs = h->max_seqs; lim.max_head_dim = h->max_head_dim; lim.max_splits = h->max_splits;
    lim.max_pairs = (int64_t)h->max_seqs * h->max_heads;
    lim.max_parts = lim.max_pairs * h->max_splits;
    lim.part_acc = h->part_acc; lim.part_ml = h->part_ml; lim.seq_done = h->seq_done;
    lim.clear_counters = false;
    return decode_with_scratch(lim, a, stream);
}

int tsattn_debug_read_counters(tsattn_handle_t h, int32_t *dst, int n, void *stream)
{
    if (!h || !dst || n < 0 || n > h->max_seqs) return fail(TSATTN_ERR_BAD_ARG, "tsattn_debug_read_counters: bad argument");
    if (n == 0) return TSATTN_OK;
    hipError_t e = hipMemcpyAsync(dst, h->seq_done, (size_t)n * sizeof(int32_t), hipMemcpyDeviceToDevice, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "counter copy");
    return TSATTN_OK;
}

int tsattn_decode_static(const tsattn_decode_args *a, void *stream)
{
    if (!a) return fail(TSATTN_ERR_BAD_ARG, "tsattn_decode_static: null argument");
    int dev = -1;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_fail(e, "hipGetDevice");
    if (dev < 0 || dev >= STATIC_MAX_DEVICES) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_decode_static: device %d (ordinals below %d)", dev, STATIC_MAX_DEVICES);
    uint8_t *base;
    {
        // Set-up, once per device and with that device current: the array's name is a host-side stand-in; the address of
        // this device's copy comes from the runtime and is what every use below goes through.
        std::lock_guard<std::mutex> lock(g_static_mutex);
        if (!g_static_ptr[dev]) {
            void *ptr = nullptr;
            e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(g_decode_scratch));
            if (e != hipSuccess || !ptr) return hip_fail(e, "hipGetSymbolAddress(decode scratch)");
            g_static_ptr[dev] = (uint8_t *)ptr;
        }
        base = g_static_ptr[dev];
    }
    DecodeScratch lim;
    lim.max_seqs = TSATTN_STATIC_MAX_SEQS; lim.max_head_dim = 128; lim.max_splits = DEFAULT_MAX_SPLITS;
    lim.max_pairs = TSATTN_STATIC_MAX_PARTS; lim.max_parts = TSATTN_STATIC_MAX_PARTS;
    lim.part_acc = (float *)base;
    lim.part_ml = (float *)(base + STATIC_ACC_BYTES);
    lim.seq_done = (int32_t *)(base + STATIC_ACC_BYTES + STATIC_ML_BYTES);
    lim.clear_counters = true;
    return decode_with_scratch(lim, a, stream);
}

int tsattn_cache_append(tsattn_handle_t h, const tsattn_append_args *a, void *stream)
{
    if (!h || !a) return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_append: null argument");
    if (!head_dim_ok(a->head_dim)) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_cache_append: head_dim %d (64 or 128 supported)", a->head_dim);
    if (a->n_seqs < 0 || a->n_heads <= 0 || a->max_len < 0) return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_append: negative size");
    if (a->n_seqs == 0) return TSATTN_OK;
    if (!a->k_new || !a->v_new || !a->k_cache || !a->v_cache || !a->cache_len) return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_append: null data pointer");
    if ((a->k_scale_new && !a->k_scale) || (a->v_scale_new && !a->v_scale)) return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_append: new scales given without scale planes");
    if (a->new_pitch % 16 || a->tok_stride % 16 || a->head_stride % 16 || a->seq_stride % 16 || a->tok_stride < a->head_dim)
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_append: pitches and strides must be multiples of 16 bytes");
    if (!aligned16(a->k_new) || !aligned16(a->v_new) || !aligned16(a->k_cache) || !aligned16(a->v_cache))
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_append: pointers must be 16-byte aligned");
    tsattn::AppendParams p;
    p.k_new = (const uint8_t *)a->k_new; p.v_new = (const uint8_t *)a->v_new; p.new_pitch = a->new_pitch;
    p.ks_new = a->k_scale_new; p.vs_new = a->v_scale_new;
    p.k = (uint8_t *)a->k_cache; p.v = (uint8_t *)a->v_cache;
    p.seq_stride = a->seq_stride; p.head_stride = a->head_stride; p.tok_stride = a->tok_stride;
    p.ks = a->k_scale; p.vs = a->v_scale; p.s_seq_stride = a->s_seq_stride; p.s_head_stride = a->s_head_stride;
    p.cache_len = a->cache_len; p.max_len = a->max_len; p.n_heads = a->n_heads; p.head_dim = a->head_dim;
    hipError_t e = tsattn::launch_cache_append(p, a->n_seqs, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "cache append launch");
    return TSATTN_OK;
}

int64_t tsattn_span_tiles_count(int64_t n_tokens)
{
    return n_tokens <= 0 ? 0 : (n_tokens + 127) / 128;
}

int tsattn_build_span_tiles(tsattn_handle_t h, int64_t n_tokens, const int32_t *span_start, const int32_t *span_finish,
                            int32_t *tiles, void *stream)
{
    if (!h) return fail(TSATTN_ERR_BAD_ARG, "tsattn_build_span_tiles: null handle");
    if (n_tokens < 0 || n_tokens > 0x7fffffff) return fail(TSATTN_ERR_BAD_ARG, "tsattn_build_span_tiles: n_tokens %lld", (long long)n_tokens);
    if (n_tokens == 0) return TSATTN_OK;
    if (!span_start || !span_finish || !tiles) return fail(TSATTN_ERR_BAD_ARG, "tsattn_build_span_tiles: null data pointer");
    if ((uintptr_t)tiles % 16) return fail(TSATTN_ERR_BAD_ARG, "tsattn_build_span_tiles: tiles must be 16-byte aligned");
    hipError_t e = tsattn::launch_build_span_tiles(n_tokens, span_start, span_finish, tiles, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "span tiles launch");
    return TSATTN_OK;
}

int tsattn_merge_lookups(tsattn_handle_t h, const tsattn_merge_args *a, void *stream)
{
    if (!h || !a) return fail(TSATTN_ERR_BAD_ARG, "tsattn_merge_lookups: null argument");
    if (a->n_parts < 1 || a->n_parts > 64) return fail(TSATTN_ERR_BAD_ARG, "tsattn_merge_lookups: n_parts %d (1..64)", a->n_parts);
    if (a->n_tokens < 0 || a->n_heads <= 0 || a->head_dim <= 0 || a->head_dim % 4)
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_merge_lookups: n_tokens %lld, n_heads %d, head_dim %d (a multiple of 4)", (long long)a->n_tokens, a->n_heads, a->head_dim);
    if (a->out_dtype != TSATTN_OUT_F32 && a->out_dtype != TSATTN_OUT_F16) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_merge_lookups: out_dtype %d", a->out_dtype);
    if (a->n_tokens == 0) return TSATTN_OK;
    if (!a->part_out || !a->part_swl || !a->out) return fail(TSATTN_ERR_BAD_ARG, "tsattn_merge_lookups: null data pointer");
    const int64_t row = (int64_t)a->n_heads * a->head_dim;
    if (a->part_out_pitch < row || a->part_out_pitch % 4 || a->part_out_stride % 4 || !aligned16(a->part_out) ||
        (a->n_parts > 1 && a->part_out_stride < a->n_tokens * a->part_out_pitch))
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_merge_lookups: parts must be 16-byte aligned, rows of part_out_pitch >= %lld floats (a multiple of 4), parts a whole result apart", (long long)row);
    if (a->scale_pitch < a->n_tokens || (a->n_parts > 1 && a->part_swl_stride < (int64_t)a->n_heads * a->scale_pitch))
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_merge_lookups: scale_pitch below n_tokens or sum_weight_log planes that overlap");
    const int64_t out_row = row * (a->out_dtype == TSATTN_OUT_F16 ? 2 : 4);
    if (a->out_pitch < out_row || a->out_pitch % 16 || !aligned16(a->out))
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_merge_lookups: out must be 16-byte aligned with a pitch >= %lld bytes, a multiple of 16", (long long)out_row);
    tsattn::MergeParams p;
    p.n_parts = a->n_parts; p.n_tokens = a->n_tokens; p.n_heads = a->n_heads; p.head_dim = a->head_dim;
    p.part_out = a->part_out; p.part_out_pitch = a->part_out_pitch; p.part_out_stride = a->part_out_stride;
    p.part_swl = a->part_swl; p.scale_pitch = a->scale_pitch; p.part_swl_stride = a->part_swl_stride;
    p.out = a->out; p.out_pitch = a->out_pitch; p.swl = a->sum_weight_log;
    const hipError_t e = tsattn::launch_merge_lookups(p, a->out_dtype == TSATTN_OUT_F16, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "merge launch");
    return TSATTN_OK;
}

int tsattn_cache_fill(tsattn_handle_t h, const tsattn_fill_args *a, void *stream)
{
    if (!h || !a) return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_fill: null argument");
    if (!head_dim_ok(a->head_dim)) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_cache_fill: head_dim %d (64 or 128 supported)", a->head_dim);
    if (a->n_seqs < 0 || a->n_heads <= 0 || a->max_len < 0 || a->n_tokens < 0) return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_fill: negative size");
    if (a->n_heads > 65535) return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_fill: too many heads");
    if (a->n_seqs == 0 || a->n_tokens == 0) return TSATTN_OK;
    if (!a->seq_offset || !a->k || !a->v || !a->k_cache || !a->v_cache || !a->cache_len) return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_fill: null data pointer");
    if ((a->k_scale && !a->k_scale_cache) || (a->v_scale && !a->v_scale_cache)) return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_fill: scales given without scale planes");
    if (a->pitch % 16 || a->tok_stride % 16 || a->head_stride % 16 || a->seq_stride % 16 || a->tok_stride < a->head_dim ||
        a->pitch < (int64_t)a->n_heads * a->head_dim)
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_fill: pitches and strides must be multiples of 16 bytes and cover a row");
    if (!aligned16(a->k) || !aligned16(a->v) || !aligned16(a->k_cache) || !aligned16(a->v_cache))
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_fill: pointers must be 16-byte aligned");
    if ((a->k_scale || a->v_scale) && a->scale_pitch < a->n_tokens) return fail(TSATTN_ERR_BAD_ARG, "tsattn_cache_fill: scale_pitch below n_tokens");
    tsattn::FillParams p;
    p.seq_offset = a->seq_offset; p.k_src = (const uint8_t *)a->k; p.v_src = (const uint8_t *)a->v; p.pitch = a->pitch;
    p.ks_src = a->k_scale; p.vs_src = a->v_scale; p.scale_pitch = a->scale_pitch;
    p.k = (uint8_t *)a->k_cache; p.v = (uint8_t *)a->v_cache;
    p.seq_stride = a->seq_stride; p.head_stride = a->head_stride; p.tok_stride = a->tok_stride;
    p.ks = a->k_scale_cache; p.vs = a->v_scale_cache; p.s_seq_stride = a->s_seq_stride; p.s_head_stride = a->s_head_stride;
    p.cache_len = a->cache_len; p.max_len = a->max_len; p.n_seqs = a->n_seqs; p.n_heads = a->n_heads; p.head_dim = a->head_dim;
    p.n_tokens = a->n_tokens;
    hipError_t e = tsattn::launch_cache_fill(p, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "cache fill launch");
    return TSATTN_OK;
}

// Checks a producer call's arguments and translates them; `who` names the entry point in messages.  Returns TSATTN_OK
// with *empty set when there are no rows.
static int fill_produce(const tsattn_produce_args *a, const char *who, tsattn::ProduceParams *out, bool *empty)
{
    *empty = false;
    if (!dtype_ok(a->dst_dtype) || (a->src_dtype != TSATTN_SRC_F32 && a->src_dtype != TSATTN_SRC_I32))
        return fail(TSATTN_ERR_UNSUPPORTED, "%s: dtypes %d -> %d", who, a->src_dtype, a->dst_dtype);
    // groups wider than a head (the feed-forward groups of 128 * ReluMult): int8 results, no rotation
    const bool wide_group = a->head_dim == 256 || a->head_dim == 384 || a->head_dim == 512;
    if (!head_dim_ok(a->head_dim) && !wide_group)
        return fail(TSATTN_ERR_UNSUPPORTED, "%s: head_dim %d (64, 128; 256, 384, 512 without rotation)", who, a->head_dim);
    if (wide_group && (a->pos || a->dst_dtype != TSATTN_I8))
        return fail(TSATTN_ERR_UNSUPPORTED, "%s: groups of %d values are normalised to int8 and not rotated", who, a->head_dim);
    if (a->n_rows < 0 || a->n_heads <= 0) return fail(TSATTN_ERR_BAD_ARG, "%s: negative size", who);
    if (a->n_rows == 0) { *empty = true; return TSATTN_OK; }
    if (!a->src || !a->dst) return fail(TSATTN_ERR_BAD_ARG, "%s: null data pointer", who);
    if (a->pos && (!a->rope || a->rope_len <= 0)) return fail(TSATTN_ERR_BAD_ARG, "%s: positions given without a rope table", who);
    const int64_t row = (int64_t)a->n_heads * a->head_dim;
    if (a->src_pitch < row || a->dst_pitch < row || a->dst_pitch % 16 || a->src_pitch % 4 || !aligned16(a->dst) || !aligned16(a->src) ||
        (a->rope && !aligned16(a->rope)))
        return fail(TSATTN_ERR_BAD_ARG, "%s: pitches must cover a row; src, dst and rope 16-byte aligned, pitches multiples of 16 bytes", who);
    const int64_t row_stride = a->scale_row_stride ? a->scale_row_stride : 1;
    if (a->scale_head_count < 0 || a->scale_head_begin < 0 || a->scale_head_begin + a->scale_head_count > a->n_heads)
        return fail(TSATTN_ERR_BAD_ARG, "%s: scale head range outside the heads", who);
    const int scale_heads = a->scale_head_count > 0 ? a->scale_head_count : a->n_heads;
    if (a->scale && (row_stride < 0 || a->scale_pitch <= 0 ||
                     !((row_stride == 1 && a->scale_pitch >= a->n_rows) || (a->scale_pitch == 1 && row_stride >= scale_heads))))
        return fail(TSATTN_ERR_BAD_ARG, "%s: scale layout must be [heads][scale_pitch >= n_rows] or [n_rows][scale_row_stride >= heads]", who);
    if (a->src_planes < 0 || a->src_planes > 16 || (a->src_planes > 1 && (a->src_dtype != TSATTN_SRC_I32 || a->src_plane_stride < a->n_rows * a->src_pitch ||
                                                                           a->src_plane_stride % 4)))
        return fail(TSATTN_ERR_BAD_ARG, "%s: up to 16 int32 source planes, at least n_rows * src_pitch elements apart, 16-byte aligned", who);
    if (a->rope_heads < 0 || a->rope_heads > a->n_heads) return fail(TSATTN_ERR_BAD_ARG, "%s: rope_heads outside the heads", who);
    if (a->resid && (a->resid_pitch < row || a->resid_pitch % 4 || !aligned16(a->resid)))
        return fail(TSATTN_ERR_BAD_ARG, "%s: resid must be 16-byte aligned with a pitch that covers a row", who);
    if (a->relu && a->dst_dtype != TSATTN_I8) return fail(TSATTN_ERR_UNSUPPORTED, "%s: relu with an int8 result only", who);
    tsattn::ProduceParams &p = *out;
    p.src = a->src; p.src_pitch = a->src_pitch; p.n_rows = a->n_rows; p.n_heads = a->n_heads;
    p.pos = a->pos; p.rope = a->rope; p.rope_len = a->rope_len;
    p.rotate_dir = a->rotate_dir; p.vec_scale = a->vec_scale; p.scale_mult = a->scale_mult;
    p.dst = (uint8_t *)a->dst; p.dst_pitch = a->dst_pitch; p.scale = a->scale; p.scale_pitch = a->scale_pitch;
    p.scale_row_stride = row_stride; p.relu = a->relu;
    p.src_planes = a->src_planes > 1 ? a->src_planes : 1; p.src_plane_stride = a->src_plane_stride;
    p.rope_heads = a->rope_heads > 0 ? a->rope_heads : a->n_heads;
    p.scale_head_begin = a->scale_head_count > 0 ? a->scale_head_begin : 0; p.scale_head_count = scale_heads;
    p.resid = a->resid; p.resid_pitch = a->resid_pitch; p.resid_scale = a->resid_scale;
    return TSATTN_OK;
}

int tsattn_rope_normalize_rows(tsattn_handle_t h, const tsattn_produce_args *a, void *stream)
{
    if (!h || !a) return fail(TSATTN_ERR_BAD_ARG, "tsattn_rope_normalize_rows: null argument");
    tsattn::ProduceParams p;
    bool empty;
    const int rc = fill_produce(a, "tsattn_rope_normalize_rows", &p, &empty);
    if (rc != TSATTN_OK || empty) return rc;
    hipError_t e = tsattn::launch_rope_normalize(p, a->dst_dtype, a->head_dim, a->src_dtype == TSATTN_SRC_I32, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "rope normalize launch");
    return TSATTN_OK;
}

int tsattn_kv_product(tsattn_handle_t h, int64_t n_rows, int n_heads, int head_dim, int rep, const void *k, int64_t k_pitch,
                      int value_dtype, const void *value, int64_t value_pitch, float mult, void *kv, int64_t kv_pitch,
                      void *stream)
{
    if (!h) return fail(TSATTN_ERR_BAD_ARG, "tsattn_kv_product: null handle");
    if (!head_dim_ok(head_dim)) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_kv_product: head_dim %d (64 or 128 supported)", head_dim);
    if (rep < 1 || rep > 4) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_kv_product: rep %d (1..4 supported)", rep);
    if (value_dtype != TSATTN_OUT_F32 && value_dtype != TSATTN_OUT_F16) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_kv_product: value dtype %d", value_dtype);
    if (n_rows < 0 || n_heads <= 0) return fail(TSATTN_ERR_BAD_ARG, "tsattn_kv_product: negative size");
    if (n_rows == 0) return TSATTN_OK;
    if (!k || !value || !kv) return fail(TSATTN_ERR_BAD_ARG, "tsattn_kv_product: null data pointer");
    const int64_t row = (int64_t)n_heads * head_dim;
    const int vsz = value_dtype == TSATTN_OUT_F16 ? 2 : 4;
    if (k_pitch < row || value_pitch < row || kv_pitch < row * rep || k_pitch % 16 || kv_pitch % 16 || (value_pitch * vsz) % 16 ||
        !aligned16(k) || !aligned16(value) || !aligned16(kv))
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_kv_product: pitches must cover a row and, like the pointers, be multiples of 16 bytes");
    tsattn::KvProductParams p;
    p.k = (const uint8_t *)k; p.k_pitch = k_pitch; p.val = value; p.val_pitch = value_pitch; p.n_rows = n_rows;
    p.n_heads = n_heads; p.head_dim = head_dim; p.rep = rep; p.mult = mult; p.kv = (uint8_t *)kv; p.kv_pitch = kv_pitch;
    hipError_t e = tsattn::launch_kv_product(p, value_dtype == TSATTN_OUT_F16, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "kv product launch");
    return TSATTN_OK;
}

int tsattn_matmul_i8(tsattn_handle_t h, const tsattn_matmul_args *a, void *stream)
{
    if (!h || !a) return fail(TSATTN_ERR_BAD_ARG, "tsattn_matmul_i8: null argument");
    if (a->mode != TSATTN_MM_I32 && a->mode != TSATTN_MM_F32 && a->mode != TSATTN_MM_ADD_SCALED && a->mode != TSATTN_MM_I32_PLANES)
        return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_matmul_i8: mode %d", a->mode);
    if (a->mode == TSATTN_MM_I32_PLANES && !a->planes_out) return fail(TSATTN_ERR_BAD_ARG, "tsattn_matmul_i8: planes_out is needed for the planes mode");
    if (a->mode == TSATTN_MM_I32_PLANES && a->out_pitch != a->n) return fail(TSATTN_ERR_BAD_ARG, "tsattn_matmul_i8: the planes are dense: out_pitch must equal n");
    if (a->m < 0 || a->n < 0) return fail(TSATTN_ERR_BAD_ARG, "tsattn_matmul_i8: negative size");
    if (a->k <= 0 || a->k % 64) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_matmul_i8: k %lld (a positive multiple of 64)", (long long)a->k);
    if (a->m == 0 || a->n == 0) return TSATTN_OK;
    if (!a->a || !a->w || !a->out) return fail(TSATTN_ERR_BAD_ARG, "tsattn_matmul_i8: null data pointer");
    if (a->a_pitch < a->k || a->w_pitch < a->k || a->out_pitch < a->n || a->a_pitch % 16 || a->w_pitch % 16 || !aligned16(a->a) ||
        !aligned16(a->w) || (uintptr_t)a->out % 4)
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_matmul_i8: pitches must cover a row; a, w and their pitches multiples of 16 bytes");
    // (the kernels address up to 256 rows of a tile with signed 32-bit offsets)
    if (a->a_pitch > (1 << 23) || a->w_pitch > (1 << 23)) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_matmul_i8: row pitch above 8 MiB");
    tsattn::GemmParams p = {};
    if (a->epilogue) {
        // the producer on the int32 result: its source is the product
        if (a->mode != TSATTN_MM_I32_PLANES) return fail(TSATTN_ERR_BAD_ARG, "tsattn_matmul_i8: an epilogue goes with the planes mode");
        tsattn_produce_args e = *a->epilogue;
        if (e.head_dim <= 0 || a->n % e.head_dim) return fail(TSATTN_ERR_BAD_ARG, "tsattn_matmul_i8: n %lld is not a whole number of the epilogue's heads", (long long)a->n);
        e.src_dtype = TSATTN_SRC_I32; e.src = a->out; e.src_pitch = a->n; e.n_rows = a->m; e.n_heads = (int)(a->n / e.head_dim);
        e.src_planes = 1; e.src_plane_stride = 0;
        bool empty;
        const int rc = fill_produce(&e, "tsattn_matmul_i8 (epilogue)", &p.ep, &empty);
        if (rc != TSATTN_OK) return rc;
        p.ep_head_dim = e.head_dim; p.ep_dst_dtype = e.dst_dtype;
    }
    p.a = (const uint8_t *)a->a; p.w = (const uint8_t *)a->w; p.a_pitch = a->a_pitch; p.w_pitch = a->w_pitch;
    p.m = a->m; p.n = a->n; p.k = a->k; p.mode = a->mode; p.scale = a->scale; p.out = a->out; p.out_pitch = a->out_pitch;
    const bool ws_ok = a->workspace && a->workspace_bytes > 0 && aligned16(a->workspace);
    p.workspace = ws_ok ? a->workspace : nullptr; p.workspace_bytes = ws_ok ? a->workspace_bytes : 0; p.split_stride = 0;
    hipError_t e = tsattn::launch_matmul_i8(p, (hipStream_t)stream, a->planes_out);
    if (e != hipSuccess) return hip_fail(e, "matmul launch");
    return TSATTN_OK;
}

int tsattn_embed_rows(tsattn_handle_t h, int64_t n_rows, int dim, const int32_t *labels, int labels_per_row, const void *embed,
                      int64_t embed_pitch, int64_t n_labels, float embed_scale, float *state, int64_t state_pitch, void *stream)
{
    if (!h) return fail(TSATTN_ERR_BAD_ARG, "tsattn_embed_rows: null handle");
    if (n_rows < 0 || dim <= 0 || dim % 16 || labels_per_row <= 0 || n_labels <= 0) return fail(TSATTN_ERR_BAD_ARG, "tsattn_embed_rows: sizes (dim a multiple of 16)");
    if (n_rows == 0) return TSATTN_OK;
    if (!labels || !embed || !state) return fail(TSATTN_ERR_BAD_ARG, "tsattn_embed_rows: null data pointer");
    if (embed_pitch < dim || embed_pitch % 16 || state_pitch < dim || state_pitch % 4 || !aligned16(embed) || !aligned16(state))
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_embed_rows: pitches must cover a row; embed, state and their pitches multiples of 16 bytes");
    tsattn::HeadParams p = {};
    p.n_rows = n_rows; p.dim = dim; p.labels = labels; p.labels_per_row = labels_per_row; p.embed = (const uint8_t *)embed;
    p.embed_pitch = embed_pitch; p.n_labels = n_labels; p.embed_scale = embed_scale; p.state = state; p.state_pitch = state_pitch;
    hipError_t e = tsattn::launch_embed_rows(p, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "embed launch");
    return TSATTN_OK;
}

int tsattn_softmax_rows(tsattn_handle_t h, int64_t n_rows, int64_t n, const int32_t *src, int src_planes, int64_t src_plane_stride,
                        int64_t src_pitch, float scale, const float *bias, float *prob, int64_t prob_pitch, int32_t *argmax,
                        void *stream)
{
    if (!h) return fail(TSATTN_ERR_BAD_ARG, "tsattn_softmax_rows: null handle");
    if (n_rows < 0 || n < 0 || n > 0x7fffffff) return fail(TSATTN_ERR_BAD_ARG, "tsattn_softmax_rows: sizes");
    if (n_rows == 0 || n == 0) return TSATTN_OK;
    if (!src || (!prob && !argmax)) return fail(TSATTN_ERR_BAD_ARG, "tsattn_softmax_rows: null data pointer");
    if (src_pitch < n || (prob && prob_pitch < n)) return fail(TSATTN_ERR_BAD_ARG, "tsattn_softmax_rows: pitches must cover a row");
    if (src_planes < 0 || src_planes > 16 || (src_planes > 1 && src_plane_stride < n_rows * src_pitch))
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_softmax_rows: up to 16 source planes, at least n_rows * src_pitch elements apart");
    tsattn::HeadParams p = {};
    p.n_rows = n_rows; p.n = n; p.src = src; p.src_planes = src_planes > 1 ? src_planes : 1; p.src_plane_stride = src_plane_stride;
    p.src_pitch = src_pitch; p.scale = scale; p.bias = bias; p.prob = prob; p.prob_pitch = prob_pitch; p.argmax = argmax;
    hipError_t e = tsattn::launch_softmax_rows(p, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "softmax launch");
    return TSATTN_OK;
}

int tsattn_sample_rows(tsattn_handle_t h, int64_t n_rows, int64_t n, const float *prob, int64_t prob_pitch, float temperature,
                       const uint32_t *rnd, int64_t rnd_pitch, uint64_t seed, uint64_t offset, int32_t *choice, void *stream)
{
    if (!h) return fail(TSATTN_ERR_BAD_ARG, "tsattn_sample_rows: null handle");
    if (n_rows < 0 || n <= 0 || n > 0x7fffffff) return fail(TSATTN_ERR_BAD_ARG, "tsattn_sample_rows: sizes");
    if (n_rows == 0) return TSATTN_OK;
    if (!prob || !choice) return fail(TSATTN_ERR_BAD_ARG, "tsattn_sample_rows: null data pointer");
    if (prob_pitch < n || (rnd && rnd_pitch < n)) return fail(TSATTN_ERR_BAD_ARG, "tsattn_sample_rows: pitches must cover a row");
    if (!(temperature > 0.0f)) return fail(TSATTN_ERR_BAD_ARG, "tsattn_sample_rows: temperature %g must be positive", (double)temperature);
    tsattn::HeadParams p = {};
    p.n_rows = n_rows; p.n = n; p.prob = const_cast<float *>(prob); p.prob_pitch = prob_pitch; p.temperature = temperature;
    p.rnd = rnd; p.rnd_pitch = rnd_pitch; p.seed = seed; p.offset = offset; p.argmax = choice;
    hipError_t e = tsattn::launch_sample_rows(p, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "sampling launch");
    return TSATTN_OK;
}

void tsattn_fill_rope_table(int head_dim, int64_t max_len, float *table)
{
    if (!table || head_dim <= 0 || head_dim % 64 || max_len <= 0) return;
    tsattn::fill_rope_table(head_dim, max_len, table);
}

int tsattn_quantize_rows(tsattn_handle_t h, int src_dtype, int dst_dtype, const void *src, int64_t src_pitch, int64_t n_rows,
                         int n_heads, int head_dim, void *dst, int64_t dst_pitch, float *scale, int64_t scale_pitch, void *stream)
{
    if (!h) return fail(TSATTN_ERR_BAD_ARG, "tsattn_quantize_rows: null handle");
    if (!dtype_ok(dst_dtype) || (src_dtype != TSATTN_SRC_F32 && src_dtype != TSATTN_SRC_BF16))
        return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_quantize_rows: dtypes %d -> %d", src_dtype, dst_dtype);
    if (head_dim <= 0 || head_dim % 64 || head_dim > 256) return fail(TSATTN_ERR_UNSUPPORTED, "tsattn_quantize_rows: head_dim %d (multiple of 64 up to 256)", head_dim);
    if (n_rows < 0 || n_heads <= 0) return fail(TSATTN_ERR_BAD_ARG, "tsattn_quantize_rows: negative size");
    if (n_rows == 0) return TSATTN_OK;
    if (!src || !dst || !scale) return fail(TSATTN_ERR_BAD_ARG, "tsattn_quantize_rows: null data pointer");
    const int64_t row = (int64_t)n_heads * head_dim;
    if (src_pitch < row * (src_dtype == TSATTN_SRC_F32 ? 4 : 2) || dst_pitch < row || scale_pitch < n_rows)
        return fail(TSATTN_ERR_BAD_ARG, "tsattn_quantize_rows: pitch too small");
    hipError_t e = tsattn::launch_quantize_rows(src_dtype, dst_dtype, src, src_pitch, n_rows, n_heads, head_dim, dst, dst_pitch, scale,
                                                scale_pitch, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "quantize launch");
    return TSATTN_OK;
}

int tsattn_build_spans(tsattn_handle_t h, int n_seqs, const int32_t *seq_offset, int64_t n_tokens, const uint8_t *doc_start_flag,
                       int64_t window, int32_t *span_start, int32_t *span_finish, void *stream)
{
    if (!h) return fail(TSATTN_ERR_BAD_ARG, "tsattn_build_spans: null handle");
    if (n_seqs < 0 || n_tokens < 0 || window < 0) return fail(TSATTN_ERR_BAD_ARG, "tsattn_build_spans: negative size");
    if (n_tokens == 0) return TSATTN_OK;
    if (n_seqs == 0 || !seq_offset || !span_start || !span_finish) return fail(TSATTN_ERR_BAD_ARG, "tsattn_build_spans: null data pointer");
    hipError_t e = tsattn::launch_build_spans(n_seqs, seq_offset, n_tokens, doc_start_flag, window, span_start, span_finish, (hipStream_t)stream);
    if (e != hipSuccess) return hip_fail(e, "build spans launch");
    return TSATTN_OK;
}

} // extern "C"
