#include "att_compute.h"

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdio.h>
#include <stdlib.h>

namespace NTsAttn {

// the reference aborts on a failed precondition (Y_VERIFY, util/eden_core.h:111)
#define TS_VERIFY(cond, ...)                                                                  \
    do {                                                                                      \
        if (!(cond)) {                                                                        \
            fprintf(stderr, "tsattn host: %s:%d: ", __FILE__, __LINE__);                      \
            fprintf(stderr, __VA_ARGS__);                                                     \
            fprintf(stderr, "\n");                                                            \
            abort();                                                                          \
        }                                                                                     \
    } while (0)

static void Check(int status, const char *what)
{
    TS_VERIFY(status == TSATTN_OK, "%s failed: %s", what, tsattn_last_error());
}

static void CheckHip(hipError_t e, const char *what)
{
    TS_VERIFY(e == hipSuccess, "%s failed: %s", what, hipGetErrorString(e));
}

void AddWindowSpans(int ptr, int len, int limitWindow, const uint8_t *docStartFlag, TAttentionInfo *pAtt)
{
    if (pAtt->SpanPtr.empty()) {
        pAtt->Init();
    }
    int docStart = 0;
    for (int t = 0; t < len; ++t) {
        if (docStartFlag && t > 0 && docStartFlag[t]) {
            docStart = t;
        }
        if (limitWindow == 0) {
            pAtt->AddSpan(TAttentionSpan(ptr + t, ptr + t));
        } else {
            int attStart = (docStart > t - limitWindow) ? docStart : t - limitWindow;
            int attFinish = t - 1;
            if (attFinish >= attStart) {
                pAtt->AddSpan(TAttentionSpan(ptr + attStart, ptr + attFinish));
            }
        }
        pAtt->AddSample();
    }
}

TAttentionComputer::TAttentionComputer(const TModelDims &dims, float alibiSlope, int deviceId, int maxLen, int maxSeqs)
    : Dims(dims), AlibiSlope(alibiSlope), MaxLen(maxLen)
{
    TS_VERIFY(dims.QDim == dims.TTDim, "QDim %d != TTDim %d", dims.QDim, dims.TTDim);
    tsattn_config cfg = {};
    cfg.device = deviceId;
    cfg.max_seqs = maxSeqs;
    cfg.max_heads = dims.HeadCount;
    cfg.max_head_dim = dims.QDim;
    Check(tsattn_create(&cfg, &Handle), "tsattn_create");
    CheckHip(hipMalloc((void **)&SpanStart, sizeof(int32_t) * (size_t)maxLen), "hipMalloc(spans)");
    CheckHip(hipMalloc((void **)&SpanFinish, sizeof(int32_t) * (size_t)maxLen), "hipMalloc(spans)");
    CheckHip(hipMalloc((void **)&SpanTiles, sizeof(int32_t) * TSATTN_SPAN_TILE_INTS * (size_t)tsattn_span_tiles_count(maxLen)), "hipMalloc(span tiles)");
    CheckHip(hipMalloc((void **)&SumWeightLog, sizeof(float) * (size_t)maxLen * dims.HeadCount), "hipMalloc(sumWeightLog)");
}

TAttentionComputer::~TAttentionComputer()
{
    (void)hipFree(SpanStart);
    (void)hipFree(SpanFinish);
    (void)hipFree(SpanTiles);
    (void)hipFree(SumWeightLog);
    tsattn_destroy(Handle);
}

void TAttentionComputer::SetAttention(const TAttentionInfo &attInfo, void *stream)
{
    int len = (int)attInfo.GetSampleCount();
    TS_VERIFY(len <= MaxLen, "%d samples exceed the context's %d", len, MaxLen);
    std::vector<int32_t> st(len), fi(len);
    for (int t = 0; t < len; ++t) {
        int a = attInfo.SpanPtr[t], b = attInfo.SpanPtr[t + 1];
        TS_VERIFY(b - a <= 1, "row %d has %d spans; one span per row is supported", t, b - a);
        if (b > a) {
            st[t] = attInfo.Spans[a].Start;
            fi[t] = attInfo.Spans[a].Finish;
        } else {
            st[t] = t;
            fi[t] = t - 1;
        }
    }
    Len = len;
    // Launch-order hint: rows without keys mark sequence starts; if they are equally spaced, cover the batch and
    // the window is wide (the last row of a sequence sees at least half of it), the batch has a causal period.
    CausalPeriod = 0;
    {
        int period = 0, last = -1;
        bool regular = len > 0 && fi[0] < st[0];
        for (int t = 0; t < len && regular; ++t) {
            if (fi[t] < st[t]) {
                if (last >= 0) {
                    if (period == 0) period = t - last;
                    else if (t - last != period) regular = false;
                }
                last = t;
            }
        }
        if (regular && period == 0) period = len; // a single sequence
        if (regular && period > 0 && len % period == 0 && last == len - period) {
            const int tail = len - 1;
            if (fi[tail] - st[tail] + 1 >= period / 2) CausalPeriod = period;
        }
    }
    // pageable source: the copy has returned from the host's point of view when the call returns
    CheckHip(hipMemcpyAsync(SpanStart, st.data(), sizeof(int32_t) * len, hipMemcpyHostToDevice, (hipStream_t)stream), "span copy");
    CheckHip(hipMemcpyAsync(SpanFinish, fi.data(), sizeof(int32_t) * len, hipMemcpyHostToDevice, (hipStream_t)stream), "span copy");
    Check(tsattn_build_span_tiles(Handle, len, SpanStart, SpanFinish, SpanTiles, stream), "tsattn_build_span_tiles");
    CheckHip(hipStreamSynchronize((hipStream_t)stream), "span copy");
}

void TAttentionComputer::ComputeValLookup(int len, int dtype, const TQuantRows &qk, const TQuantRows &qv, const TQuantRows &v,
                                          const float *qvGlobalScale, void *valLookup, int64_t valLookupPitchBytes,
                                          bool outF16, void *stream)
{
    TS_VERIFY(len == Len, "len %d differs from the %d samples set by SetAttention", len, Len);
    tsattn_prefill_args a = {};
    a.dtype = dtype;
    a.out_dtype = outF16 ? TSATTN_OUT_F16 : TSATTN_OUT_F32;
    a.n_tokens = len;
    a.n_heads = Dims.HeadCount;
    a.head_dim = Dims.QDim;
    a.q = qk.Data; a.k = qv.Data; a.v = v.Data;
    a.q_pitch = qk.PitchBytes; a.k_pitch = qv.PitchBytes; a.v_pitch = v.PitchBytes;
    a.q_scale = qk.Scale; a.k_scale = qv.Scale; a.v_scale = v.Scale;
    a.scale_pitch = MaxLen;
    a.q_scale_const = qk.ConstScale; a.k_scale_const = qv.ConstScale; a.v_scale_const = v.ConstScale;
    a.k_global_scale = qvGlobalScale;
    a.span_start = SpanStart; a.span_finish = SpanFinish;
    a.span_tiles = SpanTiles;
    a.alibi_slope = AlibiSlope;
    a.out = valLookup; a.out_pitch = valLookupPitchBytes;
    a.sum_weight_log = SumWeightLog;
    a.causal_period = CausalPeriod;
    Check(tsattn_prefill(Handle, &a, stream), "tsattn_prefill");
}

TAttentionVecHistory::TAttentionVecHistory(tsattn_handle_t handle, int dtype, int seqCount, int headCount, int maxLen, int headDim)
    : Handle(handle), DType(dtype), SeqCount(seqCount), HeadCount(headCount), MaxLen(maxLen), HeadDim(headDim)
{
    size_t rows = (size_t)seqCount * headCount * maxLen;
    CheckHip(hipMalloc((void **)&QVState, rows * headDim), "hipMalloc(cache)");
    CheckHip(hipMalloc((void **)&VState, rows * headDim), "hipMalloc(cache)");
    CheckHip(hipMalloc((void **)&QVStateScale, rows * sizeof(float)), "hipMalloc(cache)");
    CheckHip(hipMalloc((void **)&VStateScale, rows * sizeof(float)), "hipMalloc(cache)");
    CheckHip(hipMalloc((void **)&Length, sizeof(int32_t) * (size_t)seqCount), "hipMalloc(cache)");
    CheckHip(hipMemset(Length, 0, sizeof(int32_t) * (size_t)seqCount), "hipMemset(cache length)");
}

TAttentionVecHistory::~TAttentionVecHistory()
{
    (void)hipFree(QVState);
    (void)hipFree(VState);
    (void)hipFree(QVStateScale);
    (void)hipFree(VStateScale);
    (void)hipFree(Length);
}

void TAttentionVecHistory::AddVectors(const void *qv, const float *qvScale, const void *v, const float *vScale, void *stream)
{
    tsattn_append_args a = {};
    a.n_seqs = SeqCount; a.n_heads = HeadCount; a.head_dim = HeadDim;
    a.k_new = qv; a.v_new = v;
    a.new_pitch = (int64_t)HeadCount * HeadDim;
    a.k_scale_new = qvScale; a.v_scale_new = vScale;
    a.k_cache = QVState; a.v_cache = VState;
    a.seq_stride = (int64_t)HeadCount * MaxLen * HeadDim;
    a.head_stride = (int64_t)MaxLen * HeadDim;
    a.tok_stride = HeadDim;
    a.k_scale = QVStateScale; a.v_scale = VStateScale;
    a.s_seq_stride = (int64_t)HeadCount * MaxLen;
    a.s_head_stride = MaxLen;
    a.cache_len = Length;
    a.max_len = MaxLen;
    Check(tsattn_cache_append(Handle, &a, stream), "tsattn_cache_append");
}

void ComputeValLookup(int width, float alibiSlope, const TAttentionVecHistory &h, const void *qk, const float *qkScale,
                      float qkConstScale, float *valLookup, void *stream)
{
    tsattn_decode_args a = {};
    a.dtype = h.DType;
    a.q_dtype = TSATTN_Q_8BIT;
    a.n_seqs = h.SeqCount; a.n_heads = h.HeadCount; a.head_dim = h.HeadDim;
    a.q = qk;
    a.q_pitch = (int64_t)h.HeadCount * h.HeadDim;
    a.q_scale = qkScale; a.q_scale_const = qkConstScale;
    a.k_cache = h.QVState; a.v_cache = h.VState;
    a.seq_stride = (int64_t)h.HeadCount * h.MaxLen * h.HeadDim;
    a.head_stride = (int64_t)h.MaxLen * h.HeadDim;
    a.tok_stride = h.HeadDim;
    a.k_scale = h.QVStateScale; a.v_scale = h.VStateScale;
    a.s_seq_stride = (int64_t)h.HeadCount * h.MaxLen;
    a.s_head_stride = h.MaxLen;
    a.cache_len = h.Length;
    a.max_len = h.MaxLen;
    a.window = width;
    a.alibi_slope = alibiSlope;
    a.out = valLookup;
    Check(tsattn_decode(h.Handle, &a, stream), "tsattn_decode");
}

// ---- one layer of the int8 inference path ----------------------------------------------------------------------

TLayerComputer::TLayerComputer(tsattn_handle_t handle, const TModelDims &dims, int seqCount)
    : Handle(handle), Dims(dims), SeqCount(seqCount)
{
    TS_VERIFY(dims.QDim == dims.TTDim && (dims.QDim == 64 || dims.QDim == 128), "QDim %d TTDim %d: equal, 64 or 128", dims.QDim, dims.TTDim);
    TS_VERIFY(dims.Dim % STATE_NORM_TILE == 0, "Dim %d is not a multiple of %d", dims.Dim, STATE_NORM_TILE);
    ReluDim = dims.HeadCount * dims.QDim;
    const size_t n = (size_t)seqCount, qsum = (size_t)dims.GetQSum();
    auto alloc = [](void **p, size_t bytes) { CheckHip(hipMalloc(p, bytes), "hipMalloc(layer buffers)"); };
    alloc((void **)&NormState, n * dims.Dim);
    alloc((void **)&Qk, n * qsum); alloc((void **)&Qv, n * qsum); alloc((void **)&K, n * qsum); alloc((void **)&V, n * qsum);
    alloc((void **)&Kv, n * qsum * COMBINER_REP);
    alloc((void **)&Relu, n * ReluDim);
    alloc((void **)&QkSrc, n * qsum * 4); alloc((void **)&QvSrc, n * qsum * 4);
    alloc((void **)&KSrc, n * qsum * 4); alloc((void **)&VSrc, n * qsum * 4);
    alloc((void **)&ReluSrc, n * ReluDim * 4);
    alloc((void **)&QvHeadScale, n * dims.HeadCount * 4); alloc((void **)&VHeadScale, n * dims.HeadCount * 4);
    alloc((void **)&ValLookup, n * qsum * 4);
    // room for the matrix products to split K (few rows): 16 planes of the widest result
    size_t widest = qsum > (size_t)dims.Dim ? qsum : (size_t)dims.Dim;
    if ((size_t)ReluDim > widest) widest = ReluDim;
    WorkspaceBytes = (int64_t)(16 * 4 * n * widest);
    alloc(&Workspace, (size_t)WorkspaceBytes);
    // values carry the constant VEC_SCALE (cpu_infer.cpp:454)
    std::vector<float> vs(n * dims.HeadCount, VEC_SCALE);
    CheckHip(hipMemcpy(VHeadScale, vs.data(), vs.size() * sizeof(float), hipMemcpyHostToDevice), "hipMemcpy(value scales)");
}

TLayerComputer::~TLayerComputer()
{
    void *all[] = {NormState, Qk, Qv, K, V, Kv, Relu, QkSrc, QvSrc, KSrc, VSrc, ReluSrc, QvHeadScale, VHeadScale, ValLookup, Workspace};
    for (void *p : all) (void)hipFree(p);
}

void TLayerComputer::AddLookupProduct(const int32_t *t, const float *ropeBuf, int64_t ropeLen, const TAttentionMatrices &att,
                                      TAttentionVecHistory *pKVCache, float *state, void *stream)
{
    TAttentionVecHistory &kvCache = *pKVCache;
    const int dim = Dims.Dim, headCount = Dims.HeadCount, headDim = Dims.QDim, qsum = Dims.GetQSum();
    TS_VERIFY(kvCache.SeqCount == SeqCount && kvCache.HeadCount == headCount && kvCache.HeadDim == headDim && kvCache.DType == TSATTN_I8,
              "the KV cache does not match the layer (%d sequences, %d heads of %d, int8)", SeqCount, headCount, headDim);

    // NormalizeState: per group of `groupDim` values, to int8; optionally rope first, the groups' scales, ReLU
    auto normalize = [&](const void *src, bool srcI32, int groups, int groupDim, const int32_t *pos, uint8_t *dst, float *headScale,
                         float scaleMult, bool relu) {
        tsattn_produce_args a = {};
        a.src_dtype = srcI32 ? TSATTN_SRC_I32 : TSATTN_SRC_F32;
        a.dst_dtype = TSATTN_I8;
        a.n_rows = SeqCount; a.n_heads = groups; a.head_dim = groupDim;
        a.src = src; a.src_pitch = (int64_t)groups * groupDim;
        a.pos = pos; a.rope = pos ? ropeBuf : nullptr; a.rope_len = pos ? ropeLen : 0;
        a.rotate_dir = 1; a.vec_scale = VEC_SCALE; a.scale_mult = scaleMult;
        a.dst = dst; a.dst_pitch = (int64_t)groups * groupDim;
        a.scale = headScale; a.scale_pitch = 1; a.scale_row_stride = groups; // [seq][head], what the cache append reads
        a.relu = relu ? 1 : 0;
        Check(tsattn_rope_normalize_rows(Handle, &a, stream), "tsattn_rope_normalize_rows");
    };
    // MulForward / AddScaled
    auto mulForward = [&](const uint8_t *vec, int k, const int8_t *matr, int n, int mode, float scale, void *res) {
        tsattn_matmul_args a = {};
        a.m = SeqCount; a.n = n; a.k = k;
        a.a = vec; a.a_pitch = k; a.w = matr; a.w_pitch = k;
        a.mode = mode; a.scale = scale; a.out = res; a.out_pitch = n;
        a.workspace = Workspace; a.workspace_bytes = WorkspaceBytes;
        Check(tsattn_matmul_i8(Handle, &a, stream), "tsattn_matmul_i8");
    };

    normalize(state, false, dim / STATE_NORM_TILE, STATE_NORM_TILE, nullptr, NormState, nullptr, 1, false);
    mulForward(NormState, dim, att.QK, qsum, TSATTN_MM_F32, 1, QkSrc);
    mulForward(NormState, dim, att.QV, qsum, TSATTN_MM_F32, 1, QvSrc);
    mulForward(NormState, dim, att.K, qsum, TSATTN_MM_I32, 1, KSrc);
    mulForward(NormState, dim, att.V, qsum, TSATTN_MM_I32, 1, VSrc);
    normalize(QkSrc, false, headCount, headDim, t, Qk, nullptr, 1, false);
    // the cached key scale takes the matrix scale: qvMult *= att.QVScale * VEC_SCALE * CalcDotScale(dim)
    normalize(QvSrc, false, headCount, headDim, t, Qv, QvHeadScale, att.QVScale * VEC_SCALE * sqrtf(1.0f / (float)dim), false);
    normalize(KSrc, true, headCount, headDim, nullptr, K, nullptr, 1, false);
    normalize(VSrc, true, headCount, headDim, nullptr, V, nullptr, 1, false);

    // kvCache.AddVectors(qv, qvHeadScale, v) and ComputeValLookup(width, slope, dims, kvCache, qk, &valLookup) in one call
    // (width 0 would make the token attend to the row being written: two calls then)
    if (att.AttentionWidth == 0) {
        kvCache.AddVectors(Qv, QvHeadScale, V, VHeadScale, stream);
        ComputeValLookup(att.AttentionWidth, att.AlibiSlope, kvCache, Qk, nullptr, VEC_SCALE, ValLookup, stream);
    } else {
        tsattn_decode_args a = {};
        a.dtype = TSATTN_I8; a.q_dtype = TSATTN_Q_8BIT;
        a.n_seqs = SeqCount; a.n_heads = headCount; a.head_dim = headDim;
        a.q = Qk; a.q_pitch = qsum; a.q_scale = nullptr; a.q_scale_const = VEC_SCALE;
        a.k_cache = kvCache.QVState; a.v_cache = kvCache.VState;
        a.seq_stride = (int64_t)headCount * kvCache.MaxLen * headDim;
        a.head_stride = (int64_t)kvCache.MaxLen * headDim;
        a.tok_stride = headDim;
        a.k_scale = kvCache.QVStateScale; a.v_scale = kvCache.VStateScale;
        a.s_seq_stride = (int64_t)headCount * kvCache.MaxLen; a.s_head_stride = kvCache.MaxLen;
        a.cache_len = kvCache.Length; a.max_len = kvCache.MaxLen;
        a.window = att.AttentionWidth; a.alibi_slope = att.AlibiSlope;
        a.out = ValLookup;
        a.k_new = Qv; a.v_new = V; a.new_pitch = qsum; a.k_scale_new = QvHeadScale; a.v_scale_new = VHeadScale;
        Check(tsattn_decode(Handle, &a, stream), "tsattn_decode");
    }

    Check(tsattn_kv_product(Handle, SeqCount, headCount, headDim, COMBINER_REP, K, qsum, TSATTN_OUT_F32, ValLookup, qsum, 1.0f, Kv,
                            (int64_t)qsum * COMBINER_REP, stream), "tsattn_kv_product");
    const int kvDim = qsum * COMBINER_REP;
    mulForward(Kv, kvDim, att.Combiner, dim, TSATTN_MM_ADD_SCALED, att.CombinerScale * VEC_SCALE * sqrtf(1.0f / (float)kvDim), state);

    // relu
    normalize(state, false, dim / STATE_NORM_TILE, STATE_NORM_TILE, nullptr, NormState, nullptr, 1, false);
    mulForward(NormState, dim, att.Expand, ReluDim, TSATTN_MM_I32, 1, ReluSrc);
    normalize(ReluSrc, true, headCount, ReluDim / headCount, nullptr, Relu, nullptr, 1, true);
    mulForward(Relu, ReluDim, att.Contract, dim, TSATTN_MM_ADD_SCALED, att.ContractScale * VEC_SCALE * sqrtf(1.0f / (float)ReluDim), state);
}

} // namespace NTsAttn
