#include "att_compute.h"

#include <hip/hip_runtime.h>
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

} // namespace NTsAttn
