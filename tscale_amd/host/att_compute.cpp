#include "att_compute.h"

#include <hip/hip_runtime.h>

#include <algorithm>
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

static int FlattenSpans(const TAttentionInfo &attInfo, std::vector<int32_t> *pStart, std::vector<int32_t> *pFinish, int part = 0,
                        bool oneSpanPerRow = true);

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
    CheckHip(hipMalloc((void **)&SumWeightLog, sizeof(float) * (size_t)maxLen * dims.HeadCount), "hipMalloc(sumWeightLog)");
    // room for the long-span kernel's copy of V where a batch can have such spans at all
    WorkspaceBytes = maxLen >= TSATTN_PREFILL_LONG_SPAN ? tsattn_prefill_workspace_bytes(maxLen, dims.HeadCount, dims.QDim) : 0;
    if (WorkspaceBytes) CheckHip(hipMalloc(&Workspace, WorkspaceBytes), "hipMalloc(prefill workspace)");
    Reserve(1);
}

// room for the spans of `parts` parts; with more than one also for the parts' results
void TAttentionComputer::Reserve(int parts)
{
    if (parts <= PartCapacity) return;
    void *old[] = {SpanStart, SpanFinish, SpanTiles, PartOut, PartSwl};
    for (void *p : old) (void)hipFree(p);
    SpanStart = SpanFinish = SpanTiles = nullptr;
    PartOut = PartSwl = nullptr;
    const size_t n = (size_t)parts * MaxLen;
    CheckHip(hipMalloc((void **)&SpanStart, sizeof(int32_t) * n), "hipMalloc(spans)");
    CheckHip(hipMalloc((void **)&SpanFinish, sizeof(int32_t) * n), "hipMalloc(spans)");
    CheckHip(hipMalloc((void **)&SpanTiles, sizeof(int32_t) * TSATTN_SPAN_TILE_INTS * (size_t)tsattn_span_tiles_count(MaxLen) * parts), "hipMalloc(span tiles)");
    if (parts > 1) {
        CheckHip(hipMalloc((void **)&PartOut, sizeof(float) * n * Dims.HeadCount * Dims.TTDim), "hipMalloc(parts)");
        CheckHip(hipMalloc((void **)&PartSwl, sizeof(float) * n * Dims.HeadCount), "hipMalloc(parts)");
    }
    PartCapacity = parts;
}

TAttentionComputer::~TAttentionComputer()
{
    (void)hipFree(SpanStart);
    (void)hipFree(SpanFinish);
    (void)hipFree(SpanTiles);
    (void)hipFree(SumWeightLog);
    (void)hipFree(PartOut);
    (void)hipFree(PartSwl);
    (void)hipFree(Workspace);
    tsattn_destroy(Handle);
}

void TAttentionComputer::SetAttention(const TAttentionInfo &attInfo, void *stream)
{
    int len = (int)attInfo.GetSampleCount();
    TS_VERIFY(len <= MaxLen, "%d samples exceed the context's %d", len, MaxLen);
    int parts = 1;
    for (int t = 0; t < len; ++t) parts = std::max(parts, attInfo.SpanPtr[t + 1] - attInfo.SpanPtr[t]);
    TS_VERIFY(parts <= 64, "a row with %d spans; up to 64 are supported", parts);
    CheckHip(hipStreamSynchronize((hipStream_t)stream), "stream"); // nothing may still use what Reserve frees
    Reserve(parts);
    Parts = parts;
    Len = len;
    const int64_t tileInts = TSATTN_SPAN_TILE_INTS * tsattn_span_tiles_count(len); // the parts' summaries follow one another
    // every part's host arrays live until the copies have been waited for below
    std::vector<std::vector<int32_t>> st(parts), fi(parts);
    int64_t keys = 0;
    for (int i = 0; i < parts; ++i) {
        const int period = FlattenSpans(attInfo, &st[i], &fi[i], i, false); // (and the launch-order hint)
        CausalPeriod = parts == 1 ? period : 0;
        for (int t = 0; t < len; ++t) keys += std::max(0, fi[i][t] - st[i][t] + 1);
        CheckHip(hipMemcpyAsync(SpanStart + (size_t)i * MaxLen, st[i].data(), sizeof(int32_t) * len, hipMemcpyHostToDevice, (hipStream_t)stream), "span copy");
        CheckHip(hipMemcpyAsync(SpanFinish + (size_t)i * MaxLen, fi[i].data(), sizeof(int32_t) * len, hipMemcpyHostToDevice, (hipStream_t)stream), "span copy");
        Check(tsattn_build_span_tiles(Handle, len, SpanStart + (size_t)i * MaxLen, SpanFinish + (size_t)i * MaxLen, SpanTiles + i * tileInts, stream),
              "tsattn_build_span_tiles");
    }
    // keys per row of the longer rows (a causal window over sequences of S tokens averages S / 2): the library's hint
    SpanLenHint = len > 0 ? 2 * keys / ((int64_t)len * parts) : 0;
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
    a.alibi_slope = AlibiSlope;
    a.workspace = Workspace; a.workspace_bytes = (int64_t)WorkspaceBytes; a.span_len_hint = SpanLenHint;
    if (Parts == 1) {
        a.span_start = SpanStart; a.span_finish = SpanFinish;
        a.span_tiles = SpanTiles;
        a.out = valLookup; a.out_pitch = valLookupPitchBytes;
        a.sum_weight_log = SumWeightLog;
        a.causal_period = CausalPeriod;
        Check(tsattn_prefill(Handle, &a, stream), "tsattn_prefill");
        return;
    }
    if (!MergeParts) {
        // one launch walks every row's spans part by part: one softmax over all of them (gpt_cpu.cpp:405-436)
        a.span_start = SpanStart; a.span_finish = SpanFinish; a.span_tiles = SpanTiles;
        a.n_span_parts = Parts; a.span_part_stride = MaxLen;
        a.out = valLookup; a.out_pitch = valLookupPitchBytes;
        a.sum_weight_log = SumWeightLog;
        Check(tsattn_prefill(Handle, &a, stream), "tsattn_prefill");
        return;
    }
    // the same as one launch per part and their results combined by their weights
    const int64_t row = (int64_t)Dims.HeadCount * Dims.TTDim, tileInts = TSATTN_SPAN_TILE_INTS * tsattn_span_tiles_count(len);
    a.out_dtype = TSATTN_OUT_F32;
    a.out_pitch = row * 4;
    for (int i = 0; i < Parts; ++i) {
        a.span_start = SpanStart + (size_t)i * MaxLen; a.span_finish = SpanFinish + (size_t)i * MaxLen;
        a.span_tiles = SpanTiles + i * tileInts;
        a.out = PartOut + (size_t)i * MaxLen * row;
        a.sum_weight_log = PartSwl + (size_t)i * Dims.HeadCount * MaxLen;
        Check(tsattn_prefill(Handle, &a, stream), "tsattn_prefill");
    }
    tsattn_merge_args m = {};
    m.n_parts = Parts; m.n_tokens = len; m.n_heads = Dims.HeadCount; m.head_dim = Dims.TTDim;
    m.part_out = PartOut; m.part_out_pitch = row; m.part_out_stride = (int64_t)MaxLen * row;
    m.part_swl = PartSwl; m.scale_pitch = MaxLen; m.part_swl_stride = (int64_t)Dims.HeadCount * MaxLen;
    m.out_dtype = outF16 ? TSATTN_OUT_F16 : TSATTN_OUT_F32;
    m.out = valLookup; m.out_pitch = valLookupPitchBytes;
    m.sum_weight_log = SumWeightLog;
    Check(tsattn_merge_lookups(Handle, &m, stream), "tsattn_merge_lookups");
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

TLayerComputer::TLayerComputer(tsattn_handle_t handle, const TModelDims &dims, int maxRows, int64_t maxOutputs)
    : Handle(handle), Dims(dims), MaxRows(maxRows)
{
    TS_VERIFY(dims.QDim == dims.TTDim && (dims.QDim == 64 || dims.QDim == 128), "QDim %d TTDim %d: equal, 64 or 128", dims.QDim, dims.TTDim);
    TS_VERIFY(dims.Dim % STATE_NORM_TILE == 0, "Dim %d is not a multiple of %d", dims.Dim, STATE_NORM_TILE);
    // NormalizeState(relu, headCount) takes groups of 128 * ReluMult whatever the head width (gpt/train/cpu_infer.cpp:519-524,
    // model_dim.h:66); the producer kernels normalise groups of up to 512
    TS_VERIFY(dims.ReluMult >= 1 && dims.ReluMult <= 4, "ReluMult %d: feed-forward groups of 128 to 512 values are supported", dims.ReluMult);
    ReluDim = dims.GetReluDim();
    const size_t n = (size_t)maxRows, qsum = (size_t)dims.GetQSum();
    auto alloc = [](void **p, size_t bytes) { CheckHip(hipMalloc(p, bytes), "hipMalloc(layer buffers)"); };
    alloc((void **)&NormState, n * dims.Dim);
    alloc((void **)&Q4, n * qsum * 4);
    alloc((void **)&Kv, n * qsum * COMBINER_REP);
    alloc((void **)&Relu, n * ReluDim);
    alloc((void **)&QvHeadScale, n * dims.HeadCount * 4);
    alloc((void **)&VHeadScale, n * dims.HeadCount * 4);
    alloc((void **)&ValLookup, n * qsum * 4);
    // the int32 results of the matrix products: 16 planes of the widest one with few rows (K split over workgroups), one
    // plane otherwise
    size_t widest = 4 * qsum > (size_t)dims.Dim ? 4 * qsum : (size_t)dims.Dim;
    if ((size_t)ReluDim > widest) widest = ReluDim;
    if ((size_t)maxOutputs > widest) widest = (size_t)maxOutputs;
    const size_t fewRows = n < 128 ? n : 128;
    const size_t planeElems = (16 * fewRows > n ? 16 * fewRows : n) * widest;
    alloc((void **)&Planes, planeElems * 4);
    WorkspaceBytes = (int64_t)(16 * 4 * fewRows * dims.Dim);
    alloc(&Workspace, (size_t)WorkspaceBytes);
    // values carry the constant VEC_SCALE (cpu_infer.cpp:454)
    std::vector<float> vs(n * dims.HeadCount, VEC_SCALE);
    CheckHip(hipMemcpy(VHeadScale, vs.data(), vs.size() * sizeof(float), hipMemcpyHostToDevice), "hipMemcpy(value scales)");
}

TLayerComputer::~TLayerComputer()
{
    void *all[] = {NormState, Q4, Kv, Relu, QvHeadScale, VHeadScale, ValLookup, Planes, Workspace};
    for (void *p : all) (void)hipFree(p);
}

// MulForward, result left as int32 planes in Planes (their sum is the product); returns the number of planes
int TLayerComputer::MulForwardPlanes(int rows, const uint8_t *vec, int k, const int8_t *matr, int n, void *stream)
{
    tsattn_matmul_args a = {};
    int planes = 0;
    a.m = rows; a.n = n; a.k = k;
    a.a = vec; a.a_pitch = k; a.w = matr; a.w_pitch = k;
    a.mode = TSATTN_MM_I32_PLANES; a.out = Planes; a.out_pitch = n; a.planes_out = &planes;
    Check(tsattn_matmul_i8(Handle, &a, stream), "tsattn_matmul_i8");
    return planes;
}

// MulForward with NormalizeState (and whatever else `a` asks of the producer) as its epilogue: one library call; large
// products never write their int32 sums, small ones leave them in Planes for the producer's launch
void TLayerComputer::MulForwardNormalize(int rows, const uint8_t *vec, int k, const int8_t *matr, tsattn_produce_args a, int groups,
                                         int groupDim, uint8_t *dst, void *stream)
{
    a.dst_dtype = TSATTN_I8; a.head_dim = groupDim;
    a.rotate_dir = 1; a.vec_scale = VEC_SCALE;
    if (a.scale_mult == 0) a.scale_mult = 1;
    a.dst = dst; a.dst_pitch = (int64_t)groups * groupDim;
    tsattn_matmul_args m = {};
    int planes = 0;
    m.m = rows; m.n = groups * groupDim; m.k = k;
    m.a = vec; m.a_pitch = k; m.w = matr; m.w_pitch = k;
    m.mode = TSATTN_MM_I32_PLANES; m.out = Planes; m.out_pitch = m.n; m.planes_out = &planes;
    m.epilogue = &a;
    Check(tsattn_matmul_i8(Handle, &m, stream), "tsattn_matmul_i8");
}

// NormalizeState on int32 planes or on a float array: per group of groupDim values, to int8 (fields of `a` preset by the
// caller select rotation, scale output, ReLU, the residual update)
static void Normalize(tsattn_handle_t handle, tsattn_produce_args a, int rows, const void *src, bool srcI32, int planes, int groups,
                      int groupDim, uint8_t *dst, void *stream)
{
    a.src_dtype = srcI32 ? TSATTN_SRC_I32 : TSATTN_SRC_F32;
    a.dst_dtype = TSATTN_I8;
    a.n_rows = rows; a.n_heads = groups; a.head_dim = groupDim;
    a.src = src; a.src_pitch = (int64_t)groups * groupDim;
    a.src_planes = planes; a.src_plane_stride = (int64_t)rows * groups * groupDim;
    a.rotate_dir = 1; a.vec_scale = VEC_SCALE;
    if (a.scale_mult == 0) a.scale_mult = 1;
    a.dst = dst; a.dst_pitch = (int64_t)groups * groupDim;
    Check(tsattn_rope_normalize_rows(handle, &a, stream), "tsattn_rope_normalize_rows");
}

// NormalizeState(state) into NormState; a state update left pending by the previous call (the contract product's parts
// in Planes) is done first, by the same launch
void TLayerComputer::NormalizeState(int rows, float *state, void *stream)
{
    const int dim = Dims.Dim;
    if (NormReadyRows > 0) { // the previous call's last product normalised the updated state as its epilogue
        TS_VERIFY(rows == NormReadyRows, "the normalised state of %d rows is at hand, this call has %d", NormReadyRows, rows);
        NormReadyRows = 0;
        return;
    }
    if (PendingPlanes > 0) {
        TS_VERIFY(rows == PendingRows, "a state update of %d rows is pending, this call has %d", PendingRows, rows);
        tsattn_produce_args a = {};
        a.resid = state; a.resid_pitch = dim; a.resid_scale = PendingScale;
        Normalize(Handle, a, rows, Planes, true, PendingPlanes, dim / STATE_NORM_TILE, STATE_NORM_TILE, NormState, stream);
        PendingPlanes = 0;
    } else {
        Normalize(Handle, {}, rows, state, false, 1, dim / STATE_NORM_TILE, STATE_NORM_TILE, NormState, stream);
    }
}

const uint8_t *TLayerComputer::FlushState(int rows, float *state, void *stream)
{
    NormalizeState(rows, state, stream);
    return NormState;
}

// state -> NormalizeState -> the four projections -> ApplyRope on qk and qv, NormalizeState per head on all four: Q4 holds
// rows of qk, qv, k, v heads; QvHeadScale the key scales as [row][head] (token form) or [head][row] planes (prompt form)
void TLayerComputer::Projections(int rows, const int32_t *pos, const float *ropeBuf, int64_t ropeLen, const TAttentionMatrices &att,
                                 bool scalePlanes, float *state, void *stream)
{
    const int dim = Dims.Dim, headCount = Dims.HeadCount, headDim = Dims.QDim, qsum = Dims.GetQSum();
    TS_VERIFY(rows <= MaxRows, "%d rows, buffers for %d", rows, MaxRows);
    NormalizeState(rows, state, stream);
    // Matrices that lie one after the other in memory (QK, QV, K, V) are one product; the result rows hold the qk, qv, k
    // and v heads in that order either way.
    const size_t matBytes = (size_t)qsum * dim;
    // the cached key scale takes the matrix scale: qvMult *= att.QVScale * VEC_SCALE * CalcDotScale(dim)
    tsattn_produce_args a = {};
    a.pos = pos; a.rope = ropeBuf; a.rope_len = ropeLen; a.rope_heads = 2 * headCount;
    a.scale = QvHeadScale;
    if (scalePlanes) { a.scale_pitch = rows; a.scale_row_stride = 1; }           // [head][row], what tsattn_prefill reads
    else { a.scale_pitch = 1; a.scale_row_stride = headCount; }                   // [row][head], what the cache append reads
    a.scale_head_begin = headCount; a.scale_head_count = headCount;
    a.scale_mult = att.QVScale * VEC_SCALE * sqrtf(1.0f / (float)dim);
    if ((const int8_t *)att.QV == att.QK + matBytes && att.K == att.QV + matBytes && att.V == att.K + matBytes) {
        MulForwardNormalize(rows, NormState, dim, att.QK, a, 4 * headCount, headDim, Q4, stream);
        return;
    }
    {
        const int8_t *mats[4] = {att.QK, att.QV, att.K, att.V};
        for (int i = 0; i < 4; ++i) {
            tsattn_matmul_args mm = {};
            mm.m = rows; mm.n = qsum; mm.k = dim;
            mm.a = NormState; mm.a_pitch = dim; mm.w = mats[i]; mm.w_pitch = dim;
            mm.mode = TSATTN_MM_I32; mm.out = Planes + (size_t)i * qsum; mm.out_pitch = 4 * qsum;
            mm.workspace = Workspace; mm.workspace_bytes = WorkspaceBytes;
            Check(tsattn_matmul_i8(Handle, &mm, stream), "tsattn_matmul_i8");
        }
    }
    Normalize(Handle, a, rows, Planes, true, 1, 4 * headCount, headDim, Q4, stream);
}

// KVProduct (unless the attention call made it), combiner (its AddScaled done by the normalisation that follows:
// state += delta * scale, then normalise),
// expand, per-head normalisation + ReLU, contract + AddScaled
void TLayerComputer::AfterAttention(int rows, const TAttentionMatrices &att, bool kvDone, bool deferStateUpdate, float *state, void *stream)
{
    const int dim = Dims.Dim, headCount = Dims.HeadCount, headDim = Dims.QDim, qsum = Dims.GetQSum();
    const uint8_t *k = Q4 + 2 * (size_t)qsum;
    if (!kvDone) {
        Check(tsattn_kv_product(Handle, rows, headCount, headDim, COMBINER_REP, k, 4 * (int64_t)qsum, TSATTN_OUT_F32, ValLookup, qsum, 1.0f, Kv,
                                (int64_t)qsum * COMBINER_REP, stream), "tsattn_kv_product");
    }
    const int kvDim = qsum * COMBINER_REP;
    {
        tsattn_produce_args a = {};
        a.resid = state; a.resid_pitch = dim; a.resid_scale = att.CombinerScale * VEC_SCALE * sqrtf(1.0f / (float)kvDim);
        MulForwardNormalize(rows, Kv, kvDim, att.Combiner, a, dim / STATE_NORM_TILE, STATE_NORM_TILE, NormState, stream);
    }
    {
        tsattn_produce_args a = {};
        a.relu = 1;
        MulForwardNormalize(rows, NormState, dim, att.Expand, a, headCount, ReluDim / headCount, Relu, stream);
    }
    const float contractScale = att.ContractScale * VEC_SCALE * sqrtf(1.0f / (float)ReluDim);
    if (deferStateUpdate && rows > 128) {
        // many rows: the product updates the state and normalises it in its own epilogue; nothing is left pending but
        // the next call's first normalisation is already done
        tsattn_produce_args a = {};
        a.resid = state; a.resid_pitch = dim; a.resid_scale = contractScale;
        MulForwardNormalize(rows, Relu, ReluDim, att.Contract, a, dim / STATE_NORM_TILE, STATE_NORM_TILE, NormState, stream);
        NormReadyRows = rows;
        return;
    }
    if (deferStateUpdate) {
        PendingPlanes = MulForwardPlanes(rows, Relu, ReluDim, att.Contract, dim, stream);
        PendingScale = contractScale;
        PendingRows = rows;
        return;
    }
    tsattn_matmul_args ca = {};
    ca.m = rows; ca.n = dim; ca.k = ReluDim;
    ca.a = Relu; ca.a_pitch = ReluDim; ca.w = att.Contract; ca.w_pitch = ReluDim;
    ca.mode = TSATTN_MM_ADD_SCALED; ca.scale = contractScale;
    ca.out = state; ca.out_pitch = dim; ca.workspace = Workspace; ca.workspace_bytes = WorkspaceBytes;
    Check(tsattn_matmul_i8(Handle, &ca, stream), "tsattn_matmul_i8");
}

void TLayerComputer::AddLookupProduct(const int32_t *t, const float *ropeBuf, int64_t ropeLen, const TAttentionMatrices &att,
                                      TAttentionVecHistory *pKVCache, float *state, void *stream, bool deferStateUpdate)
{
    TAttentionVecHistory &kvCache = *pKVCache;
    const int headCount = Dims.HeadCount, headDim = Dims.QDim, qsum = Dims.GetQSum(), rows = kvCache.SeqCount;
    TS_VERIFY(kvCache.HeadCount == headCount && kvCache.HeadDim == headDim && kvCache.DType == TSATTN_I8,
              "the KV cache does not match the layer (%d heads of %d, int8)", headCount, headDim);
    Projections(rows, t, ropeBuf, ropeLen, att, false, state, stream);
    const uint8_t *qk = Q4, *qv = Q4 + qsum, *v = Q4 + 3 * (size_t)qsum;
    const int64_t pitch4 = 4 * (int64_t)qsum;

    // kvCache.AddVectors(qv, qvHeadScale, v) and ComputeValLookup(width, slope, dims, kvCache, qk, &valLookup)
    tsattn_decode_args da = {};
    da.dtype = TSATTN_I8; da.q_dtype = TSATTN_Q_8BIT;
    da.n_seqs = rows; da.n_heads = headCount; da.head_dim = headDim;
    da.q = qk; da.q_pitch = pitch4; da.q_scale = nullptr; da.q_scale_const = VEC_SCALE;
    da.k_cache = kvCache.QVState; da.v_cache = kvCache.VState;
    da.seq_stride = (int64_t)headCount * kvCache.MaxLen * headDim;
    da.head_stride = (int64_t)kvCache.MaxLen * headDim;
    da.tok_stride = headDim;
    da.k_scale = kvCache.QVStateScale; da.v_scale = kvCache.VStateScale;
    da.s_seq_stride = (int64_t)headCount * kvCache.MaxLen; da.s_head_stride = kvCache.MaxLen;
    da.cache_len = kvCache.Length; da.max_len = kvCache.MaxLen;
    da.window = att.AttentionWidth; da.alibi_slope = att.AlibiSlope;
    da.out = ValLookup;
    // KVProduct(k, valLookup) is written by the attention launches themselves
    da.kv_k = Q4 + 2 * (size_t)qsum; da.kv_k_pitch = pitch4; da.kv_out = Kv; da.kv_out_pitch = (int64_t)qsum * COMBINER_REP;
    da.kv_rep = COMBINER_REP; da.kv_mult = 1.0f;
    if (att.AttentionWidth == 0) {
        // the token attends to the row being written: append first, in its own call
        tsattn_append_args aa = {};
        aa.n_seqs = rows; aa.n_heads = headCount; aa.head_dim = headDim;
        aa.k_new = qv; aa.v_new = v; aa.new_pitch = pitch4; aa.k_scale_new = QvHeadScale; aa.v_scale_new = VHeadScale;
        aa.k_cache = kvCache.QVState; aa.v_cache = kvCache.VState;
        aa.seq_stride = da.seq_stride; aa.head_stride = da.head_stride; aa.tok_stride = da.tok_stride;
        aa.k_scale = kvCache.QVStateScale; aa.v_scale = kvCache.VStateScale;
        aa.s_seq_stride = da.s_seq_stride; aa.s_head_stride = da.s_head_stride;
        aa.cache_len = kvCache.Length; aa.max_len = kvCache.MaxLen;
        Check(tsattn_cache_append(Handle, &aa, stream), "tsattn_cache_append");
    } else {
        da.k_new = qv; da.v_new = v; da.new_pitch = pitch4; da.k_scale_new = QvHeadScale; da.v_scale_new = VHeadScale;
    }
    Check(tsattn_decode(Handle, &da, stream), "tsattn_decode");
    AfterAttention(rows, att, true, deferStateUpdate, state, stream);
}

void TLayerComputer::AddLookupProductPrompt(int len, const int32_t *seqOffset, const int32_t *pos, const float *ropeBuf, int64_t ropeLen,
                                            const TAttentionMatrices &att, const int32_t *spanStart, const int32_t *spanFinish,
                                            const int32_t *spanTiles, int64_t causalPeriod, TAttentionVecHistory *pKVCache, float *state,
                                            void *stream, bool deferStateUpdate, int nSpanParts, int64_t spanPartStride)
{
    const int headCount = Dims.HeadCount, headDim = Dims.QDim, qsum = Dims.GetQSum();
    TS_VERIFY(!pKVCache || (pKVCache->HeadCount == headCount && pKVCache->HeadDim == headDim && pKVCache->DType == TSATTN_I8),
              "the KV cache does not match the layer (%d heads of %d, int8)", headCount, headDim);
    Projections(len, pos, ropeBuf, ropeLen, att, true, state, stream);
    const uint8_t *qk = Q4, *qv = Q4 + qsum, *v = Q4 + 3 * (size_t)qsum;
    const int64_t pitch4 = 4 * (int64_t)qsum;
    // every token's attention over the earlier tokens of its fragment: the prefill form of ComputeValLookup
    tsattn_prefill_args pa = {};
    pa.dtype = TSATTN_I8; pa.out_dtype = TSATTN_OUT_F32;
    pa.n_tokens = len; pa.n_heads = headCount; pa.head_dim = headDim;
    pa.q = qk; pa.k = qv; pa.v = v; pa.q_pitch = pa.k_pitch = pa.v_pitch = pitch4;
    pa.q_scale = nullptr; pa.q_scale_const = VEC_SCALE; pa.k_scale = QvHeadScale; pa.v_scale = nullptr; pa.v_scale_const = VEC_SCALE;
    pa.scale_pitch = len;
    pa.span_start = spanStart; pa.span_finish = spanFinish; pa.span_tiles = spanTiles; pa.causal_period = causalPeriod;
    pa.n_span_parts = nSpanParts; pa.span_part_stride = spanPartStride;
    pa.alibi_slope = att.AlibiSlope;
    pa.out = WriteValLookup ? ValLookup : nullptr; pa.out_pitch = (int64_t)qsum * 4;
    // KVProduct (cpu_infer.cpp:511) as the attention kernel's last step
    pa.kv_k = Q4 + 2 * (size_t)qsum; pa.kv_k_pitch = pitch4; pa.kv_out = Kv; pa.kv_out_pitch = (int64_t)qsum * COMBINER_REP;
    pa.kv_rep = COMBINER_REP; pa.kv_mult = 1.0f;
    Check(tsattn_prefill(Handle, &pa, stream), "tsattn_prefill");
    // kvCache.AddVectors for every token at once (a forward pass over fragments that nobody continues has no cache)
    if (pKVCache) {
    TAttentionVecHistory &kvCache = *pKVCache;
    tsattn_fill_args fa = {};
    fa.n_seqs = kvCache.SeqCount; fa.n_heads = headCount; fa.head_dim = headDim; fa.n_tokens = len;
    fa.seq_offset = seqOffset; fa.k = qv; fa.v = v; fa.pitch = pitch4;
    fa.k_scale = QvHeadScale; fa.v_scale = VHeadScale; fa.scale_pitch = len; // VHeadScale: the constant in every slot
    fa.k_cache = kvCache.QVState; fa.v_cache = kvCache.VState;
    fa.seq_stride = (int64_t)headCount * kvCache.MaxLen * headDim;
    fa.head_stride = (int64_t)kvCache.MaxLen * headDim;
    fa.tok_stride = headDim;
    fa.k_scale_cache = kvCache.QVStateScale; fa.v_scale_cache = kvCache.VStateScale;
    fa.s_seq_stride = (int64_t)headCount * kvCache.MaxLen; fa.s_head_stride = kvCache.MaxLen;
    fa.cache_len = kvCache.Length; fa.max_len = kvCache.MaxLen;
    Check(tsattn_cache_fill(Handle, &fa, stream), "tsattn_cache_fill");
    }
    AfterAttention(len, att, true, deferStateUpdate, state, stream);
}

void ComputePrediction(TLayerComputer &layer, const TInferModel &model, const std::vector<TAttentionVecHistory *> &kvCaches,
                       const int32_t *labels, const int32_t *t, const float *ropeBuf, int64_t ropeLen, float *state,
                       float *prediction, int32_t *choice, void *stream)
{
    TS_VERIFY(kvCaches.size() == model.LayerArr.size() && !kvCaches.empty(), "%d caches for %d layers", (int)kvCaches.size(), (int)model.LayerArr.size());
    const int dim = layer.Dims.Dim, rows = kvCaches[0]->SeqCount;
    // embedding
    Check(tsattn_embed_rows(layer.Handle, rows, dim, labels, 1, model.LabelEmbed, dim, model.LabelCount, model.LabelEmbedScale, state, dim, stream),
          "tsattn_embed_rows");
    // apply layers
    // every layer leaves its last state update to the next one's first normalisation, the last layer to FlushState
    for (size_t d = 0; d < model.LayerArr.size(); ++d) layer.AddLookupProduct(t, ropeBuf, ropeLen, model.LayerArr[d], kvCaches[d], state, stream, true);
    layer.FlushState(rows, state, stream); // NormalizeState of the final state
    if (prediction || choice) {
        const int planes = layer.MulForwardPlanes(rows, layer.NormState, dim, model.FinalLayer, (int)model.VocabSize, stream);
        // finalScale = CalcDotScale(dim) * CalcFinalLayerMult() * params.FinalLayerScale * VEC_SCALE
        const float finalScale = sqrtf(1.0f / (float)dim) * (1.0f / 0.693147f) * model.FinalLayerScale * VEC_SCALE;
        Check(tsattn_softmax_rows(layer.Handle, rows, model.VocabSize, layer.Planes, planes, (int64_t)rows * model.VocabSize, model.VocabSize, finalScale,
                                  model.Bias, prediction, model.VocabSize, choice, stream), "tsattn_softmax_rows");
    }
}

void SampleFromDistr(tsattn_handle_t handle, int rows, int64_t vocabSize, const float *prediction, float temperature, uint64_t seed,
                     uint64_t offset, int32_t *choice, void *stream)
{
    Check(tsattn_sample_rows(handle, rows, vocabSize, prediction, vocabSize, temperature, nullptr, 0, seed, offset, choice, stream),
          "tsattn_sample_rows");
}

// ---- TNodesBatch, TComputeContext ----------------------------------------------------------------------------------

void TNodesBatch::Init(int attentionWidthCount)
{
    SampleIndex.resize(0);
    LabelArr.resize(0);
    LabelPtr.assign(1, 0u);
    Target.resize(0);
    AttArr.resize(attentionWidthCount);
    for (TAttentionInfo &att : AttArr) att.Init();
}

void TNodesBatch::AddSample(int idx, const std::vector<int32_t> &labels, const std::vector<std::vector<TAttentionSpan>> &attSpansArr)
{
    SampleIndex.push_back(idx);
    LabelArr.insert(LabelArr.end(), labels.begin(), labels.end());
    LabelPtr.push_back((uint32_t)LabelArr.size());
    TS_VERIFY(AttArr.size() == attSpansArr.size(), "%d span lists for %d attention widths", (int)attSpansArr.size(), (int)AttArr.size());
    for (size_t k = 0; k < AttArr.size(); ++k) {
        for (const TAttentionSpan &span : attSpansArr[k]) AttArr[k].AddSpan(span);
        AttArr[k].AddSample();
    }
}

// One inclusive span per row (rows without keys: an empty one) from the reference's span lists, and the launch-order
// hint: rows without keys mark fragment starts; if they are equally spaced, cover the batch and the window is wide
// (the last row of a fragment sees at least half of it), the batch has a causal period.
static int FlattenSpans(const TAttentionInfo &attInfo, std::vector<int32_t> *pStart, std::vector<int32_t> *pFinish, int part, bool oneSpanPerRow)
{
    const int len = (int)attInfo.GetSampleCount();
    std::vector<int32_t> &st = *pStart, &fi = *pFinish;
    st.resize(len);
    fi.resize(len);
    for (int t = 0; t < len; ++t) {
        const int a = attInfo.SpanPtr[t] + part, b = attInfo.SpanPtr[t + 1];
        if (oneSpanPerRow) TS_VERIFY(b - a <= 1, "row %d has %d spans; one span per row is supported here", t, b - a);
        if (b > a) {
            st[t] = attInfo.Spans[a].Start;
            fi[t] = attInfo.Spans[a].Finish;
        } else {
            st[t] = t;
            fi[t] = t - 1;
        }
    }
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
    if (regular && period == 0) period = len; // a single fragment
    if (regular && period > 0 && len % period == 0 && last == len - period) {
        const int tail = len - 1;
        if (fi[tail] - st[tail] + 1 >= period / 2) return period;
    }
    return 0;
}

TComputeContext::TComputeContext(tsattn_handle_t handle, const TModelDims &dims, const TInferModel &model, const std::vector<int> &layerWidthId,
                                 int attentionWidthCount, int maxNodeCount, int maxLabelsPerNode)
    : Handle(handle), Dims(dims), Model(model), LayerWidthId(layerWidthId), AttentionWidthCount(attentionWidthCount), MaxNodeCount(maxNodeCount),
      MaxLabelsPerNode(maxLabelsPerNode), Layer(handle, dims, maxNodeCount, model.VocabSize)
{
    TS_VERIFY(layerWidthId.size() == model.LayerArr.size(), "%d width ids for %d layers", (int)layerWidthId.size(), (int)model.LayerArr.size());
    for (int id : layerWidthId) TS_VERIFY(id >= 0 && id < attentionWidthCount, "attention width id %d of %d", id, attentionWidthCount);
    TS_VERIFY(maxNodeCount > 0 && maxLabelsPerNode > 0, "empty context");
    Nodes.Init(attentionWidthCount);
    const size_t n = (size_t)maxNodeCount;
    CheckHip(hipMalloc((void **)&Labels, n * maxLabelsPerNode * sizeof(int32_t)), "hipMalloc(labels)");
    CheckHip(hipMalloc((void **)&Pos, n * sizeof(int32_t)), "hipMalloc(positions)");
    CheckHip(hipMalloc((void **)&State, n * dims.Dim * sizeof(float)), "hipMalloc(state)");
    CheckHip(hipMalloc((void **)&Prediction, n * (size_t)model.VocabSize * sizeof(float)), "hipMalloc(prediction)");
    CheckHip(hipMalloc((void **)&RopeBuf, n * dims.QDim * sizeof(float)), "hipMalloc(rope table)");
    SpanStart.assign(attentionWidthCount, nullptr);
    SpanFinish.assign(attentionWidthCount, nullptr);
    SpanTiles.assign(attentionWidthCount, nullptr);
    CausalPeriod.assign(attentionWidthCount, 0);
    SpanParts.assign(attentionWidthCount, 1);
    SpanPartCapacity.assign(attentionWidthCount, 0);
    for (int k = 0; k < attentionWidthCount; ++k) ReserveSpans(k, 1);
    // FillRopeBuf for every node index of the largest batch, and the nodes' positions (their indices), once
    std::vector<float> rope(n * dims.QDim);
    tsattn_fill_rope_table(dims.QDim, maxNodeCount, rope.data());
    std::vector<int32_t> pos(n);
    for (size_t i = 0; i < n; ++i) pos[i] = (int32_t)i;
    CheckHip(hipMemcpy(RopeBuf, rope.data(), rope.size() * sizeof(float), hipMemcpyHostToDevice), "rope table copy");
    CheckHip(hipMemcpy(Pos, pos.data(), n * sizeof(int32_t), hipMemcpyHostToDevice), "position copy");
}

TComputeContext::~TComputeContext()
{
    for (void *p : {(void *)Labels, (void *)Pos, (void *)State, (void *)Prediction, (void *)RopeBuf}) (void)hipFree(p);
    for (int k = 0; k < AttentionWidthCount; ++k) {
        (void)hipFree(SpanStart[k]);
        (void)hipFree(SpanFinish[k]);
        (void)hipFree(SpanTiles[k]);
    }
}

// room for `parts` spans per row of width k's span list (more than one only where a batch has such rows)
void TComputeContext::ReserveSpans(int k, int parts)
{
    if (parts <= SpanPartCapacity[k]) return;
    (void)hipFree(SpanStart[k]);
    (void)hipFree(SpanFinish[k]);
    (void)hipFree(SpanTiles[k]);
    const size_t n = (size_t)MaxNodeCount * parts;
    CheckHip(hipMalloc((void **)&SpanStart[k], n * sizeof(int32_t)), "hipMalloc(spans)");
    CheckHip(hipMalloc((void **)&SpanFinish[k], n * sizeof(int32_t)), "hipMalloc(spans)");
    CheckHip(hipMalloc((void **)&SpanTiles[k], (size_t)((MaxNodeCount + 127) / 128) * parts * TSATTN_SPAN_TILE_INTS * sizeof(int32_t)), "hipMalloc(span summary)");
    SpanPartCapacity[k] = parts;
}

TNodesBatch &TComputeContext::GetNodes(int deviceId)
{
    TS_VERIFY(deviceId == 0, "device %d of 1", deviceId);
    return Nodes;
}

// Per batch: the nodes' labels and every width's spans go to the device (gpt_cpu.cpp:862-883, gpt_cuda.cu:1350-1376).
void TComputeContext::Init(int deviceId, EInitType initType)
{
    (void)initType; // (no dropout on this path: a training batch is computed like a test batch)
    TS_VERIFY(deviceId == 0, "device %d of 1", deviceId);
    const int len = Nodes.GetNodeCount();
    TS_VERIFY(len <= MaxNodeCount, "%d nodes exceed the context's %d", len, MaxNodeCount);
    TS_VERIFY((int)Nodes.LabelPtr.size() == len + 1 && (int)Nodes.AttArr.size() == AttentionWidthCount, "inconsistent batch");
    Len = len;
    KeepTarget = Nodes.Target;
    // labels as rows of equal width; unused slots hold -1 (an empty slot for the embedding)
    int perRow = 1;
    for (int i = 0; i < len; ++i) perRow = std::max(perRow, (int)(Nodes.LabelPtr[i + 1] - Nodes.LabelPtr[i]));
    TS_VERIFY(perRow <= MaxLabelsPerNode, "%d labels on a node exceed the context's %d", perRow, MaxLabelsPerNode);
    LabelsPerRow = perRow;
    std::vector<int32_t> labels((size_t)len * perRow, -1);
    for (int i = 0; i < len; ++i)
        for (uint32_t j = Nodes.LabelPtr[i]; j < Nodes.LabelPtr[i + 1]; ++j) labels[(size_t)i * perRow + (j - Nodes.LabelPtr[i])] = Nodes.LabelArr[j];
    if (len > 0) CheckHip(hipMemcpy(Labels, labels.data(), labels.size() * sizeof(int32_t), hipMemcpyHostToDevice), "label copy");
    std::vector<int32_t> st, fi;
    const int64_t tileInts = TSATTN_SPAN_TILE_INTS * tsattn_span_tiles_count(len);
    for (int k = 0; k < AttentionWidthCount; ++k) {
        const TAttentionInfo &att = Nodes.AttArr[k];
        TS_VERIFY((int)att.GetSampleCount() == len, "span list %d has %d samples for %d nodes", k, (int)att.GetSampleCount(), len);
        // rows may hold several spans (the reference's ComputeFragmentPredictions takes any TAttentionInfo,
        // gpt_cpu.cpp:405-436): part i is every row's i-th span, walked by the one attention launch of the layer
        int parts = 1;
        for (int t = 0; t < len; ++t) parts = std::max(parts, att.SpanPtr[t + 1] - att.SpanPtr[t]);
        TS_VERIFY(parts <= 64, "a node with %d spans; up to 64 are supported", parts);
        if (parts > SpanPartCapacity[k]) CheckHip(hipDeviceSynchronize(), "before the span arrays grow");
        ReserveSpans(k, parts);
        SpanParts[k] = parts;
        for (int i = 0; i < parts; ++i) {
            const int period = FlattenSpans(att, &st, &fi, i, false);
            CausalPeriod[k] = parts == 1 ? period : 0;
            if (len == 0) continue;
            int32_t *const ds = SpanStart[k] + (size_t)i * MaxNodeCount, *const df = SpanFinish[k] + (size_t)i * MaxNodeCount;
            CheckHip(hipMemcpy(ds, st.data(), sizeof(int32_t) * len, hipMemcpyHostToDevice), "span copy"); // (blocking: st, fi are reused)
            CheckHip(hipMemcpy(df, fi.data(), sizeof(int32_t) * len, hipMemcpyHostToDevice), "span copy");
            Check(tsattn_build_span_tiles(Handle, len, ds, df, SpanTiles[k] + i * tileInts, nullptr), "tsattn_build_span_tiles");
        }
    }
    CheckHip(hipDeviceSynchronize(), "batch set-up");
}

// ComputeForward (gpt_cpu.cpp:886-938) up to the normalised final state
const uint8_t *TComputeContext::ComputeForward(void *stream)
{
    TS_VERIFY(Len > 0, "Init() with a non-empty batch comes first");
    const int dim = Dims.Dim;
    Check(tsattn_embed_rows(Handle, Len, dim, Labels, LabelsPerRow, Model.LabelEmbed, dim, Model.LabelCount, Model.LabelEmbedScale, State, dim, stream),
          "tsattn_embed_rows");
    for (size_t d = 0; d < Model.LayerArr.size(); ++d) {
        const int k = LayerWidthId[d];
        Layer.AddLookupProductPrompt(Len, nullptr, Pos, RopeBuf, MaxNodeCount, Model.LayerArr[d], SpanStart[k], SpanFinish[k], SpanTiles[k],
                                     CausalPeriod[k], nullptr, State, stream, true, SpanParts[k], MaxNodeCount);
    }
    return Layer.FlushState(Len, State, stream);
}

void TComputeContext::ComputeFinalStateVectors(std::vector<std::vector<float>> *pStateVectors)
{
    ComputeForward(nullptr);
    std::vector<float> flat((size_t)Len * Dims.Dim);
    CheckHip(hipMemcpy(flat.data(), State, flat.size() * sizeof(float), hipMemcpyDeviceToHost), "state copy");
    pStateVectors->resize(Len);
    for (int i = 0; i < Len; ++i) (*pStateVectors)[i].assign(flat.begin() + (size_t)i * Dims.Dim, flat.begin() + (size_t)(i + 1) * Dims.Dim);
}

void TComputeContext::ComputeFragmentPredictions(std::vector<std::vector<float>> *pPrediction)
{
    const uint8_t *norm = ComputeForward(nullptr);
    const int dim = Dims.Dim;
    const int64_t vocab = Model.VocabSize;
    const int planes = Layer.MulForwardPlanes(Len, norm, dim, Model.FinalLayer, (int)vocab, nullptr);
    // finalScale = CalcDotScale(dim) * CalcFinalLayerMult() * params.FinalLayerScale * VEC_SCALE (cpu_infer.cpp:574-579)
    const float finalScale = sqrtf(1.0f / (float)dim) * (1.0f / 0.693147f) * Model.FinalLayerScale * VEC_SCALE;
    Check(tsattn_softmax_rows(Handle, Len, vocab, Layer.Planes, planes, (int64_t)Len * vocab, vocab, finalScale, Model.Bias, Prediction, vocab, nullptr,
                              nullptr), "tsattn_softmax_rows");
    std::vector<float> flat((size_t)Len * vocab);
    CheckHip(hipMemcpy(flat.data(), Prediction, flat.size() * sizeof(float), hipMemcpyDeviceToHost), "prediction copy");
    pPrediction->resize(Len);
    for (int i = 0; i < Len; ++i) (*pPrediction)[i].assign(flat.begin() + (size_t)i * vocab, flat.begin() + (size_t)(i + 1) * vocab);
}

void TComputeContext::ComputeFragmentPredictions(std::vector<float> *pPrediction)
{
    std::vector<std::vector<float>> prediction;
    ComputeFragmentPredictions(&prediction);
    pPrediction->assign(prediction.size(), 0.0f);
    for (const TNodeTarget &nt : KeepTarget) (*pPrediction)[nt.Node] = prediction[nt.Node][nt.TargetId];
}

float TComputeContext::ComputeScore()
{
    std::vector<std::vector<float>> prediction;
    ComputeFragmentPredictions(&prediction);
    double sum = 0;
    int64_t count = 0;
    for (const TNodeTarget &nt : KeepTarget) {
        sum += log(prediction[nt.Node][nt.TargetId]);
        count += 1;
    }
    return (float)(sum / (double)count);
}

} // namespace NTsAttn
