// C++ host side of the attention path: keeps the shape of the reference's attention call sites so
// that a model/layer implementation written against them can switch to the gfx950 kernels.
//
//   reference                                                     here
//   TAttentionSpan / TAttentionInfo        gpt/att/att.h:4-47      NTsAttn::TAttentionSpan / TAttentionInfo
//   AddAttSpans + GenerateAttentionGraph   gpt/att/sliding_window.cpp:80-87,205-223   NTsAttn::AddWindowSpans
//   TAttentionComputer::ComputeValLookup   gpt/compute/gpt_cpu.cpp:391-441 (call :633),
//   CudaCall(c, Fp8Att)...                 gpt/compute/gpt_cuda.cu:503-507            TAttentionComputer::ComputeValLookup
//   TAttentionVecHistory::AddVectors       gpt/train/cpu_infer.cpp:397-410            TAttentionVecHistory::AddVectors
//   ComputeValLookup (KV cache)            gpt/train/cpu_infer.cpp:413-460 (call :509) NTsAttn::ComputeValLookup
//   TCPUModelParams::TAttentionMatrices    gpt/train/cpu_infer.cpp:60-77              NTsAttn::TAttentionMatrices
//   AddLookupProduct                       gpt/train/cpu_infer.cpp:465-527            TLayerComputer::AddLookupProduct(Prompt)
//   ComputePrediction                      gpt/train/cpu_infer.cpp:552-582            NTsAttn::ComputePrediction
//   SampleFromDistr                        gpt/train/cpu_infer.cpp:585-599            NTsAttn::SampleFromDistr
//   TNodeTarget / TNodesBatch              gpt/att/nodes_batch.h:10-36                NTsAttn::TNodeTarget / TNodesBatch
//   IComputeContext (the forward half)     gpt/compute/model.h:55-155                 NTsAttn::TComputeContext
//
// All arithmetic runs in libtsattn.so through the C ABI of include/tsattn.h; this layer owns the
// per-context device buffers (allocated once, like TAttentionComputeCtx::AllocateCuda,
// gpt/compute/gpt_cuda.cu:231-302) and aborts on errors the way the reference's Y_VERIFY does.
#pragma once

#include <stddef.h>
#include <stdint.h>

#include <vector>

#include "../../include/tsattn.h"

namespace NTsAttn {

struct TAttentionSpan {
    // inclusive borders
    int Start = 0;
    int Finish = 0;
    TAttentionSpan() {}
    TAttentionSpan(int start, int finish) : Start(start), Finish(finish) {}
};

struct TAttentionInfo {
    std::vector<TAttentionSpan> Spans;
    std::vector<int> SpanPtr;

    void Init()
    {
        Spans.resize(0);
        SpanPtr.assign(1, 0);
    }
    size_t GetSampleCount() const { return SpanPtr.size() - 1; }
    bool IsEmpty() const { return SpanPtr.size() <= 1; }
    void AddSpan(const TAttentionSpan &span) { Spans.push_back(span); }
    void AddSample() { SpanPtr.push_back((int)Spans.size()); }
};

struct TModelDims {
    int Dim = 256;
    int QDim = 128;
    int TTDim = 128;
    int HeadCount = 1;
    int ReluMult = 1; // feed-forward width in units of 128 per head (gpt/model_params/model_dim.h:66)
    int GetReluDim() const { return HeadCount * 128 * ReluMult; }
    int GetQSum() const { return QDim * HeadCount; }
    int GetTTSum() const { return TTDim * HeadCount; }
};

// Appends the samples of one fragment of `len` tokens that starts at node `ptr` of the batch:
// token t sees [max(docStart, t - limitWindow), t - 1]; limitWindow == 0 means itself only;
// docStartFlag (nullable, per token of the fragment) marks document starts inside the fragment.
void AddWindowSpans(int ptr, int len, int limitWindow, const uint8_t *docStartFlag, TAttentionInfo *pAtt);

// Quantised per-row operands as the projection epilogues leave them on the device.
struct TQuantRows {
    const void *Data = nullptr;   // [len][headCount*dim] 8-bit, device
    int64_t PitchBytes = 0;
    const float *Scale = nullptr; // [headCount][scalePitch] device, or nullptr = ConstScale
    float ConstScale = 1;
};

class TAttentionComputer
{
    tsattn_handle_t Handle = nullptr;
    TModelDims Dims;
    float AlibiSlope = 0;
    int MaxLen = 0;
    int Len = 0;
    int CausalPeriod = 0; // launch-order hint derived from the spans by SetAttention
    int64_t SpanLenHint = 0; // typical keys per row of the spans set (tsattn_prefill_args.span_len_hint)
    void *Workspace = nullptr; // device scratch of the long-span kernel (tsattn_prefill_args.workspace), if maxLen can need it
    size_t WorkspaceBytes = 0;
    // Rows may hold several spans: part i of the batch is every row's i-th span (an empty one for rows with fewer)
    int Parts = 1, PartCapacity = 0;
    int32_t *SpanStart = nullptr; // device [PartCapacity][MaxLen]
    int32_t *SpanFinish = nullptr;
    int32_t *SpanTiles = nullptr; // per part: per-128-row summary of the spans (tsattn_build_span_tiles)
    float *SumWeightLog = nullptr; // device [headCount][MaxLen]
    float *PartOut = nullptr;      // device [PartCapacity][MaxLen][headCount*TTDim], only with more than one part
    float *PartSwl = nullptr;      // device [PartCapacity][headCount][MaxLen]
    void Reserve(int parts);

  public:
    // Rows with several spans: false = one launch that walks them (n_span_parts of tsattn_prefill_args), true = one launch
    // per span of the rows and tsattn_merge_lookups.  The same result up to rounding.
    bool MergeParts = false;
    // maxSeqs > 0 also provisions the handle for KV-cache decode of that many sequences
    TAttentionComputer(const TModelDims &dims, float alibiSlope, int deviceId, int maxLen, int maxSeqs = 0);
    ~TAttentionComputer();
    TAttentionComputer(const TAttentionComputer &) = delete;
    TAttentionComputer &operator=(const TAttentionComputer &) = delete;

    // Per batch, like TComputeContext::Init copying the spans to the device (gpt_cuda.cu:1362-1376).
    // Rows with several spans (TAttentionInfo allows any number) cost one attention launch per span of the rows and
    // one launch that combines them (tsattn_merge_lookups).
    void SetAttention(const TAttentionInfo &attInfo, void *stream);
    int GetPartCount() const { return Parts; }

    // valLookup: device [len][headCount*TTDim] fp32 (outF16 = false) or fp16.
    void ComputeValLookup(int len, int dtype, const TQuantRows &qk, const TQuantRows &qv, const TQuantRows &v,
                          const float *qvGlobalScale, void *valLookup, int64_t valLookupPitchBytes, bool outF16,
                          void *stream);
    const float *GetSumWeightLog() const { return SumWeightLog; }
    int GetSumWeightLogPitch() const { return MaxLen; }
    tsattn_handle_t GetHandle() const { return Handle; }
};

// Device-resident KV cache: planar [seq][head][maxLen][dim] 8-bit planes and [seq][head][maxLen] fp32
// key and value row scales.
struct TAttentionVecHistory {
    tsattn_handle_t Handle = nullptr;
    int DType = TSATTN_I8;
    int SeqCount = 0, HeadCount = 0, MaxLen = 0, HeadDim = 0;
    uint8_t *QVState = nullptr;        // keys
    uint8_t *VState = nullptr;         // values
    float *QVStateScale = nullptr;
    float *VStateScale = nullptr;
    int32_t *Length = nullptr;         // device [seqCount]

    TAttentionVecHistory(tsattn_handle_t handle, int dtype, int seqCount, int headCount, int maxLen, int headDim);
    ~TAttentionVecHistory();
    TAttentionVecHistory(const TAttentionVecHistory &) = delete;
    TAttentionVecHistory &operator=(const TAttentionVecHistory &) = delete;

    // qv, v: device [seqCount][headCount*headDim]; scales device [seqCount][headCount]
    void AddVectors(const void *qv, const float *qvScale, const void *v, const float *vScale, void *stream);
};

// One new token per sequence; qk: device [seqCount][headCount*headDim] 8-bit with qkScale
// [seqCount][headCount] (nullptr = qkConstScale).  valLookup: device [seqCount][headCount*headDim] fp32.
void ComputeValLookup(int width, float alibiSlope, const TAttentionVecHistory &history, const void *qk,
                      const float *qkScale, float qkConstScale, float *valLookup, void *stream);

// One layer's matrices of the int8 inference path, on the device: int8, one row per output (the layout MulForward
// reads), with the scales ConvertMatrix returned.
struct TAttentionMatrices {
    const int8_t *QK = nullptr, *QV = nullptr, *K = nullptr, *V = nullptr; // [HeadCount*QDim][Dim]
    const int8_t *Combiner = nullptr;                                       // [Dim][HeadCount*TTDim*COMBINER_REP]
    const int8_t *Expand = nullptr;                                         // [ReluDim][Dim]
    const int8_t *Contract = nullptr;                                       // [Dim][ReluDim]
    float QVScale = 0, CombinerScale = 0, ContractScale = 0;
    int AttentionWidth = 0;
    float AlibiSlope = 0;
};

constexpr float VEC_SCALE = 1.0f / 24; // gpt/train/cpu_infer.cpp:16
constexpr int STATE_NORM_TILE = 128;   // gpt/model_params/model_dim.h:22
constexpr int COMBINER_REP = 4;        // gpt/model_params/model_dim.h:12

// AddLookupProduct for a batch of rows.  Token form: one new token per sequence, every sequence with its own state row
// and KV cache (append + attention over the cache).  Prompt form: all tokens of a batch of fragments at once (one
// prefill launch, one cache fill).  Owns the intermediate vectors (allocated once for maxRows rows).  10 or 11 launches
// per token call: the four projections are one product when QK, QV, K and V lie one after the other in memory, the
// normalisations that follow them are one call, K-split products leave their parts for the consumer to add up, and the
// combiner's AddScaled is done by the normalisation after it.  QDim == TTDim == 64 or 128; the feed-forward width is
// reluDim = HeadCount * 128 * ReluMult with ReluMult 1 to 4.
struct TInferModel; // below

class TLayerComputer
{
    tsattn_handle_t Handle = nullptr;
    TModelDims Dims;
    int MaxRows = 0, ReluDim = 0;
    uint8_t *NormState = nullptr, *Q4 = nullptr, *Kv = nullptr, *Relu = nullptr; // Q4: rows of qk, qv, k, v heads
    float *QvHeadScale = nullptr, *VHeadScale = nullptr, *ValLookup = nullptr;
    int32_t *Planes = nullptr; // int32 results of the matrix products: up to 16 planes with few rows, one otherwise
    void *Workspace = nullptr;
    int64_t WorkspaceBytes = 0;
    int PendingPlanes = 0, PendingRows = 0; // a deferred state update: the contract product's parts in Planes
    int NormReadyRows = 0;                  // NormState already holds NormalizeState of the caller's state (that many rows)
    float PendingScale = 0;

    int MulForwardPlanes(int rows, const uint8_t *vec, int k, const int8_t *matr, int n, void *stream);
    void MulForwardNormalize(int rows, const uint8_t *vec, int k, const int8_t *matr, tsattn_produce_args a, int groups, int groupDim,
                             uint8_t *dst, void *stream);
    void Projections(int rows, const int32_t *pos, const float *ropeBuf, int64_t ropeLen, const TAttentionMatrices &att, bool scalePlanes,
                     float *state, void *stream);
    void AfterAttention(int rows, const TAttentionMatrices &att, bool kvDone, bool deferStateUpdate, float *state, void *stream);
    void NormalizeState(int rows, float *state, void *stream);
    friend void ComputePrediction(TLayerComputer &, const TInferModel &, const std::vector<TAttentionVecHistory *> &, const int32_t *,
                                  const int32_t *, const float *, int64_t, float *, float *, int32_t *, void *);
    friend class TComputeContext;

  public:
    // maxOutputs: the widest matrix product a caller will run through this object's buffers (the vocabulary size for
    // ComputePrediction; 0 = the layer's own products only)
    TLayerComputer(tsattn_handle_t handle, const TModelDims &dims, int maxRows, int64_t maxOutputs = 0);
    ~TLayerComputer();
    TLayerComputer(const TLayerComputer &) = delete;
    TLayerComputer &operator=(const TLayerComputer &) = delete;

    // t: device int32 [seqCount], the new tokens' positions; ropeBuf: device table of FillRopeBuf with ropeLen rows;
    // state: device [seqCount][Dim] fp32, updated in place; the cache gets the new rows and its lengths grow by one.
    // deferStateUpdate (layers that follow one another on the same state rows): with few rows the layer's last state
    // update (contract's AddScaled) is left to the first normalisation of the next call, or to FlushState -- one launch
    // less per layer; until then `state` lacks that update.  With many rows the last product updates the state and
    // normalises it for the next call as its epilogue.  Either way finish with FlushState.
    void AddLookupProduct(const int32_t *t, const float *ropeBuf, int64_t ropeLen, const TAttentionMatrices &att,
                          TAttentionVecHistory *pKVCache, float *state, void *stream, bool deferStateUpdate = false);
    // Does a pending state update and returns NormalizeState(state) (device, int8 [rows][Dim]), which is what
    // ComputePrediction multiplies with the final layer.
    const uint8_t *FlushState(int rows, float *state, void *stream);
    // len tokens of the cache's sequences, concatenated (seqOffset: device int32 [seqCount + 1]); pos: device int32 [len],
    // each token's position in its sequence; spans (and optionally their summary and the launch-order hint) of
    // att.AttentionWidth as for tsattn_prefill; state: device [len][Dim]; the tokens' rows are appended to the cache
    // (pKVCache and seqOffset may be null: nothing is kept for later tokens).
    void AddLookupProductPrompt(int len, const int32_t *seqOffset, const int32_t *pos, const float *ropeBuf, int64_t ropeLen,
                                const TAttentionMatrices &att, const int32_t *spanStart, const int32_t *spanFinish,
                                const int32_t *spanTiles, int64_t causalPeriod, TAttentionVecHistory *pKVCache, float *state,
                                void *stream, bool deferStateUpdate = false, int nSpanParts = 1, int64_t spanPartStride = 0);
    const float *GetValLookup() const { return ValLookup; } // [rows][HeadCount*TTDim] of the last call
    // false: AddLookupProductPrompt does not write the attention output (its KVProduct, made by the same kernel, is all
    // the layer reads); GetValLookup() is then stale after that call
    bool WriteValLookup = true;
};

// The model around the layers: TCPUModelParams of the reference (gpt/train/cpu_infer.cpp:58-86), device copies.
struct TInferModel {
    const int8_t *LabelEmbed = nullptr; // [LabelCount][Dim]
    float LabelEmbedScale = 0;
    int64_t LabelCount = 0;
    std::vector<TAttentionMatrices> LayerArr;
    const int8_t *FinalLayer = nullptr; // [VocabSize][Dim]
    float FinalLayerScale = 0;
    int64_t VocabSize = 0;
    const float *Bias = nullptr;        // [VocabSize]
};

// ComputePrediction (gpt/train/cpu_infer.cpp:552-582) for one new token per sequence: embedding of `labels` (device
// int32 [seqCount], one label per token) -> every layer's AddLookupProduct on its own cache -> NormalizeState,
// MulForward(FinalLayer), SoftMax.  state: device scratch [seqCount][Dim].  prediction (device [seqCount][VocabSize],
// nullable) receives the distribution, choice (device int32 [seqCount], nullable) the most likely label.
void ComputePrediction(TLayerComputer &layer, const TInferModel &model, const std::vector<TAttentionVecHistory *> &kvCaches,
                       const int32_t *labels, const int32_t *t, const float *ropeBuf, int64_t ropeLen, float *state,
                       float *prediction, int32_t *choice, void *stream);

// SampleFromDistr (gpt/train/cpu_infer.cpp:585-599) for every row of a batch of distributions: the Gumbel-max choice at
// the given temperature.  The random words come from the library's counter-based generator (same seed and offset:
// same choices; advance offset by rows * vocabSize per call), not from the reference's MT19937 stream.
void SampleFromDistr(tsattn_handle_t handle, int rows, int64_t vocabSize, const float *prediction, float temperature, uint64_t seed,
                     uint64_t offset, int32_t *choice, void *stream);

// The batch a context computes on, filled by the caller exactly as the reference's MakeTest / MakeTrain fill theirs
// (gpt/att/nodes_batch.h:10-36, nodes_batch.cpp:5-31): a node is one token position of one fragment; LabelArr /
// LabelPtr hold every node's embedding labels, AttArr one span list per attention width of the model, Target the
// (node, label) pairs whose probability is asked for.
struct TNodeTarget {
    int64_t Node = 0;
    int64_t TargetId = 0;
    TNodeTarget() {}
    TNodeTarget(int64_t nodeId, int64_t targetId) : Node(nodeId), TargetId(targetId) {}
};

struct TNodesBatch {
    std::vector<int32_t> LabelArr;
    std::vector<uint32_t> LabelPtr;
    std::vector<int> SampleIndex;
    std::vector<TNodeTarget> Target;
    std::vector<TAttentionInfo> AttArr;

    void Init(int attentionWidthCount);
    void AddSample(int idx, const std::vector<int32_t> &labels, const std::vector<std::vector<TAttentionSpan>> &attSpansArr);
    int GetNodeCount() const { return (int)SampleIndex.size(); }
};

// The forward half of the reference's IComputeContext (gpt/compute/model.h:55-155; its CPU form
// gpt/compute/gpt_cpu.cpp:795-967) over the int8 model: fill GetNodes(0), Init(0, INIT_TEST), then
// ComputeFragmentPredictions / ComputeFinalStateVectors / ComputeScore, which run the batch form of every layer
// (AddLookupProductPrompt on the spans of the layer's attention width; a node's RoPE position is its index in the
// batch, gpt/att/rope.cpp:53-62).  One device; nothing of the training half (Backprop, the gradient and parameter
// accessors) exists here.
class TComputeContext
{
  public:
    enum EInitType { INIT_TRAIN, INIT_TEST };

  private:
    tsattn_handle_t Handle = nullptr;
    TModelDims Dims;
    TInferModel Model;
    std::vector<int> LayerWidthId; // per layer: which of the batch's span lists it attends over (AttentionWidthId)
    int AttentionWidthCount = 0, MaxNodeCount = 0, MaxLabelsPerNode = 0;
    TLayerComputer Layer;
    TNodesBatch Nodes;
    std::vector<TNodeTarget> KeepTarget;
    int Len = 0, LabelsPerRow = 1;
    int32_t *Labels = nullptr, *Pos = nullptr;
    std::vector<int32_t *> SpanStart, SpanFinish, SpanTiles; // per attention width, device
    std::vector<int> CausalPeriod;
    std::vector<int> SpanParts, SpanPartCapacity; // per width: spans per row of the batch set, and what the arrays hold
    void ReserveSpans(int k, int parts);
    float *State = nullptr, *RopeBuf = nullptr, *Prediction = nullptr;

    const uint8_t *ComputeForward(void *stream); // returns NormalizeState of the final state (device)

  public:
    // model: device copies of the int8 matrices, one TAttentionMatrices per layer; layerWidthId[d] in
    // [0, attentionWidthCount).  maxLabelsPerNode bounds LabelPtr[i + 1] - LabelPtr[i].
    TComputeContext(tsattn_handle_t handle, const TModelDims &dims, const TInferModel &model, const std::vector<int> &layerWidthId,
                    int attentionWidthCount, int maxNodeCount, int maxLabelsPerNode = 1);
    ~TComputeContext();
    TComputeContext(const TComputeContext &) = delete;
    TComputeContext &operator=(const TComputeContext &) = delete;

    int GetDeviceCount() const { return 1; }
    const TModelDims &GetModelDims() const { return Dims; }
    TNodesBatch &GetNodes(int deviceId);
    void Init(int deviceId, EInitType initType);
    void ComputeFinalStateVectors(std::vector<std::vector<float>> *pStateVectors);
    void ComputeFragmentPredictions(std::vector<std::vector<float>> *pPrediction);
    void ComputeFragmentPredictions(std::vector<float> *pPrediction);
    float ComputeScore();
};

} // namespace NTsAttn
