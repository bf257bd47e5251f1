// Thin C wrapper around the reference's OWN mask, layer-schedule and e4m3 code, compiled from the
// reference checkout where it lies (see build_ref.sh).  Test infrastructure only: it validates the
// restatements in tsattn_oracle.c.  Only the reference files that build without the CUDA SDK are
// used; gpt/compute/gpt_cpu.cpp and gpt/train/cpu_infer.cpp (the attention arithmetic itself) need
// cuda_runtime.h through lib/cuda/cuda_arrays.h and are therefore not part of this library.
#include <util/eden_core.h>
#include <util/fp8.h>
#include <gpt/att/sliding_window.h>
#include <gpt/att/att.h>
#include <gpt/data/data.h>
#include <gpt/model_params/model_dim.h>
#include <gpt/att/rope.h>

extern "C" {

// InitModelDescr + InitAlibi (gpt/model_params/model_dim.cpp:55-120): per-layer window width and slope
int ref_layer_schedule(const char *descr, int max_layers, long long *width, float *slope)
{
    TModelDescr md;
    InitModelDescr(&md, descr, ALIBI_V3, 1000, 0);
    int n = (int)YSize(md.Layers);
    for (int i = 0; i < n && i < max_layers; ++i) {
        width[i] = md.AttentionWidthArr[md.Layers[i].AttentionWidthId];
        slope[i] = md.Layers[i].AlibiSlope;
    }
    return n;
}

// InitLabelData / GenerateAttentionGraph (gpt/att/sliding_window.cpp:91-290) on fragments given as
// token arrays; returns per node the first span of window `width_id` and the number of spans.
int ref_spans(const char *descr, int n_frag, const int *frag_len, const int *tokens, int doc_start_token,
              int width_id, int *span_start, int *span_finish, int *span_count)
{
    TModelDescr md;
    InitModelDescr(&md, descr, ALIBI_V3, 1000, 0);
    if (doc_start_token >= 0) {
        md.SetDocStartToken(doc_start_token);
    }
    TVector<TFragment> frags;
    int ptr = 0;
    for (int f = 0; f < n_frag; ++f) {
        TFragment fr;
        fr.Offset = ptr;
        for (int t = 0; t < frag_len[f]; ++t) {
            fr.Text.push_back(tokens[ptr + t]);
        }
        ptr += frag_len[f];
        frags.push_back(fr);
    }
    TNodesBatch nodes;
    InitLabelData(md, NopRng, 1., frags, ATT_GRAPH_TEST_LOSS, &nodes);
    if (width_id < 0 || width_id >= (int)YSize(nodes.AttArr)) {
        return -1;
    }
    const TAttentionInfo &att = nodes.AttArr[width_id];
    int n = (int)att.GetSampleCount();
    for (int i = 0; i < n; ++i) {
        int a = att.SpanPtr[i], b = att.SpanPtr[i + 1];
        span_count[i] = b - a;
        if (b > a) {
            span_start[i] = att.Spans[a].Start;
            span_finish[i] = att.Spans[a].Finish;
        } else {
            span_start[i] = i;
            span_finish[i] = i - 1;
        }
    }
    return n;
}

// GroupAttention<64,128> (gpt/att/att.h:95-181): the reference's tile-skip list for one-span rows.
// Returns the number of groups; group g of 64-row block b covers keys [start, finish] (aligned to 128).
int ref_group_attention(int n_rows, const int *span_start, const int *span_finish, int max_groups,
                        int *group_block, int *group_start, int *group_finish)
{
    TAttentionInfo att;
    att.Init();
    for (int i = 0; i < n_rows; ++i) {
        if (span_finish[i] >= span_start[i]) {
            att.AddSpan(TAttentionSpan(span_start[i], span_finish[i]));
        }
        att.AddSample();
    }
    TAttentionInfoGrouped<64> grouped;
    GroupAttention<64, 128>(att, &grouped);
    int n = 0;
    for (yint b = 0; b < grouped.GetGroupCount(); ++b) {
        for (int k = grouped.SpanGroupPtr[b]; k < grouped.SpanGroupPtr[b + 1]; ++k) {
            if (n < max_groups) {
                group_block[n] = (int)b;
                group_start[n] = grouped.SpanGroups[k].Start;
                group_finish[n] = grouped.SpanGroups[k].Finish;
            }
            ++n;
        }
    }
    return n;
}

// util/fp8.h:4-21
float ref_e4m3_to_float(int code) { return ConvertE4toFloat((i8)code); }

// constants of gpt/model_params/model_dim.h:19-33 as the reference's preprocessor sees them
float ref_att_dot_scale(int dim) { return CalcDotScale(dim) * CalcAttentionMult(); }
float ref_attention_decay(int dist, float slope) { return GetAttentionDecay(dist, slope); }


// FillRopeBuf (gpt/att/rope.cpp:4-24): rope[t][x], row-major [max_len][width]
void ref_fill_rope(int width, long long max_len, float *rope)
{
    TArray2D<float> buf;
    FillRopeBuf(&buf, width, max_len);
    for (long long t = 0; t < max_len; ++t) {
        for (int x = 0; x < width; ++x) {
            rope[t * width + x] = buf[t][x];
        }
    }
}

// ApplyRope (gpt/att/rope.cpp:48-53) on one vector of `dim` floats at position t
void ref_apply_rope(int width, long long max_len, float rotate_dir, long long t, int dim, float *vec)
{
    TArray2D<float> buf;
    FillRopeBuf(&buf, width, max_len);
    TVector<float> v;
    for (int i = 0; i < dim; ++i) {
        v.push_back(vec[i]);
    }
    ApplyRope(buf, rotate_dir, t, &v);
    for (int i = 0; i < dim; ++i) {
        vec[i] = v[i];
    }
}
}
