#include "model_init.h"

#include <math.h>
#include <stdio.h>
#include <stdlib.h>

#include <algorithm>

namespace NTsAttn {

// gpt/model_params/model_dim.cpp:55-97
void InitAlibi(TLayerSchedule *p, EAlibi alibi, int depth, int wideLimitWindow)
{
    p->AttentionWidthArr.clear();
    p->Layers.assign(depth, TAttentionPosParams());
    if (depth == 1) { // the attention-profiling model: one wide layer with a small slope
        p->AttentionWidthArr.push_back(wideLimitWindow);
        p->Layers[0] = TAttentionPosParams(0.1f, 0);
        return;
    }
    if (alibi == ALIBI_NONE) {
        p->AttentionWidthArr.assign(1, 0);
    } else if (alibi == ALIBI_ABS_POS_ENCODING) {
        p->AttentionWidthArr.assign(1, wideLimitWindow);
    } else if (alibi == ALIBI_V3) {
        const int widths[4] = {0, 1, 64, wideLimitWindow};
        p->AttentionWidthArr.assign(widths, widths + 4);
        p->Layers.clear();
        if (depth > 0) {
            const int groupCount = (depth + 1) / 2;
            const int w1count = std::max(1, groupCount / 6);
            for (int k = 0; k < w1count; ++k) {
                p->Layers.push_back(TAttentionPosParams(0, 1));
                p->Layers.push_back(TAttentionPosParams(0, 1));
            }
            for (int k = w1count; k < groupCount; ++k) {
                p->Layers.push_back(TAttentionPosParams(0.5f, 2));
                p->Layers.push_back(TAttentionPosParams(0, 3));
            }
        }
    } else {
        fprintf(stderr, "InitAlibi: unknown alibi version %d\n", (int)alibi);
        abort();
    }
}

static uint64_t SplitMix(uint64_t &s)
{
    uint64_t z = (s += 0x9E3779B97F4A7C15ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

TFastNormalRng::TFastNormalRng(uint64_t seed) : Buf(BUF_SIZE), State(seed)
{
    for (int k = 0; k < BUF_SIZE; k += 2) {
        const double u1 = ((SplitMix(State) >> 11) + 0.5) / 9007199254740992.0, u2 = ((SplitMix(State) >> 11) + 0.5) / 9007199254740992.0;
        const float val = (float)(sqrt(-2 * log(u1)) * cos(6.283185307179586 * u2));
        Buf[k] = val;
        Buf[k + 1] = -val;
    }
}

uint32_t TFastNormalRng::GenRand() { return (uint32_t)(SplitMix(State) >> 32); }

// gpt/model_params/model_params.cpp:33-45
void InitMatrixNormal(float *data, int64_t xSize, int64_t ySize, TFastNormalRng &rng, float sko)
{
    const float bound = sko * 0.5f;
    for (int64_t i = 0; i < xSize * ySize; ++i) data[i] = rng.Gen() * bound;
}

static int8_t ConvertToInt8(float x)
{
    const float r = nearbyintf(x); // the reference rounds with cvtss2si: to nearest, ties to even
    return (int8_t)std::min(127.0f, std::max(-127.0f, r));
}

// gpt/train/cpu_infer.cpp:94-121
float ConvertMatrix(const float *data, int64_t xSize, int64_t ySize, int8_t *dst)
{
    float sum2 = 0;
    for (int64_t i = 0; i < xSize * ySize; ++i) sum2 += data[i] * data[i];
    const float sko = sqrtf(sum2 / (xSize * ySize));
    const float discrScale = sko * MODEL_DISCR_SCALE;
    const float mult = (sko == 0) ? 0 : (1 / discrScale);
    for (int64_t i = 0; i < xSize * ySize; ++i) dst[i] = ConvertToInt8(data[i] * mult);
    return discrScale;
}

static float RandomInt8(std::vector<int8_t> *dst, std::vector<float> &tmp, int64_t xSize, int64_t ySize, TFastNormalRng &rng, float sko)
{
    tmp.resize(xSize * ySize);
    InitMatrixNormal(tmp.data(), xSize, ySize, rng, sko);
    dst->resize(xSize * ySize);
    return ConvertMatrix(tmp.data(), xSize, ySize, dst->data());
}

// gpt/model_params/model_params.cpp:47-151 (InitEmbedMatrix, InitAttention, InitModel) + gpt/train/cpu_infer.cpp:128-161
void InitModel(THostModel *p, uint64_t seed, int dim, int headCount, int headDim, int reluMult, int depth, int wideLimitWindow,
               int64_t labelCount, int64_t vocabSize, ECombinerInit combinerInit)
{
    TFastNormalRng rng(seed);
    std::vector<float> tmp;
    p->Dim = dim, p->QDim = headDim, p->TTDim = headDim, p->HeadCount = headCount, p->ReluMult = reluMult;
    p->ReluDim = headCount * 128 * reluMult; // TModelDims::GetReluDim, gpt/model_params/model_dim.h:66
    p->LabelCount = labelCount, p->VocabSize = vocabSize;
    // embedding: plain table values (not halved), the noise labels' rows zero
    tmp.assign((size_t)labelCount * dim, 0.0f);
    for (int64_t y = NOISE_LABELS_COUNT; y < labelCount; ++y)
        for (int x = 0; x < dim; ++x) tmp[y * dim + x] = rng.Gen();
    p->LabelEmbed.resize((size_t)labelCount * dim);
    p->LabelEmbedScale = ConvertMatrix(tmp.data(), dim, labelCount, p->LabelEmbed.data());
    p->FinalLayerScale = RandomInt8(&p->FinalLayer, tmp, dim, vocabSize, rng, 1);
    TLayerSchedule sched;
    InitAlibi(&sched, ALIBI_V3, depth, wideLimitWindow);
    p->LayerArr.resize(sched.Layers.size());
    const int qSum = headCount * headDim;
    const float outSko = combinerInit == COMBINER_INIT_RANDOM ? 1.0f : 0.0f;
    for (size_t d = 0; d < p->LayerArr.size(); ++d) {
        THostAttention &a = p->LayerArr[d];
        RandomInt8(&a.QK, tmp, dim, qSum, rng, 1);
        a.QVScale = RandomInt8(&a.QV, tmp, dim, qSum, rng, 1);
        RandomInt8(&a.K, tmp, dim, qSum, rng, 1);
        a.VScale = RandomInt8(&a.V, tmp, dim, qSum, rng, 1);
        a.CombinerScale = RandomInt8(&a.Combiner, tmp, (int64_t)qSum * 4, dim, rng, outSko);
        a.ContractScale = RandomInt8(&a.Contract, tmp, p->ReluDim, dim, rng, outSko);
        RandomInt8(&a.Expand, tmp, dim, p->ReluDim, rng, 1);
        a.AttentionWidth = sched.GetAttentionWidth((int)d);
        a.AlibiSlope = sched.GetAlibiSlope((int)d);
    }
    p->Bias.assign(vocabSize, 0.0f);
}

} // namespace NTsAttn

extern "C" {

int tshost_init_alibi(int alibi, int depth, int wide_limit_window, int *widths, float *slopes, int capacity)
{
    NTsAttn::TLayerSchedule s;
    NTsAttn::InitAlibi(&s, (NTsAttn::EAlibi)alibi, depth, wide_limit_window);
    for (size_t d = 0; d < s.Layers.size() && (int)d < capacity; ++d) {
        widths[d] = s.GetAttentionWidth((int)d);
        slopes[d] = s.GetAlibiSlope((int)d);
    }
    return (int)s.Layers.size();
}

void tshost_init_model_shapes(int dim, int head_count, int head_dim, int relu_mult, int64_t shapes[7][2])
{
    // a model of one layer and the smallest tables: only the layer's matrix sizes are looked at
    NTsAttn::THostModel m;
    NTsAttn::InitModel(&m, 1, dim, head_count, head_dim, relu_mult, 1, 64, NTsAttn::NOISE_LABELS_COUNT + 1, 1, NTsAttn::COMBINER_INIT_RANDOM);
    const NTsAttn::THostAttention &a = m.LayerArr[0];
    const int64_t q_sum = (int64_t)head_count * head_dim;
    const std::vector<int8_t> *mats[7] = {&a.QK, &a.QV, &a.K, &a.V, &a.Combiner, &a.Expand, &a.Contract};
    const int64_t cols[7] = {dim, dim, dim, dim, q_sum * 4, dim, m.ReluDim};
    for (int i = 0; i < 7; ++i) {
        shapes[i][1] = cols[i];
        shapes[i][0] = (int64_t)mats[i]->size() / cols[i];
    }
}

float tshost_convert_matrix(const float *data, int64_t x_size, int64_t y_size, int8_t *dst) { return NTsAttn::ConvertMatrix(data, x_size, y_size, dst); }

void tshost_init_matrix_normal(uint64_t seed, float sko, int64_t x_size, int64_t y_size, float *data)
{
    NTsAttn::TFastNormalRng rng(seed);
    NTsAttn::InitMatrixNormal(data, x_size, y_size, rng, sko);
}

void tshost_random_int8_matrices(uint64_t seed, float sko, int64_t x_size, int64_t y_size, int n_matrices, int8_t *dst, float *scales)
{
    NTsAttn::TFastNormalRng rng(seed);
    std::vector<float> tmp((size_t)x_size * y_size);
    for (int m = 0; m < n_matrices; ++m) {
        NTsAttn::InitMatrixNormal(tmp.data(), x_size, y_size, rng, sko);
        scales[m] = NTsAttn::ConvertMatrix(tmp.data(), x_size, y_size, dst + (size_t)m * x_size * y_size);
    }
}
}
