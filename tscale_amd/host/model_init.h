// Host-side set-up of a TScale model for the int8 inference path: the per-layer attention schedule, a random model,
// and the conversion of its float matrices to int8 with their scales.
//
//   reference                                                          here
//   InitAlibi, TModelDescr::AddLayer   gpt/model_params/model_dim.cpp:55-97, model_dim.h:83-117   NTsAttn::InitAlibi
//   TFastNormalRNG, InitMatrixNormal   gpt/model_params/model_params.cpp:7-45                      NTsAttn::TFastNormalRng, InitMatrixNormal
//   InitEmbedMatrix, InitAttention, InitModel   gpt/model_params/model_params.cpp:47-151           NTsAttn::InitModel
//   ConvertMatrix, ConvertAtt, ConvertModel     gpt/train/cpu_infer.cpp:94-161                      NTsAttn::ConvertMatrix, ConvertModel
//
// Pure host code (no device calls).  The random numbers are this repository's own (splitmix64 + Box-Muller where the
// reference has MT19937 + the polar method): same distribution and the same table-of-65536 structure, other values.
#pragma once

#include <stdint.h>

#include <vector>

namespace NTsAttn {

enum EAlibi { ALIBI_NONE = 0, ALIBI_V3 = 1, ALIBI_ABS_POS_ENCODING = 2 };

struct TAttentionPosParams {
    float AlibiSlope = 0;
    int AttentionWidthId = 0;
    TAttentionPosParams() {}
    TAttentionPosParams(float slope, int id) : AlibiSlope(slope), AttentionWidthId(id) {}
};

// The part of TModelDescr the attention path reads: the table of widths and every layer's (slope, width id).
struct TLayerSchedule {
    std::vector<int> AttentionWidthArr;
    std::vector<TAttentionPosParams> Layers;
    int GetAttentionWidth(int layer) const { return AttentionWidthArr[Layers[layer].AttentionWidthId]; }
    float GetAlibiSlope(int layer) const { return Layers[layer].AlibiSlope; }
};

void InitAlibi(TLayerSchedule *p, EAlibi alibi, int depth, int wideLimitWindow);

constexpr float MODEL_DISCR_SCALE = 1.0f / 32; // gpt/model_params/model_dim.h:9
constexpr int NOISE_LABELS_COUNT = 32;         // gpt/model_params/model_dim.h:15 (labels whose embedding starts at zero)

// 65536 normal values in pairs (x, -x); Gen() picks one by 16 random bits.
struct TFastNormalRng {
    enum { BUF_SIZE = 1 << 16 };
    std::vector<float> Buf;
    uint64_t State;
    explicit TFastNormalRng(uint64_t seed);
    uint32_t GenRand();
    float Gen() { return Buf[GenRand() & (BUF_SIZE - 1)]; }
};

// data[y][x] = rng.Gen() * sko * 0.5, y < ySize, x < xSize (row-major, one row per output)
void InitMatrixNormal(float *data, int64_t xSize, int64_t ySize, TFastNormalRng &rng, float sko);

enum ECombinerInit { COMBINER_INIT_RANDOM = 0, COMBINER_INIT_ZERO = 1 };

// int8 = round-to-nearest-even(value / (rms * MODEL_DISCR_SCALE)) clamped to [-127, 127]; returns rms * MODEL_DISCR_SCALE
// (0 for an all-zero matrix, whose int8 form is all zero).
float ConvertMatrix(const float *data, int64_t xSize, int64_t ySize, int8_t *dst);

struct THostAttention {                       // one layer, int8, one row per output
    std::vector<int8_t> QK, QV, K, V;          // [HeadCount*QDim][Dim]
    std::vector<int8_t> Combiner;              // [Dim][HeadCount*TTDim*4]
    std::vector<int8_t> Expand, Contract;      // [ReluDim][Dim], [Dim][ReluDim]
    float QVScale = 0, VScale = 0, CombinerScale = 0, ContractScale = 0;
    int AttentionWidth = 0;
    float AlibiSlope = 0;
};

struct THostModel {                            // TCPUModelParams of the reference, on the host
    int Dim = 0, QDim = 0, TTDim = 0, HeadCount = 0, ReluMult = 1;
    int ReluDim = 0;                           // HeadCount * 128 * ReluMult whatever the head width (gpt/model_params/model_dim.h:66)
    int64_t LabelCount = 0, VocabSize = 0;
    std::vector<int8_t> LabelEmbed, FinalLayer; // [LabelCount][Dim], [VocabSize][Dim]
    float LabelEmbedScale = 0, FinalLayerScale = 0;
    std::vector<THostAttention> LayerArr;
    std::vector<float> Bias;
    int BaseLabel = 1 + NOISE_LABELS_COUNT;
};

// InitModel followed by ConvertModel, matrix by matrix (the float form of one matrix at a time is all that is held).
// combinerInit: the reference's create_model() starts combiner and contract at zero, which cuts the attention output off
// from the result; a random-init model that is to exercise attention uses COMBINER_INIT_RANDOM, as the reference's own
// CPU/GPU comparison does (gpt/train/main_gpt.cpp:274).
// reluMult: the feed-forward block's width in units of 128 per head (TModelDims::ReluMult).
void InitModel(THostModel *p, uint64_t seed, int dim, int headCount, int headDim, int reluMult, int depth, int wideLimitWindow,
               int64_t labelCount, int64_t vocabSize, ECombinerInit combinerInit);

} // namespace NTsAttn

// The same through a C ABI (libtshost.so), for callers that are not C++.
extern "C" {
// Every layer's attention width and ALiBi slope.  Returns the number of layers the schedule has -- depth rounded up to
// an even number for ALIBI_V3, whose layers come in pairs (gpt/model_params/model_dim.cpp:63-79) -- and writes the first
// min(that, capacity) of them; call with capacity 0 to ask for the count.
int tshost_init_alibi(int alibi, int depth, int wide_limit_window, int *widths, float *slopes, int capacity);
// the sizes InitModel gives the matrices of one layer: {QK, QV, K, V} rows x cols, Combiner, Expand, Contract (rows, cols each)
void tshost_init_model_shapes(int dim, int head_count, int head_dim, int relu_mult, int64_t shapes[7][2]);
float tshost_convert_matrix(const float *data, int64_t x_size, int64_t y_size, int8_t *dst);
// data[y_size][x_size] floats as InitMatrixNormal makes them from a generator seeded with `seed`
void tshost_init_matrix_normal(uint64_t seed, float sko, int64_t x_size, int64_t y_size, float *data);
// int8 matrix + scale of InitMatrixNormal + ConvertMatrix, n_matrices of them from one generator, one after the other in dst
void tshost_random_int8_matrices(uint64_t seed, float sko, int64_t x_size, int64_t y_size, int n_matrices, int8_t *dst, float *scales);
}
