// The two ends of the int8 inference path around the layers (ComputePrediction, gpt/train/cpu_infer.cpp:552-582):
// the embedding sum that makes the first state, and the softmax over the final layer's products with the greedy
// choice of the next token; and the sampled choice (SampleFromDistr, :585-599).
#include "common.hpp"
#include "kernels.hpp"

namespace tsattn {

#pragma clang fp contract(off)

// state[row][x] = sum over the row's labels of embed[label][x] * scale, added in label order starting from 0
// (cpu_infer.cpp:559-565).  One thread per 16 consecutive x.
__global__ __launch_bounds__(256) void embed_rows_kernel(HeadParams p)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int chunks = p.dim / 16;
    if (i >= p.n_rows * chunks) return;
    const int64_t row = i / chunks;
    const int x0 = (int)(i - row * chunks) * 16;
    float acc[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) acc[j] = 0.0f;
    for (int l = 0; l < p.labels_per_row; ++l) {
        const int label = p.labels[row * p.labels_per_row + l];
        if (label < 0 || label >= p.n_labels) continue; // an empty slot
        const v4i w = *(const v4i *)(p.embed + (int64_t)label * p.embed_pitch + x0);
        const int ww[4] = {w.x, w.y, w.z, w.w};
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const int8_t e = (int8_t)((ww[j / 4] >> (8 * (j % 4))) & 0xff);
            acc[j] = acc[j] + (float)e * p.embed_scale;
        }
    }
    float *o = p.state + row * p.state_pitch + x0;
#pragma unroll
    for (int j = 0; j < 16; j += 4) *(v4f *)(o + j) = v4f{acc[j], acc[j + 1], acc[j + 2], acc[j + 3]};
}

// One workgroup per row.  w[k] = vec[k] * scale + bias[k]; M = max(0, max w) (the buffer's maximum starts at 0,
// cpu_infer.cpp:226-244); p[k] = 2^(w[k] - M) / sum (base 2: the scale carries 1/ln 2).  The choice is the first k of
// the largest w.  A row is 200 KB of sums and as much bias for one workgroup: 1024 threads, eight independent
// requests per thread and round, so that a pass is a handful of memory round trips and not two hundred.
constexpr int SM_THREADS = 1024;
constexpr int SM_U = 8;

__device__ inline float softmax_logit(const HeadParams &p, int64_t row, int64_t k)
{
    int v = p.src[row * p.src_pitch + k];
    for (int pl = 1; pl < p.src_planes; ++pl) v += p.src[pl * p.src_plane_stride + row * p.src_pitch + k];
    const float w = (float)v * p.scale;
    return p.bias ? w + p.bias[k] : w;
}

__global__ __launch_bounds__(SM_THREADS) void softmax_rows_kernel(HeadParams p)
{
    __shared__ float s_max[SM_THREADS / WAVE];
    __shared__ int s_arg[SM_THREADS / WAVE];
    __shared__ float s_sum[SM_THREADS / WAVE];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    // pass 1: maximum and where it is first reached
    float best = -INFINITY;
    int arg = 0x7fffffff;
    for (int64_t k0 = tid; k0 < p.n; k0 += SM_U * SM_THREADS) {
        float w[SM_U];
#pragma unroll
        for (int u = 0; u < SM_U; ++u) {
            const int64_t k = k0 + u * SM_THREADS;
            w[u] = k < p.n ? softmax_logit(p, row, k) : -INFINITY;
        }
#pragma unroll
        for (int u = 0; u < SM_U; ++u) // (ascending k: the first of equal values stays)
            if (w[u] > best) { best = w[u]; arg = (int)(k0 + u * SM_THREADS); }
    }
    for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, WAVE);
        const int oa = __shfl_xor(arg, o, WAVE);
        if (ob > best || (ob == best && oa < arg)) { best = ob; arg = oa; }
    }
    if (lane == 0) { s_max[wave] = best; s_arg[wave] = arg; }
    __syncthreads();
    best = s_max[0]; arg = s_arg[0];
    for (int w = 1; w < SM_THREADS / WAVE; ++w) {
        if (s_max[w] > best || (s_max[w] == best && s_arg[w] < arg)) { best = s_max[w]; arg = s_arg[w]; }
    }
    if (tid == 0 && p.argmax) p.argmax[row] = arg;
    if (!p.prob) return;
    const float M = fmaxf(0.0f, best);
    // pass 2: sum of the weights
    float sum = 0.0f;
    for (int64_t k0 = tid; k0 < p.n; k0 += SM_U * SM_THREADS) {
        float w[SM_U];
#pragma unroll
        for (int u = 0; u < SM_U; ++u) {
            const int64_t k = k0 + u * SM_THREADS;
            w[u] = k < p.n ? softmax_logit(p, row, k) : -INFINITY;
        }
#pragma unroll
        for (int u = 0; u < SM_U; ++u)
            if (k0 + u * SM_THREADS < p.n) sum += fast_exp2(fmaxf(w[u] - M, -127.0f));
    }
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, WAVE);
    if (lane == 0) s_sum[wave] = sum;
    __syncthreads();
    sum = 0.0f;
    for (int w = 0; w < SM_THREADS / WAVE; ++w) sum += s_sum[w];
    const float inv = 1.0f / sum;
    // pass 3: the probabilities
    for (int64_t k0 = tid; k0 < p.n; k0 += SM_U * SM_THREADS) {
        float w[SM_U];
#pragma unroll
        for (int u = 0; u < SM_U; ++u) {
            const int64_t k = k0 + u * SM_THREADS;
            w[u] = k < p.n ? softmax_logit(p, row, k) : -INFINITY;
        }
#pragma unroll
        for (int u = 0; u < SM_U; ++u) {
            const int64_t k = k0 + u * SM_THREADS;
            if (k < p.n) p.prob[row * p.prob_pitch + k] = fast_exp2(fmaxf(w[u] - M, -127.0f)) * inv;
        }
    }
}


// SampleFromDistr (cpu_infer.cpp:585-599), the Gumbel-max choice, one workgroup per row:
// score[k] = (float)(logf(prob[k]) / temperature - log(-log(u))), u = (r + 0.5) / 2^32 in double (GenRandReal3 of the
// reference's 32-bit generator); the first k of the largest score above -1e38, else 0.  r: the caller's words, or a
// 64-bit mix of (seed, offset + row * n + k), the output function of splitmix64 on a counter.
__device__ inline uint32_t mix32(uint64_t seed, uint64_t index)
{
    uint64_t z = seed + (index + 1) * 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (uint32_t)(z >> 32);
}

__global__ __launch_bounds__(SM_THREADS) void sample_rows_kernel(HeadParams p)
{
    __shared__ float s_max[SM_THREADS / WAVE];
    __shared__ int s_arg[SM_THREADS / WAVE];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    float best = -1e38f;
    int arg = 0x7fffffff;
    for (int64_t k = tid; k < p.n; k += SM_THREADS) {
        const uint32_t r = p.rnd ? p.rnd[row * p.rnd_pitch + k] : mix32(p.seed, p.offset + (uint64_t)(row * p.n + k));
        const double u = ((double)r + 0.5) * (1.0 / 4294967296.0);
        const float score = (float)((double)(logf(p.prob[row * p.prob_pitch + k]) / p.temperature) - log(-log(u)));
        if (score > best) { best = score; arg = (int)k; }
    }
    for (int o = 32; o > 0; o >>= 1) {
        const float ob = __shfl_xor(best, o, WAVE);
        const int oa = __shfl_xor(arg, o, WAVE);
        if (ob > best || (ob == best && oa < arg)) { best = ob; arg = oa; }
    }
    if (lane == 0) { s_max[wave] = best; s_arg[wave] = arg; }
    __syncthreads();
    if (tid == 0) {
        for (int w = 1; w < SM_THREADS / WAVE; ++w) {
            if (s_max[w] > best || (s_max[w] == best && s_arg[w] < arg)) { best = s_max[w]; arg = s_arg[w]; }
        }
        p.argmax[row] = arg == 0x7fffffff ? 0 : arg;
    }
}

hipError_t launch_embed_rows(const HeadParams &p, hipStream_t st)
{
    const int64_t n = p.n_rows * (p.dim / 16);
    if (n == 0) return hipSuccess;
    hipLaunchKernelGGL(embed_rows_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, p);
    return hipGetLastError();
}

hipError_t launch_softmax_rows(const HeadParams &p, hipStream_t st)
{
    if (p.n_rows == 0 || p.n == 0) return hipSuccess;
    hipLaunchKernelGGL(softmax_rows_kernel, dim3((unsigned)p.n_rows), dim3(SM_THREADS), 0, st, p);
    return hipGetLastError();
}

hipError_t launch_sample_rows(const HeadParams &p, hipStream_t st)
{
    if (p.n_rows == 0) return hipSuccess;
    hipLaunchKernelGGL(sample_rows_kernel, dim3((unsigned)p.n_rows), dim3(SM_THREADS), 0, st, p);
    return hipGetLastError();
}

} // namespace tsattn
