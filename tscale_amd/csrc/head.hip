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
// the largest w.  A row is 200 KB of sums and as much bias for one CU, and what a CU gets per microsecond is what it
// has in flight: 1024 threads, four requests of 16 bytes (rows start at any multiple of 4 bytes) per thread and round,
// so that a pass is two rounds of memory latency and not two hundred.
constexpr int SM_THREADS = 1024;
constexpr int SM_U = 4;
typedef int v4i_any __attribute__((ext_vector_type(4), aligned(4)));
typedef float v4f_any __attribute__((ext_vector_type(4), aligned(4)));

__device__ inline float softmax_logit(const HeadParams &p, int64_t row, int64_t k)
{
    int v = p.src[row * p.src_pitch + k];
    for (int pl = 1; pl < p.src_planes; ++pl) v += p.src[pl * p.src_plane_stride + row * p.src_pitch + k];
    const float w = (float)v * p.scale;
    return p.bias ? w + p.bias[k] : w;
}

// the same for k .. k + 3
__device__ inline v4f softmax_logit4(const HeadParams &p, int64_t row, int64_t k)
{
    v4i v = *(const v4i_any *)(p.src + row * p.src_pitch + k);
    for (int pl = 1; pl < p.src_planes; ++pl) v += *(const v4i_any *)(p.src + pl * p.src_plane_stride + row * p.src_pitch + k);
    v4f w = v4f{(float)v.x * p.scale, (float)v.y * p.scale, (float)v.z * p.scale, (float)v.w * p.scale};
    if (p.bias) {
        const v4f b = *(const v4f_any *)(p.bias + k);
        w = v4f{w.x + b.x, w.y + b.y, w.z + b.z, w.w + b.w};
    }
    return w;
}

// Walks a row: groups of four from the front, SM_U requests per thread out before the first is used (none under a
// branch: a group past the end asks for the last whole group again), then the up to three values that are left.
template <typename F>
__device__ inline void softmax_walk(const HeadParams &p, int64_t row, int tid, F &&f)
{
    const int64_t n4 = p.n & ~(int64_t)3;
    for (int64_t base = 0; base < n4; base += 4 * SM_THREADS * SM_U) {
        v4f w[SM_U];
#pragma unroll
        for (int u = 0; u < SM_U; ++u) {
            const int64_t k = base + 4 * (tid + (int64_t)u * SM_THREADS);
            w[u] = softmax_logit4(p, row, k < n4 ? k : n4 - 4);
        }
#pragma unroll
        for (int u = 0; u < SM_U; ++u) {
            const int64_t k = base + 4 * (tid + (int64_t)u * SM_THREADS);
            if (k < n4) { f(k, w[u].x); f(k + 1, w[u].y); f(k + 2, w[u].z); f(k + 3, w[u].w); }
        }
    }
    if (n4 + tid < p.n) f(n4 + tid, softmax_logit(p, row, n4 + tid));
}

__global__ __launch_bounds__(SM_THREADS) void softmax_rows_kernel(HeadParams p)
{
    __shared__ float s_max[SM_THREADS / WAVE];
    __shared__ int s_arg[SM_THREADS / WAVE];
    __shared__ float s_sum[SM_THREADS / WAVE];
    const int64_t row = blockIdx.x;
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wave = tid / WAVE;
    // pass 1: maximum and where it is first reached (a thread sees its k in ascending order)
    float best = -INFINITY;
    int arg = 0x7fffffff;
    softmax_walk(p, row, tid, [&](int64_t k, float w) {
        if (w > best) { best = w; arg = (int)k; }
    });
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
    softmax_walk(p, row, tid, [&](int64_t, float w) { sum += fast_exp2(fmaxf(w - M, -127.0f)); });
    for (int o = 32; o > 0; o >>= 1) sum += __shfl_xor(sum, o, WAVE);
    if (lane == 0) s_sum[wave] = sum;
    __syncthreads();
    sum = 0.0f;
    for (int w = 0; w < SM_THREADS / WAVE; ++w) sum += s_sum[w];
    const float inv = 1.0f / sum;
    // pass 3: the probabilities
    float *const prob = p.prob + row * p.prob_pitch;
    softmax_walk(p, row, tid, [&](int64_t k, float w) { prob[k] = fast_exp2(fmaxf(w - M, -127.0f)) * inv; });
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
    auto take = [&](int64_t k, float prob, uint32_t r) {
        const double u = ((double)r + 0.5) * (1.0 / 4294967296.0);
        const float score = (float)((double)(logf(prob) / p.temperature) - log(-log(u)));
        if (score > best) { best = score; arg = (int)k; }
    };
    // groups of four from the front (16-byte requests, all of a round out before the first is used; a thread sees its k
    // in ascending order), then the up to three values that are left
    const float *const prob = p.prob + row * p.prob_pitch;
    const uint32_t *const rnd = p.rnd ? p.rnd + row * p.rnd_pitch : nullptr;
    const int64_t n4 = p.n & ~(int64_t)3;
    for (int64_t base = 0; base < n4; base += 4 * SM_THREADS * SM_U) {
        v4f q[SM_U];
        v4i r[SM_U];
#pragma unroll
        for (int u = 0; u < SM_U; ++u) {
            const int64_t k = base + 4 * (tid + (int64_t)u * SM_THREADS), kc = k < n4 ? k : n4 - 4;
            q[u] = *(const v4f_any *)(prob + kc);
            r[u] = rnd ? (v4i)*(const v4i_any *)(rnd + kc) : v4i{0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < SM_U; ++u) {
            const int64_t k = base + 4 * (tid + (int64_t)u * SM_THREADS);
            if (k >= n4) continue;
            const float qq[4] = {q[u].x, q[u].y, q[u].z, q[u].w};
            const int rr[4] = {r[u].x, r[u].y, r[u].z, r[u].w};
#pragma unroll
            for (int j = 0; j < 4; ++j)
                take(k + j, qq[j], rnd ? (uint32_t)rr[j] : mix32(p.seed, p.offset + (uint64_t)(row * p.n + k + j)));
        }
    }
    if (n4 + tid < p.n) {
        const int64_t k = n4 + tid;
        take(k, prob[k], rnd ? rnd[k] : mix32(p.seed, p.offset + (uint64_t)(row * p.n + k)));
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
