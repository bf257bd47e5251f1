// Small kernels around the attention path: the absmax row quantiser, the span (window metadata)
// builder, the KV-cache append and the combination of attention results over several spans per row.
#include "common.hpp"
#include "kernels.hpp"

namespace tsattn {

// One wave per (row, head).  scale = absmax/127 (int8) or absmax/256 (e4m3); values times 1/scale,
// rounded to nearest even (lib/cuda/cuda_matmul.cuh:237-249, lib/cuda/cuda_util.cuh:286-297).
template <int SRC, int DST>
__global__ __launch_bounds__(256) void quantize_rows_kernel(const uint8_t *src, int64_t src_pitch, int64_t n_rows, int n_heads,
                                                            int head_dim, uint8_t *dst, int64_t dst_pitch, float *scale,
                                                            int64_t scale_pitch)
{
    const int lane = threadIdx.x & (WAVE - 1);
    const int64_t job = (int64_t)blockIdx.x * (blockDim.x / WAVE) + threadIdx.x / WAVE;
    if (job >= n_rows * n_heads) return;
    const int64_t row = job / n_heads;
    const int head = (int)(job % n_heads);
    const int per = head_dim / WAVE; // head_dim is a multiple of 64, at most 256
    float x[4];
    float amax = 0;
    for (int i = 0; i < per; ++i) {
        int e = head * head_dim + i * WAVE + lane;
        if (SRC == TSATTN_SRC_F32) x[i] = ((const float *)(src + row * src_pitch))[e];
        else x[i] = bf16_to_float(((const uint16_t *)(src + row * src_pitch))[e]);
        amax = fmaxf(amax, fabsf(x[i]));
    }
    amax = wave_max(amax);
    float discr = 0, mult = 0;
    if (amax > 0) {
        discr = (DST == TSATTN_I8) ? amax / 127.0f : amax / 256.0f;
        mult = 1.0f / discr;
    }
    for (int i = 0; i < per; ++i) {
        float y = x[i] * mult;
        uint8_t b = (DST == TSATTN_I8) ? (uint8_t)float_to_i8(y) : float_to_e4m3(y);
        dst[row * dst_pitch + head * head_dim + i * WAVE + lane] = b;
    }
    if (lane == 0) scale[head * scale_pitch + row] = discr;
}

hipError_t launch_quantize_rows(int src_dtype, int dst_dtype, const void *src, int64_t src_pitch, int64_t n_rows,
                                int n_heads, int head_dim, void *dst, int64_t dst_pitch, float *scale,
                                int64_t scale_pitch, hipStream_t st)
{
    int64_t jobs = n_rows * n_heads;
    if (jobs == 0) return hipSuccess;
    dim3 grid((unsigned)((jobs + 3) / 4)), block(256);
#define TSATTN_QR(S, D)                                                                                              \
    hipLaunchKernelGGL((quantize_rows_kernel<S, D>), grid, block, 0, st, (const uint8_t *)src, src_pitch, n_rows,   \
                       n_heads, head_dim, (uint8_t *)dst, dst_pitch, scale, scale_pitch)
    if (src_dtype == TSATTN_SRC_F32 && dst_dtype == TSATTN_I8) TSATTN_QR(TSATTN_SRC_F32, TSATTN_I8);
    else if (src_dtype == TSATTN_SRC_F32 && dst_dtype == TSATTN_E4M3) TSATTN_QR(TSATTN_SRC_F32, TSATTN_E4M3);
    else if (src_dtype == TSATTN_SRC_BF16 && dst_dtype == TSATTN_I8) TSATTN_QR(TSATTN_SRC_BF16, TSATTN_I8);
    else if (src_dtype == TSATTN_SRC_BF16 && dst_dtype == TSATTN_E4M3) TSATTN_QR(TSATTN_SRC_BF16, TSATTN_E4M3);
    else return hipErrorInvalidValue;
#undef TSATTN_QR
    return hipGetLastError();
}

// One thread per token: span = [max(docStart, t - W), t - 1] shifted by the sequence's first token;
// W == 0 means the token itself (gpt/att/sliding_window.cpp:80-87, 213-220).  A flagged token
// starts a document unless it is the first token of its sequence (:150-154).
__global__ __launch_bounds__(256) void build_spans_kernel(int n_seqs, const int32_t *seq_offset, int64_t n_tokens,
                                                          const uint8_t *flag, int64_t window, int32_t *span_start,
                                                          int32_t *span_finish)
{
    const int64_t tok = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (tok >= n_tokens) return;
    int lo = 0, hi = n_seqs; // last sequence whose offset <= tok
    while (hi - lo > 1) {
        int mid = (lo + hi) / 2;
        if (seq_offset[mid] <= tok) lo = mid; else hi = mid;
    }
    const int64_t base = seq_offset[lo];
    const int64_t t = tok - base;
    int64_t a, b;
    if (window == 0) {
        a = t; b = t;
    } else {
        a = t - window;
        if (a < 0) a = 0;
        b = t - 1;
        if (flag) {
            // the latest document start in (a, t] clips the span
            for (int64_t u = t; u > a; --u) {
                if (flag[base + u]) { a = u; break; }
            }
        }
        if (b < a) { a = t; b = t - 1; }
    }
    span_start[tok] = (int32_t)(a + base);
    span_finish[tok] = (int32_t)(b + base);
}

hipError_t launch_build_spans(int n_seqs, const int32_t *seq_offset, int64_t n_tokens, const uint8_t *doc_start_flag,
                              int64_t window, int32_t *span_start, int32_t *span_finish, hipStream_t st)
{
    if (n_tokens == 0) return hipSuccess;
    hipLaunchKernelGGL(build_spans_kernel, dim3((unsigned)((n_tokens + 255) / 256)), dim3(256), 0, st, n_seqs, seq_offset,
                       n_tokens, doc_start_flag, window, span_start, span_finish);
    return hipGetLastError();
}

// Span summary for the prefill kernel: one workgroup of 128 threads per 128 query rows, one wave half (32 lanes)
// per 32-row group.  Rows without keys (span_finish < span_start) and rows past the end do not count.
__global__ __launch_bounds__(128) void span_tiles_kernel(int64_t n_tokens, const int32_t *span_start, const int32_t *span_finish, int32_t *tiles)
{
    __shared__ int red[8];
    const int tid = threadIdx.x;
    const int64_t row = (int64_t)blockIdx.x * 128 + tid;
    int a = 1, b = 0;
    if (row < n_tokens) {
        a = span_start[row];
        b = span_finish[row];
    }
    const bool has = b >= a;
    int min_a = has ? a : 0x7fffffff, max_a = has ? a : -1, min_b = has ? b : 0x7fffffff, max_b = has ? b : -1;
    int all = has ? 1 : 0;
    for (int o = 16; o > 0; o >>= 1) { // within each 32-lane half
        min_a = min(min_a, __shfl_xor(min_a, o, WAVE));
        max_a = max(max_a, __shfl_xor(max_a, o, WAVE));
        min_b = min(min_b, __shfl_xor(min_b, o, WAVE));
        max_b = max(max_b, __shfl_xor(max_b, o, WAVE));
        all &= __shfl_xor(all, o, WAVE);
    }
    int32_t *out = tiles + (int64_t)blockIdx.x * SPAN_TILE_INTS;
    const int grp = tid >> 5;
    if ((tid & 31) == 0) {
        int32_t *w = out + SPAN_TILE_WAVE0 + grp * SPAN_TILE_WAVE_INTS;
        w[0] = min_a; w[1] = max_a; w[2] = min_b; w[3] = max_b; w[4] = all;
        red[grp] = min_a;
        red[4 + grp] = max_b;
    }
    __syncthreads();
    if (tid == 0) {
        out[SPAN_TILE_MIN_A] = min(min(red[0], red[1]), min(red[2], red[3]));
        out[SPAN_TILE_MAX_B] = max(max(red[4], red[5]), max(red[6], red[7]));
        out[2] = 0; out[3] = 0;
        for (int i = SPAN_TILE_WAVE0 + 4 * SPAN_TILE_WAVE_INTS; i < SPAN_TILE_INTS; ++i) out[i] = 0;
    }
}

hipError_t launch_build_span_tiles(int64_t n_tokens, const int32_t *span_start, const int32_t *span_finish, int32_t *tiles, hipStream_t st)
{
    if (n_tokens <= 0) return hipSuccess;
    hipLaunchKernelGGL(span_tiles_kernel, dim3((unsigned)((n_tokens + 127) / 128)), dim3(128), 0, st, n_tokens, span_start, span_finish, tiles);
    return hipGetLastError();
}

// TAttentionVecHistory::AddVectors (gpt/train/cpu_infer.cpp:403-408) for a planar cache: one thread
// copies 16 bytes of the new K and V rows to row cache_len[seq]; a second kernel bumps the lengths.
__global__ __launch_bounds__(256) void cache_append_kernel(AppendParams p, int n_seqs)
{
    const int chunks = p.head_dim / 16;
    const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = (int64_t)n_seqs * p.n_heads * chunks;
    if (id >= total) return;
    const int c = (int)(id % chunks);
    const int head = (int)((id / chunks) % p.n_heads);
    const int seq = (int)(id / ((int64_t)chunks * p.n_heads));
    const int pos = p.cache_len[seq];
    if (pos < 0 || pos >= p.max_len) return;
    const int64_t src = (int64_t)seq * p.new_pitch + head * p.head_dim + c * 16;
    const int64_t dst = (int64_t)seq * p.seq_stride + (int64_t)head * p.head_stride + (int64_t)pos * p.tok_stride + c * 16;
    *(v4i *)(p.k + dst) = *(const v4i *)(p.k_new + src);
    *(v4i *)(p.v + dst) = *(const v4i *)(p.v_new + src);
    if (c == 0) {
        const int64_t sd = (int64_t)seq * p.s_seq_stride + (int64_t)head * p.s_head_stride + pos;
        if (p.ks_new) p.ks[sd] = p.ks_new[seq * p.n_heads + head];
        if (p.vs_new) p.vs[sd] = p.vs_new[seq * p.n_heads + head];
    }
}

__global__ void cache_len_bump_kernel(int32_t *cache_len, int n_seqs, int max_len)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n_seqs && cache_len[i] >= 0 && cache_len[i] < max_len) cache_len[i] += 1;
}

__global__ void zero_i32_kernel(int32_t *p, int n)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0;
}

hipError_t launch_zero_i32(int32_t *p, int n, hipStream_t st)
{
    if (n <= 0) return hipSuccess;
    hipLaunchKernelGGL(zero_i32_kernel, dim3((n + 255) / 256), dim3(256), 0, st, p, n);
    return hipGetLastError();
}

hipError_t launch_cache_append(const AppendParams &p, int n_seqs, hipStream_t st)
{
    if (n_seqs == 0) return hipSuccess;
    const int64_t total = (int64_t)n_seqs * p.n_heads * (p.head_dim / 16);
    hipLaunchKernelGGL(cache_append_kernel, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, st, p, n_seqs);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(cache_len_bump_kernel, dim3((unsigned)((n_seqs + 255) / 256)), dim3(256), 0, st, p.cache_len, n_seqs, p.max_len);
    return hipGetLastError();
}

// Bulk form of the append: the K/V rows of a prefill batch ([token][head*d]) go to the planar cache.
// A workgroup handles 16 consecutive tokens with all their heads: a wave reads 1 KiB of a row at a time, four
// requests of K and four of V per thread are out before the first store, and every token is looked up in the
// sequence offsets once, not once per thread.
constexpr int FILL_TOKENS = 16;

__global__ __launch_bounds__(256) void cache_fill_kernel(FillParams p)
{
    __shared__ int s_seq[FILL_TOKENS];
    __shared__ int64_t s_pos[FILL_TOKENS]; // -1: nothing to write for this token
    const int64_t tok0 = (int64_t)blockIdx.x * FILL_TOKENS;
    if (threadIdx.x < FILL_TOKENS) {
        const int64_t tok = tok0 + threadIdx.x;
        int seq = 0;
        int64_t pos = -1;
        if (tok < p.n_tokens) {
            // sequence of this token: last s with seq_offset[s] <= tok
            int lo = 0, hi = p.n_seqs;
            while (hi - lo > 1) {
                const int mid = (lo + hi) >> 1;
                if (p.seq_offset[mid] <= tok) lo = mid; else hi = mid;
            }
            seq = lo;
            const int64_t first = p.seq_offset[seq];
            if (tok >= first && tok < p.seq_offset[seq + 1]) {
                pos = (int64_t)p.cache_len[seq] + (tok - first);
                if (pos < 0 || pos >= p.max_len) pos = -1;
            }
        }
        s_seq[threadIdx.x] = seq;
        s_pos[threadIdx.x] = pos;
    }
    __syncthreads();
    const int chunks_head = p.head_dim / 16, chunks_row = p.n_heads * chunks_head;
    const int total = FILL_TOKENS * chunks_row;
    for (int base = 0; base < total; base += 4 * 256) {
        v4i kk[4], vv[4];
        int64_t dst[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
            const int id = base + u * 256 + (int)threadIdx.x;
            const int t = id / chunks_row, c = id % chunks_row;
            dst[u] = -1;
            if (id < total && s_pos[t] >= 0) {
                const int head = c / chunks_head, within = c % chunks_head;
                const int64_t src = (tok0 + t) * p.pitch + c * 16;
                dst[u] = (int64_t)s_seq[t] * p.seq_stride + (int64_t)head * p.head_stride + s_pos[t] * p.tok_stride + within * 16;
                kk[u] = *(const v4i *)(p.k_src + src);
                vv[u] = *(const v4i *)(p.v_src + src);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (dst[u] >= 0) {
                *(v4i *)(p.k + dst[u]) = kk[u];
                *(v4i *)(p.v + dst[u]) = vv[u];
            }
    }
    for (int id = threadIdx.x; id < FILL_TOKENS * p.n_heads; id += 256) { // scales: consecutive lanes, consecutive tokens
        const int head = id / FILL_TOKENS, t = id % FILL_TOKENS;
        if (s_pos[t] < 0) continue;
        const int64_t sd = (int64_t)s_seq[t] * p.s_seq_stride + (int64_t)head * p.s_head_stride + s_pos[t];
        if (p.ks_src) p.ks[sd] = p.ks_src[(int64_t)head * p.scale_pitch + tok0 + t];
        if (p.vs_src) p.vs[sd] = p.vs_src[(int64_t)head * p.scale_pitch + tok0 + t];
    }
}

__global__ void cache_len_add_kernel(int32_t *cache_len, const int32_t *seq_offset, int n_seqs, int max_len)
{
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_seqs) return;
    const int len = cache_len[i];
    if (len < 0) return;
    const int64_t grown = (int64_t)len + (seq_offset[i + 1] - seq_offset[i]);
    cache_len[i] = (int32_t)(grown < max_len ? grown : max_len);
}

hipError_t launch_cache_fill(const FillParams &p, hipStream_t st)
{
    if (p.n_seqs == 0 || p.n_tokens == 0) return hipSuccess;
    hipLaunchKernelGGL(cache_fill_kernel, dim3((unsigned)((p.n_tokens + FILL_TOKENS - 1) / FILL_TOKENS)), dim3(256), 0, st, p);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    hipLaunchKernelGGL(cache_len_add_kernel, dim3((unsigned)((p.n_seqs + 255) / 256)), dim3(256), 0, st, p.cache_len, p.seq_offset,
                       p.n_seqs, p.max_len);
    return hipGetLastError();
}

// Rows whose keys come as several spans: tsattn_prefill has been run once per span of the rows, part i over every row's
// i-th span, each part with the zero vector among its keys.  The weights of the parts add up and the zero vector counts
// once: with W_i = 2^swl_i the total weight of part i (zero vector included, weight 1),
//   out = sum_i out_i W_i / (sum_i W_i - (n - 1)),   swl = log2 of that denominator
// -- what the reference's loop over a row's spans computes in one go (compute/gpt_cpu.cpp:405-436).  Evaluated against
// the largest swl_i so that nothing overflows.  One thread per four consecutive values of a (row, head).
template <bool OUT_F16>
__global__ __launch_bounds__(256) void merge_lookups_kernel(MergeParams p)
{
    const int per_head = p.head_dim / 4;
    const int64_t id = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= p.n_tokens * p.n_heads * per_head) return;
    const int c = (int)(id % per_head);
    const int64_t pair = id / per_head;
    const int head = (int)(pair % p.n_heads);
    const int64_t row = pair / p.n_heads;
    const int64_t s_at = (int64_t)head * p.scale_pitch + row;
    const int64_t o_at = row * p.part_out_pitch + (int64_t)head * p.head_dim + 4 * c;
    float top = 0.0f; // every swl_i is >= 0: the zero vector alone weighs 1
    for (int i = 0; i < p.n_parts; ++i) top = fmaxf(top, p.part_swl[i * p.part_swl_stride + s_at]);
    v4f acc = v4f{0.0f, 0.0f, 0.0f, 0.0f};
    float total = 0.0f;
    for (int i = 0; i < p.n_parts; ++i) {
        const float w = exp2f(p.part_swl[i * p.part_swl_stride + s_at] - top);
        const v4f x = *(const v4f *)(p.part_out + i * p.part_out_stride + o_at);
        acc += x * w;
        total += w;
    }
    total -= (float)(p.n_parts - 1) * exp2f(-top);
    const v4f res = acc * (1.0f / total);
    if (OUT_F16) {
        uint8_t *dst = (uint8_t *)p.out + row * p.out_pitch + ((int64_t)head * p.head_dim + 4 * c) * 2;
        *(v4h *)dst = v4h{(_Float16)res.x, (_Float16)res.y, (_Float16)res.z, (_Float16)res.w};
    } else {
        uint8_t *dst = (uint8_t *)p.out + row * p.out_pitch + ((int64_t)head * p.head_dim + 4 * c) * 4;
        *(v4f *)dst = res;
    }
    if (p.swl && c == 0) p.swl[s_at] = top + log2f(total);
}

hipError_t launch_merge_lookups(const MergeParams &p, bool out_f16, hipStream_t st)
{
    const int64_t n = p.n_tokens * p.n_heads * (p.head_dim / 4);
    if (n == 0) return hipSuccess;
    const dim3 grid((unsigned)((n + 255) / 256)), block(256);
    if (out_f16) hipLaunchKernelGGL((merge_lookups_kernel<true>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((merge_lookups_kernel<false>), grid, block, 0, st, p);
    return hipGetLastError();
}

} // namespace tsattn
