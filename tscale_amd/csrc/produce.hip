// Producer of the attention operands: RoPE, per-head RMS normalisation and 8-bit conversion of a projection
// result, with the per-(row, head) scale the attention kernels consume.  Follows the reference's CPU inference
// (ApplyRope + NormalizeState, gpt/train/cpu_infer.cpp:486-499, :358-391; gpt/att/rope.cpp:28-46) operation by
// operation: the same float products, the sum of squares taken in index order, no fused multiply-adds, so the
// bytes and scales are identical to a CPU evaluation in that order.
//
// A workgroup takes 32 (8 in a small launch) consecutive (row, head) pairs.  The rotated values go to LDS (row pitch d+1 floats, so
// that 32 lanes walking 32 different pairs in step hit 32 different banks); then lane j of the first wave sums
// pair j's squares one after the other, which keeps the summation order while 32 sums advance together; then
// all threads convert and write the bytes out, sixteen per thread, consecutively.
#include <math.h>

#include "common.hpp"
#include "kernels.hpp"

namespace tsattn {

constexpr int PR_PAIRS = 32;       // (row, head) pairs per workgroup
constexpr int PR_PAIRS_FEW = 8;    // ... of a small launch: more workgroups, each with less to wait for

// every float operation below is meant as written: no fused multiply-adds
#pragma clang fp contract(off)

template <int D, int DST, bool SRC_I32, int PAIRS>
__global__ __launch_bounds__(256) void rope_normalize_kernel(ProduceParams p)
{
    constexpr int PITCH = D + 1;
    __shared__ float vals[PAIRS * PITCH];
    __shared__ float mults[PAIRS];
    __shared__ int64_t s_row[PAIRS];
    __shared__ int s_head[PAIRS], s_pos[PAIRS];
    const int tid = threadIdx.x;
    const int64_t pair0 = (int64_t)blockIdx.x * PAIRS;
    const int64_t n_pairs = p.n_rows * p.n_heads;
    const int n_here = (int)(n_pairs - pair0 < PAIRS ? n_pairs - pair0 : PAIRS);

    if (tid < n_here) {
        const int64_t pair = pair0 + tid;
        const int64_t row = pair / p.n_heads;
        s_row[tid] = row;
        s_head[tid] = (int)(pair - row * p.n_heads);
        int t = p.pos ? p.pos[row] : 0;
        s_pos[tid] = t < 0 ? 0 : (t >= p.rope_len ? (int)p.rope_len - 1 : t);
    }
    __syncthreads();

    // ---- load + rotate: four (k, k+32) couples per thread and step, 16-byte loads; all loads of a thread are
    //      issued before the first is used ------------------------------------------------------------------
    constexpr int PER_PAIR = D / 8;
    constexpr int STEPS = (PAIRS * PER_PAIR + 255) / 256;
    v4f v0[STEPS], v1[STEPS], cs[STEPS], sn[STEPS];
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
        const int j = tid + st * 256;
        const int pr = j / PER_PAIR, c = j % PER_PAIR;
        if (pr >= n_here) continue;
        const int x0 = (c / 8) * 64 + (c % 8) * 4, x1 = x0 + 32;
        const int64_t e = s_row[pr] * p.src_pitch + (int64_t)s_head[pr] * D;
        if (SRC_I32) {
            v4i a = *(const v4i *)((const int32_t *)p.src + e + x0), b = *(const v4i *)((const int32_t *)p.src + e + x1);
            for (int pl = 1; pl < p.src_planes; ++pl) { // the parts of a product whose K was split: exact integer sums
                a += *(const v4i *)((const int32_t *)p.src + pl * p.src_plane_stride + e + x0);
                b += *(const v4i *)((const int32_t *)p.src + pl * p.src_plane_stride + e + x1);
            }
            v0[st] = v4f{(float)a.x, (float)a.y, (float)a.z, (float)a.w};
            v1[st] = v4f{(float)b.x, (float)b.y, (float)b.z, (float)b.w};
        } else {
            v0[st] = *(const v4f *)((const float *)p.src + e + x0);
            v1[st] = *(const v4f *)((const float *)p.src + e + x1);
        }
        if (p.pos) { // heads that are not rotated read their row too and then turn by the identity: no divergent branch
            const float *rr = p.rope + (int64_t)s_pos[pr] * D;
            cs[st] = *(const v4f *)(rr + x0);
            sn[st] = *(const v4f *)(rr + x1);
        }
    }
    if (p.resid) {
        // state += delta * scale, written back; the updated state is what gets normalised.  (In loops of their own, after
        // every request above has been issued: a store in between would keep the compiler from issuing them together.)
        v4f u0[STEPS], u1[STEPS];
#pragma unroll
        for (int st = 0; st < STEPS; ++st) {
            const int j = tid + st * 256;
            const int pr = j / PER_PAIR, c = j % PER_PAIR;
            if (pr >= n_here) continue;
            const int x0 = (c / 8) * 64 + (c % 8) * 4;
            const float *r0 = p.resid + s_row[pr] * p.resid_pitch + (int64_t)s_head[pr] * D + x0;
            u0[st] = *(const v4f *)r0;
            u1[st] = *(const v4f *)(r0 + 32);
        }
#pragma unroll
        for (int st = 0; st < STEPS; ++st) {
            const int j = tid + st * 256;
            const int pr = j / PER_PAIR, c = j % PER_PAIR;
            if (pr >= n_here) continue;
            const int x0 = (c / 8) * 64 + (c % 8) * 4;
            float *r0 = p.resid + s_row[pr] * p.resid_pitch + (int64_t)s_head[pr] * D + x0;
            v0[st] = u0[st] + v0[st] * p.resid_scale;
            v1[st] = u1[st] + v1[st] * p.resid_scale;
            *(v4f *)r0 = v0[st];
            *(v4f *)(r0 + 32) = v1[st];
        }
    }
#pragma unroll
    for (int st = 0; st < STEPS; ++st) {
        const int j = tid + st * 256;
        const int pr = j / PER_PAIR, c = j % PER_PAIR;
        if (pr >= n_here) continue;
        const int x0 = (c / 8) * 64 + (c % 8) * 4, x1 = x0 + 32;
        if (p.pos) {
            const bool turn = s_head[pr] < p.rope_heads;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float cos_value = turn ? cs[st][i] : 1.0f;
                const float sin_value = turn ? sn[st][i] * p.rotate_dir : 0.0f;
                const float r0 = v0[st][i] * cos_value - v1[st][i] * sin_value;
                const float r1 = v0[st][i] * sin_value + v1[st][i] * cos_value;
                v0[st][i] = r0;
                v1[st][i] = r1;
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            vals[pr * PITCH + x0 + i] = v0[st][i];
            vals[pr * PITCH + x1 + i] = v1[st][i];
        }
    }
    __syncthreads();

    // ---- per pair: sum of squares in index order, scale -----------------------------------------------------
    if (tid < n_here) {
        const float *v = vals + tid * PITCH;
        float sum2 = 0.0f;
#pragma unroll 8
        for (int x = 0; x < D; ++x) sum2 = sum2 + v[x] * v[x];
        float discr = 0.0f, mult = 0.0f;
        if (sum2 != 0.0f) {
            // the single-precision square root instruction is one ulp off now and then; the double-precision routine
            // is exact to well below a float ulp, and rounding its result to float gives the correctly rounded root
            const float sko = (float)sqrt((double)(sum2 / (float)D));
            discr = sko * p.vec_scale;
            mult = 1.0f / discr;
        }
        mults[tid] = mult;
        const int sh = s_head[tid] - p.scale_head_begin;
        if (p.scale && sh >= 0 && sh < p.scale_head_count) p.scale[sh * p.scale_pitch + s_row[tid] * p.scale_row_stride] = discr * p.scale_mult;
    }
    __syncthreads();

    // ---- convert and store, 16 bytes per thread and step ------------------------------------------------------
    constexpr int OUT_PER_PAIR = D / 16;
    for (int j = tid; j < n_here * OUT_PER_PAIR; j += 256) {
        const int pr = j / OUT_PER_PAIR, x = (j % OUT_PER_PAIR) * 16;
        const float mult = mults[pr];
        uint32_t w[4];
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            w[k] = 0;
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const float y = vals[pr * PITCH + x + 4 * k + i] * mult;
                // a head of zeros is written as zero bytes whatever the signs of its (rotated) zeros
                uint32_t b = mult == 0.0f ? 0u : ((DST == TSATTN_I8) ? (uint8_t)float_to_i8(y) : float_to_e4m3(y));
                if (DST == TSATTN_I8 && p.relu && (b & 0x80u)) b = 0u; // x = max(0, x)
                w[k] |= b << (8 * i);
            }
        }
        *(v4i *)(p.dst + s_row[pr] * p.dst_pitch + (int64_t)s_head[pr] * D + x) = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
    }
}

hipError_t launch_rope_normalize(const ProduceParams &p, int dst_dtype, int head_dim, bool src_i32, hipStream_t st)
{
    const int64_t n_pairs = p.n_rows * p.n_heads;
    if (n_pairs == 0) return hipSuccess;
    // a small launch (one token per sequence) is a chain of waits -- positions, rows, the ordered sums -- that more,
    // smaller workgroups get through sooner; a large one is bound by memory and takes 32 pairs per workgroup
    // (groups wider than a head -- the feed-forward groups of 128 * ReluMult -- always: 32 of them would not fit in LDS)
    const bool few = n_pairs <= 4096 || head_dim > 128;
    const int per_wg = few ? PR_PAIRS_FEW : PR_PAIRS;
    dim3 grid((unsigned)((n_pairs + per_wg - 1) / per_wg)), block(256);
#define TSATTN_PR(D_, DST_, I32_)                                                                                   \
    do {                                                                                                            \
        if (few) hipLaunchKernelGGL((rope_normalize_kernel<D_, DST_, I32_, PR_PAIRS_FEW>), grid, block, 0, st, p);  \
        else hipLaunchKernelGGL((rope_normalize_kernel<D_, DST_, I32_, PR_PAIRS>), grid, block, 0, st, p);          \
    } while (0)
    if (head_dim == 128 && dst_dtype == TSATTN_I8 && !src_i32) TSATTN_PR(128, TSATTN_I8, false);
    else if (head_dim == 128 && dst_dtype == TSATTN_I8 && src_i32) TSATTN_PR(128, TSATTN_I8, true);
    else if (head_dim == 128 && dst_dtype == TSATTN_E4M3 && !src_i32) TSATTN_PR(128, TSATTN_E4M3, false);
    else if (head_dim == 128 && dst_dtype == TSATTN_E4M3 && src_i32) TSATTN_PR(128, TSATTN_E4M3, true);
    else if (head_dim == 64 && dst_dtype == TSATTN_I8 && !src_i32) TSATTN_PR(64, TSATTN_I8, false);
    else if (head_dim == 64 && dst_dtype == TSATTN_I8 && src_i32) TSATTN_PR(64, TSATTN_I8, true);
    else if (head_dim == 64 && dst_dtype == TSATTN_E4M3 && !src_i32) TSATTN_PR(64, TSATTN_E4M3, false);
    else if (head_dim == 64 && dst_dtype == TSATTN_E4M3 && src_i32) TSATTN_PR(64, TSATTN_E4M3, true);
#define TSATTN_PR_WIDE(D_)                                                                                          \
    else if (head_dim == D_ && dst_dtype == TSATTN_I8 && !src_i32)                                                  \
        hipLaunchKernelGGL((rope_normalize_kernel<D_, TSATTN_I8, false, PR_PAIRS_FEW>), grid, block, 0, st, p);     \
    else if (head_dim == D_ && dst_dtype == TSATTN_I8 && src_i32)                                                   \
        hipLaunchKernelGGL((rope_normalize_kernel<D_, TSATTN_I8, true, PR_PAIRS_FEW>), grid, block, 0, st, p);
    TSATTN_PR_WIDE(256)
    TSATTN_PR_WIDE(384)
    TSATTN_PR_WIDE(512)
#undef TSATTN_PR_WIDE
    else return hipErrorInvalidValue;
#undef TSATTN_PR
    return hipGetLastError();
}

// KVProduct, gpt/train/cpu_infer.cpp:320-337 (GPU form compute/gpt_combiner.cuh:13-37): the step after attention,
// kv[head][blk][z] = int8(k[head][z ^ blk] * value[head][z] * mult) for blk < 4.  One thread per 16 consecutive z of a
// (row, head): z ^ blk stays inside an aligned group of four, so a thread needs only its own 16 key bytes.
template <bool VAL_F16>
__global__ __launch_bounds__(256) void kv_product_kernel(KvProductParams p)
{
    const int chunks = p.head_dim / 16;
    const int64_t id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const int64_t total = p.n_rows * p.n_heads * chunks;
    if (id >= total) return;
    const int c = (int)(id % chunks);
    const int head = (int)((id / chunks) % p.n_heads);
    const int64_t row = id / ((int64_t)chunks * p.n_heads);
    const int64_t e = (int64_t)head * p.head_dim + c * 16;
    const v4i kw = *(const v4i *)(p.k + row * p.k_pitch + e);
    const int kws[4] = {kw.x, kw.y, kw.z, kw.w};
    float key[16], val[16];
#pragma unroll
    for (int i = 0; i < 16; ++i) key[i] = (float)(int8_t)((kws[i / 4] >> (8 * (i % 4))) & 0xff);
    if (VAL_F16) {
        const v8h a = *(const v8h *)((const _Float16 *)p.val + row * p.val_pitch + e);
        const v8h b = *(const v8h *)((const _Float16 *)p.val + row * p.val_pitch + e + 8);
#pragma unroll
        for (int i = 0; i < 8; ++i) { val[i] = (float)a[i]; val[8 + i] = (float)b[i]; }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const v4f a = *(const v4f *)((const float *)p.val + row * p.val_pitch + e + 4 * i);
            val[4 * i] = a.x; val[4 * i + 1] = a.y; val[4 * i + 2] = a.z; val[4 * i + 3] = a.w;
        }
    }
#pragma unroll
    for (int blk = 0; blk < 4; ++blk) {
        if (blk >= p.rep) break;
        uint32_t w[4] = {0, 0, 0, 0};
#pragma unroll
        for (int z = 0; z < 16; ++z) {
            const float y = (key[z ^ blk] * val[z]) * p.mult;
            w[z / 4] |= (uint32_t)(uint8_t)float_to_i8(y) << (8 * (z % 4));
        }
        *(v4i *)(p.kv + row * p.kv_pitch + ((int64_t)head * p.rep + blk) * p.head_dim + c * 16) = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
    }
}

hipError_t launch_kv_product(const KvProductParams &p, bool val_f16, hipStream_t st)
{
    const int64_t total = p.n_rows * p.n_heads * (p.head_dim / 16);
    if (total == 0) return hipSuccess;
    dim3 grid((unsigned)((total + 255) / 256)), block(256);
    if (val_f16) hipLaunchKernelGGL((kv_product_kernel<true>), grid, block, 0, st, p);
    else hipLaunchKernelGGL((kv_product_kernel<false>), grid, block, 0, st, p);
    return hipGetLastError();
}

// FillRopeBuf, gpt/att/rope.cpp:4-24 (host): table[t][base + k] = cos(t f), table[t][base + k + 32] = sin(t f),
// f = theta^-(2 (base/2 + k) / width), theta = 500000.  The float/double mix follows the reference's C++ overloads.
void fill_rope_table(int width, int64_t max_len, float *table)
{
    const float theta = 500000;
    for (int64_t t = 0; t < max_len; ++t) {
        for (int base = 0; base < width; base += 64) {
            for (int k = 0; k < 32; ++k) {
                const float freq = (float)exp((double)(-logf(theta)) * ((base / 2 + k) * 2. / width));
                const float angle = t * freq;
                table[t * width + base + k] = cosf(angle);
                table[t * width + base + k + 32] = sinf(angle);
            }
        }
    }
}

} // namespace tsattn
