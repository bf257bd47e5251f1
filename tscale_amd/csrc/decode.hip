// Single-token attention over a planar int8 / e4m3 KV cache: bandwidth-bound split-KV kernel plus
// the cross-split merge.
//
// Work decomposition.  grid = (n_splits, n_heads, n_seqs), 256 threads.  A (sequence, head) pair owns
// two contiguous planes, K[L][d] and V[L][d]; a split owns a contiguous run of cache rows.  Inside
// a wave, d/16 neighbouring lanes share one cache row and each lane reads 16 B of it, so one wave
// load instruction covers 1 KiB of consecutive memory (8 rows at d=128, 16 rows at d=64).  Each lane
// group keeps its own online-softmax state (running max, sum, 16 value accumulators) across all the
// rows it visits; states are merged only once, at the end: across lane groups by wave shuffles,
// across the four waves through LDS, across splits by merge_kernel.
//
// Semantics follow ComputeValLookup of gpt/train/cpu_infer.cpp:413-460: keys cur-1 ... cur-min(cur,W)
// (cur itself when W == 0), a leading logit 0 of value zero (:444), logit =
// dot * key_scale * attDotScale * q_scale - slope * (cur - to) (:448), value weight times the value
// scale (:454).  The running max starts at 0 in every split, which is what the zero logit makes it
// in the reference anyway, so no split ever needs a -inf state.
#include "common.hpp"
#include "kernels.hpp"

namespace tsattn {

constexpr int DEC_THREADS = 256;
constexpr int DEC_WAVES = DEC_THREADS / WAVE;
constexpr int DEC_U = 8; // cache rows per lane group kept in flight per step

template <int DTYPE>
struct QFrag;

template <>
struct QFrag<TSATTN_I8> {
    int w[4];
    __device__ void set(const uint8_t *b)
    {
        const int *p = (const int *)b;
        w[0] = p[0]; w[1] = p[1]; w[2] = p[2]; w[3] = p[3];
    }
    // exact int32 dot product of 16 bytes of the row with this lane's slice of q
    __device__ float dot_partial_as_bits(v4i kv) const
    {
        int acc = 0;
        acc = __builtin_amdgcn_sdot4(kv.x, w[0], acc, false);
        acc = __builtin_amdgcn_sdot4(kv.y, w[1], acc, false);
        acc = __builtin_amdgcn_sdot4(kv.z, w[2], acc, false);
        acc = __builtin_amdgcn_sdot4(kv.w, w[3], acc, false);
        return __int_as_float(acc);
    }
};

template <>
struct QFrag<TSATTN_E4M3> {
    float f[16];
    __device__ void set(const uint8_t *b)
    {
        const int *p = (const int *)b;
        for (int i = 0; i < 4; ++i) {
            v2f lo = e4m3x2_to_float(p[i], false);
            v2f hi = e4m3x2_to_float(p[i], true);
            f[4 * i + 0] = lo.x; f[4 * i + 1] = lo.y; f[4 * i + 2] = hi.x; f[4 * i + 3] = hi.y;
        }
    }
    __device__ float dot_partial_as_bits(v4i kv) const
    {
        float acc = 0;
        int kw[4] = {kv.x, kv.y, kv.z, kv.w};
        for (int i = 0; i < 4; ++i) {
            v2f lo = e4m3x2_to_float(kw[i], false);
            v2f hi = e4m3x2_to_float(kw[i], true);
            acc = fmaf(lo.x, f[4 * i + 0], acc);
            acc = fmaf(lo.y, f[4 * i + 1], acc);
            acc = fmaf(hi.x, f[4 * i + 2], acc);
            acc = fmaf(hi.y, f[4 * i + 3], acc);
        }
        return acc;
    }
};

// sum over the LPK lanes that share a cache row; every one of them ends with the total
template <int DTYPE, int LPK>
__device__ inline float group_sum_bits(float bits)
{
    if (DTYPE == TSATTN_I8) {
        int a = __float_as_int(bits);
        a += dpp_xor1(a);
        a += dpp_xor2(a);
        if (LPK == 8) {
            a += dpp_half_mirror(a);
        }
        return __int_as_float(a);
    } else {
        float a = bits;
        a += __int_as_float(dpp_xor1(__float_as_int(a)));
        a += __int_as_float(dpp_xor2(__float_as_int(a)));
        if (LPK == 8) {
            a += __int_as_float(dpp_half_mirror(__float_as_int(a)));
        }
        return a;
    }
}

template <int DTYPE>
__device__ inline void accumulate_values(float w, v4i vv, float *acc)
{
    int vw[4] = {vv.x, vv.y, vv.z, vv.w};
    if (DTYPE == TSATTN_I8) {
        for (int i = 0; i < 4; ++i) {
            int x = vw[i];
            acc[4 * i + 0] = fmaf(w, (float)(int8_t)(x & 0xff), acc[4 * i + 0]);
            acc[4 * i + 1] = fmaf(w, (float)(int8_t)((x >> 8) & 0xff), acc[4 * i + 1]);
            acc[4 * i + 2] = fmaf(w, (float)(int8_t)((x >> 16) & 0xff), acc[4 * i + 2]);
            acc[4 * i + 3] = fmaf(w, (float)(x >> 24), acc[4 * i + 3]);
        }
    } else {
        for (int i = 0; i < 4; ++i) {
            v2f lo = e4m3x2_to_float(vw[i], false);
            v2f hi = e4m3x2_to_float(vw[i], true);
            acc[4 * i + 0] = fmaf(w, lo.x, acc[4 * i + 0]);
            acc[4 * i + 1] = fmaf(w, lo.y, acc[4 * i + 1]);
            acc[4 * i + 2] = fmaf(w, hi.x, acc[4 * i + 2]);
            acc[4 * i + 3] = fmaf(w, hi.y, acc[4 * i + 3]);
        }
    }
}

// KVProduct of a finished output element (gpt/train/cpu_infer.cpp:320-337): kv[head][blk][x] = int8((k[head][x ^ blk] *
// value) * mult) for blk < rep; x ^ blk stays inside x's aligned group of four key bytes.  The same arithmetic as
// kv_product_kernel on the stored output.
template <int D>
__device__ inline void kv_product_store(const uint8_t *kv_k, int64_t kv_k_pitch, uint8_t *kv_out, int64_t kv_out_pitch, int rep, float mult,
                                        int64_t seq, int head, int x, float value)
{
    const uint32_t kw = *(const uint32_t *)(kv_k + seq * kv_k_pitch + (int64_t)head * D + (x & ~3));
    for (int blk = 0; blk < rep; ++blk) {
        const float key = (float)(int8_t)((kw >> (8 * ((x ^ blk) & 3))) & 0xff);
        const float y = (key * value) * mult;
        kv_out[seq * kv_out_pitch + ((int64_t)head * rep + blk) * D + x] = (uint8_t)float_to_i8(y);
    }
}

template <int DTYPE, int D, bool QBF16, bool DUMP>
__global__ __launch_bounds__(DEC_THREADS) void decode_split_kernel(DecodeParams p)
{
    constexpr int LPK = D / 16;      // lanes per cache row
    constexpr int KPL = WAVE / LPK;  // rows per wave load
    constexpr int ROWS_PER_STEP = DEC_U * KPL;

    const int split = blockIdx.x;
    const int head = blockIdx.y;
    const int seq = blockIdx.z;
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid / WAVE;
    const int c = lane % LPK;        // which 16-byte slice of the row
    const int g = lane / LPK;        // which row of a wave load

    __shared__ float sm_m[DEC_WAVES];
    __shared__ float sm_l[DEC_WAVES];
    __shared__ float sm_acc[DEC_WAVES][D];

    // ---- key range of this block --------------------------------------------------------------
    // With a fused append the cache holds cache_len rows and the new token's row is being added as row cache_len
    // by the first split's workgroup of each head (a full cache drops it, as the separate append does).
    int cur = p.cache_len[seq] - 1;
    if (p.k_new && cur + 1 < p.max_len) {
        cur += 1;
        if (split == 0 && tid < 2 * LPK) {
            const int pl = tid / LPK, ch = tid % LPK; // plane (K or V), 16-byte chunk
            const int64_t src = (int64_t)seq * p.new_pitch + head * D + ch * 16;
            const int64_t dst = (int64_t)seq * p.seq_stride + (int64_t)head * p.head_stride + (int64_t)cur * p.tok_stride + ch * 16;
            if (pl == 0) *(v4i *)(const_cast<uint8_t *>(p.k) + dst) = *(const v4i *)(p.k_new + src);
            else *(v4i *)(const_cast<uint8_t *>(p.v) + dst) = *(const v4i *)(p.v_new + src);
            if (ch == 0) {
                const int64_t sd = (int64_t)seq * p.s_seq_stride + (int64_t)head * p.s_head_stride + cur;
                if (pl == 0 && p.ks_new) const_cast<float *>(p.ks)[sd] = p.ks_new[seq * p.n_heads + head];
                if (pl == 1 && p.vs_new) const_cast<float *>(p.vs)[sd] = p.vs_new[seq * p.n_heads + head];
            }
        }
    }
    const bool direct = p.n_splits == 1; // no merge kernel follows: this workgroup writes the output
    // A single-split launch with a fused append has no merge kernel to count the new row either: every workgroup
    // of a sequence (one per head) reports when it is done with the old length, and the last to report adds one.
    // (The counter is back at zero when the launch ends; launches that share a handle must not overlap.)
    auto report_done = [&]() {
        if (tid == 0) {
            const int done = atomicAdd(&p.seq_done[seq], 1);
            if (done == p.n_heads - 1) {
                p.seq_done[seq] = 0;
                const int len = p.cache_len_rw[seq];
                if (len >= 0 && len < p.max_len) p.cache_len_rw[seq] = len + 1;
            }
        }
    };
    const bool count_row = direct && p.k_new != nullptr;
    int lo, n;
    if (cur < 0) {
        lo = 0; n = 0;
    } else if (p.window == 0) {
        lo = cur; n = 1;
    } else {
        n = (int)((p.window < (int64_t)cur) ? p.window : (int64_t)cur);
        lo = cur - n;
    }
    int per = (n + p.n_splits - 1) / p.n_splits;
    per = ((per + KPL - 1) / KPL) * KPL;
    const int s0 = lo + split * per;
    int s1 = s0 + per;
    if (s1 > lo + n) s1 = lo + n;

    const int64_t part = ((int64_t)seq * p.n_heads + head) * p.n_splits + split;
    if (s0 >= s1) { // nothing to do: neutral partial (max 0, sum 0, zeros)
        if (direct) {
            if (tid < D) {
                p.out[((int64_t)seq * p.n_heads + head) * D + tid] = 0.0f;
                if (p.kv_out) kv_product_store<D>(p.kv_k, p.kv_k_pitch, p.kv_out, p.kv_out_pitch, p.kv_rep, p.kv_mult, seq, head, tid, 0.0f);
            }
            if (count_row) {
                __syncthreads(); // every thread has read the old length
                report_done();
            }
            return;
        }
        if (tid < D) p.part_acc[part * D + tid] = 0.0f;
        if (tid == 0) { p.part_ml[part * 2] = 0.0f; p.part_ml[part * 2 + 1] = 0.0f; }
        return;
    }

    // ---- query slice of this lane ----------------------------------------------------------------
    QFrag<DTYPE> qf;
    float qs;
    {
        __attribute__((aligned(16))) uint8_t qb[16];
        if (QBF16) {
            const uint16_t *src = (const uint16_t *)(p.q + (int64_t)seq * p.q_pitch) + head * D + c * 16;
            float x[16];
            float amax = 0;
            for (int i = 0; i < 16; ++i) {
                x[i] = bf16_to_float(src[i]);
                amax = fmaxf(amax, fabsf(x[i]));
            }
            for (int o = 1; o < LPK; o <<= 1) {
                amax = fmaxf(amax, __shfl_xor(amax, o, WAVE));
            }
            // absmax rule of lib/cuda/cuda_matmul.cuh:237-249
            float discr = 0, mult = 0;
            if (amax > 0) {
                discr = (DTYPE == TSATTN_I8) ? amax / 127.0f : amax / 256.0f;
                mult = 1.0f / discr;
            }
            for (int i = 0; i < 16; ++i) {
                float y = x[i] * mult;
                qb[i] = (DTYPE == TSATTN_I8) ? (uint8_t)float_to_i8(y) : float_to_e4m3(y);
            }
            qs = discr;
        } else {
            const v4i *src = (const v4i *)(p.q + (int64_t)seq * p.q_pitch + head * D + c * 16);
            *(v4i *)qb = *src;
            qs = p.q_scale ? p.q_scale[seq * p.n_heads + head] : p.q_scale_const;
        }
        qf.set(qb);
    }

    const uint8_t *kbase = p.k + (int64_t)seq * p.seq_stride + (int64_t)head * p.head_stride + c * 16;
    const uint8_t *vbase = p.v + (int64_t)seq * p.seq_stride + (int64_t)head * p.head_stride + c * 16;
    const float *ksb = p.ks ? p.ks + (int64_t)seq * p.s_seq_stride + (int64_t)head * p.s_head_stride : nullptr;
    const float *vsb = p.vs ? p.vs + (int64_t)seq * p.s_seq_stride + (int64_t)head * p.s_head_stride : nullptr;
    const float ads = att_dot_scale(D);

    float m = 0.0f, l = 0.0f;
    float acc[16];
    for (int i = 0; i < 16; ++i) acc[i] = 0.0f;

    for (int base = s0 + wave * ROWS_PER_STEP; base < s1; base += DEC_WAVES * ROWS_PER_STEP) {
        v4i kreg[DEC_U], vreg[DEC_U];
        float ksr[DEC_U], vsr[DEC_U];
        int row[DEC_U];
#pragma unroll
        for (int u = 0; u < DEC_U; ++u) {
            int r = base + u * KPL + g;
            row[u] = r;
            int rc = (r < s1) ? r : s1 - 1; // clamp the address, mask the logit below
            kreg[u] = __builtin_nontemporal_load((const v4i *)(kbase + (int64_t)rc * p.tok_stride));
            ksr[u] = ksb ? ksb[rc] : p.ks_const;
        }
#pragma unroll
        for (int u = 0; u < DEC_U; ++u) {
            int rc = (row[u] < s1) ? row[u] : s1 - 1;
            vreg[u] = __builtin_nontemporal_load((const v4i *)(vbase + (int64_t)rc * p.tok_stride));
            vsr[u] = vsb ? vsb[rc] : p.vs_const;
        }
        float s[DEC_U];
        float m_new = m;
#pragma unroll
        for (int u = 0; u < DEC_U; ++u) {
            float bits = group_sum_bits<DTYPE, LPK>(qf.dot_partial_as_bits(kreg[u]));
            float accf = (DTYPE == TSATTN_I8) ? (float)__float_as_int(bits) : bits;
            if (DUMP) {
                if (c == 0 && row[u] < s1) {
                    ((float *)p.dbg)[((int64_t)seq * p.n_heads + head) * p.dbg_pitch + row[u]] = bits;
                }
            }
            float dp = accf * ksr[u] * ads * qs - p.slope * (float)(cur - row[u]);
            s[u] = (row[u] < s1) ? dp : -INFINITY;
            m_new = fmaxf(m_new, s[u]);
        }
        float alpha = fast_exp2(m - m_new);
        m = m_new;
        l *= alpha;
#pragma unroll
        for (int i = 0; i < 16; ++i) acc[i] *= alpha;
#pragma unroll
        for (int u = 0; u < DEC_U; ++u) {
            float pu = fast_exp2(s[u] - m_new);
            l += pu;
            accumulate_values<DTYPE>(pu * vsr[u], vreg[u], acc);
        }
    }

    // ---- merge the lane groups of this wave ---------------------------------------------------
#pragma unroll
    for (int o = LPK; o < WAVE; o <<= 1) {
        float m_o = __shfl_xor(m, o, WAVE);
        float l_o = __shfl_xor(l, o, WAVE);
        float m_n = fmaxf(m, m_o);
        float a = fast_exp2(m - m_n), b = fast_exp2(m_o - m_n);
        l = l * a + l_o * b;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            float acc_o = __shfl_xor(acc[i], o, WAVE);
            acc[i] = acc[i] * a + acc_o * b;
        }
        m = m_n;
    }
    if (g == 0) {
#pragma unroll
        for (int i = 0; i < 16; ++i) sm_acc[wave][c * 16 + i] = acc[i];
        if (c == 0) { sm_m[wave] = m; sm_l[wave] = l; }
    }
    __syncthreads();
    // ---- merge the waves, write this split's partial --------------------------------------------
    if (tid < D) {
        float M = sm_m[0];
        for (int w = 1; w < DEC_WAVES; ++w) M = fmaxf(M, sm_m[w]);
        float o = 0, L = 0;
        for (int w = 0; w < DEC_WAVES; ++w) {
            float f = fast_exp2(sm_m[w] - M);
            o += sm_acc[w][tid] * f;
            L += sm_l[w] * f;
        }
        if (direct) {
            // the only split: add the zero vector's weight 2^-M (M >= 0 by construction) and normalise here
            const float res = o / (L + fast_exp2(-M));
            p.out[((int64_t)seq * p.n_heads + head) * D + tid] = res;
            if (p.kv_out) kv_product_store<D>(p.kv_k, p.kv_k_pitch, p.kv_out, p.kv_out_pitch, p.kv_rep, p.kv_mult, seq, head, tid, res);
        } else {
            p.part_acc[part * D + tid] = o;
            if (tid == 0) { p.part_ml[part * 2] = M; p.part_ml[part * 2 + 1] = L; }
        }
    }
    if (count_row) report_done(); // after the barrier above: every thread has read the old length
}

// out = sum_s acc_s 2^(m_s - M) / (2^-M + sum_s l_s 2^(m_s - M)),  M = max(0, max_s m_s)
template <int D>
__global__ __launch_bounds__(D) void decode_merge_kernel(const float *part_acc, const float *part_ml, int n_splits, float *out,
                                                         int32_t *bump_len, int n_heads, int max_len, const uint8_t *kv_k,
                                                         int64_t kv_k_pitch, uint8_t *kv_out, int64_t kv_out_pitch, int kv_rep, float kv_mult)
{
    const int64_t sh = blockIdx.x; // seq * n_heads + head
    const int x = threadIdx.x;
    // after a fused append: every split kernel has finished with the old length, count the new row
    if (bump_len && x == 0 && sh % n_heads == 0) {
        const int64_t seq = sh / n_heads;
        const int len = bump_len[seq];
        if (len >= 0 && len < max_len) bump_len[seq] = len + 1;
    }
    float M = 0.0f;
    for (int s = 0; s < n_splits; ++s) M = fmaxf(M, part_ml[(sh * n_splits + s) * 2]);
    float L = fast_exp2(-M); // the zero vector of weight 1 (cpu_infer.cpp:444)
    float o = 0;
    for (int s = 0; s < n_splits; ++s) {
        float f = fast_exp2(part_ml[(sh * n_splits + s) * 2] - M);
        L += part_ml[(sh * n_splits + s) * 2 + 1] * f;
        o += part_acc[(sh * n_splits + s) * D + x] * f;
    }
    const float res = o / L;
    out[sh * D + x] = res;
    if (kv_out) kv_product_store<D>(kv_k, kv_k_pitch, kv_out, kv_out_pitch, kv_rep, kv_mult, sh / n_heads, (int)(sh % n_heads), x, res);
}

template <int DTYPE, int D>
static void launch_decode_dd(const DecodeParams &p, bool qbf16, bool dump, dim3 grid, hipStream_t st)
{
    if (qbf16) {
        if (dump) hipLaunchKernelGGL((decode_split_kernel<DTYPE, D, true, true>), grid, dim3(DEC_THREADS), 0, st, p);
        else hipLaunchKernelGGL((decode_split_kernel<DTYPE, D, true, false>), grid, dim3(DEC_THREADS), 0, st, p);
    } else {
        if (dump) hipLaunchKernelGGL((decode_split_kernel<DTYPE, D, false, true>), grid, dim3(DEC_THREADS), 0, st, p);
        else hipLaunchKernelGGL((decode_split_kernel<DTYPE, D, false, false>), grid, dim3(DEC_THREADS), 0, st, p);
    }
}

hipError_t launch_decode(const DecodeParams &p, int dtype, int head_dim, bool qbf16, int n_seqs, float *out, hipStream_t st)
{
    dim3 grid(p.n_splits, p.n_heads, n_seqs);
    const bool dump = p.dbg != nullptr;
    if (dtype == TSATTN_I8 && head_dim == 128) launch_decode_dd<TSATTN_I8, 128>(p, qbf16, dump, grid, st);
    else if (dtype == TSATTN_I8 && head_dim == 64) launch_decode_dd<TSATTN_I8, 64>(p, qbf16, dump, grid, st);
    else if (dtype == TSATTN_E4M3 && head_dim == 128) launch_decode_dd<TSATTN_E4M3, 128>(p, qbf16, dump, grid, st);
    else if (dtype == TSATTN_E4M3 && head_dim == 64) launch_decode_dd<TSATTN_E4M3, 64>(p, qbf16, dump, grid, st);
    else return hipErrorInvalidValue;
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    if (p.n_splits == 1) return hipSuccess; // the split kernel wrote the output (and counted a fused append's row) itself
    dim3 mgrid((unsigned)(n_seqs * p.n_heads));
    int32_t *bump = p.k_new ? p.cache_len_rw : nullptr;
    if (head_dim == 128) hipLaunchKernelGGL((decode_merge_kernel<128>), mgrid, dim3(128), 0, st, p.part_acc, p.part_ml, p.n_splits, out, bump, p.n_heads, p.max_len, p.kv_k, p.kv_k_pitch, p.kv_out, p.kv_out_pitch, p.kv_rep, p.kv_mult);
    else hipLaunchKernelGGL((decode_merge_kernel<64>), mgrid, dim3(64), 0, st, p.part_acc, p.part_ml, p.n_splits, out, bump, p.n_heads, p.max_len, p.kv_k, p.kv_k_pitch, p.kv_out, p.kv_out_pitch, p.kv_rep, p.kv_mult);
    return hipGetLastError();
}

} // namespace tsattn
