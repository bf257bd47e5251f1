// Prefill attention for int8 / e4m3 Q,K,V with per-row scales: flash-style tiling on the gfx950
// matrix cores.
//
// One workgroup (4 waves) owns 128 consecutive query rows of one head; each wave owns 32 of them.
// The key range [min span start, max span finish] of the workgroup is walked in tiles of 64 keys;
// tiles outside a wave's own rows' spans are skipped by that wave, tiles fully inside run without
// the per-element mask.  Per tile:
//   S^T = K . Q^T   with v_mfma_f32_32x32x64_f8f6f4 (e4m3) or v_mfma_i32_32x32x32_i8 (int8, exact);
//                   computing the transpose puts one query in each lane (column) and 16 keys of a
//                   32-key sub-tile in its registers, so all softmax state is per lane;
//   online softmax  in fp32 registers, base 2, running max starting at 0 (the zero vector's logit);
//   O^T += V^T . P^T with v_mfma_f32_32x32x16_f16: P goes from the S^T registers straight into the B
//                   operand (no LDS round trip); V is widened to f16 with its row scale folded in
//                   when the tile is staged, and read back transposed with ds_read_b64_tr_b16.
// Semantics: gpt/compute/gpt_cpu.cpp:391-441 (two-pass form of the same sums) with the 8-bit
// operand handling of gpt/compute/gpt_att_fp8.cuh:139-152 / gpt_att_fp16.cuh:184-189.
#include "common.hpp"
#include "kernels.hpp"

namespace tsattn {

constexpr int PF_THREADS = 256;
constexpr int PF_WAVES = 4;
constexpr int PF_BM = 128; // queries per workgroup
constexpr int PF_BN = 64;  // keys per tile

template <int D>
struct PfLayout {
    static constexpr int K_PITCH = D + 16;                  // bytes; 16-lane b128 reads hit 64 distinct banks
    static constexpr int V_PITCH = (D == 128) ? 320 : 192;  // bytes of an f16 row; row stride = 16 banks (mod 64)
    static constexpr int K_BYTES = PF_BN * K_PITCH;
    static constexpr int V_BYTES = PF_BN * V_PITCH;
};

template <int DTYPE, int D>
struct QkMma;

template <int D>
struct QkMma<TSATTN_E4M3, D> {
    static constexpr int STEPS = D / 64;
    typedef v16f acc_t;
    v8i q[STEPS];
    __device__ void load_q(const uint8_t *row, int g)
    {
        for (int s = 0; s < STEPS; ++s) {
            const v4i *p = (const v4i *)(row + 64 * s + 32 * g);
            v4i a = p[0], b = p[1];
            q[s] = v8i{a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
        }
    }
    __device__ void clear_q()
    {
        for (int s = 0; s < STEPS; ++s) q[s] = v8i{0, 0, 0, 0, 0, 0, 0, 0};
    }
    // acc = K[32 keys] . Q^T ; krow points at this lane's key row in LDS
    __device__ acc_t mma(const uint8_t *krow, int g) const
    {
        acc_t acc = {0};
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            const v4i *p = (const v4i *)(krow + 64 * s + 32 * g);
            v4i a = p[0], b = p[1];
            v8i kk = v8i{a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
            acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kk, q[s], acc, 0, 0, 0, 0, 0, 0);
        }
        return acc;
    }
    __device__ static float to_float(const acc_t &a, int r) { return a[r]; }
    __device__ static float bits(const acc_t &a, int r) { return a[r]; }
};

template <int D>
struct QkMma<TSATTN_I8, D> {
    static constexpr int STEPS = D / 32;
    typedef v16i acc_t;
    v4i q[STEPS];
    __device__ void load_q(const uint8_t *row, int g)
    {
        for (int s = 0; s < STEPS; ++s) q[s] = *(const v4i *)(row + 32 * s + 16 * g);
    }
    __device__ void clear_q()
    {
        for (int s = 0; s < STEPS; ++s) q[s] = v4i{0, 0, 0, 0};
    }
    __device__ acc_t mma(const uint8_t *krow, int g) const
    {
        acc_t acc = {0};
#pragma unroll
        for (int s = 0; s < STEPS; ++s) {
            v4i kk = *(const v4i *)(krow + 32 * s + 16 * g);
            acc = __builtin_amdgcn_mfma_i32_32x32x32_i8(kk, q[s], acc, 0, 0, 0);
        }
        return acc;
    }
    __device__ static float to_float(const acc_t &a, int r) { return (float)a[r]; }
    __device__ static float bits(const acc_t &a, int r) { return __int_as_float(a[r]); }
};

// 16 bytes of one V row -> 16 halves scaled by the row's value scale
template <int DTYPE>
__device__ inline void widen_v(v4i raw, float vs, v8h &lo, v8h &hi)
{
    int w[4] = {raw.x, raw.y, raw.z, raw.w};
    _Float16 h[16];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        float f0, f1, f2, f3;
        if (DTYPE == TSATTN_I8) {
            f0 = (float)(int8_t)(w[i] & 0xff);
            f1 = (float)(int8_t)((w[i] >> 8) & 0xff);
            f2 = (float)(int8_t)((w[i] >> 16) & 0xff);
            f3 = (float)(w[i] >> 24);
        } else {
            v2f a = e4m3x2_to_float(w[i], false), b = e4m3x2_to_float(w[i], true);
            f0 = a.x; f1 = a.y; f2 = b.x; f3 = b.y;
        }
        h[4 * i + 0] = (_Float16)(f0 * vs);
        h[4 * i + 1] = (_Float16)(f1 * vs);
        h[4 * i + 2] = (_Float16)(f2 * vs);
        h[4 * i + 3] = (_Float16)(f3 * vs);
    }
    lo = v8h{h[0], h[1], h[2], h[3], h[4], h[5], h[6], h[7]};
    hi = v8h{h[8], h[9], h[10], h[11], h[12], h[13], h[14], h[15]};
}

typedef __attribute__((address_space(3))) v4s *lds_v4s_ptr;

template <int DTYPE, int D, bool OUT_F16, bool DUMP>
__global__ __launch_bounds__(PF_THREADS) void prefill_kernel(PrefillParams p)
{
    typedef PfLayout<D> L;
    typedef QkMma<DTYPE, D> Qk;
    constexpr int DT = D / 32;       // 32-row tiles of O^T
    constexpr int CHUNKS = D / 16;   // 16-byte chunks per 8-bit row

    __shared__ __attribute__((aligned(16))) uint8_t k_lds[L::K_BYTES];
    __shared__ __attribute__((aligned(16))) uint8_t v_lds[L::V_BYTES];
    __shared__ __attribute__((aligned(16))) float ks_lds[PF_BN];
    __shared__ int red_lds[2 * PF_WAVES];

    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid / WAVE;
    const int qi = lane & 31; // query column of this lane
    const int g = lane >> 5;  // which half of the contraction this lane feeds
    const int head = blockIdx.y;
    const int tile = (int)gridDim.x - 1 - (int)blockIdx.x; // long rows first
    const int q0 = tile * PF_BM + wave * 32;
    const int from = q0 + qi;
    const bool row_ok = from < p.n_tokens;
    const int64_t hoff = (int64_t)head * D;

    // ---- spans --------------------------------------------------------------------------------
    int sp_a = 1, sp_b = 0;
    if (row_ok) {
        sp_a = p.span_start[from];
        sp_b = p.span_finish[from];
    }
    const bool has_keys = sp_b >= sp_a;
    const bool w_all_have_keys = __all(has_keys);
    int w_min_a = has_keys ? sp_a : 0x7fffffff, w_max_a = has_keys ? sp_a : -1;
    int w_min_b = has_keys ? sp_b : 0x7fffffff, w_max_b = has_keys ? sp_b : -1;
    for (int o = 16; o > 0; o >>= 1) {
        w_min_a = min(w_min_a, __shfl_xor(w_min_a, o, WAVE));
        w_max_a = max(w_max_a, __shfl_xor(w_max_a, o, WAVE));
        w_min_b = min(w_min_b, __shfl_xor(w_min_b, o, WAVE));
        w_max_b = max(w_max_b, __shfl_xor(w_max_b, o, WAVE));
    }
    if (lane == 0) {
        red_lds[wave] = w_min_a;
        red_lds[PF_WAVES + wave] = w_max_b;
    }
    __syncthreads();
    int b_min_a = red_lds[0], b_max_b = red_lds[PF_WAVES];
    for (int w = 1; w < PF_WAVES; ++w) {
        b_min_a = min(b_min_a, red_lds[w]);
        b_max_b = max(b_max_b, red_lds[PF_WAVES + w]);
    }

    // ---- query operand and per-row constants -------------------------------------------------------
    Qk qk;
    if (row_ok) qk.load_q(p.q + (int64_t)from * p.q_pitch + hoff, g);
    else qk.clear_q();
    const float qs = row_ok ? (p.qs ? p.qs[(int64_t)head * p.scale_pitch + from] : p.qs_const) : 0.0f;
    float ads = att_dot_scale(D);
    if (p.k_global_scale) ads *= *p.k_global_scale;

    v16f o_acc[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i) o_acc[i] = v16f{0};
    float m = 0.0f; // the zero vector's logit takes part in the maximum
    float l = 0.0f; // this lane's share of the sum (its 32 of every 64 keys)

    if (b_max_b >= b_min_a) {
        const int kb_first = (b_min_a / PF_BN) * PF_BN;
        for (int kb = kb_first; kb <= b_max_b; kb += PF_BN) {
            // ---- stage K (8-bit, as is) and V (f16 * row scale) in LDS ----------------------------------
            __syncthreads();
#pragma unroll
            for (int i = 0; i < (PF_BN * CHUNKS) / PF_THREADS; ++i) {
                int ch = tid + i * PF_THREADS;
                int r = ch / CHUNKS, c = ch % CHUNKS;
                int key = min(kb + r, p.n_tokens - 1);
                v4i kraw = *(const v4i *)(p.k + (int64_t)key * p.k_pitch + hoff + c * 16);
                v4i vraw = *(const v4i *)(p.v + (int64_t)key * p.v_pitch + hoff + c * 16);
                float vs = p.vs ? p.vs[(int64_t)head * p.scale_pitch + key] : p.vs_const;
                *(v4i *)(k_lds + r * L::K_PITCH + c * 16) = kraw;
                v8h lo, hi;
                widen_v<DTYPE>(vraw, vs, lo, hi);
                *(v8h *)(v_lds + r * L::V_PITCH + c * 32) = lo;
                *(v8h *)(v_lds + r * L::V_PITCH + c * 32 + 16) = hi;
            }
            if (tid < PF_BN) {
                int key = min(kb + tid, p.n_tokens - 1);
                float ks = p.ks ? p.ks[(int64_t)head * p.scale_pitch + key] : p.ks_const;
                ks_lds[tid] = ks * ads;
            }
            __syncthreads();

            // ---- does this wave need the tile at all, and does it need the mask? -----------------------
            if (kb + PF_BN - 1 < w_min_a || kb > w_max_b) continue;
            const bool interior = w_all_have_keys && (kb >= w_max_a) && (kb + PF_BN - 1 <= w_min_b);

            // ---- S^T = K . Q^T, scale, mask ---------------------------------------------------------------
            float s[2][16];
            float tmax = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
                typename Qk::acc_t acc = qk.mma(k_lds + (kt * 32 + qi) * L::K_PITCH, g);
#pragma unroll
                for (int c4 = 0; c4 < 4; ++c4) {
                    const int koff = kt * 32 + 8 * c4 + 4 * g;
                    v4f ksv = *(const v4f *)(ks_lds + koff);
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        const int r = c4 * 4 + j;
                        const int key = kb + koff + j;
                        if (DUMP) {
                            if (row_ok && key >= sp_a && key <= sp_b) {
                                ((float *)p.dbg)[((int64_t)head * p.n_tokens + from) * p.dbg_pitch + key] = Qk::bits(acc, r);
                            }
                        }
                        float dp = Qk::to_float(acc, r) * ksv[j] * qs - p.slope * (float)(from - key);
                        if (!interior) {
                            dp = (key >= sp_a && key <= sp_b) ? dp : -INFINITY;
                        }
                        s[kt][r] = dp;
                        tmax = fmaxf(tmax, dp);
                    }
                }
            }
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
            const float m_new = fmaxf(m, tmax);
            if (__any(m_new != m)) {
                const float alpha = fast_exp2(m - m_new);
                l *= alpha;
#pragma unroll
                for (int i = 0; i < DT; ++i) o_acc[i] *= alpha;
            }
            m = m_new;

            // ---- P = 2^(S - m), O^T += V^T . P^T --------------------------------------------------------------
#pragma unroll
            for (int kt = 0; kt < 2; ++kt) {
#pragma unroll
                for (int i = 0; i < 2; ++i) {
                    float pw[8];
#pragma unroll
                    for (int x = 0; x < 8; ++x) {
                        pw[x] = fast_exp2(s[kt][8 * i + x] - m_new);
                        l += pw[x];
                    }
                    v8h pb = v8h{(_Float16)pw[0], (_Float16)pw[1], (_Float16)pw[2], (_Float16)pw[3],
                                 (_Float16)pw[4], (_Float16)pw[5], (_Float16)pw[6], (_Float16)pw[7]};
                    // keys of this MFMA for lane group g: kt*32 + 16*i + 4*g + {0..3} and the same + 8
                    const int i16 = lane & 15, dh = (lane >> 4) & 1;
                    const int key0 = kt * 32 + 16 * i + 4 * g + (i16 >> 2);
#pragma unroll
                    for (int dt = 0; dt < DT; ++dt) {
                        const uint8_t *base = v_lds + key0 * L::V_PITCH + (dt * 32 + 16 * dh + 4 * (i16 & 3)) * 2;
                        v4s a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)(base));
                        v4s a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)(base + 8 * L::V_PITCH));
                        v8h va = __builtin_bit_cast(v8h, __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7));
                        o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va, pb, o_acc[dt], 0, 0, 0);
                    }
                }
            }
        }
    }

    // ---- epilogue: add the zero vector's weight, normalise, store -----------------------------------
    float l_all = l + __shfl_xor(l, 32, WAVE);
    l_all += fast_exp2(-m);
    const float inv = 1.0f / l_all;
    if (row_ok) {
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) {
                const int dcol = dt * 32 + 8 * c4 + 4 * g;
                float o0 = o_acc[dt][c4 * 4 + 0] * inv, o1 = o_acc[dt][c4 * 4 + 1] * inv;
                float o2 = o_acc[dt][c4 * 4 + 2] * inv, o3 = o_acc[dt][c4 * 4 + 3] * inv;
                if (OUT_F16) {
                    v4h hv = v4h{(_Float16)o0, (_Float16)o1, (_Float16)o2, (_Float16)o3};
                    *(v4h *)((uint8_t *)p.out + (int64_t)from * p.out_pitch + (hoff + dcol) * 2) = hv;
                } else {
                    *(v4f *)((uint8_t *)p.out + (int64_t)from * p.out_pitch + (hoff + dcol) * 4) = v4f{o0, o1, o2, o3};
                }
            }
        }
        if (p.sum_weight_log && g == 0) {
            p.sum_weight_log[(int64_t)head * p.scale_pitch + from] = m + __log2f(l_all);
        }
    }
}

template <int DTYPE, int D>
static void launch_prefill_dd(const PrefillParams &p, int out_dtype, dim3 grid, hipStream_t st)
{
    const bool dump = p.dbg != nullptr;
    const bool f16 = out_dtype == TSATTN_OUT_F16;
    dim3 block(PF_THREADS);
    if (f16) {
        if (dump) hipLaunchKernelGGL((prefill_kernel<DTYPE, D, true, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((prefill_kernel<DTYPE, D, true, false>), grid, block, 0, st, p);
    } else {
        if (dump) hipLaunchKernelGGL((prefill_kernel<DTYPE, D, false, true>), grid, block, 0, st, p);
        else hipLaunchKernelGGL((prefill_kernel<DTYPE, D, false, false>), grid, block, 0, st, p);
    }
}

hipError_t launch_prefill(const PrefillParams &p, int dtype, int head_dim, int out_dtype, hipStream_t st)
{
    if (p.n_tokens <= 0) return hipSuccess;
    dim3 grid((unsigned)((p.n_tokens + PF_BM - 1) / PF_BM), (unsigned)p.n_heads);
    if (dtype == TSATTN_E4M3 && head_dim == 128) launch_prefill_dd<TSATTN_E4M3, 128>(p, out_dtype, grid, st);
    else if (dtype == TSATTN_E4M3 && head_dim == 64) launch_prefill_dd<TSATTN_E4M3, 64>(p, out_dtype, grid, st);
    else if (dtype == TSATTN_I8 && head_dim == 128) launch_prefill_dd<TSATTN_I8, 128>(p, out_dtype, grid, st);
    else if (dtype == TSATTN_I8 && head_dim == 64) launch_prefill_dd<TSATTN_I8, 64>(p, out_dtype, grid, st);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

} // namespace tsattn
