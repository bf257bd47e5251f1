// Pieces shared by the prefill kernels: the K.Q^T step for each 8-bit operand type.
#pragma once

#include "common.hpp"
#include "kernels.hpp"

namespace tsattn {

constexpr int PF_THREADS = 256;
constexpr int PF_WAVES = 4;
constexpr int PF_BM = 128; // queries per workgroup (the C ABI's causal_period hint is counted in these)

// A logit may exceed the reference maximum by this much (log2 units) before the accumulators are
// rescaled: weights then stay below 2^8, far inside f16 and f32 range, and ordinary inputs never
// trigger a rescale because the reference maximum starts at the zero vector's logit 0.
constexpr float PF_RESCALE_THRESHOLD = 8.0f;

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
    // the same in single steps, for code that places each LDS read and MFMA itself
    typedef v8i kop_t;
    __device__ static kop_t load_k(const uint8_t *krow, int g, int s)
    {
        const v4i *p = (const v4i *)(krow + 64 * s + 32 * g);
        v4i a = p[0], b = p[1];
        return v8i{a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
    }
    __device__ acc_t step(kop_t kk, int s, acc_t acc) const { return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(kk, q[s], acc, 0, 0, 0, 0, 0, 0); }
    // the same operand straight from global memory (row_off: byte offset of the key's row in the descriptor)
    __device__ static kop_t load_k_global(__amdgpu_buffer_rsrc_t kr, int row_off, int g, int s)
    {
        const v4i a = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(kr, row_off + 64 * s + 32 * g, 0, 0));
        const v4i b = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(kr, row_off + 64 * s + 32 * g + 16, 0, 0));
        return v8i{a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
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
    typedef v4i kop_t;
    __device__ static kop_t load_k(const uint8_t *krow, int g, int s) { return *(const v4i *)(krow + 32 * s + 16 * g); }
    __device__ acc_t step(kop_t kk, int s, acc_t acc) const { return __builtin_amdgcn_mfma_i32_32x32x32_i8(kk, q[s], acc, 0, 0, 0); }
    __device__ static kop_t load_k_global(__amdgpu_buffer_rsrc_t kr, int row_off, int g, int s)
    {
        return __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(kr, row_off + 32 * s + 16 * g, 0, 0));
    }
    __device__ static float to_float(const acc_t &a, int r) { return (float)a[r]; }
    __device__ static float bits(const acc_t &a, int r) { return __int_as_float(a[r]); }
};

} // namespace tsattn
