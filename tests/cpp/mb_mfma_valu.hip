// Microbenchmark behind the prefill kernel's schedule: how much of the softmax's vector work runs under the P.V matrix
// instructions on gfx950.  One workgroup per compute unit, one or two waves per SIMD; every wave repeats
// [v_mfma_f32_32x32x16_f16 ; a block of vector instructions] on registers of its own (no memory traffic).  Printed per
// such pair, in ns: the matrix instructions alone (accumulators in VGPRs or in AGPRs), the vector block alone, both.
// Vector blocks: 8 two-register multiplies; 8 three-register fmas; 4 v_exp_f32; the weights of two (query, key)
// pairs as the kernel computes them (mul, fma, exp, add per element, one v_cvt_pk_f16_f32 per two).
// Then the same work as two groups of four waves a phase apart (one group issues 8 matrix instructions while the
// other does 8 vector blocks), with and without barriers between the phases and raised priority on the matrix phase.
// Build: make -C tests/cpp mb_mfma_valu; run on the GPU: ./tests/cpp/mb_mfma_valu
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));

#define MFMA_V(c) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+v"(c) : "v"(a), "v"(b))
#define MFMA_A(c) asm volatile("v_mfma_f32_32x32x16_f16 %0, %1, %2, %0" : "+a"(c) : "v"(a), "v"(b))
// 8 vector instructions: KIND 0: two-register multiplies; 1: three-register fma; 2: exp; 3: mix as in the softmax (mul, fma, exp, add, cvt_pk per 2)
template <int KIND>
__device__ inline void valu8(float (&x)[8], float s, float t)
{
    if (KIND == 0) {
#pragma unroll
        for (int i = 0; i < 8; ++i) asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[i]) : "v"(s));
    } else if (KIND == 1) {
#pragma unroll
        for (int i = 0; i < 8; ++i) asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[i]) : "v"(s), "v"(t));
    } else if (KIND == 2) {
#pragma unroll
        for (int i = 0; i < 4; ++i) asm volatile("v_exp_f32 %0, %0" : "+v"(x[i]));
    } else {
        // two elements: mul, mul, fma, fma, exp, exp (2 slots each), add, add, cvt_pk (2 slots) = 13 slots
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[0]) : "v"(s));
        asm volatile("v_mul_f32 %0, %0, %1" : "+v"(x[1]) : "v"(s));
        asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[0]) : "v"(s), "v"(t));
        asm volatile("v_fma_f32 %0, %0, %1, %2" : "+v"(x[1]) : "v"(s), "v"(t));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[0]));
        asm volatile("v_exp_f32 %0, %0" : "+v"(x[1]));
        asm volatile("v_add_f32 %0, %0, %1" : "+v"(x[2]) : "v"(x[0]));
        asm volatile("v_add_f32 %0, %0, %1" : "+v"(x[3]) : "v"(x[1]));
        asm volatile("v_cvt_pk_f16_f32 %0, %1, %2" : "=v"(x[4]) : "v"(x[0]), "v"(x[1]));
    }
}

template <bool AGPR, bool DO_MFMA, bool DO_VALU, int KIND>
__global__ __launch_bounds__(512) void mb_kernel(float *out, int iters, float s, float t)
{
    v16f c[4];
    for (int k = 0; k < 4; ++k) for (int i = 0; i < 16; ++i) c[k][i] = 0.0f;
    v8h a, b;
    for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(threadIdx.x * 0.001f); b[i] = (_Float16)0.5f; }
    float x[8];
    for (int i = 0; i < 8; ++i) x[i] = s * (threadIdx.x + i);
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            if (DO_MFMA) { if (AGPR) MFMA_A(c[k]); else MFMA_V(c[k]); }
            if (DO_VALU) valu8<KIND>(x, s, t);
        }
    }
    float r = 0.0f;
    for (int k = 0; k < 4; ++k) for (int i = 0; i < 16; ++i) r += c[k][i];
    for (int i = 0; i < 8; ++i) r += x[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = r;
}

// two groups of four waves a phase apart: while one issues its matrix instructions the other does its vector work
template <int KIND, bool BARRIER, bool PRIO>
__global__ __launch_bounds__(512) void pp_kernel(float *out, int iters, float s, float t)
{
    v16f c[4];
    for (int k = 0; k < 4; ++k) for (int i = 0; i < 16; ++i) c[k][i] = 0.0f;
    v8h a, b;
    for (int i = 0; i < 8; ++i) { a[i] = (_Float16)(threadIdx.x * 0.001f); b[i] = (_Float16)0.5f; }
    float x[8];
    for (int i = 0; i < 8; ++i) x[i] = s * (threadIdx.x + i);
    const int grp = __builtin_amdgcn_readfirstlane(threadIdx.x >> 8);
    auto mm = [&]() __attribute__((always_inline)) {
        if (PRIO) __builtin_amdgcn_s_setprio(2);
#pragma unroll
        for (int r = 0; r < 2; ++r)
#pragma unroll
            for (int k = 0; k < 4; ++k) MFMA_V(c[k]);
        if (PRIO) __builtin_amdgcn_s_setprio(0);
    };
    auto vv = [&]() __attribute__((always_inline)) {
#pragma unroll
        for (int r = 0; r < 8; ++r) valu8<KIND>(x, s, t);
    };
    if (grp == 0) {
        for (int it = 0; it < iters; ++it) {
            mm();
            if (BARRIER) __builtin_amdgcn_s_barrier();
            vv();
            if (BARRIER) __builtin_amdgcn_s_barrier();
        }
    } else {
        for (int it = 0; it < iters; ++it) {
            vv();
            if (BARRIER) __builtin_amdgcn_s_barrier();
            mm();
            if (BARRIER) __builtin_amdgcn_s_barrier();
        }
    }
    float r = 0.0f;
    for (int k = 0; k < 4; ++k) for (int i = 0; i < 16; ++i) r += c[k][i];
    for (int i = 0; i < 8; ++i) r += x[i];
    out[blockIdx.x * blockDim.x + threadIdx.x] = r;
}

template <int KIND, bool BARRIER, bool PRIO>
static float run_pp(float *out, int iters)
{
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    pp_kernel<KIND, BARRIER, PRIO><<<256, 512>>>(out, 10, 1.0001f, 0.0f);
    hipDeviceSynchronize();
    hipEventRecord(e0);
    pp_kernel<KIND, BARRIER, PRIO><<<256, 512>>>(out, iters, 1.0001f, 0.0f);
    hipEventRecord(e1); hipEventSynchronize(e1);
    float ms; hipEventElapsedTime(&ms, e0, e1);
    return ms;
}

template <bool AGPR, bool M, bool V, int KIND>
static float run(int threads, float *out, int iters)
{
    hipEvent_t e0, e1; hipEventCreate(&e0); hipEventCreate(&e1);
    mb_kernel<AGPR, M, V, KIND><<<256, threads>>>(out, 10, 1.0001f, 0.0f);
    hipDeviceSynchronize();
    hipEventRecord(e0);
    mb_kernel<AGPR, M, V, KIND><<<256, threads>>>(out, iters, 1.0001f, 0.0f);
    hipEventRecord(e1); hipEventSynchronize(e1);
    float ms; hipEventElapsedTime(&ms, e0, e1);
    return ms;
}

template <int KIND>
static void table(float *out, int iters, const char *name)
{
    for (int threads = 256; threads <= 512; threads += 256) {
        const float m_v = run<false, true, false, KIND>(threads, out, iters), m_a = run<true, true, false, KIND>(threads, out, iters);
        const float v = run<false, false, true, KIND>(threads, out, iters);
        const float b_v = run<false, true, true, KIND>(threads, out, iters), b_a = run<true, true, true, KIND>(threads, out, iters);
        // per iteration-quarter (one MFMA + one VALU block), in ns -> cycles at 2.4 GHz nominal are only indicative
        const double q = 1e6 / (4.0 * iters);
        printf("%-8s waves/SIMD %d: MFMA(vgpr) %.1f ns  MFMA(agpr) %.1f  VALU %.1f  both(vgpr) %.1f  both(agpr) %.1f\n", name, threads / 256,
               m_v * q, m_a * q, v * q, b_v * q, b_a * q);
        fflush(stdout);
    }
}

int main()
{
    float *out; hipMalloc(&out, 256 * 512 * 4);
    const int iters = 20000;
    table<0>(out, iters, "mul2src");
    table<1>(out, iters, "fma3src");
    table<2>(out, iters, "exp x4");
    table<3>(out, iters, "softmax");
    // per (one MFMA + one vector block) of each wave, as above: two waves per SIMD -> compare with the 2-wave "both" column
    {
        const int it8 = iters / 2;
        const double q = 1e6 / (8.0 * it8);
        printf("ping-pong mul2src: barrier+prio %.1f ns  barrier %.1f  free-running %.1f\n", run_pp<0, true, true>(out, it8) * q, run_pp<0, true, false>(out, it8) * q, run_pp<0, false, false>(out, it8) * q);
        printf("ping-pong softmax: barrier+prio %.1f ns  barrier %.1f  free-running %.1f\n", run_pp<3, true, true>(out, it8) * q, run_pp<3, true, false>(out, it8) * q, run_pp<3, false, false>(out, it8) * q);
    }
    return 0;
}
