// Shared device helpers for the gfx950 attention kernels.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/tsattn.h"

namespace tsattn {

constexpr int WAVE = 64;

// TScale's logit scale: sqrtf(1/d) * (0.5f / 0.693147f)  (gpt/model_params/model_dim.h:19-31).
__host__ __device__ inline float att_dot_scale(int head_dim)
{
    return sqrtf(1.0f / (float)head_dim) * (0.5f / 0.693147f);
}

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 v2h __attribute__((ext_vector_type(2)));
typedef _Float16 v4h __attribute__((ext_vector_type(4)));
typedef _Float16 v8h __attribute__((ext_vector_type(8)));
typedef short v4s __attribute__((ext_vector_type(4)));

__device__ inline float fast_exp2(float x)
{
    return __builtin_amdgcn_exp2f(x); // v_exp_f32
}

// Two-operand maximum kept out of the compiler's v_max3_f32 fusion: VALU instructions that read
// three different VGPRs do not execute alongside an MFMA on gfx950, two-operand ones do.
__device__ inline float max2(float a, float b)
{
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(a), "v"(b));
    return r;
}

__device__ inline float bf16_to_float(uint16_t b)
{
    return __uint_as_float((uint32_t)b << 16);
}

// e4m3 (OCP fn) <-> f32 through the gfx950 conversion instructions.
__device__ inline v2f e4m3x2_to_float(int packed, bool high_word)
{
    return high_word ? __builtin_amdgcn_cvt_pk_f32_fp8(packed, true) : __builtin_amdgcn_cvt_pk_f32_fp8(packed, false);
}

// Round-to-nearest-even, saturating to +-448 (the conversion alone would produce NaN on overflow).
__device__ inline uint8_t float_to_e4m3(float x)
{
    float c = __builtin_amdgcn_fmed3f(x, -448.0f, 448.0f);
    c = (x != x) ? x : c;
    int r = __builtin_amdgcn_cvt_pk_fp8_f32(c, c, 0, false);
    return (uint8_t)(r & 0xff);
}

// Round-to-nearest-even, clamped to [-127,127] (gpt/train/cpu_infer.cpp:88-92).
__device__ inline int8_t float_to_i8(float x)
{
    float r = rintf(x);
    r = fminf(fmaxf(r, -127.0f), 127.0f);
    return (int8_t)(int)r;
}

// Four floats to four int8 in one word (first value in the low byte): what float_to_i8 gives for each, with the lower
// bound a parameter (-127, or 0 where negative results are dropped).  Clamping before rounding gives what rounding
// before clamping gives, the bounds being whole numbers (one median-of-three instruction; a NaN comes out as the lower
// bound, as it does from fmaxf/fminf); adding 1.5 * 2^23 rounds to nearest even and leaves the whole number, in two's
// complement, in the low bits of the float.
__device__ inline uint32_t pack_i8x4(float y0, float y1, float y2, float y3, float low)
{
    const uint32_t b0 = __float_as_uint(__builtin_amdgcn_fmed3f(y0, low, 127.0f) + 12582912.0f);
    const uint32_t b1 = __float_as_uint(__builtin_amdgcn_fmed3f(y1, low, 127.0f) + 12582912.0f);
    const uint32_t b2 = __float_as_uint(__builtin_amdgcn_fmed3f(y2, low, 127.0f) + 12582912.0f);
    const uint32_t b3 = __float_as_uint(__builtin_amdgcn_fmed3f(y3, low, 127.0f) + 12582912.0f);
    // byte 0 of each
    return __builtin_amdgcn_perm(__builtin_amdgcn_perm(b3, b2, 0x0c0c0400u), __builtin_amdgcn_perm(b1, b0, 0x0c0c0400u), 0x05040100u);
}

// Butterfly exchange inside a wave through DPP where the pattern allows it.
template <int CTRL>
__device__ inline int dpp_mov(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
__device__ inline int dpp_xor1(int v) { return dpp_mov<0xB1>(v); }        // quad_perm [1,0,3,2]
__device__ inline int dpp_xor2(int v) { return dpp_mov<0x4E>(v); }        // quad_perm [2,3,0,1]
__device__ inline int dpp_half_mirror(int v) { return dpp_mov<0x141>(v); } // lane i <-> 7-i in each 8
__device__ inline int dpp_mirror(int v) { return dpp_mov<0x140>(v); }      // lane i <-> 15-i in each 16

__device__ inline float wave_max(float v)
{
    for (int o = 32; o > 0; o >>= 1) {
        v = fmaxf(v, __shfl_xor(v, o, WAVE));
    }
    return v;
}

__device__ inline float wave_sum(float v)
{
    for (int o = 32; o > 0; o >>= 1) {
        v += __shfl_xor(v, o, WAVE);
    }
    return v;
}

} // namespace tsattn
