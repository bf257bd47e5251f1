// The LDS access patterns of prefill_kernel (d = 128), each alone in a kernel of its own, to be run under the LDS
// counters: which of them has bank conflicts?  Kernels pat<0..5>: K operand reads, key-scale reads, transposing V^T
// operand reads, the staging stores (K and V together, K alone, V alone).
// Build: make -C tests/cpp mb_lds_patterns
// Run:   rocprofv3 --pmc SQ_LDS_BANK_CONFLICT SQ_LDS_IDX_ACTIVE SQ_INSTS_LDS -d out -o r --output-format csv -- ./tests/cpp/mb_lds_patterns
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdint.h>
typedef int v4i __attribute__((ext_vector_type(4)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef short v4s __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4s *lds_v4s_ptr;
constexpr int K_PITCH = 144, V_PITCH = 320, BN = 64;
constexpr int K_BYTES = BN * K_PITCH, V_BYTES = BN * V_PITCH;
__shared__ __attribute__((aligned(16))) uint8_t lds[2 * K_BYTES + 2 * V_BYTES + 2 * BN * 4];

template <int KIND>
__global__ __launch_bounds__(256) void pat(int iters, int *out)
{
    const int tid = threadIdx.x, lane = tid & 63, qi = lane & 31, g = lane >> 5;
    for (int i = tid; i < (int)sizeof(lds) / 4; i += 256) ((int *)lds)[i] = i;
    __syncthreads();
    int acc = 0;
    uint8_t *k_lds = lds, *v_lds = lds + 2 * K_BYTES;
    float *ks_lds = (float *)(lds + 2 * K_BYTES + 2 * V_BYTES);
    for (int it = 0; it < iters; ++it) {
        const int buf = it & 1;
        if (KIND == 0) { // K operand reads: lane's key row, 2 x 16 bytes per step, 2 steps, 2 sub-tiles
            for (int kt = 0; kt < 2; ++kt)
                for (int s = 0; s < 2; ++s) {
                    const v4i *p = (const v4i *)(k_lds + buf * K_BYTES + (kt * 32 + qi) * K_PITCH + 64 * s + 32 * g);
                    v4i a = p[0], b = p[1];
                    asm volatile("" ::"v"(a), "v"(b)); acc += a.x + b.y;
                }
        } else if (KIND == 1) { // key scales: 4 x 16 bytes per sub-tile, the same for the 32 lanes of a half
            for (int kt = 0; kt < 2; ++kt)
                for (int c4 = 0; c4 < 4; ++c4) {
                    v4f v = *(const v4f *)(ks_lds + buf * BN + 4 * g + 32 * kt + 8 * c4);
                    asm volatile("" ::"v"(v)); acc += (int)v.x;
                }
        } else if (KIND == 2) { // V^T operand reads (transposing)
            const int i16 = lane & 15, dh = (lane >> 4) & 1;
            const int key0 = 4 * g + (i16 >> 2);
            for (int grp = 0; grp < 4; ++grp)
                for (int dt = 0; dt < 4; ++dt) {
                    const uint8_t *vb = v_lds + buf * V_BYTES + grp * 16 * V_PITCH + key0 * V_PITCH + (dt * 32 + 16 * dh + 4 * (i16 & 3)) * 2;
                    v4s a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)(vb));
                    v4s a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)(vb + 8 * V_PITCH));
                    acc += a0.x + a1.y;
                }
        } else if (KIND == 3) { // staging stores: K chunk, two V halves per chunk, two chunks per thread
            for (int i = 0; i < 2; ++i) {
                const int ch = tid + i * 256, r = ch / 8, c = ch % 8;
                *(v4i *)(k_lds + buf * K_BYTES + r * K_PITCH + c * 16) = v4i{acc, it, i, c};
                *(v4i *)(v_lds + buf * V_BYTES + r * V_PITCH + c * 32) = v4i{acc, it, i, r};
                *(v4i *)(v_lds + buf * V_BYTES + r * V_PITCH + c * 32 + 16) = v4i{it, acc, i, r};
            }
        } else if (KIND == 4) { // K stores only
            for (int i = 0; i < 2; ++i) {
                const int ch = tid + i * 256, r = ch / 8, c = ch % 8;
                *(v4i *)(k_lds + buf * K_BYTES + r * K_PITCH + c * 16) = v4i{acc, it, i, c};
            }
        } else if (KIND == 5) { // V stores only
            for (int i = 0; i < 2; ++i) {
                const int ch = tid + i * 256, r = ch / 8, c = ch % 8;
                *(v4i *)(v_lds + buf * V_BYTES + r * V_PITCH + c * 32) = v4i{acc, it, i, r};
                *(v4i *)(v_lds + buf * V_BYTES + r * V_PITCH + c * 32 + 16) = v4i{it, acc, i, r};
            }
        }
        asm volatile("" ::: "memory");
    }
    __syncthreads();
    out[blockIdx.x * 256 + tid] = acc + ((int *)lds)[tid];
}

int main()
{
    int *out; hipMalloc(&out, 256 * 256 * 4);
    const int iters = 2000;
    pat<0><<<256, 256>>>(iters, out);
    pat<1><<<256, 256>>>(iters, out);
    pat<2><<<256, 256>>>(iters, out);
    pat<3><<<256, 256>>>(iters, out);
    pat<4><<<256, 256>>>(iters, out);
    pat<5><<<256, 256>>>(iters, out);
    hipDeviceSynchronize();
    printf("done\n");
    return 0;
}
