// int8 x int8 -> int32 matrix product with the epilogues of the reference's int8 inference path:
//   out[m][n] = sum_k a[m][k] * w[n][k]
// MulForward (gpt/train/cpu_infer.cpp:294-305: one weight row per output, exact int32 sums, result as int32 or
// converted to float) and AddScaled (:308-316: state += delta * scale).
//
// Two kernels.  Many rows (a prompt): 128 x 128 output tiles, K in steps of 64 bytes through LDS, four waves of
// 64 x 64 each, v_mfma_i32_32x32x32_i8; bound by the matrix cores.  Few rows (one token per sequence): the
// weights are read once from HBM, 32 weight rows per workgroup with K split over its four waves; bound by HBM.
// Integer sums are exact, so every decomposition gives the same bits.
#include <type_traits>
#include "common.hpp"
#include "kernels.hpp"

namespace tsattn {

namespace {

constexpr int GT_THREADS = 256;
constexpr int GT_BN = 128, GT_BK = 64;
constexpr int GT_PITCH = GT_BK + 16; // LDS row pitch: 16-lane phases of a 16-byte read hit distinct banks

__device__ inline __amdgpu_buffer_rsrc_t rows_rsrc(const void *base, int64_t rows, int64_t pitch, int64_t row_bytes)
{
    // the last row ends after row_bytes, not after a whole pitch
    int64_t bytes = rows <= 0 ? 0 : (rows - 1) * pitch + row_bytes;
    const uint32_t n = bytes > 0xffffffffll ? 0xffffffffu : (uint32_t)bytes;
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)n, 0x00020000);
}

template <int MODE>
__device__ inline void store_out(const GemmParams &p, int64_t m, int64_t n, int acc)
{
#pragma clang fp contract(off) // delta * scale is rounded before it is added, as in the reference's two statements
    if (MODE == TSATTN_MM_I32) {
        ((int32_t *)p.out)[m * p.out_pitch + n] = acc;
    } else if (MODE == TSATTN_MM_F32) {
        ((float *)p.out)[m * p.out_pitch + n] = (float)acc * p.scale;
    } else {
        float *o = (float *)p.out + m * p.out_pitch + n;
        *o += (float)acc * p.scale; // (*pRes)[k] += delta[k] * scale
    }
}

// ---- many rows --------------------------------------------------------------------------------------------------
// Products too small for the wide tiles below: output tiles of 64 MT x 128 (MT = 2 in use), K in steps of 64 bytes
// through LDS (two buffers), four waves as 2 x 2, each wave 32 MT x 64 = MT x 2 MFMA tiles.  One 32x32x32 MFMA takes 32
// cycles and two KiB of operands, so operands have to be used several times from registers.
template <int MODE, int MT>
__global__ __launch_bounds__(GT_THREADS, 2) void gemm_tiled_kernel(GemmParams p)
{
    constexpr int BM = 64 * MT;
    constexpr int A_CH = BM * GT_BK / 16 / GT_THREADS, W_CH = GT_BN * GT_BK / 16 / GT_THREADS; // 16-byte chunks per thread
    __shared__ __attribute__((aligned(16))) uint8_t a_lds[2][BM * GT_PITCH];
    __shared__ __attribute__((aligned(16))) uint8_t w_lds[2][GT_BN * GT_PITCH];
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid / WAVE;
    const int wm = wave >> 1, wn = wave & 1;
    const int li = lane & 31, g = lane >> 5;

    // Which output tile.  The 8 XCDs take workgroups round-robin and each has its own L2; the 64 or so workgroups an
    // XCD runs at a time walk through K at about the same pace, so its L2 only has to hold the current slices of the
    // rows they use.  Give those 64 an 8 x 8 block of tiles: 8 tiles of activations and 8 of weights cross the fabric
    // per 64 output tiles instead of up to 64 + 8.  Shapes that do not divide that way walk along rows of tiles.
    const int64_t tiles_n = (p.n + GT_BN - 1) / GT_BN, tiles_m = (p.m + BM - 1) / BM;
    int64_t tile_m, tile_n;
    if (tiles_n % 8 == 0 && tiles_m % 8 == 0 && ((tiles_n >> 3) * (tiles_m >> 3)) % 8 == 0) { // whole blocks, eight at a time
        const int64_t x = blockIdx.x & 7, l = blockIdx.x >> 3;
        const int64_t sb = (l >> 6) * 8 + x, within = l & 63; // super-block of 8 x 8 tiles, tile inside it
        const int64_t sb_per_row = tiles_n >> 3;
        tile_m = (sb / sb_per_row) * 8 + (within >> 3);
        tile_n = (sb % sb_per_row) * 8 + (within & 7);
    } else {
        tile_m = blockIdx.x / tiles_n;
        tile_n = blockIdx.x % tiles_n;
    }
    const int64_t m0 = tile_m * BM, n0 = tile_n * GT_BN;

    const __amdgpu_buffer_rsrc_t ar = rows_rsrc(p.a + m0 * p.a_pitch, p.m - m0 < BM ? p.m - m0 : BM, p.a_pitch, p.k);
    const __amdgpu_buffer_rsrc_t wr = rows_rsrc(p.w + n0 * p.w_pitch, p.n - n0 < GT_BN ? p.n - n0 : GT_BN, p.w_pitch, p.k);
    // staging: a row of 64 bytes is four chunks of 16
    int a_off[A_CH], w_off[W_CH], a_dst[A_CH], w_dst[W_CH];
#pragma unroll
    for (int i = 0; i < A_CH; ++i) {
        const int ch = tid + i * GT_THREADS, r = ch >> 2, c = ch & 3;
        a_off[i] = r * (int)p.a_pitch + c * 16;
        a_dst[i] = r * GT_PITCH + c * 16;
    }
#pragma unroll
    for (int i = 0; i < W_CH; ++i) {
        const int ch = tid + i * GT_THREADS, r = ch >> 2, c = ch & 3;
        w_off[i] = r * (int)p.w_pitch + c * 16;
        w_dst[i] = r * GT_PITCH + c * 16;
    }
    // two sets of staging registers: what is requested at the end of step s is the tile of step s + 3 and has two
    // whole steps to arrive before it is written to LDS
    v4i ra[2][A_CH], rw[2][W_CH];
    auto load = [&](int set, int kb) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < A_CH; ++i) ra[set][i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ar, a_off[i], kb, 0));
#pragma unroll
        for (int i = 0; i < W_CH; ++i) rw[set][i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(wr, w_off[i], kb, 0));
    };
    auto stage = [&](int set, int buf) __attribute__((always_inline)) {
#pragma unroll
        for (int i = 0; i < A_CH; ++i) *(v4i *)(a_lds[buf] + a_dst[i]) = ra[set][i];
#pragma unroll
        for (int i = 0; i < W_CH; ++i) *(v4i *)(w_lds[buf] + w_dst[i]) = rw[set][i];
    };

    v16i acc[MT][2];
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = v16i{0};

    const int n_steps = (int)(p.k / GT_BK);
    auto compute = [&](int buf) __attribute__((always_inline)) {
        const uint8_t *ab = a_lds[buf] + (wm * (BM / 2) + li) * GT_PITCH + 16 * g;
        const uint8_t *wb = w_lds[buf] + (wn * 64 + li) * GT_PITCH + 16 * g;
        // all of the step's operands are asked for before the first MFMA: the LDS latency is paid once per step
        v4i a[2][MT], w[2][2];
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
            for (int j = 0; j < 2; ++j) w[ks][j] = *(const v4i *)(wb + j * 32 * GT_PITCH + 32 * ks);
#pragma unroll
            for (int i = 0; i < MT; ++i) a[ks][i] = *(const v4i *)(ab + i * 32 * GT_PITCH + 32 * ks);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int ks = 0; ks < 2; ++ks)
#pragma unroll
            for (int i = 0; i < MT; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[ks][i], w[ks][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    // step s computes from LDS buffer s & 1, then writes the tile of step s + 1 (register set (s + 1) & 1) to the
    // other buffer and asks for the tile of step s + 3 into the set just emptied
    // (Requests and LDS writes are unconditional: past K a request reads zeros or other rows of the tile, never
    // outside it, and nobody computes from what it leaves in LDS.  With branches around them the compiler loses track
    // of which request is which and waits for all of them before every write.)
    load(0, 0);
    stage(0, 0);
    load(1, GT_BK);
    load(0, 2 * GT_BK);
    __syncthreads();
    for (int s = 0; s < n_steps; s += 2) {
        compute(0);
        stage(1, 1);
        load(1, (s + 3) * GT_BK);
        __syncthreads();
        if (s + 1 < n_steps) compute(1);
        stage(0, 0);
        load(0, (s + 4) * GT_BK);
        __syncthreads();
    }

    // accumulator register r of tile (i, j): row m0 + wm*(BM/2) + i*32 + 8*(r/4) + 4*g + r%4, column n0 + wn*64 + j*32 + li
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int64_t n = n0 + wn * 64 + j * 32 + li;
            if (n >= p.n) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int64_t m = m0 + wm * (BM / 2) + i * 32 + 8 * (r / 4) + 4 * g + (r & 3);
                if (m < p.m) store_out<MODE>(p, m, n, acc[i][j][r]);
            }
        }
}

// Wide tiles for the largest products: 256 x 256 outputs by eight waves of 128 x 64, K in steps of 64 bytes, one
// workgroup per compute unit; per MFMA cycle this moves a third less through LDS and the caches than 256 x 128 tiles.
// Each SIMD holds two of the waves, one from each half of the workgroup, and the halves run half a step apart: while
// one half issues the 16 MFMAs of its step, the other does its memory work (requests its share of the tile three
// steps on, which memory writes straight into LDS, and reads its operands of the next step from LDS), then they swap
// at a barrier.  The MFMA pipe always has a wave feeding it and no wave waits for memory while it feeds.  Four LDS
// buffers of 32 KiB: one being read, three tiles on their way (a request has two whole steps to land).
// LDS rows are 64 bytes without padding; the 16-byte chunks of a row are permuted by (row / 4) % 4, which keeps the
// row-per-lane operand reads free of bank conflicts; a memory-to-LDS request writes the 64 lanes' 16 bytes one after
// the other, so the permutation is applied to the addresses the lanes request.  K must be a multiple of 64.
constexpr int GW_THREADS = 512, GW_BM = 256, GW_BN = 256, GW_BK = 64, GW_NBUF = 4;
constexpr int GW_BUF = (GW_BM + GW_BN) * GW_BK;
constexpr int GW_LDS_BYTES = GW_NBUF * GW_BUF;
// with the producer as epilogue: the floats of 128 rows (row pitch head width + 4), a multiplier per (row, head), 256 positions
constexpr int ep_lds_bytes(int head_dim) { return head_dim == 0 ? 0 : (128 * (GW_BN / head_dim) * (head_dim + 4) + 128 * (GW_BN / head_dim) + GW_BM) * 4; }
constexpr int gw_lds_bytes(int head_dim) { return ep_lds_bytes(head_dim) > GW_LDS_BYTES ? ep_lds_bytes(head_dim) : GW_LDS_BYTES; }

template <int MODE, int EP_D>
__global__ __launch_bounds__(GW_THREADS, 1) void gemm_wide_kernel(GemmParams p)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t gw_lds[];
    typedef __attribute__((address_space(3))) void *lds_ptr;
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int half = wave >> 2; // waves 0-3 and 4-7 land on SIMDs 0-3 each
    const int wm = wave >> 2, wn = wave & 3;
    const int li = lane & 31, g = lane >> 5;

    // 8 x 8 blocks of tiles per XCD where the shape allows (see gemm_tiled_kernel)
    const int64_t tiles_n = (p.n + GW_BN - 1) / GW_BN, tiles_m = (p.m + GW_BM - 1) / GW_BM;
    int64_t tile_m, tile_n;
    if (tiles_n % 8 == 0 && tiles_m % 8 == 0 && ((tiles_n >> 3) * (tiles_m >> 3)) % 8 == 0) {
        const int64_t x = blockIdx.x & 7, l = blockIdx.x >> 3;
        const int64_t sb = (l >> 6) * 8 + x, within = l & 63;
        const int64_t sb_per_row = tiles_n >> 3;
        tile_m = (sb / sb_per_row) * 8 + (within >> 3);
        tile_n = (sb % sb_per_row) * 8 + (within & 7);
    } else {
        tile_m = blockIdx.x / tiles_n;
        tile_n = blockIdx.x % tiles_n;
    }
    const int64_t m0 = tile_m * GW_BM, n0 = tile_n * GW_BN;
    const __amdgpu_buffer_rsrc_t ar = rows_rsrc(p.a + m0 * p.a_pitch, p.m - m0 < GW_BM ? p.m - m0 : GW_BM, p.a_pitch, p.k);
    const __amdgpu_buffer_rsrc_t wr = rows_rsrc(p.w + n0 * p.w_pitch, p.n - n0 < GW_BN ? p.n - n0 : GW_BN, p.w_pitch, p.k);
    // A buffer holds 256 rows of A, then 256 rows of W.  A wave's request fills 16 rows (1 KiB): lane L writes the
    // chunk at position L % 4 of row L / 4, which is chunk (L % 4) ^ perm(row) of the matrix row.  Rows
    // wave * 16 + 128 i: perm depends on the lane only.
    const int sr = wave * 16 + (lane >> 2), sc = (lane & 3) ^ ((lane >> 4) & 3);
    const int a_off0 = sr * (int)p.a_pitch + sc * 16, a_off1 = a_off0 + 128 * (int)p.a_pitch;
    const int w_off0 = sr * (int)p.w_pitch + sc * 16, w_off1 = w_off0 + 128 * (int)p.w_pitch;
    auto request = [&](int kb, uint8_t *buf) __attribute__((always_inline)) { // tile at K offset kb -> buf
        uint8_t *const d = buf + wave * 16 * GW_BK;
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ar, (lds_ptr)(d), 16, a_off0, kb, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(ar, (lds_ptr)(d + 128 * GW_BK), 16, a_off1, kb, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(wr, (lds_ptr)(d + 256 * GW_BK), 16, w_off0, kb, 0, 0);
        __builtin_amdgcn_raw_ptr_buffer_load_lds(wr, (lds_ptr)(d + 384 * GW_BK), 16, w_off1, kb, 0, 0);
    };
    // operands: row li of each 32-row block, chunk 2 * h + g of its 64 bytes (h: which 32 bytes of the step)
    const int f_perm = (li >> 2) & 3;
    const int f_a = (wm * 128 + li) * GW_BK + ((g ^ f_perm) << 4);
    const int f_w = (GW_BM + wn * 64 + li) * GW_BK + ((g ^ f_perm) << 4);
    v4i fa[2][4], fw[2][2];
    v16i acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = v16i{0};

    // A barrier that waits for this wave's LDS reads only: __syncthreads() would also wait for every tile still on its
    // way into LDS, which is exactly what must stay in flight.  What has to have landed is waited for by count.
#define GW_BARRIER                                              \
    do {                                                        \
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");      \
        __builtin_amdgcn_s_barrier();                           \
        asm volatile("" ::: "memory");                          \
    } while (0)
    const int n_steps = (int)(p.k / GW_BK);
    // (with the producer as epilogue: the position of tile row tid, asked for now, so that the epilogue's rope rows do not
    // wait for it)
    int row_pos = 0;
    if constexpr (EP_D != 0) {
        if (p.ep.pos && tid < GW_BM && m0 + tid < p.m) row_pos = p.ep.pos[m0 + tid];
    }
    // requests past K fetch bytes that are never computed with (or zeros past the rows' end)
    request(0, gw_lds);
    request(GW_BK, gw_lds + GW_BUF);
    request(2 * GW_BK, gw_lds + 2 * GW_BUF);
    asm volatile("s_waitcnt vmcnt(8)" ::: "memory"); // this wave's share of the first tile has landed
    GW_BARRIER;
    if (half == 1) GW_BARRIER; // the second half of the workgroup runs half a step behind the first
#define GW_FENCE __builtin_amdgcn_sched_barrier(0)
    for (int s = 0; s < n_steps; ++s) {
        uint8_t *const cur = gw_lds + (s & 3) * GW_BUF;
        // memory half: request the tile of step s + 3 into the buffer step s - 1 was read from, read this step's
        // operands, make sure this wave's share of the tile of step s + 1 has landed before the barrier
        GW_FENCE;
        request((s + 3) * GW_BK, gw_lds + ((s + 3) & 3) * GW_BUF);
        GW_FENCE;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
#pragma unroll
            for (int i = 0; i < 4; ++i) fa[h][i] = *(const v4i *)(cur + ((f_a + i * 32 * GW_BK) ^ (h * 32)));
#pragma unroll
            for (int j = 0; j < 2; ++j) fw[h][j] = *(const v4i *)(cur + ((f_w + j * 32 * GW_BK) ^ (h * 32)));
        }
        GW_FENCE;
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");
        GW_BARRIER;
        // MFMA half
        GW_FENCE;
        __builtin_amdgcn_s_setprio(1);
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fa[h][i], fw[h][j], acc[i][j], 0, 0, 0);
        __builtin_amdgcn_s_setprio(0);
        GW_FENCE;
        GW_BARRIER;
    }
#undef GW_FENCE
    if (half == 0) GW_BARRIER;
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); // nothing may still be on its way into LDS when the workgroup ends
#undef GW_BARRIER
    if constexpr (EP_D != 0) {
        // The producer as the product's epilogue (the reference's projection kernels end the same way,
        // TStoreRowTileNormalizeRope, gpt/compute/gpt_rope.cuh:4-66): the int32 sums never go to memory.  The tile's
        // 256 columns are whole heads of EP_D; 128 of its rows at a time (blocks 2 s and 2 s + 1 of both row halves) go
        // through LDS as floats -- after the residual update or the rotation, which are lane-local: a wave's 64 columns
        // are one rotation block, x in acc[.][0] and x + 32 in acc[.][1] -- so that one thread per (row, head) can add up
        // the squares in index order, as the producer kernel and the CPU path do (that chain of additions is the longest
        // wait of the epilogue: the more pairs a step has, the more threads walk their chains side by side).  Every
        // float operation as written there.  A residual update and a rotation in one call are left to the producer
        // kernel by the launcher.
#pragma clang fp contract(off)
        constexpr int HEADS_T = GW_BN / EP_D;  // heads per tile
        constexpr int PAIRS = 128 * HEADS_T;   // (row, head) pairs per step
        constexpr int PITCH = EP_D + 4;        // rows 16 bytes aligned, 16 lanes' 16-byte reads on 64 different banks
        static_assert(ep_lds_bytes(EP_D) == (PAIRS * PITCH + PAIRS + GW_BM) * 4 && PAIRS <= GW_THREADS, "the epilogue's LDS and threads");
        float *const vals = (float *)gw_lds;
        float *const mults = vals + PAIRS * PITCH;
        int *const tile_pos = (int *)(mults + PAIRS); // positions of the tile's 256 rows
        const ProduceParams &e = p.ep;
        const int head_t = (wn * 64) / EP_D, xbase = (wn * 64) % EP_D;
        const int head = (int)(n0 / EP_D) + head_t;
        const bool head_ok = head < e.n_heads;
        const bool turn = head < e.rope_heads;
        __syncthreads(); // every wave is done with the operand buffers
        if (tid < GW_BM) tile_pos[tid] = row_pos < 0 ? 0 : (row_pos >= e.rope_len ? (int)e.rope_len - 1 : row_pos);
        __syncthreads();
        // Addresses inside the tile are 32-bit offsets from a base that is the same for the whole wave (the launcher
        // checks that the pitches allow it): one add per access instead of a 64-bit multiply.
        const int rows_here = (int)(p.m - m0 < GW_BM ? p.m - m0 : GW_BM);
        const bool rotate = e.pos && turn;
        const char *const rope_base = (const char *)(e.rope + xbase);
        char *const resid_base = (char *)(e.resid + m0 * e.resid_pitch + (int64_t)head * EP_D + xbase);
        const uint32_t resid_pitch_bytes = (uint32_t)e.resid_pitch * 4u;
        // Everything a block of rows needs from memory is requested before any of it is used or stored (row by row, each
        // row's stores would have to be waited for before the next row's loads, which they might overlap), and the next
        // step's requests go out before this step's sums and conversion, which they pass under.  Per block two values
        // per row and lane: the old state's, or cos and sin.
        float xa[2][16], xb[2][16];
        auto request = [&](int i, int set) __attribute__((always_inline)) {
            if (e.resid) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = wm * 128 + i * 32 + 8 * (r / 4) + 4 * g + (r & 3);
                    const bool ok = row < rows_here && head_ok;
                    const float *const q0 = (const float *)(resid_base + ((uint32_t)row * resid_pitch_bytes + (uint32_t)li * 4u));
                    xa[set][r] = ok ? q0[0] : 0.0f;
                    xb[set][r] = ok ? q0[32] : 0.0f;
                }
            } else if (rotate) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const uint32_t t = (uint32_t)tile_pos[wm * 128 + i * 32 + 8 * (r / 4) + 4 * g + (r & 3)];
                    const float *const rope_row = (const float *)(rope_base + (t * (uint32_t)(EP_D * 4) + (uint32_t)li * 4u));
                    xa[set][r] = rope_row[0];
                    xb[set][r] = rope_row[32];
                }
            }
        };
        request(0, 0);
        request(1, 1);
#pragma unroll // (the accumulators are registers: no run-time index into them)
        for (int s = 0; s < 2; ++s) {
#pragma unroll
            for (int b = 0; b < 2; ++b) {
                const int i = 2 * s + b;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int rr = 8 * (r / 4) + 4 * g + (r & 3);
                    const int row = wm * 128 + i * 32 + rr;
                    float v0 = (float)acc[i][0][r], v1 = (float)acc[i][1][r];
                    if (e.resid) { // state += delta * scale, written back; the updated state is what gets normalised
                        v0 = xa[b][r] + v0 * e.resid_scale;
                        v1 = xb[b][r] + v1 * e.resid_scale;
                        if (row < rows_here && head_ok) {
                            float *const q0 = (float *)(resid_base + ((uint32_t)row * resid_pitch_bytes + (uint32_t)li * 4u));
                            q0[0] = v0;
                            q0[32] = v1;
                        }
                    } else if (rotate) {
                        const float cos_value = xa[b][r];
                        const float sin_value = xb[b][r] * e.rotate_dir;
                        const float r0 = v0 * cos_value - v1 * sin_value;
                        const float r1 = v0 * sin_value + v1 * cos_value;
                        v0 = r0;
                        v1 = r1;
                    } // (a head that is not rotated: cos 1 and sin 0 leave the values as they are)
                    float *const dst = vals + ((b * 64 + wm * 32 + rr) * HEADS_T + head_t) * PITCH + xbase + li;
                    dst[0] = v0;
                    dst[32] = v1;
                }
                if (s == 0) request(2 + b, b);
            }
            __syncthreads();
            if (tid < PAIRS) { // sum of squares in index order, scale
                const int rc = tid / HEADS_T, ht = tid % HEADS_T;
                const int64_t m = m0 + ((rc % 64) / 32) * 128 + (2 * s + rc / 64) * 32 + (rc % 32);
                const int hd = (int)(n0 / EP_D) + ht;
                const float *const v = vals + tid * PITCH;
                float sum2 = 0.0f;
#pragma unroll
                for (int x = 0; x < EP_D; x += 32) { // 32 values per round of LDS reads, added in index order
                    v4f q[8];
#pragma unroll
                    for (int c = 0; c < 8; ++c) q[c] = *(const v4f *)(v + x + 4 * c);
#pragma unroll
                    for (int c = 0; c < 8; ++c) {
                        sum2 = sum2 + q[c].x * q[c].x;
                        sum2 = sum2 + q[c].y * q[c].y;
                        sum2 = sum2 + q[c].z * q[c].z;
                        sum2 = sum2 + q[c].w * q[c].w;
                    }
                }
                float discr = 0.0f, mult = 0.0f;
                if (sum2 != 0.0f) {
                    const float sko = (float)sqrt((double)(sum2 / (float)EP_D)); // correctly rounded (see the producer kernel)
                    discr = sko * e.vec_scale;
                    mult = 1.0f / discr;
                }
                mults[tid] = mult;
                const int sh = hd - e.scale_head_begin;
                if (e.scale && m < p.m && hd < e.n_heads && sh >= 0 && sh < e.scale_head_count)
                    e.scale[sh * e.scale_pitch + m * e.scale_row_stride] = discr * e.scale_mult;
            }
            __syncthreads();
            // Convert and store, 16 bytes per thread and step.  A head of zeros has mult 0: zero bytes.
            constexpr int OUT_PER_PAIR = EP_D / 16;
            static_assert((PAIRS * OUT_PER_PAIR) % GW_THREADS == 0, "whole steps of the workgroup");
            const float low = e.relu ? 0.0f : -127.0f;
            uint8_t *const dst_base = e.dst + m0 * e.dst_pitch + n0;
#pragma unroll
            for (int j0 = 0; j0 < PAIRS * OUT_PER_PAIR; j0 += GW_THREADS) {
                const int j = j0 + tid;
                const int pr = j / OUT_PER_PAIR, x = (j % OUT_PER_PAIR) * 16;
                const int rc = pr / HEADS_T, ht = pr % HEADS_T;
                const int row = ((rc % 64) / 32) * 128 + (2 * s + rc / 64) * 32 + (rc % 32);
                const float mult = mults[pr];
                v4f q[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) q[k] = *(const v4f *)(vals + pr * PITCH + x + 4 * k);
                uint32_t w[4];
#pragma unroll
                for (int k = 0; k < 4; ++k) w[k] = pack_i8x4(q[k].x * mult, q[k].y * mult, q[k].z * mult, q[k].w * mult, low);
                if (row < rows_here && (int)(n0 / EP_D) + ht < e.n_heads)
                    *(v4i *)(dst_base + ((uint32_t)row * (uint32_t)e.dst_pitch + (uint32_t)(ht * EP_D + x))) = v4i{(int)w[0], (int)w[1], (int)w[2], (int)w[3]};
            }
            __syncthreads(); // before the next step overwrites the values
        }
    } else if constexpr (MODE == TSATTN_MM_ADD_SCALED) {
        // state += sum * scale: the 32 old values of a block of rows are requested together, then updated and stored
        // (element by element every store would have to be waited for before the next load, which it might overlap;
        // with one workgroup per compute unit nothing else runs under those waits)
#pragma clang fp contract(off)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float old[2][16];
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int64_t n = n0 + wn * 64 + j * 32 + li;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t m = m0 + wm * 128 + i * 32 + 8 * (r / 4) + 4 * g + (r & 3);
                    old[j][r] = (n < p.n && m < p.m) ? ((const float *)p.out)[m * p.out_pitch + n] : 0.0f;
                }
            }
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int64_t n = n0 + wn * 64 + j * 32 + li;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t m = m0 + wm * 128 + i * 32 + 8 * (r / 4) + 4 * g + (r & 3);
                    if (n < p.n && m < p.m) ((float *)p.out)[m * p.out_pitch + n] = old[j][r] + (float)acc[i][j][r] * p.scale;
                }
            }
        }
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) {
                const int64_t n = n0 + wn * 64 + j * 32 + li;
                if (n >= p.n) continue;
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int64_t m = m0 + wm * 128 + i * 32 + 8 * (r / 4) + 4 * g + (r & 3);
                    if (m < p.m) store_out<MODE>(p, m, n, acc[i][j][r]);
                }
            }
    }
}

// ---- few rows ---------------------------------------------------------------------------------------------------
// One workgroup per 32 weight rows and part of K.  K is walked in slabs of 1024 bytes: every wave instruction asks
// for 1 KiB of consecutive memory of one row (the weights are read once, so what matters is that HBM sees long
// consecutive requests and that many are in flight), the slab goes through LDS, and there the rows are read back the
// way the MFMA wants them (32 bytes of a row per lane and step).  The four waves each take a quarter of the slab
// and add their sums up in LDS.
constexpr int GS_THREADS = 256;
constexpr int GS_WAVES = GS_THREADS / WAVE;
constexpr int GS_BN = 32;      // weight rows per workgroup
constexpr int GS_MB = 4;       // blocks of 32 activation rows handled by this kernel
constexpr int GS_SLAB = 1024;  // bytes of K per slab
constexpr int GS_PITCH = GS_SLAB + 16;
constexpr int GS_LD = 32 * GS_SLAB / 16 / GS_THREADS; // 16-byte chunks per thread and slab: 8

template <int MODE>
__global__ __launch_bounds__(GS_THREADS) void gemm_skinny_kernel(GemmParams p)
{
    __shared__ __attribute__((aligned(16))) uint8_t w_lds[32 * GS_PITCH];
    __shared__ __attribute__((aligned(16))) uint8_t x_lds[32 * GS_PITCH];
    static_assert(GS_MB * 16 * WAVE * 4 <= 32 * GS_PITCH, "the waves' sums are added up in the activations' slab");
    int(*red)[16 * WAVE] = (int(*)[16 * WAVE]) x_lds;
    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid / WAVE;
    const int li = lane & 31, g = lane >> 5;
    const int64_t n0 = (int64_t)blockIdx.x * GS_BN;

    // this workgroup's part of K (blockIdx.y of gridDim.y parts, in whole steps of 64 bytes); with more than one
    // part the sums go to this part's plane of the workspace
    const int all_steps = (int)(p.k / 64);
    const int split_steps = (all_steps + (int)gridDim.y - 1) / (int)gridDim.y;
    const int k_begin = (int)blockIdx.y * split_steps * 64, k_end = min(all_steps, ((int)blockIdx.y + 1) * split_steps) * 64;
    p.out = (uint8_t *)p.out + (int64_t)blockIdx.y * p.split_stride * 4;

    const int n_mb = (int)((p.m + 31) / 32);
    const __amdgpu_buffer_rsrc_t wr = rows_rsrc(p.w + n0 * p.w_pitch, p.n - n0 < GS_BN ? p.n - n0 : GS_BN, p.w_pitch, p.k);
    const __amdgpu_buffer_rsrc_t ar = rows_rsrc(p.a, p.m, p.a_pitch, p.k);
    // chunk i of this thread: row 4*i + wave, bytes 16*lane.. of the slab: one wave instruction = one row's KiB
    v16i acc[GS_MB];
#pragma unroll
    for (int j = 0; j < GS_MB; ++j) acc[j] = v16i{0};

    // the weights of a slab are requested while the slab before it is being multiplied
    auto request_w = [&](int kb, v4i (&dst)[GS_LD]) __attribute__((always_inline)) {
        const bool in_slab = 16 * lane < min(GS_SLAB, k_end - kb);
#pragma unroll
        for (int i = 0; i < GS_LD; ++i) {
            const int row = 4 * i + wave;
            dst[i] = in_slab ? __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(wr, row * (int)p.w_pitch + 16 * lane, kb, 0)) : v4i{0, 0, 0, 0};
        }
    };
    v4i rw[GS_LD], rw_next[GS_LD];
    if (k_begin < k_end) request_w(k_begin, rw);
    for (int kb = k_begin; kb < k_end; kb += GS_SLAB) {
        const int slab = min(GS_SLAB, k_end - kb); // bytes of K in this slab, a multiple of 64
        const bool in_slab = 16 * lane < slab;
        const bool more = kb + GS_SLAB < k_end;
#pragma unroll
        for (int j = 0; j < GS_MB; ++j) {
            if (j < n_mb) { // uniform
                v4i rx[GS_LD];
#pragma unroll
                for (int i = 0; i < GS_LD; ++i) {
                    const int row = 32 * j + 4 * i + wave;
                    rx[i] = in_slab ? __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(ar, row * (int)p.a_pitch + 16 * lane, kb, 0)) : v4i{0, 0, 0, 0};
                }
                if (j == 0 && more) request_w(kb + GS_SLAB, rw_next);
                __syncthreads(); // the previous block's reads of x_lds (and, for j == 0, of w_lds) are done
                if (j == 0) {
#pragma unroll
                    for (int i = 0; i < GS_LD; ++i) *(v4i *)(w_lds + (4 * i + wave) * GS_PITCH + 16 * lane) = rw[i];
                }
#pragma unroll
                for (int i = 0; i < GS_LD; ++i) *(v4i *)(x_lds + (4 * i + wave) * GS_PITCH + 16 * lane) = rx[i];
                __syncthreads();
                // this wave's quarter of the slab: steps 4*wave .. 4*wave+3 (those inside the slab)
                const uint8_t *wb = w_lds + li * GS_PITCH + 32 * g, *xb = x_lds + li * GS_PITCH + 32 * g;
#pragma unroll
                for (int u = 0; u < 4; ++u) {
                    const int off = (4 * wave + u) * 64;
                    if (off < slab) { // uniform
                        const v4i w0 = *(const v4i *)(wb + off), w1 = *(const v4i *)(wb + off + 16);
                        const v4i x0 = *(const v4i *)(xb + off), x1 = *(const v4i *)(xb + off + 16);
                        acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w0, x0, acc[j], 0, 0, 0);
                        acc[j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(w1, x1, acc[j], 0, 0, 0);
                    }
                }
            }
        }
        if (more) {
#pragma unroll
            for (int i = 0; i < GS_LD; ++i) rw[i] = rw_next[i];
        }
    }
    // sum the waves' shares in LDS; register r of block j: weight row n0 + 8*(r/4) + 4*g + r%4, activation row 32*j + li
    __syncthreads(); // the slab has been read
    for (int i = tid; i < GS_MB * 16 * WAVE; i += GS_THREADS) (&red[0][0])[i] = 0;
    __syncthreads();
#pragma unroll
    for (int j = 0; j < GS_MB; ++j) {
        if (j < n_mb) {
#pragma unroll
            for (int r = 0; r < 16; ++r) atomicAdd(&red[j][r * WAVE + lane], acc[j][r]);
        }
    }
    __syncthreads();
    for (int r = wave; r < 16; r += GS_WAVES) {
        const int64_t n = n0 + 8 * (r / 4) + 4 * g + (r & 3);
        for (int j = 0; j < n_mb; ++j) {
            const int64_t m = 32 * j + li;
            if (n < p.n && m < p.m) store_out<MODE>(p, m, n, red[j][r * WAVE + lane]);
        }
    }
}

// sums the planes of the workspace and applies the epilogue: one thread per output element
template <int MODE>
__global__ __launch_bounds__(256) void gemm_reduce_kernel(GemmParams p, const int32_t *ws, int n_split)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= p.m * p.n) return;
    int sum = 0;
    for (int s = 0; s < n_split; ++s) sum += ws[s * p.split_stride + i];
    store_out<MODE>(p, i / p.n, i % p.n, sum);
}

template <int MODE>
void launch_mode(const GemmParams &p, hipStream_t st)
{
    if (p.m > 32 * GS_MB) {
        // wide tiles when there are two rounds of them for every compute unit, 128 x 128 tiles otherwise
        const int64_t tiles_n = (p.n + GT_BN - 1) / GT_BN;
        const int64_t wide = ((p.m + GW_BM - 1) / GW_BM) * ((p.n + GW_BN - 1) / GW_BN);
        if (wide >= 512) hipLaunchKernelGGL((gemm_wide_kernel<MODE, 0>), dim3((unsigned)wide), dim3(GW_THREADS), GW_LDS_BYTES, st, p);
        else hipLaunchKernelGGL((gemm_tiled_kernel<MODE, 2>), dim3((unsigned)(((p.m + 127) / 128) * tiles_n)), dim3(GT_THREADS), 0, st, p);
        return;
    }
    hipLaunchKernelGGL((gemm_skinny_kernel<MODE>), dim3((unsigned)((p.n + GS_BN - 1) / GS_BN), 1), dim3(GS_THREADS), 0, st, p);
}

// Few rows: the weights are streamed once and every compute unit has to help.  With 32 weight rows per workgroup
// there are too few workgroups unless K is split as well, which needs room for the parts' sums.  A workgroup walks
// its slabs with the next one's weights on their way, so parts of two and more slabs cost little more than parts of
// one: about one workgroup per compute unit (measured: 1.86 ms per token step of 24 layers against 1.89 with twice as
// many parts and 1.92 with half as many).
int split_for(const GemmParams &p, int64_t room_bytes)
{
    if (p.m > 32 * GS_MB) return 1;
    const int64_t n_tiles = (p.n + GS_BN - 1) / GS_BN;
    int split = 1;
    while (split < 16 && n_tiles * split < 256 && p.k / (split * 2) >= GS_SLAB && (int64_t)(split * 2) * p.m * p.n * 4 <= room_bytes) split *= 2;
    return split;
}

} // namespace

// Once per device, before the first product: the wide-tile kernels use more LDS than a launch may ask for by default.
hipError_t prepare_matmul_i8()
{
    const struct {
        const void *kernel;
        int lds;
    } kernels[] = {{(const void *)gemm_wide_kernel<TSATTN_MM_I32, 0>, gw_lds_bytes(0)},
                   {(const void *)gemm_wide_kernel<TSATTN_MM_F32, 0>, gw_lds_bytes(0)},
                   {(const void *)gemm_wide_kernel<TSATTN_MM_ADD_SCALED, 0>, gw_lds_bytes(0)},
                   {(const void *)gemm_wide_kernel<TSATTN_MM_I32, 64>, gw_lds_bytes(64)},
                   {(const void *)gemm_wide_kernel<TSATTN_MM_I32, 128>, gw_lds_bytes(128)}};
    for (const auto &k : kernels) {
        const hipError_t e = hipFuncSetAttribute(k.kernel, hipFuncAttributeMaxDynamicSharedMemorySize, k.lds);
        if (e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_matmul_i8(const GemmParams &p, hipStream_t st, int *planes_out)
{
    if (p.m <= 0 || p.n <= 0) {
        if (planes_out) *planes_out = 1;
        return hipSuccess;
    }
    if (p.mode == TSATTN_MM_I32_PLANES) {
        // the parts' sums straight into the caller's planes (16 * m * n ints of room by contract)
        const int split = split_for(p, (int64_t)16 * p.m * p.n * 4);
        GemmParams q = p;
        q.split_stride = p.m * p.n;
        if (p.ep_head_dim) {
            // the producer on the result: in the product's own kernel where the wide tiles are used, else after it
            q.ep.src = p.out; q.ep.src_pitch = p.n; q.ep.n_rows = p.m; q.ep.n_heads = (int)(p.n / p.ep_head_dim);
            q.ep.src_planes = split; q.ep.src_plane_stride = p.m * p.n;
            *planes_out = split;
            const int64_t wide = ((p.m + GW_BM - 1) / GW_BM) * ((p.n + GW_BN - 1) / GW_BN);
            // (the epilogue addresses a tile's rows with 32-bit offsets)
            const bool offsets_fit = q.ep.dst_pitch < (1 << 23) && (!q.ep.resid || q.ep.resid_pitch < (1 << 21)) &&
                                     (!q.ep.pos || q.ep.rope_len * p.ep_head_dim * 4 < ((int64_t)1 << 31));
            const bool one_operand = !(q.ep.resid && q.ep.pos); // (registers for the old state or for cos and sin)
            const bool head_group = p.ep_head_dim == 64 || p.ep_head_dim == 128; // (wider groups: the producer's own launch)
            if (p.m > 32 * GS_MB && wide >= 512 && p.ep_dst_dtype == TSATTN_I8 && offsets_fit && one_operand && head_group) {
                if (p.ep_head_dim == 128) hipLaunchKernelGGL((gemm_wide_kernel<TSATTN_MM_I32, 128>), dim3((unsigned)wide), dim3(GW_THREADS), gw_lds_bytes(128), st, q);
                else hipLaunchKernelGGL((gemm_wide_kernel<TSATTN_MM_I32, 64>), dim3((unsigned)wide), dim3(GW_THREADS), gw_lds_bytes(64), st, q);
                return hipGetLastError();
            }
            if (split == 1) launch_mode<TSATTN_MM_I32>(q, st);
            else hipLaunchKernelGGL((gemm_skinny_kernel<TSATTN_MM_I32>), dim3((unsigned)((p.n + GS_BN - 1) / GS_BN), (unsigned)split), dim3(GS_THREADS), 0, st, q);
            const hipError_t e = hipGetLastError();
            if (e != hipSuccess) return e;
            return launch_rope_normalize(q.ep, p.ep_dst_dtype, p.ep_head_dim, true, st);
        }
        if (split == 1) launch_mode<TSATTN_MM_I32>(q, st);
        else hipLaunchKernelGGL((gemm_skinny_kernel<TSATTN_MM_I32>), dim3((unsigned)((p.n + GS_BN - 1) / GS_BN), (unsigned)split), dim3(GS_THREADS), 0, st, q);
        *planes_out = split;
        return hipGetLastError();
    }
    const int split = split_for(p, p.workspace ? p.workspace_bytes : 0);
    if (split > 1) {
        GemmParams q = p;
        q.out = p.workspace;
        q.out_pitch = p.n;
        q.split_stride = p.m * p.n;
        hipLaunchKernelGGL((gemm_skinny_kernel<TSATTN_MM_I32>), dim3((unsigned)((p.n + GS_BN - 1) / GS_BN), (unsigned)split), dim3(GS_THREADS), 0, st, q);
        GemmParams r = p;
        r.split_stride = p.m * p.n;
        const dim3 grid((unsigned)((p.m * p.n + 255) / 256));
        if (p.mode == TSATTN_MM_I32) hipLaunchKernelGGL((gemm_reduce_kernel<TSATTN_MM_I32>), grid, dim3(256), 0, st, r, (const int32_t *)p.workspace, split);
        else if (p.mode == TSATTN_MM_F32) hipLaunchKernelGGL((gemm_reduce_kernel<TSATTN_MM_F32>), grid, dim3(256), 0, st, r, (const int32_t *)p.workspace, split);
        else hipLaunchKernelGGL((gemm_reduce_kernel<TSATTN_MM_ADD_SCALED>), grid, dim3(256), 0, st, r, (const int32_t *)p.workspace, split);
        return hipGetLastError();
    }
    if (p.mode == TSATTN_MM_I32) launch_mode<TSATTN_MM_I32>(p, st);
    else if (p.mode == TSATTN_MM_F32) launch_mode<TSATTN_MM_F32>(p, st);
    else if (p.mode == TSATTN_MM_ADD_SCALED) launch_mode<TSATTN_MM_ADD_SCALED>(p, st);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

} // namespace tsattn
