// Prefill attention for long key ranges (head width 128): the same result as prefill_kernel, organised so that the
// waves' instruction streams hold almost nothing but matrix instructions and the softmax.
//
//  * A small first kernel writes V once as f16 with the row's value scale folded in, transposed ([head][x][token]) and
//    with the tokens of every 16 in the order the matrix instruction wants its keys; the attention kernel then never
//    converts or stores a V element.
//  * K (as it is), that V copy and the key scales go from memory straight into LDS (buffer loads with the LDS flag):
//    no staging registers, no LDS store instructions.  Three stages per operand; a tile is requested two tiles ahead;
//    what has to have landed is waited for by count, then one barrier per 64-key tile.  LDS rows are 128 bytes without
//    padding, their 16-byte chunks permuted by (row / 2) % 8 (applied to the addresses requested from memory) so that
//    the row-per-lane operand reads are free of bank conflicts.
//  * The work on one 32-key sub-tile is spread over three steps of the loop: step T issues K.Q^T of sub-tile T, the
//    softmax of sub-tile T-1 and V^T.P^T of sub-tile T-2, so every step has the same mix of matrix and vector
//    instructions and nothing in a step waits for a result of the same step.
//  * The weights are taken against the zero vector's logit 0 without looking at the logits (no maximum, no branch);
//    their sum comes from a 4x4x4 matrix instruction with a matrix of ones (each lane gets the sum of its own four
//    weights).  Only if a weight overflowed f16 (a logit 16 above the zero vector's: the sum is then not finite) does
//    the workgroup repeat its rows on a slower path that tracks the maximum and rescales.
// Semantics: gpt/compute/gpt_cpu.cpp:391-441 with the 8-bit operand handling of gpt/compute/gpt_att_fp8.cuh:139-152 /
// gpt_att_fp16.cuh:184-189; the transposed V copy is what the reference makes too (Transpose, gpt_cuda.cu:501).
#include <type_traits>

#include "prefill_common.hpp"

namespace tsattn {

constexpr int PL_BN = 64;     // keys per staged tile
constexpr int PL_STAGES = 3;
constexpr int PL_D = 128;
constexpr int PL_K_BYTES = PL_BN * PL_D;      // a K tile: 64 rows of 128 bytes
constexpr int PL_V_BYTES = PL_D * PL_BN * 2;  // a V tile: 128 rows (x) of 64 keys, f16
constexpr int PL_KS_BYTES = PL_BN * 4;
constexpr int PL_K_OFF = 0;
constexpr int PL_V_OFF = PL_K_OFF + PL_STAGES * PL_K_BYTES;
constexpr int PL_KS_OFF = PL_V_OFF + PL_STAGES * PL_V_BYTES;
constexpr int PL_RED_OFF = PL_KS_OFF + PL_STAGES * PL_KS_BYTES;
constexpr int PL_SPARE_OFF = PL_RED_OFF + 64;
constexpr int PL_LDS_BYTES = PL_SPARE_OFF + PL_KS_BYTES;

// ---- the V copy ---------------------------------------------------------------------------------------------------
// vt[(head * 128 + x) * vt_pitch + VT_PAD + pos(t)] = f16(v[t][head][x] * vs[head][t]), pos(t) = t with bits 2 and 3
// exchanged (positions 0..15 of every 16 tokens hold tokens 0-3, 8-11, 4-7, 12-15: the keys the two halves of a wave
// feed into one V^T.P^T instruction).  Columns that stand for no token are zero.  The column of a token is shifted by
// VT_PAD = 32 so that the tile of V a loop iteration needs (the second sub-tile of one K tile and the first of the next)
// starts at a multiple of 64 columns.
//
// With a constant query scale the same kernel also writes the key scales times that constant, the logit scale and the
// optional global key scale (ksq[head][t], pitch ksq_pitch): the attention kernel then has one multiply per logit.
template <int DTYPE>
__global__ __launch_bounds__(256) void widen_v_kernel(const uint8_t *v, int64_t v_pitch, const float *vs, int64_t scale_pitch, float vs_const,
                                                      int n_tokens, _Float16 *vt, int64_t vt_pitch, const float *ks, float ks_mult,
                                                      const float *k_global_scale, float *ksq, int64_t ksq_pitch)
{
    constexpr int D = PL_D, PITCH = 64 + 8; // halves per LDS row: 16-byte aligned, rows 36 banks apart
    __shared__ __attribute__((aligned(16))) _Float16 tile[D * PITCH];
    const int tid = threadIdx.x, head = blockIdx.y;
    const int col0 = blockIdx.x * 64; // first column of this block; column c holds position c - VT_PAD
    if (ksq && tid < 64 && col0 + tid < n_tokens) {
        const float m = k_global_scale ? ks_mult * *k_global_scale : ks_mult;
        ksq[(int64_t)head * ksq_pitch + col0 + tid] = ks[(int64_t)head * scale_pitch + col0 + tid] * m;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i) {
        const int ch = tid + i * 256;   // 64 columns x 8 chunks of 16 bytes
        const int c = ch >> 3, part = ch & 7;
        const int pos = col0 + c - VT_PAD;
        const int t = (pos & ~12) | ((pos & 4) << 1) | ((pos & 8) >> 1); // the token that sits at this position
        v4i raw = v4i{0, 0, 0, 0};
        float s = 0.0f;
        if (pos >= 0 && t < n_tokens) {
            raw = *(const v4i *)(v + (int64_t)t * v_pitch + head * D + part * 16);
            s = vs ? vs[(int64_t)head * scale_pitch + t] : vs_const;
        }
        const int w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float f[4];
            if (DTYPE == TSATTN_I8) {
#pragma unroll
                for (int b = 0; b < 4; ++b) f[b] = (float)(int8_t)((w[j] >> (8 * b)) & 0xff);
            } else {
                const v2f lo = __builtin_amdgcn_cvt_pk_f32_fp8(w[j], false), hi = __builtin_amdgcn_cvt_pk_f32_fp8(w[j], true);
                f[0] = lo[0]; f[1] = lo[1]; f[2] = hi[0]; f[3] = hi[1];
            }
#pragma unroll
            for (int b = 0; b < 4; ++b) tile[(part * 16 + j * 4 + b) * PITCH + c] = (_Float16)(f[b] * s);
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int ch = tid + i * 256;   // 128 rows x 8 chunks of 8 columns
        const int x = ch >> 3, part = ch & 7;
        const v4i w = *(const v4i *)(tile + x * PITCH + part * 8);
        if (col0 + part * 8 < vt_pitch) *(v4i *)(vt + ((int64_t)head * D + x) * vt_pitch + col0 + part * 8) = w;
    }
}

typedef __attribute__((address_space(3))) void *pl_lds_ptr;

// QS_CONST: the query scale is one number for all rows and has been multiplied into the key scales the kernel reads
// (p.ks then points at the plane the first kernel wrote, or p.ks_const holds the product).
template <int DTYPE, int D, bool OUT_F16, bool QS_CONST>
__global__ __launch_bounds__(PF_THREADS, 2) void prefill_long_kernel(PrefillParams p, int n_qtiles)
{
    static_assert(D == PL_D, "written for a head width of 128");
    typedef QkMma<DTYPE, D> Qk;
    constexpr int DT = D / 32;
    constexpr int QS = Qk::STEPS;
    extern __shared__ __attribute__((aligned(1024))) uint8_t pl_lds[];

    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = __builtin_amdgcn_readfirstlane(tid / WAVE);
    const int qi = lane & 31; // query column of this lane
    const int g = lane >> 5;  // which half of the contraction this lane feeds
    int head, tile;
    wg_locate(p.map, blockIdx.x, gridDim.x, n_qtiles, head, tile);
    const int q0 = tile * PF_BM + wave * 32;
    const int from = q0 + qi;
    const bool row_ok = from < p.n_tokens;
    const int64_t hoff = (int64_t)head * D;

    // ---- spans: the workgroup's key range and the extremes of this wave's 32 spans (as in prefill_kernel) -------
    bool w_all_have_keys = false;
    int w_min_a = 0, w_max_a = 0, w_min_b = 0, w_max_b = 0, b_min_a = 0, b_max_b = 0;
    const bool have_summary = p.span_tiles != nullptr;
    if (have_summary) {
        typedef __attribute__((address_space(4))) const int32_t *const_i32_ptr;
        const const_i32_ptr t = (const_i32_ptr)(p.span_tiles + (int64_t)tile * SPAN_TILE_INTS);
        const const_i32_ptr w = t + SPAN_TILE_WAVE0 + wave * SPAN_TILE_WAVE_INTS;
        b_min_a = t[SPAN_TILE_MIN_A];
        b_max_b = t[SPAN_TILE_MAX_B];
        w_min_a = w[0];
        w_max_a = w[1];
        w_min_b = w[2];
        w_max_b = w[3];
        w_all_have_keys = w[4] != 0;
    }
    int sp_a = 1, sp_b = 0;
    if (row_ok) {
        sp_a = p.span_start[from];
        sp_b = p.span_finish[from];
    }
    Qk qk;
    if (row_ok) qk.load_q(p.q + (int64_t)from * p.q_pitch + hoff, g);
    else qk.clear_q();
    float qs = row_ok ? (p.qs ? p.qs[(int64_t)head * p.scale_pitch + from] : p.qs_const) : 0.0f;
    int *const red = (int *)(pl_lds + PL_RED_OFF);
    if (!have_summary) {
        const bool hk = sp_b >= sp_a;
        w_all_have_keys = __all(hk);
        w_min_a = hk ? sp_a : 0x7fffffff, w_max_a = hk ? sp_a : -1;
        w_min_b = hk ? sp_b : 0x7fffffff, w_max_b = hk ? sp_b : -1;
        for (int o = 16; o > 0; o >>= 1) {
            w_min_a = min(w_min_a, __shfl_xor(w_min_a, o, WAVE));
            w_max_a = max(w_max_a, __shfl_xor(w_max_a, o, WAVE));
            w_min_b = min(w_min_b, __shfl_xor(w_min_b, o, WAVE));
            w_max_b = max(w_max_b, __shfl_xor(w_max_b, o, WAVE));
        }
        if (lane == 0) {
            red[wave] = w_min_a;
            red[PF_WAVES + wave] = w_max_b;
        }
        __syncthreads();
        b_min_a = red[0], b_max_b = red[PF_WAVES];
        for (int w = 1; w < PF_WAVES; ++w) {
            b_min_a = min(b_min_a, red[w]);
            b_max_b = max(b_max_b, red[PF_WAVES + w]);
        }
        __syncthreads(); // red is used again at the end
    }
    // the logit scale goes into the query's scale: the key scales arrive in LDS as they are in memory
    if (!QS_CONST) {
        float ads = att_dot_scale(D);
        if (p.k_global_scale) ads *= *p.k_global_scale;
        qs *= ads;
    } else {
        qs = 1.0f; // (rows past the end have zero operands)
    }
    w_min_a = __builtin_amdgcn_readfirstlane(w_min_a);
    w_max_a = __builtin_amdgcn_readfirstlane(w_max_a);
    w_min_b = __builtin_amdgcn_readfirstlane(w_min_b);
    w_max_b = __builtin_amdgcn_readfirstlane(w_max_b);

    v16f o_acc[DT];
    v4f l4;     // this lane's share of the weight sum (all four registers hold it)
    float m_ref; // reference maximum: the zero vector's logit unless the slow path raises it
    bool redo = false;

    if (b_max_b >= b_min_a) {
        const int kb_first = __builtin_amdgcn_readfirstlane((b_min_a / PL_BN) * PL_BN);
        const int n_tiles = __builtin_amdgcn_readfirstlane((b_max_b - kb_first) / PL_BN + 1);
        const int n_sub = 2 * n_tiles;
        // this wave's sub-tiles (32 keys each, counted from kb_first): needed [ua, ub], inside every span [fa, fb]
        int ua = 1, ub = 0, fa = 1, fb = 0;
        if (w_max_b >= w_min_a) {
            ua = (w_min_a - kb_first) >> 5;
            ub = (w_max_b - kb_first) >> 5;
            if (w_all_have_keys) {
                fa = (w_max_a - kb_first + 31) >> 5;
                fb = ((w_min_b + 1 - kb_first) >> 5) - 1;
            }
        }
        // Iterations [it_f0, it_f1): both steps complete and no span cuts through them -- K.Q^T of sub-tiles 2 it and
        // 2 it + 1, softmax of 2 it - 1 and 2 it (inside every span), V^T.P^T of 2 it - 2 and 2 it - 1.  Before and after
        // them, up to it_last (the iteration of the wave's last V^T.P^T), the steps look at the spans; a key outside a
        // row's span -- a sub-tile the wave does not need at all included -- gets the weight zero.
        int it_f0 = max((ua + 3) >> 1, (fa + 2) >> 1);
        int it_f1 = min(fb >> 1, (ub - 1) >> 1) + 1; // one past the last
        int it_last = (ub + 2) >> 1;
        if (ub < ua) it_last = -1, it_f0 = it_f1 = 0;
        else if (fb < fa || it_f1 <= it_f0) it_f0 = it_f1 = 0;
        it_last = min(it_last, n_tiles);
        it_f0 = __builtin_amdgcn_readfirstlane(it_f0);
        it_f1 = __builtin_amdgcn_readfirstlane(it_f1);
        it_last = __builtin_amdgcn_readfirstlane(it_last);
        // in span <=> (unsigned)(key - sp_a) <= sp_b - sp_a; per lane the keys are first key + 4 g + {0..3, 8..11, ...}
        const int mask_lo = sp_b >= sp_a ? sp_a - 4 * g : 0x40000000;
        const unsigned mask_w = sp_b >= sp_a ? (unsigned)(sp_b - sp_a) : 0u;

        // ---- requests: memory -> LDS ------------------------------------------------------------------------
        auto rsrc = [](const void *base, int64_t bytes) {
            const uint32_t n = bytes <= 0 ? 0u : (bytes > 0xffffffffll ? 0xffffffffu : (uint32_t)bytes);
            return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)n, 0x00020000);
        };
        // (the launcher has checked that the byte offsets inside K fit 31 bits)
        const __amdgpu_buffer_rsrc_t kr = rsrc(p.k + hoff + (int64_t)kb_first * p.k_pitch, (int64_t)(p.n_tokens - 1 - kb_first) * p.k_pitch + D);
        const int64_t vt_row_bytes = p.vt_pitch * 2;
        const __amdgpu_buffer_rsrc_t vr = rsrc((const uint8_t *)p.vt + (int64_t)head * D * vt_row_bytes + (int64_t)kb_first * 2, D * vt_row_bytes - (int64_t)kb_first * 2);
        const bool ks_plane = p.ks != nullptr;
        const float *ks_ptr = ks_plane ? p.ks + (int64_t)head * p.ks_pitch + kb_first : nullptr;
        const __amdgpu_buffer_rsrc_t ksr = rsrc(ks_ptr, ks_plane ? (int64_t)(p.n_tokens - kb_first) * 4 : 0);
        if (!ks_plane && tid < PL_STAGES * PL_BN) ((float *)(pl_lds + PL_KS_OFF))[tid] = p.ks_const; // (the first barrier of the loop follows)
        // A request of one wave fills 1 KiB of LDS = 8 rows of 128 bytes: lane L writes position L % 8 of row L / 8,
        // which holds chunk (L % 8) ^ ((row / 2) % 8) of the row.
        int kd_voff[2], vd_voff[4];
#pragma unroll
        for (int j = 0; j < 2; ++j) {
            const int row = 8 * (2 * wave + j) + (lane >> 3);
            kd_voff[j] = row * (int)p.k_pitch + (((lane & 7) ^ ((row >> 1) & 7)) << 4);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int row = 8 * (4 * wave + j) + (lane >> 3);
            vd_voff[j] = row * (int)vt_row_bytes + (((lane & 7) ^ ((row >> 1) & 7)) << 4);
        }
        const int64_t k_step = (int64_t)PL_BN * p.k_pitch;
        uint32_t k_soff = 0, v_soff = 0, s_soff = 0;
        auto request_tile = [&](int dma_stage) __attribute__((always_inline)) { // the next tile in sequence -> that stage
            uint8_t *const kd = pl_lds + PL_K_OFF + dma_stage * PL_K_BYTES + wave * 2048;
            uint8_t *const vd = pl_lds + PL_V_OFF + dma_stage * PL_V_BYTES + wave * 4096;
#pragma unroll
            for (int j = 0; j < 2; ++j) __builtin_amdgcn_raw_ptr_buffer_load_lds(kr, (pl_lds_ptr)(kd + j * 1024), 16, kd_voff[j], (int)k_soff, 0, 0);
#pragma unroll
            for (int j = 0; j < 4; ++j) __builtin_amdgcn_raw_ptr_buffer_load_lds(vr, (pl_lds_ptr)(vd + j * 1024), 16, vd_voff[j], (int)v_soff, 0, 0);
            // every wave asks for the tile's 64 key scales (the same bytes to the same place: one count for all waves);
            // a constant key scale sits in all three stages from the start, and the request (of zeros: its descriptor
            // is empty) goes to a spare corner, so that the loop has no branch and one count to wait for
            __builtin_amdgcn_raw_ptr_buffer_load_lds(ksr, (pl_lds_ptr)(pl_lds + (ks_plane ? PL_KS_OFF + dma_stage * PL_KS_BYTES : PL_SPARE_OFF)), 4, lane * 4, (int)s_soff, 0, 0);
            k_soff += (uint32_t)k_step;
            v_soff += PL_BN * 2;
            s_soff += PL_BN * 4;
        };
#define PL_WAIT_TILE asm volatile("s_waitcnt vmcnt(7)" ::: "memory") // all but the newest tile's seven requests have landed
#define PL_WAIT_ALL asm volatile("s_waitcnt vmcnt(0)" ::: "memory")
#define PL_BARRIER                                          \
    do {                                                    \
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  \
        __builtin_amdgcn_s_barrier();                       \
        asm volatile("" ::: "memory");                      \
    } while (0)
#define PL_FENCE __builtin_amdgcn_sched_barrier(0)

        // ---- operand reads -------------------------------------------------------------------------------------
        const int swz = (qi >> 1) & 7;
        const int row_off = qi * 128;
        // K: row qi of the sub-tile, chunks Qk's step st needs; V: row x = dt * 32 + qi, the chunk of 8 keys
        int kx[4], vx[2][2];
        if (DTYPE == TSATTN_E4M3) {
#pragma unroll
            for (int i = 0; i < 4; ++i) kx[i] = row_off + ((((i >> 1) * 4 + 2 * g + (i & 1)) ^ swz) << 4); // step i/2, half i%2
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) kx[i] = row_off + (((2 * i + g) ^ swz) << 4); // step i
        }
#pragma unroll
        for (int sv = 0; sv < 2; ++sv)
#pragma unroll
            for (int grp = 0; grp < 2; ++grp) vx[sv][grp] = row_off + (((4 * sv + 2 * grp + g) ^ swz) << 4);
        typedef typename Qk::kop_t kop_t;
        auto read_k = [&](const uint8_t *kt, kop_t (&kop)[QS]) __attribute__((always_inline)) { // kt: the sub-tile's first row
            if constexpr (DTYPE == TSATTN_E4M3) {
#pragma unroll
                for (int st = 0; st < QS; ++st) {
                    const v4i a = *(const v4i *)(kt + kx[2 * st]), b = *(const v4i *)(kt + kx[2 * st + 1]);
                    kop[st] = v8i{a.x, a.y, a.z, a.w, b.x, b.y, b.z, b.w};
                }
            } else {
#pragma unroll
                for (int st = 0; st < QS; ++st) kop[st] = *(const v4i *)(kt + kx[st]);
            }
        };

        // ---- state of the pipeline ---------------------------------------------------------------------------------
        typename Qk::acc_t acc[2]; // acc[T & 1]: K.Q^T of sub-tile T
        v2h pw[2][8];              // pw[T & 1]: the weights of sub-tile T, two keys per register
        v8h va[2 * DT];            // V^T operands of the next step's V^T.P^T
        v4f ksv[4];                // key scales of the next step's softmax
        const v4h ones4 = v4h{(_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f};

        auto pv_mfma = [&](int m, const v2h (&pc)[8]) __attribute__((always_inline)) { // one of the eight V^T.P^T of a step
            const int grp = m / DT, dt = m % DT;
            const v8h pb = v8h{pc[4 * grp][0], pc[4 * grp][1], pc[4 * grp + 1][0], pc[4 * grp + 1][1], pc[4 * grp + 2][0], pc[4 * grp + 2][1], pc[4 * grp + 3][0], pc[4 * grp + 3][1]};
            o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[m], pb, o_acc[dt], 0, 0, 0);
        };
        auto sum_mfma = [&](int i, const v2h (&pc)[8]) __attribute__((always_inline)) { // four of a step: weights 4 i .. 4 i + 3 of the lane
            l4 = __builtin_amdgcn_mfma_f32_4x4x4f16(ones4, v4h{pc[2 * i][0], pc[2 * i][1], pc[2 * i + 1][0], pc[2 * i + 1][1]}, l4, 0, 0, 0);
        };
        auto read_v = [&](int m, const uint8_t *vt_tile, int sv) __attribute__((always_inline)) { // operand m of sub-tile half sv of a V tile
            const int grp = m / DT, dt = m % DT;
            va[m] = *(const v8h *)(vt_tile + dt * 4096 + vx[sv][grp]);
        };

        // Weights of two keys (accumulator registers 2 pr, 2 pr + 1) against the zero vector's logit: no maximum.
        // MASKED: a weight whose key lies outside the row's span becomes zero (rel_lo: the span's start relative to this
        // lane's first key of the sub-tile; span_w: its length - 1, or a bound no key meets for a row without keys).
        auto weights_pair = [&](auto masked_tag, const typename Qk::acc_t &a, int pr, int rel_lo, unsigned span_w, v2h &out) __attribute__((always_inline)) {
            constexpr bool MASKED = decltype(masked_tag)::value;
            const int r = 2 * pr;
            const v4f kq = ksv[pr >> 1];
            const float k0 = kq[2 * (pr & 1)], k1 = kq[2 * (pr & 1) + 1];
            float p0 = fast_exp2(QS_CONST ? Qk::to_float(a, r) * k0 : (Qk::to_float(a, r) * k0) * qs);
            float p1 = fast_exp2(QS_CONST ? Qk::to_float(a, r + 1) * k1 : (Qk::to_float(a, r + 1) * k1) * qs);
            if (MASKED) {
                const int off = 8 * (r >> 2) + (r & 3); // key of register r relative to the lane's first key
                p0 = ((unsigned)(off - rel_lo) <= span_w) ? p0 : 0.0f;
                p1 = ((unsigned)(off + 1 - rel_lo) <= span_w) ? p1 : 0.0f;
            }
            out = v2h{(_Float16)p0, (_Float16)p1};
        };

        // ---- one step ------------------------------------------------------------------------------------------------
        // s = T & 1.  kt: K sub-tile T; ks_next: key scales of sub-tile T (for the next step); v_next: the V tile that holds
        // sub-tile T - 1 in half s (for the next step).  MASKED: the softmax of sub-tile T - 1 (first key key0) looks at the
        // spans.  Order: four V^T.P^T, K.Q^T, four V^T.P^T, with the weight sums and eight pairs of weights between them.
        auto fast_step = [&](auto s_tag, auto masked_tag, int key0, const uint8_t *kt, const float *ks_next, const uint8_t *v_next) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value;
            typename Qk::acc_t &accC = acc[s ^ 1];
            const v2h(&pc)[8] = pw[s];
            v2h(&pn)[8] = pw[s ^ 1];
            const int rel_lo = mask_lo - key0;
            kop_t kop[QS];
            read_k(kt, kop);
            // what the previous step asked for (this step's V^T operands and key scales) has arrived once only the four
            // reads above are outstanding: one wait here instead of one in front of every first use
            __builtin_amdgcn_s_waitcnt(0xc07f | (4 << 8)); // lgkmcnt(4), the other counters untouched
            PL_FENCE;
            int pr = 0;
            typename Qk::acc_t accN = {0};
            auto pair = [&]() __attribute__((always_inline)) {
                weights_pair(masked_tag, accC, pr, rel_lo, mask_w, pn[pr]);
                ++pr;
                if ((pr & 1) == 0) ksv[(pr >> 1) - 1] = *(const v4f *)(ks_next + 8 * ((pr >> 1) - 1));
                PL_FENCE;
            };
#pragma unroll
            for (int m = 0; m < 2 * DT; ++m) {
                pv_mfma(m, pc);
                read_v(m, v_next, s);
                if (m & 1) sum_mfma(m >> 1, pc);
                PL_FENCE;
                if (m == 0 || m == 2 || m == 3 || m == 4 || m == 6 || m == 7) pair();
                if (m == DT - 1) {
#pragma unroll
                    for (int st = 0; st < QS; ++st) {
                        accN = qk.step(kop[st], st, accN);
                        PL_FENCE;
                        if (st == QS / 2 - 1 || st == QS - 1) pair();
                    }
                }
            }
            acc[s] = accN;
            PL_FENCE;
        };

        // ---- one step in general form: any of the three parts may be missing, spans may cut through the sub-tile ---------
        // SAFE: track the maximum and rescale (the repeat after an overflow).  T: the step; kt, ks_next, v_next as above.
        auto weights_masked = [&](auto safe_tag, const typename Qk::acc_t &a, int key0, v2h (&out)[8]) __attribute__((always_inline)) {
            constexpr bool SAFE = decltype(safe_tag)::value;
            const int rel_a = sp_a - key0 - 4 * g;           // span start relative to this lane's first key
            const unsigned span_w = (unsigned)(sp_b - sp_a); // in-span <=> (unsigned)(off - rel_a) <= span_w
            const bool has_keys = sp_b >= sp_a;
            // (no array of logits is kept: on the slow path they are computed twice, for the maximum and for the weights)
            auto logit = [&](int r) __attribute__((always_inline)) -> float {
                const int off = 8 * (r >> 2) + (r & 3);
                const bool in_span = (unsigned)(off - rel_a) <= span_w && has_keys;
                const float tv = (Qk::to_float(a, r) * ksv[r >> 2][r & 3]) * qs - m_ref;
                return in_span ? tv : -INFINITY;
            };
            if (SAFE) {
                float tmax = -INFINITY;
#pragma unroll
                for (int r = 0; r < 16; ++r) tmax = fmaxf(tmax, logit(r));
                // the two lanes of a query exchange their maxima only if some lane of the wave is over the threshold
                if (__any(tmax > PF_RESCALE_THRESHOLD)) {
                    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
                    const float shift = (tmax > PF_RESCALE_THRESHOLD) ? tmax : 0.0f;
                    const float alpha = fast_exp2(-shift);
                    m_ref += shift;
                    l4 *= alpha;
#pragma unroll
                    for (int i = 0; i < DT; ++i) o_acc[i] *= alpha;
                }
            }
#pragma unroll
            for (int x = 0; x < 8; ++x) out[x] = v2h{(_Float16)fast_exp2(logit(2 * x)), (_Float16)fast_exp2(logit(2 * x + 1))};
        };
        auto general_step = [&](auto s_tag, auto safe_tag, int T, const uint8_t *kt, const float *ks_next, const uint8_t *v_next) __attribute__((always_inline)) {
            constexpr int s = decltype(s_tag)::value;
            if (T - 2 >= ua && T - 2 <= ub) {
#pragma unroll
                for (int m = 0; m < 2 * DT; ++m) pv_mfma(m, pw[s]);
#pragma unroll
                for (int i = 0; i < 4; ++i) sum_mfma(i, pw[s]);
            }
#pragma unroll
            for (int m = 0; m < 2 * DT; ++m) read_v(m, v_next, s);
            if (T - 1 >= ua && T - 1 <= ub) weights_masked(safe_tag, acc[s ^ 1], kb_first + 32 * (T - 1), pw[s ^ 1]);
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) ksv[c4] = *(const v4f *)(ks_next + 8 * c4);
            if (T >= ua && T <= ub && T < n_sub) {
                kop_t kop[QS];
                read_k(kt, kop);
                typename Qk::acc_t accN = {0};
#pragma unroll
                for (int st = 0; st < QS; ++st) accN = qk.step(kop[st], st, accN);
                acc[s] = accN;
            }
        };

        // ---- the tile loop -------------------------------------------------------------------------------------------
        // Iteration `it` holds steps 2 it and 2 it + 1 and reads K tile it, the key scales of tile it and V tile it (sub-tiles
        // 2 it - 1 and 2 it); tile it + 2 is requested at its start into the stage tile it - 1 was read from.  There is one
        // iteration more than K tiles: the last V^T.P^T trail the last K.Q^T by two steps.
        auto run = [&](auto safe_tag) __attribute__((always_inline)) {
            constexpr bool SAFE = decltype(safe_tag)::value;
#pragma unroll
            for (int i = 0; i < DT; ++i) o_acc[i] = v16f{0};
            l4 = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            m_ref = 0.0f;
#pragma unroll
            for (int i = 0; i < 2; ++i) {
#pragma unroll
                for (int x = 0; x < 8; ++x) pw[i][x] = v2h{(_Float16)0.0f, (_Float16)0.0f};
                acc[i] = typename Qk::acc_t{0};
            }
#pragma unroll
            for (int m = 0; m < 2 * DT; ++m) va[m] = v8h{0};
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) ksv[c4] = v4f{0.0f, 0.0f, 0.0f, 0.0f};
            k_soff = 0, v_soff = 0, s_soff = 0;
            request_tile(0);
            request_tile(1);
            PL_WAIT_TILE;
            PL_BARRIER;
            int stage = 0, it = 0;
            // Separate loops rather than one with branches: each keeps only what it needs in registers, and a loop body
            // without branches keeps the order it was written in.  Each loop is unrolled over the three stages, entered at
            // the current one, so that every LDS address is a lane constant plus an immediate.
            auto one = [&](auto mode_tag, int st_k, int st_dma) __attribute__((always_inline)) { // st_k: a constant in the unrolled loop
                constexpr int MODE = decltype(mode_tag)::value; // 0: slow path, 1: spans looked at, 2: common, 3: nothing to compute
                const uint8_t *const kt = pl_lds + PL_K_OFF + st_k * PL_K_BYTES;
                const uint8_t *const vt_tile = pl_lds + PL_V_OFF + st_k * PL_V_BYTES;
                const float *const ksp = (const float *)(pl_lds + PL_KS_OFF + st_k * PL_KS_BYTES) + 4 * g;
                request_tile(st_dma); // (past the last tile: rows that are never computed with, or zeros past the end)
                if (MODE == 0) {
                    general_step(std::integral_constant<int, 0>{}, std::true_type{}, 2 * it, kt, ksp, vt_tile);
                    general_step(std::integral_constant<int, 1>{}, std::true_type{}, 2 * it + 1, kt + 32 * 128, ksp + 32, vt_tile);
                } else if (MODE == 1) {
                    const int key0 = kb_first + 64 * it - 32; // first key of sub-tile 2 it - 1
                    fast_step(std::integral_constant<int, 0>{}, std::true_type{}, key0, kt, ksp, vt_tile);
                    fast_step(std::integral_constant<int, 1>{}, std::true_type{}, key0 + 32, kt + 32 * 128, ksp + 32, vt_tile);
                } else if (MODE == 2) {
                    fast_step(std::integral_constant<int, 0>{}, std::false_type{}, 0, kt, ksp, vt_tile);
                    fast_step(std::integral_constant<int, 1>{}, std::false_type{}, 0, kt + 32 * 128, ksp + 32, vt_tile);
                }
                PL_WAIT_TILE;
                PL_BARRIER;
            };
            auto iterations = [&](auto mode_tag, int end) __attribute__((always_inline)) {
                constexpr int MODE = decltype(mode_tag)::value;
                // the common path runs three iterations at a time from stage 0 on, every LDS address then being a lane constant
                // plus an immediate; single iterations in front of and behind that
                for (; it < end && (MODE != 2 || stage != 0 || it + PL_STAGES > end); ++it) {
                    one(mode_tag, stage, stage == 0 ? 2 : stage - 1);
                    stage = stage == PL_STAGES - 1 ? 0 : stage + 1;
                }
                if (MODE == 2) {
                    for (; it + PL_STAGES <= end; it += PL_STAGES) {
                        one(mode_tag, 0, 2);
                        one(mode_tag, 1, 0);
                        one(mode_tag, 2, 1);
                    }
                    for (; it < end; ++it) {
                        one(mode_tag, stage, stage == 0 ? 2 : stage - 1);
                        stage = stage == PL_STAGES - 1 ? 0 : stage + 1;
                    }
                }
            };
            if (SAFE) {
                iterations(std::integral_constant<int, 0>{}, n_tiles + 1);
            } else {
                iterations(std::integral_constant<int, 1>{}, it_f0);
                iterations(std::integral_constant<int, 2>{}, it_f1);
                iterations(std::integral_constant<int, 1>{}, it_last + 1);
                iterations(std::integral_constant<int, 3>{}, n_tiles + 1);
            }
            PL_WAIT_ALL; // nothing may still be on its way into LDS
        };
        run(std::false_type{});
        // a weight that overflowed f16 leaves a sum that is not finite: then all four waves repeat on the slow path
        {
            float l = l4[0];
            l += __shfl_xor(l, 32, WAVE);
            const int any_bad = __any(!(l <= 3.0e38f)) ? 1 : 0; // (asked of all lanes, before the branch)
            if (lane == 0) red[wave] = any_bad;
            PL_BARRIER;
            redo = (red[0] | red[1] | red[2] | red[3]) != 0;
            PL_BARRIER;
        }
        if (redo) run(std::true_type{});
#undef PL_FENCE
    } else {
#pragma unroll
        for (int i = 0; i < DT; ++i) o_acc[i] = v16f{0};
        l4 = v4f{0.0f, 0.0f, 0.0f, 0.0f};
        m_ref = 0.0f;
    }

    // ---- epilogue: add the zero vector's weight, normalise, store through LDS as whole rows ------------------------
    float l_all = l4[0];
    l_all += __shfl_xor(l_all, 32, WAVE);
    l_all += fast_exp2(-m_ref);
    const float inv = 1.0f / l_all;
    if (p.out) {
        uint8_t *const stage = pl_lds + wave * (32 * (D * 2 + 16)); // the tile loop has ended with a barrier
        if constexpr (OUT_F16) {
            constexpr int OUT_PITCH = D * 2 + 16;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                for (int c4 = 0; c4 < 4; ++c4) {
                    const int dcol = dt * 32 + 8 * c4 + 4 * g;
                    const v4h hv = v4h{(_Float16)(o_acc[dt][c4 * 4 + 0] * inv), (_Float16)(o_acc[dt][c4 * 4 + 1] * inv),
                                       (_Float16)(o_acc[dt][c4 * 4 + 2] * inv), (_Float16)(o_acc[dt][c4 * 4 + 3] * inv)};
                    *(v4h *)(stage + qi * OUT_PITCH + dcol * 2) = hv;
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // this wave's values are in LDS (nobody else reads them)
            constexpr int ROW_CHUNKS = D * 2 / 16;
#pragma unroll
            for (int it = 0; it < 32 * ROW_CHUNKS / WAVE; ++it) {
                const int id = it * WAVE + lane;
                const int c = id % ROW_CHUNKS, r = id / ROW_CHUNKS;
                const v4i w = *(const v4i *)(stage + r * OUT_PITCH + c * 16);
                if (q0 + r < p.n_tokens) *(v4i *)((uint8_t *)p.out + (int64_t)(q0 + r) * p.out_pitch + hoff * 2 + c * 16) = w;
            }
        } else {
            constexpr int HALF = D / 2, OUT_PITCH = HALF * 4 + 16;
            static_assert(32 * OUT_PITCH <= 32 * (D * 2 + 16), "a wave's corner holds half rows of floats");
            constexpr int ROW_CHUNKS = HALF * 4 / 16;
#pragma unroll
            for (int half = 0; half < 2; ++half) {
#pragma unroll
                for (int dt = half * (DT / 2); dt < (half + 1) * (DT / 2); ++dt) {
#pragma unroll
                    for (int c4 = 0; c4 < 4; ++c4) {
                        const int dcol = dt * 32 + 8 * c4 + 4 * g - half * HALF;
                        *(v4f *)(stage + qi * OUT_PITCH + dcol * 4) =
                            v4f{o_acc[dt][c4 * 4 + 0] * inv, o_acc[dt][c4 * 4 + 1] * inv, o_acc[dt][c4 * 4 + 2] * inv, o_acc[dt][c4 * 4 + 3] * inv};
                    }
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
                for (int it = 0; it < 32 * ROW_CHUNKS / WAVE; ++it) {
                    const int id = it * WAVE + lane;
                    const int c = id % ROW_CHUNKS, r = id / ROW_CHUNKS;
                    const v4i w = *(const v4i *)(stage + r * OUT_PITCH + c * 16);
                    if (q0 + r < p.n_tokens) *(v4i *)((uint8_t *)p.out + (int64_t)(q0 + r) * p.out_pitch + (hoff + half * HALF) * 4 + c * 16) = w;
                }
                asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // read before the second half overwrites it
            }
        }
    }
    if (row_ok && p.sum_weight_log && g == 0) p.sum_weight_log[(int64_t)head * p.scale_pitch + from] = m_ref + __log2f(l_all);
}

// Bytes of scratch: the f16 copy of V, then (used with a constant query scale only) a plane of scaled key scales.
static int64_t ksq_pitch_of(int64_t n_tokens) { return (n_tokens + 63) / 64 * 64; }
size_t prefill_long_workspace_bytes(int64_t n_tokens, int n_heads, int head_dim)
{
    if (head_dim != PL_D || n_tokens <= 0) return 0;
    return (size_t)n_heads * PL_D * (size_t)prefill_long_vt_pitch(n_tokens) * 2 + (size_t)n_heads * (size_t)ksq_pitch_of(n_tokens) * 4;
}

template <int DTYPE, bool OUT_F16, bool QS_CONST>
static hipError_t launch_long_do(const PrefillParams &p_in, hipStream_t st)
{
    PrefillParams p = p_in;
    const int n_qtiles = (int)((p.n_tokens + PF_BM - 1) / PF_BM);
    p.ks_pitch = p.scale_pitch;
    p.map = wg_plan(n_qtiles, p.n_heads, PL_D, PF_BM, p.period_tiles, 3); // K as it is, V as f16
    auto kernel = prefill_long_kernel<DTYPE, PL_D, OUT_F16, QS_CONST>;
    const dim3 wgrid((unsigned)(p.vt_pitch / 64), (unsigned)p.n_heads);
    float *ksq = nullptr;
    const int64_t ksq_pitch = ksq_pitch_of(p.n_tokens);
    const float ks_mult = p.qs_const * att_dot_scale(PL_D);
    if (QS_CONST && p.ks) ksq = (float *)((uint8_t *)p.vt + (size_t)p.n_heads * PL_D * (size_t)p.vt_pitch * 2);
    hipLaunchKernelGGL((widen_v_kernel<DTYPE>), wgrid, dim3(256), 0, st, p.v, p.v_pitch, p.vs, p.scale_pitch, p.vs_const, p.n_tokens, (_Float16 *)p.vt, p.vt_pitch,
                       p.ks, ks_mult, p.k_global_scale, ksq, ksq_pitch);
    if (QS_CONST) {
        if (p.ks) {
            p.ks = ksq;
            p.ks_pitch = ksq_pitch;
        } else {
            if (p.k_global_scale) return hipErrorInvalidValue; // filtered out by launch_prefill_long: the product would need the device value
            p.ks_const = p.ks_const * ks_mult;
        }
    }
    hipLaunchKernelGGL(kernel, dim3((unsigned)(n_qtiles * p.n_heads)), dim3(PF_THREADS), PL_LDS_BYTES, st, p, n_qtiles);
    return hipGetLastError();
}

template <int DTYPE, bool OUT_F16, bool QS_CONST>
static hipError_t allow_lds()
{
    return hipFuncSetAttribute((const void *)prefill_long_kernel<DTYPE, PL_D, OUT_F16, QS_CONST>, hipFuncAttributeMaxDynamicSharedMemorySize, PL_LDS_BYTES);
}

// The kernels use more LDS than a launch may ask for by default: said once per device (at handle creation), so that no
// launch has to, also not the first one under a graph capture.
hipError_t prepare_prefill_long()
{
    hipError_t e = allow_lds<TSATTN_E4M3, true, true>();
    if (e == hipSuccess) e = allow_lds<TSATTN_E4M3, true, false>();
    if (e == hipSuccess) e = allow_lds<TSATTN_E4M3, false, true>();
    if (e == hipSuccess) e = allow_lds<TSATTN_E4M3, false, false>();
    if (e == hipSuccess) e = allow_lds<TSATTN_I8, true, true>();
    if (e == hipSuccess) e = allow_lds<TSATTN_I8, true, false>();
    if (e == hipSuccess) e = allow_lds<TSATTN_I8, false, true>();
    if (e == hipSuccess) e = allow_lds<TSATTN_I8, false, false>();
    return e;
}

hipError_t launch_prefill_long(const PrefillParams &p, int dtype, int out_dtype, hipStream_t st)
{
    const bool f16 = out_dtype == TSATTN_OUT_F16;
    // one multiply per logit where the query scale is a constant (and, with a constant key scale too, no device value
    // would be needed on the host to form the product)
    const bool qs_const = p.qs == nullptr && !(p.ks == nullptr && p.k_global_scale != nullptr);
    if (dtype == TSATTN_E4M3) {
        if (qs_const) return f16 ? launch_long_do<TSATTN_E4M3, true, true>(p, st) : launch_long_do<TSATTN_E4M3, false, true>(p, st);
        return f16 ? launch_long_do<TSATTN_E4M3, true, false>(p, st) : launch_long_do<TSATTN_E4M3, false, false>(p, st);
    }
    if (qs_const) return f16 ? launch_long_do<TSATTN_I8, true, true>(p, st) : launch_long_do<TSATTN_I8, false, true>(p, st);
    return f16 ? launch_long_do<TSATTN_I8, true, false>(p, st) : launch_long_do<TSATTN_I8, false, false>(p, st);
}

} // namespace tsattn
