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
#include <type_traits>

#include "prefill_common.hpp"

namespace tsattn {

constexpr int PF_BN = 64;         // keys per tile
constexpr int PF_KT = PF_BN / 32; // 32-key sub-tiles per tile
constexpr int PF_SHORT_KEYS = 192; // key range a workgroup may handle without the tile loop (see the kernel)

template <int D>
struct PfLayout {
    static constexpr int K_PITCH = D + 16;                  // bytes; 16-lane b128 reads hit 64 distinct banks
    static constexpr int V_PITCH = (D == 128) ? 320 : 192;  // bytes of an f16 row; row stride = 16 banks (mod 64)
    static constexpr int K_BYTES = PF_BN * K_PITCH;
    static constexpr int V_BYTES = PF_BN * V_PITCH;
};

// 16 bytes of one V row -> 16 halves scaled by the row's value scale.
// e4m3: v_cvt_scalef32_pk_f16_fp8 (exact widening, unit scale) then a packed f16 multiply.
// int8: byte b -> f16 bits 0x6400 | (b ^ 0x80) = 1024 + (b + 128); a packed add of -1152 gives b
//       exactly, then the packed multiply.
// SCALED = false: the values as they are (a scale that is one number for all rows is applied to the result instead).
template <int DTYPE, bool SCALED = true>
__device__ inline void widen_v(v4i raw, float vs, v8h &lo, v8h &hi)
{
    const _Float16 vsh = (_Float16)vs;
    const v2h vs2 = v2h{vsh, vsh};
    int w[4] = {raw.x, raw.y, raw.z, raw.w};
    v2h h[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        if (DTYPE == TSATTN_I8) {
            const unsigned u = (unsigned)w[i] ^ 0x80808080u;
            const unsigned a = __builtin_amdgcn_perm(u, 0x64646464u, 0x00050004u);
            const unsigned b = __builtin_amdgcn_perm(u, 0x64646464u, 0x00070006u);
            const v2h off = v2h{(_Float16)-1152.0f, (_Float16)-1152.0f};
            h[2 * i] = __builtin_bit_cast(v2h, a) + off;
            h[2 * i + 1] = __builtin_bit_cast(v2h, b) + off;
        } else {
            h[2 * i] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[i], 1.0f, false);
            h[2 * i + 1] = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w[i], 1.0f, true);
        }
        if (SCALED) {
            h[2 * i] *= vs2;
            h[2 * i + 1] *= vs2;
        }
    }
    lo = v8h{h[0][0], h[0][1], h[1][0], h[1][1], h[2][0], h[2][1], h[3][0], h[3][1]};
    hi = v8h{h[4][0], h[4][1], h[5][0], h[5][1], h[6][0], h[6][1], h[7][0], h[7][1]};
}

// one 32-bit word (4 values) of the same: two packed pairs
template <int DTYPE, bool SCALED = true>
__device__ inline void widen_v_word(int w, v2h vs2, v2h &h0, v2h &h1)
{
    if (DTYPE == TSATTN_I8) {
        const unsigned u = (unsigned)w ^ 0x80808080u;
        const unsigned a = __builtin_amdgcn_perm(u, 0x64646464u, 0x00050004u);
        const unsigned b = __builtin_amdgcn_perm(u, 0x64646464u, 0x00070006u);
        const v2h off = v2h{(_Float16)-1152.0f, (_Float16)-1152.0f};
        h0 = __builtin_bit_cast(v2h, a) + off;
        h1 = __builtin_bit_cast(v2h, b) + off;
    } else {
        h0 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false);
        h1 = __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true);
    }
    if (SCALED) {
        h0 *= vs2;
        h1 *= vs2;
    }
}

typedef __attribute__((address_space(3))) v4s *lds_v4s_ptr;

// MULTI: rows may have several spans (p.n_parts arrays of them); otherwise the one-span kernel, which needs fewer registers.
// CONSTS >= 1: the query scale is one number for all rows (TScale's own model: VEC_SCALE, gpt_att_fp8.cuh:137); it is
// multiplied into the key scales as they are staged and a logit costs one multiply-add instead of a multiply and one.
// CONSTS == 2: the value scale is one number too (cpu_infer.cpp:454): V is widened as it is -- exactly -- and the
// result multiplied by the scale.
template <int DTYPE, int D, bool OUT_F16, bool SLOPE, bool DUMP, bool MULTI, int CONSTS>
__global__ __launch_bounds__(PF_THREADS, (D == 64 && !MULTI) ? 3 : 2) void prefill_kernel(PrefillParams p, int n_qtiles)
{
    typedef PfLayout<D> L;
    typedef QkMma<DTYPE, D> Qk;
    constexpr bool QS_CONST = CONSTS >= 1, VS_CONST = CONSTS == 2;
    constexpr int DT = D / 32;                               // 32-row tiles of O^T
    constexpr int CHUNKS = D / 16;                           // 16-byte chunks per 8-bit row
    constexpr int NLD = (PF_BN * CHUNKS + PF_THREADS - 1) / PF_THREADS;
    constexpr bool LD_ALL = (PF_BN * CHUNKS) % PF_THREADS == 0; // every thread owns NLD chunks       // 16-byte chunks per thread per tile

    // One LDS block carved two ways.  Tile loop: two K tiles, two widened V tiles, two sets of key scales.
    // Short key ranges (d = 64, at most PF_SHORT_KEYS keys for the whole workgroup): every widened V row and key
    // scale of the range at once.
    constexpr int LOOP_BYTES = 2 * L::K_BYTES + 2 * L::V_BYTES + 2 * PF_BN * 4;
    constexpr int SHORT_BYTES = PF_SHORT_KEYS * L::V_PITCH + PF_SHORT_KEYS * 4;
    constexpr bool HAS_SHORT = (D == 64) && !DUMP;
    // the common-tile loop with ALiBi only where it fits into the registers without spilling
    constexpr bool FAST_LOOP = !DUMP && (!SLOPE || (D == 128 && DTYPE == TSATTN_E4M3 && !MULTI)); // (with ALiBi and a loop over parts it would spill)
    constexpr int LDS_BYTES = (HAS_SHORT && SHORT_BYTES > LOOP_BYTES) ? SHORT_BYTES : LOOP_BYTES;
    // the fused KVProduct exists where the reference has one: behind int8 attention with an f32 result (cpu_infer.cpp:509-511)
    constexpr bool KV_FUSED = DTYPE == TSATTN_I8 && !OUT_F16 && !DUMP;
    __shared__ __attribute__((aligned(16))) uint8_t lds_raw[LDS_BYTES];
    auto k_lds = [&](int b) -> uint8_t * { return lds_raw + b * L::K_BYTES; };
    auto v_lds = [&](int b) -> uint8_t * { return lds_raw + 2 * L::K_BYTES + b * L::V_BYTES; };
    auto ks_lds = [&](int b) -> float * { return (float *)(lds_raw + 2 * L::K_BYTES + 2 * L::V_BYTES) + b * PF_BN; };
    __shared__ int red_lds[2 * PF_WAVES];

    const int tid = threadIdx.x;
    const int lane = tid & (WAVE - 1);
    const int wave = tid / WAVE;
    const int qi = lane & 31; // query column of this lane
    const int g = lane >> 5;  // which half of the contraction this lane feeds
    // Ask for every kernel argument the prologue needs in one go: left to itself the compiler fetches them where
    // they are first used, which chains five scalar-load round trips in front of the first K/V request.
#define PF_TOUCH(x) asm volatile("" ::"s"(x))
    PF_TOUCH(p.q); PF_TOUCH(p.k); PF_TOUCH(p.v); PF_TOUCH(p.q_pitch); PF_TOUCH(p.k_pitch); PF_TOUCH(p.v_pitch);
    PF_TOUCH(p.qs); PF_TOUCH(p.ks); PF_TOUCH(p.vs); PF_TOUCH(p.scale_pitch); PF_TOUCH(p.span_start); PF_TOUCH(p.span_finish);
    PF_TOUCH(p.span_tiles); PF_TOUCH(p.n_tokens); PF_TOUCH(p.n_heads); PF_TOUCH(p.k_global_scale);
    PF_TOUCH(p.map.period_tiles); PF_TOUCH(p.map.period_group); PF_TOUCH(p.map.units_per_xcd); PF_TOUCH(p.map.hg_shift);
    PF_TOUCH(p.map.by_qtiles.d); PF_TOUCH(p.map.by_qtiles.m); PF_TOUCH(p.map.by_group_wgs.d); PF_TOUCH(p.map.by_group_wgs.m);
    PF_TOUCH(p.map.by_group_units.d); PF_TOUCH(p.map.by_group_units.m); PF_TOUCH(p.map.by_seqs.d); PF_TOUCH(p.map.by_seqs.m);
    PF_TOUCH(p.qs_const); PF_TOUCH(p.ks_const); PF_TOUCH(p.vs_const); PF_TOUCH(p.slope); PF_TOUCH(p.out); PF_TOUCH(p.out_pitch);
#undef PF_TOUCH
    // which (head, query tile) this workgroup computes: divisions by launch constants whose reciprocals the host
    // has prepared
    int head, tile;
    wg_locate(p.map, blockIdx.x, gridDim.x, n_qtiles, head, tile);
    const int q0 = tile * PF_BM + wave * 32;
    const int from = q0 + qi;
    const bool row_ok = from < p.n_tokens;
    const int64_t hoff = (int64_t)head * D;

    // ---- query operand and per-row constants -----------------------------------------------------------------
    Qk qk;
    if (row_ok) qk.load_q(p.q + (int64_t)from * p.q_pitch + hoff, g);
    else qk.clear_q();
    const float qs = QS_CONST ? 1.0f : (row_ok ? (p.qs ? p.qs[(int64_t)head * p.scale_pitch + from] : p.qs_const) : 0.0f);

    float ads = att_dot_scale(D);
    if (p.k_global_scale) ads *= *p.k_global_scale;
    if (QS_CONST) ads *= p.qs_const; // (rows past the end have zero operands: their logits are zero either way)
    // a logit from an accumulator, its key's staged scale and what is added to it
    auto logit = [&](float a, float k, float bias) __attribute__((always_inline)) { return QS_CONST ? fmaf(a, k, bias) : fmaf(a * k, qs, bias); };

    v16f o_acc[DT];
#pragma unroll
    for (int i = 0; i < DT; ++i) o_acc[i] = v16f{0};
    float m_ref = 0.0f; // reference maximum: starts at the zero vector's logit
    float l = 0.0f, l2 = 0.0f; // this lane's share of the weight sum (its 32 of every 64 keys), in two chains

    // Rows with several spans (TAttentionInfo allows them, gpt/att/att.h:24-47; the reference's kernel walks a list of
    // key ranges per query block, att.h:95-181, gpt_att_fp8.cuh:103-112): part i of the span arrays holds every row's
    // i-th span (an empty one where a row has fewer), and the parts are walked one after the other into the same
    // accumulators -- one softmax over all keys of all spans, a key in c spans counted c times, as the CPU loop over
    // the spans does (gpt_cpu.cpp:405-436).
    const int n_parts = MULTI ? p.n_parts : 1;
    for (int part = 0; part < n_parts; ++part) {
    const int32_t *const part_start = p.span_start + (int64_t)part * p.span_part_stride;
    const int32_t *const part_finish = p.span_finish + (int64_t)part * p.span_part_stride;
    // ---- spans --------------------------------------------------------------------------------
    // What the loop needs to know about the spans: the workgroup's key range and the extremes of this wave's 32
    // spans.  Either read from the caller's summary (scalar loads, so K and V can be requested as soon as they
    // return, without waiting for the per-row spans) or reduced below from the rows' spans (shuffles, LDS, a barrier).
    bool w_all_have_keys = false;
    int w_min_a = 0, w_max_a = 0, w_min_b = 0, w_max_b = 0, b_min_a = 0, b_max_b = 0;
    const bool have_summary = p.span_tiles != nullptr;
    if (have_summary) {
        typedef __attribute__((address_space(4))) const int32_t *const_i32_ptr;
        const const_i32_ptr t = (const_i32_ptr)(p.span_tiles + ((int64_t)part * n_qtiles + tile) * SPAN_TILE_INTS);
        const const_i32_ptr w = t + SPAN_TILE_WAVE0 + __builtin_amdgcn_readfirstlane(wave) * SPAN_TILE_WAVE_INTS;
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
        sp_a = part_start[from];
        sp_b = part_finish[from];
    }
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
            red_lds[wave] = w_min_a;
            red_lds[PF_WAVES + wave] = w_max_b;
        }
        __syncthreads();
        b_min_a = red_lds[0], b_max_b = red_lds[PF_WAVES];
        for (int w = 1; w < PF_WAVES; ++w) {
            b_min_a = min(b_min_a, red_lds[w]);
            b_max_b = max(b_max_b, red_lds[PF_WAVES + w]);
        }
    }

    if (b_max_b >= b_min_a) {
        // the same in every lane; said explicitly so that everything derived from them stays in scalar registers
        const int kb_first = __builtin_amdgcn_readfirstlane((b_min_a / PF_BN) * PF_BN);
        const int n_tiles = __builtin_amdgcn_readfirstlane((b_max_b - kb_first) / PF_BN + 1);

        // ---- staging: global -> registers -> LDS (K as is; V widened to f16 * row scale) -----------------
        // Loads go through buffer descriptors plus a scalar byte offset that advances by one tile per load, so the
        // per-lane offsets are loop constants and no vector address arithmetic is left in the loop.  A
        // descriptor ends at the last token's row: rows past it read as zeros (their logits are masked); on this
        // hardware generation the range check counts the scalar offset too.
        v4i rk[NLD], rv[NLD];
        float rvs[NLD], rks = 0.0f;
        int k_voff[NLD], v_voff[NLD];
#pragma unroll
        for (int i = 0; i < NLD; ++i) {
            const int ch = tid + i * PF_THREADS;
            const int r = ch / CHUNKS, c = ch % CHUNKS;
            k_voff[i] = r * (int)p.k_pitch + c * 16;
            v_voff[i] = r * (int)p.v_pitch + c * 16;
        }
        const int64_t k_step = (int64_t)PF_BN * p.k_pitch, v_step = (int64_t)PF_BN * p.v_pitch;
        const uint8_t *k_ptr = p.k + hoff + (int64_t)kb_first * p.k_pitch;
        const uint8_t *v_ptr = p.v + hoff + (int64_t)kb_first * p.v_pitch;
        // bytes from the tile's first row to the end of this head's part of the last row
        int64_t k_left = (int64_t)(p.n_tokens - 1 - kb_first) * p.k_pitch + D;
        int64_t v_left = (int64_t)(p.n_tokens - 1 - kb_first) * p.v_pitch + D;
        const float *vs_ptr = p.vs ? p.vs + (int64_t)head * p.scale_pitch + kb_first : nullptr;
        const float *ks_ptr = p.ks ? p.ks + (int64_t)head * p.scale_pitch + kb_first : nullptr;
        const int64_t s_left = (int64_t)(p.n_tokens - kb_first) * 4;
        auto rsrc = [](const void *base, int64_t bytes) {
            const uint32_t n = bytes <= 0 ? 0u : (bytes > 0xffffffffll ? 0xffffffffu : (uint32_t)bytes);
            return __builtin_amdgcn_make_buffer_rsrc(const_cast<void *>(base), 0, (int)n, 0x00020000);
        };
        __amdgpu_buffer_rsrc_t kr = rsrc(k_ptr, k_left), vr = rsrc(v_ptr, v_left);
        const __amdgpu_buffer_rsrc_t ksr = rsrc(ks_ptr, s_left), vsr = rsrc(vs_ptr, s_left);
        // scalar byte offsets of the next tile to load, relative to the descriptors' bases
        uint32_t k_soff = 0, v_soff = 0, s_soff = 0;
        auto load_tile = [&]() __attribute__((always_inline)) { // loads the next tile in sequence
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                if (!LD_ALL && tid + i * PF_THREADS >= PF_BN * CHUNKS) break;
                rk[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(kr, k_voff[i], (int)k_soff, 0));
                rv[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(vr, v_voff[i], (int)v_soff, 0));
            }
            if (vs_ptr) {
#pragma unroll
                for (int i = 0; i < NLD; ++i) {
                    const int r = (tid + i * PF_THREADS) / CHUNKS;
                    rvs[i] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(vsr, r * 4, (int)s_soff, 0));
                }
            } else {
#pragma unroll
                for (int i = 0; i < NLD; ++i) rvs[i] = p.vs_const;
            }
            // lanes beyond the tile's 64 keys read past it harmlessly (zeros past the end)
            if (ks_ptr) rks = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ksr, (tid & (PF_BN - 1)) * 4, (int)s_soff, 0));
            else rks = p.ks_const;
            k_soff += (uint32_t)k_step;
            v_soff += (uint32_t)v_step;
            s_soff += PF_BN * 4;
            // far into a very long key range the 32-bit offsets are folded back into the bases
            if ((k_soff | v_soff) >= 0x40000000u) {
                k_ptr += k_soff; k_left -= k_soff; k_soff = 0;
                v_ptr += v_soff; v_left -= v_soff; v_soff = 0;
                kr = rsrc(k_ptr, k_left);
                vr = rsrc(v_ptr, v_left);
            }
        };
        auto store_tile = [&](int buf) __attribute__((always_inline)) {
#pragma unroll
            for (int i = 0; i < NLD; ++i) {
                const int ch = tid + i * PF_THREADS;
                if (!LD_ALL && ch >= PF_BN * CHUNKS) break;
                const int r = ch / CHUNKS, c = ch % CHUNKS;
                *(v4i *)(k_lds(buf) + r * L::K_PITCH + c * 16) = rk[i];
                v8h lo, hi;
                widen_v<DTYPE, !VS_CONST>(rv[i], rvs[i], lo, hi);
                *(v8h *)(v_lds(buf) + r * L::V_PITCH + c * 32) = lo;
                *(v8h *)(v_lds(buf) + r * L::V_PITCH + c * 32 + 16) = hi;
            }
            if (tid < PF_BN) ks_lds(buf)[tid] = rks * ads;
        };

        // V^T operands (A of the P.V MFMA) of one group: keys kt*32 + 16*i + 4*g + {0..3} and the same + 8
        const int i16 = lane & 15, dh = (lane >> 4) & 1;
        v8h va[2][DT];
        auto vload_rows = [&](int slot, const uint8_t *rows16) __attribute__((always_inline)) { // rows16: the first of 16 consecutive V rows in LDS
            const int key0 = 4 * g + (i16 >> 2);
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const uint8_t *vb = rows16 + key0 * L::V_PITCH + (dt * 32 + 16 * dh + 4 * (i16 & 3)) * 2;
                v4s a0 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)(vb));
                v4s a1 = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_ptr)(vb + 8 * L::V_PITCH));
                va[slot][dt] = __builtin_bit_cast(v8h, __builtin_shufflevector(a0, a1, 0, 1, 2, 3, 4, 5, 6, 7));
            }
        };
        auto vload = [&](int slot, int grp, int buf) { vload_rows(slot, v_lds(buf) + grp * 16 * L::V_PITCH); };

        // ---- one 32-key sub-tile: weights from the accumulators of K.Q^T, then V^T.P^T ---------------------------
        // ksp: the sub-tile's 32 key scales in LDS; vrows: its 32 widened V rows in LDS; key0: its first key.
        // Key of accumulator register r: key0 + 8*(r/4) + 4*g + r%4.
        //
        // Weights, general form: any mix of rows; exact maximum, and the reference maximum is raised (accumulators
        // rescaled) when a logit is more than the threshold above it.
        auto weights_general = [&](const typename Qk::acc_t &acc, const float *ksp, int key0, v2h (&pp)[8], float &s0, float &s1) __attribute__((always_inline)) {
            const int rel_a = sp_a - key0 - 4 * g;           // span start relative to this lane's first key
            const unsigned span_w = (unsigned)(sp_b - sp_a); // in-span <=> (unsigned)(off - rel_a) <= span_w
            const bool has_keys = sp_b >= sp_a;
            const float dist0 = (float)(from - key0 - 4 * g);
            float t[16];
            float tmax = -INFINITY;
            const float base = SLOPE ? -(p.slope * dist0) - m_ref : -m_ref;
            float bias = base; // base + slope * off, advanced key by key
            const float slope5 = p.slope * 5.0f;
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) {
                v4f ksv = *(const v4f *)(ksp + 8 * c4 + 4 * g);
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int r = c4 * 4 + j;
                    const int off = 8 * c4 + j;
                    const bool in_span = (unsigned)(off - rel_a) <= span_w && has_keys;
                    if (DUMP) {
                        if (in_span) {
                            ((float *)p.dbg)[((int64_t)head * p.n_tokens + from) * p.dbg_pitch + key0 + off + 4 * g] = Qk::bits(acc, r);
                        }
                    }
                    float tv = logit(Qk::to_float(acc, r), ksv[j], bias);
                    if (SLOPE) bias += (j == 3) ? slope5 : p.slope;
                    tv = in_span ? tv : -INFINITY;
                    t[r] = tv;
                    tmax = fmaxf(tmax, tv);
                }
            }
            // the two lanes of a query exchange their maxima only if some lane of the wave is over the threshold
            if (__any(tmax > PF_RESCALE_THRESHOLD)) {
                tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
                const float shift = (tmax > PF_RESCALE_THRESHOLD) ? tmax : 0.0f;
                const float alpha = fast_exp2(-shift);
                m_ref += shift;
                l *= alpha;
                l2 *= alpha;
#pragma unroll
                for (int i = 0; i < DT; ++i) o_acc[i] *= alpha;
#pragma unroll
                for (int r = 0; r < 16; ++r) t[r] -= shift;
            }
            s0 = 0.0f;
            s1 = 0.0f;
#pragma unroll
            for (int x = 0; x < 8; ++x) {
                const float p0 = fast_exp2(t[2 * x]);
                const float p1 = fast_exp2(t[2 * x + 1]);
                pp[x] = v2h{(_Float16)p0, (_Float16)p1};
                s0 += p0;
                s1 += p1;
            }
        };
        // Weights with fewer instructions for the usual edge cases: every row of the wave has keys and at most one
        // end of the spans cuts through the sub-tile (LOW: some span starts after its first key; HIGH: some span
        // ends before its last).  No maximum is computed; a masked weight is zeroed after the exponential (one
        // compare against a per-lane bound and one select).  The caller checks the weight sum.
        auto weights_quick = [&](auto low_tag, auto high_tag, const typename Qk::acc_t &acc, const float *ksp, int key0, v2h (&pp)[8], float &s0, float &s1) __attribute__((always_inline)) {
            constexpr bool LOW = decltype(low_tag)::value, HIGH = decltype(high_tag)::value;
            const int lo = sp_a - key0 - 4 * g, hi = sp_b - key0 - 4 * g; // in span <=> lo <= off <= hi
            const float dist0 = (float)(from - key0 - 4 * g);
            const float base = SLOPE ? -(p.slope * dist0) - m_ref : -m_ref;
            s0 = 0.0f;
            s1 = 0.0f;
            float bias = base; // base + slope * off, advanced key by key (no per-key constants in registers)
            const float slope5 = p.slope * 5.0f;
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) {
                const v4f ksv = *(const v4f *)(ksp + 8 * c4 + 4 * g);
                float w[4];
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int off = 8 * c4 + j;
                    const float tv = logit(Qk::to_float(acc, c4 * 4 + j), ksv[j], bias);
                    if (SLOPE) bias += (j == 3) ? slope5 : p.slope;
                    float pw = fast_exp2(tv);
                    if (LOW) pw = (lo <= off) ? pw : 0.0f;
                    if (HIGH) pw = (hi >= off) ? pw : 0.0f;
                    w[j] = pw;
                }
                s0 += w[0];
                s1 += w[1];
                s0 += w[2];
                s1 += w[3];
                pp[2 * c4] = v2h{(_Float16)w[0], (_Float16)w[1]};
                pp[2 * c4 + 1] = v2h{(_Float16)w[2], (_Float16)w[3]};
            }
        };
        // The form is chosen by what the wave's spans do inside [key0, key0 + 31]; the matrix part is common.
        auto sub_tile = [&](const typename Qk::acc_t &acc, const float *ksp, const uint8_t *vrows, int key0) __attribute__((always_inline)) {
            constexpr float SUM_LIMIT = 256.0f; // = 2^PF_RESCALE_THRESHOLD: one weight above it is enough
            vload_rows(0, vrows);
            vload_rows(1, vrows + 16 * L::V_PITCH);
            v2h pp[8];
            float s0 = 0.0f, s1 = 0.0f;
            const bool low = w_max_a > key0, high = w_min_b < key0 + 31;
            bool general = DUMP || !w_all_have_keys || (low && high);
            if (!general) {
                if (low) weights_quick(std::true_type{}, std::false_type{}, acc, ksp, key0, pp, s0, s1);
                else if (high) weights_quick(std::false_type{}, std::true_type{}, acc, ksp, key0, pp, s0, s1);
                else weights_quick(std::false_type{}, std::false_type{}, acc, ksp, key0, pp, s0, s1);
                general = __any(!(s0 + s1 <= SUM_LIMIT)); // a logit far above the reference (or an overflowed sum)
            }
            if (general) weights_general(acc, ksp, key0, pp, s0, s1);
            l += s0;
            l2 += s1;
            // O^T += V^T . P^T in two groups of DT MFMAs (16 keys each)
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const v8h pb = v8h{pp[4 * i][0], pp[4 * i][1], pp[4 * i + 1][0], pp[4 * i + 1][1], pp[4 * i + 2][0], pp[4 * i + 2][1], pp[4 * i + 3][0], pp[4 * i + 3][1]};
#pragma unroll
                for (int dt = 0; dt < DT; ++dt) o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[i][dt], pb, o_acc[dt], 0, 0, 0);
            }
        };

        // ---- one 64-key tile for this wave's 32 queries ---------------------------------------------------
        // General form: any mix of rows, one 32-key sub-tile at a time (few live registers; a sub-tile outside
        // every span of the wave is skipped, which for a short window is one in four).
        auto compute_tile = [&](int buf, int kb) __attribute__((always_inline)) {
#pragma unroll
            for (int kt = 0; kt < PF_KT; ++kt) {
                if (kb + kt * 32 + 31 < w_min_a || kb + kt * 32 > w_max_b) continue;
                const typename Qk::acc_t acc = qk.mma(k_lds(buf) + (kt * 32 + qi) * L::K_PITCH, g);
                sub_tile(acc, ks_lds(buf) + kt * 32, v_lds(buf) + kt * 32 * L::V_PITCH, kb + kt * 32);
            }
        };

        // ---- the common tile: every key inside every span of the wave ------------------------------------
        // Written so that matrix and vector instructions alternate in the instruction stream (a wave issues
        // in order: vector work placed between two MFMAs runs while the first one executes):
        //   block 1: K.Q^T of both 32-key sub-tiles; the weights of sub-tile 0 overlap the MFMAs of sub-tile 1
        //   block 2: V^T.P^T of sub-tile 0 overlaps the weights of sub-tile 1
        //   block 3: V^T.P^T of sub-tile 1 overlaps the staging (widening, LDS stores) of the next tile
        // Weights are computed against the reference maximum without looking at the logits' maximum; if a
        // sub-tile's weight sum shows that a logit was more than the threshold above it, the sub-tile is redone
        // on the slow path with a raised reference.
        constexpr float PF_SUM_LIMIT = 256.0f; // = 2^PF_RESCALE_THRESHOLD: one weight above it is enough to exceed it
        // weights of four keys (accumulator registers 4*c4 .. 4*c4+3)
        // nbase: minus the reference maximum plus, with ALiBi, the term of the quarter's first key; advanced here
        // to the next quarter's first key (+8 keys)
        auto weights_quarter = [&](const typename Qk::acc_t &acc, int c4, v4f ksv, float &nbase, v2h &pa, v2h &pb, float &s0, float &s1) __attribute__((always_inline)) {
            const int r = 4 * c4;
            float b1 = nbase, b2 = nbase, b3 = nbase;
            if (SLOPE) {
                b1 = nbase + p.slope;
                b2 = b1 + p.slope;
                b3 = b2 + p.slope;
            }
            const float p0 = fast_exp2(logit(Qk::to_float(acc, r), ksv[0], nbase));
            const float p1 = fast_exp2(logit(Qk::to_float(acc, r + 1), ksv[1], b1));
            const float p2 = fast_exp2(logit(Qk::to_float(acc, r + 2), ksv[2], b2));
            const float p3 = fast_exp2(logit(Qk::to_float(acc, r + 3), ksv[3], b3));
            if (SLOPE) nbase = b3 + 5.0f * p.slope;
            s0 += p0;
            s1 += p1;
            s0 += p2;
            s1 += p3;
            pa = v2h{(_Float16)p0, (_Float16)p1};
            pb = v2h{(_Float16)p2, (_Float16)p3};
        };
        auto weights_sub_rescale = [&](const typename Qk::acc_t &acc, const float *ksp, float bias0, v8h &pa, v8h &pb, float &s0, float &s1) __attribute__((always_inline)) {
            float xs[16];
            float tmax = -INFINITY;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const float bias = SLOPE ? bias0 + p.slope * (float)(8 * (r / 4) + (r & 3)) : bias0;
                xs[r] = logit(Qk::to_float(acc, r), ksp[8 * (r / 4) + (r & 3)], bias);
                tmax = fmaxf(tmax, xs[r]);
            }
            tmax = fmaxf(tmax, __shfl_xor(tmax, 32, WAVE));
            const float shift = (tmax > PF_RESCALE_THRESHOLD) ? tmax : 0.0f;
            const float alpha = fast_exp2(-shift);
            m_ref += shift;
            l *= alpha;
            l2 *= alpha;
#pragma unroll
            for (int i = 0; i < DT; ++i) o_acc[i] *= alpha;
            s0 = 0.0f;
            s1 = 0.0f;
            v2h pp[8];
#pragma unroll
            for (int r = 0; r < 16; r += 2) {
                const float p0 = fast_exp2(xs[r] - shift), p1 = fast_exp2(xs[r + 1] - shift);
                s0 += p0;
                s1 += p1;
                pp[r / 2] = v2h{(_Float16)p0, (_Float16)p1};
            }
            pa = v8h{pp[0][0], pp[0][1], pp[1][0], pp[1][1], pp[2][0], pp[2][1], pp[3][0], pp[3][1]};
            pb = v8h{pp[4][0], pp[4][1], pp[5][0], pp[5][1], pp[6][0], pp[6][1], pp[7][0], pp[7][1]};
        };
#define PF_FENCE __builtin_amdgcn_sched_barrier(0)
        auto fast_tile = [&](int buf, int kb) __attribute__((always_inline)) {
            static_assert(PF_KT == 2, "the common-tile path is written for 64-key tiles");
            constexpr int QS = Qk::STEPS;
            const uint8_t *kr0 = k_lds(buf) + qi * L::K_PITCH, *kr1 = kr0 + 32 * L::K_PITCH;
            const float *ksp = ks_lds(buf) + 4 * g;
            // ---- block 1: K.Q^T; sub-tile 0's weights between sub-tile 1's MFMAs ----
            typename Qk::kop_t k0[QS], k1[QS];
#pragma unroll
            for (int st = 0; st < QS; ++st) k0[st] = Qk::load_k(kr0, g, st);
#pragma unroll
            for (int st = 0; st < QS; ++st) k1[st] = Qk::load_k(kr1, g, st);
            PF_FENCE;
            typename Qk::acc_t acc0 = {0}, acc1 = {0};
#pragma unroll
            for (int st = 0; st < QS; ++st) acc0 = qk.step(k0[st], st, acc0);
            acc1 = qk.step(k1[0], 0, acc1);
            v4f ksv[4];
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) ksv[c4] = *(const v4f *)(ksp + 8 * c4);
            vload(0, 0, buf);
            vload(1, 1, buf);
            PF_FENCE;
            v2h pp0[8], pp1[8];
            float s0 = 0.0f, s1 = 0.0f;
            // ALiBi: -slope * (from - key), key of register r = kb + 8*(r/4) + 4*g + r%4 (+32 in sub-tile 1)
            const float alibi0 = SLOPE ? -(p.slope * (float)(from - kb - 4 * g)) : 0.0f;
            const float bias00 = alibi0 - m_ref;
            float nbase = bias00;
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) {
                weights_quarter(acc0, c4, ksv[c4], nbase, pp0[2 * c4], pp0[2 * c4 + 1], s0, s1);
                PF_FENCE;
                if (c4 + 1 < QS) {
                    acc1 = qk.step(k1[c4 + 1], c4 + 1, acc1);
                    PF_FENCE;
                }
            }
            v8h p0a = v8h{pp0[0][0], pp0[0][1], pp0[1][0], pp0[1][1], pp0[2][0], pp0[2][1], pp0[3][0], pp0[3][1]};
            v8h p0b = v8h{pp0[4][0], pp0[4][1], pp0[5][0], pp0[5][1], pp0[6][0], pp0[6][1], pp0[7][0], pp0[7][1]};
            if (__any(!(s0 + s1 <= PF_SUM_LIMIT))) weights_sub_rescale(acc0, ksp, bias00, p0a, p0b, s0, s1);
            l += s0;
            l2 += s1;
            // ---- block 2: V^T.P^T of sub-tile 0; sub-tile 1's weights between the MFMAs ----
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) ksv[c4] = *(const v4f *)(ksp + 32 + 8 * c4);
            s0 = 0.0f;
            s1 = 0.0f;
            const float bias10 = alibi0 + (SLOPE ? 32.0f * p.slope : 0.0f) - m_ref; // m_ref may have been raised above
            float nbase1 = bias10;
            PF_FENCE;
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4) {
                // MFMAs c4*DT/2 .. of the 2*DT of this block: group 0 (operand p0a) first, then group 1 (p0b)
#pragma unroll
                for (int j = 0; j < DT / 2; ++j) {
                    const int m = c4 * (DT / 2) + j, grp = m / DT, dt = m % DT;
                    o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[grp][dt], grp == 0 ? p0a : p0b, o_acc[dt], 0, 0, 0);
                }
                weights_quarter(acc1, c4, ksv[c4], nbase1, pp1[2 * c4], pp1[2 * c4 + 1], s0, s1);
                if (c4 == 1) vload(0, 2, buf); // group 0's operands have been consumed
                PF_FENCE;
            }
            vload(1, 3, buf);
            v8h p1a = v8h{pp1[0][0], pp1[0][1], pp1[1][0], pp1[1][1], pp1[2][0], pp1[2][1], pp1[3][0], pp1[3][1]};
            v8h p1b = v8h{pp1[4][0], pp1[4][1], pp1[5][0], pp1[5][1], pp1[6][0], pp1[6][1], pp1[7][0], pp1[7][1]};
            if (__any(!(s0 + s1 <= PF_SUM_LIMIT))) weights_sub_rescale(acc1, ksp + 32, bias10, p1a, p1b, s0, s1);
            l += s0;
            l2 += s1;
            // ---- block 3: V^T.P^T of sub-tile 1; the next tile's staging between the MFMAs ----
            static_assert(LD_ALL && 4 * NLD == 2 * DT, "one 32-bit word of V per MFMA");
            v2h hh[NLD][8];
            PF_FENCE;
#pragma unroll
            for (int m = 0; m < 2 * DT; ++m) {
                const int grp = m / DT, dt = m % DT;
                o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(va[grp][dt], grp == 0 ? p1a : p1b, o_acc[dt], 0, 0, 0);
                const int i = m / 4, w = m % 4;
                const _Float16 vsh = (_Float16)rvs[i];
                widen_v_word<DTYPE, !VS_CONST>(rv[i][w], v2h{vsh, vsh}, hh[i][2 * w], hh[i][2 * w + 1]);
                if (w == 3) {
                    const int ch = tid + i * PF_THREADS;
                    const int r = ch / CHUNKS, c = ch % CHUNKS;
                    uint8_t *vdst = v_lds(buf ^ 1) + r * L::V_PITCH + c * 32;
                    *(v4i *)(k_lds(buf ^ 1) + r * L::K_PITCH + c * 16) = rk[i];
                    *(v8h *)(vdst) = v8h{hh[i][0][0], hh[i][0][1], hh[i][1][0], hh[i][1][1], hh[i][2][0], hh[i][2][1], hh[i][3][0], hh[i][3][1]};
                    *(v8h *)(vdst + 16) = v8h{hh[i][4][0], hh[i][4][1], hh[i][5][0], hh[i][5][1], hh[i][6][0], hh[i][6][1], hh[i][7][0], hh[i][7][1]};
                }
                PF_FENCE;
            }
            if (tid < PF_BN) ks_lds(buf ^ 1)[tid] = rks * ads;
        };
#undef PF_FENCE

        // ---- short key ranges: no tile loop ------------------------------------------------------------------
        // When the whole workgroup needs at most PF_SHORT_KEYS keys (a short window, or the first rows of a
        // sequence) everything is requested at once: the V rows and key scales of the range (widened into LDS by
        // all threads) and each wave's K operands (straight into registers: a key's row slice is exactly what the
        // MFMA operand of that lane holds).  One round trip to memory and one barrier instead of one per tile.
        bool short_done = false;
        if constexpr (HAS_SHORT) {
            if (n_tiles * PF_BN <= PF_SHORT_KEYS) {
                short_done = true;
                const int n_keys = n_tiles * PF_BN;
                uint8_t *const v_short = lds_raw;
                float *const ks_short = (float *)(lds_raw + PF_SHORT_KEYS * L::V_PITCH);
                constexpr int NSH = PF_SHORT_KEYS * CHUNKS / PF_THREADS;
                static_assert(PF_SHORT_KEYS * CHUNKS % PF_THREADS == 0 && PF_SHORT_KEYS <= PF_THREADS, "short range layout");
                v4i svv[NSH];
                float svs[NSH], sks = 0.0f;
#pragma unroll
                for (int i = 0; i < NSH; ++i) {
                    const int ch = tid + i * PF_THREADS;
                    const int r = ch / CHUNKS, c = ch % CHUNKS;
                    svv[i] = v4i{0, 0, 0, 0};
                    svs[i] = 0.0f;
                    if (r < n_keys) {
                        svv[i] = __builtin_bit_cast(v4i, __builtin_amdgcn_raw_buffer_load_b128(vr, r * (int)p.v_pitch + c * 16, 0, 0));
                        svs[i] = vs_ptr ? __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(vsr, r * 4, 0, 0)) : p.vs_const;
                    }
                }
                if (tid < n_keys) sks = ks_ptr ? __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ksr, tid * 4, 0, 0)) : p.ks_const;
                // this wave's 32-key sub-tiles: [s_lo, s_hi] (empty if none of its rows has keys)
                const int s_lo = __builtin_amdgcn_readfirstlane(max(0, (w_min_a - kb_first) >> 5));
                const int s_hi = __builtin_amdgcn_readfirstlane(min(n_keys / 32 - 1, (w_max_b - kb_first) >> 5));
                constexpr int QS = Qk::STEPS;
                constexpr int KREG = 3; // sub-tiles whose K operands are requested up front
                typename Qk::kop_t kk[KREG][QS];
#pragma unroll
                for (int j = 0; j < KREG; ++j) {
                    if (s_lo + j <= s_hi) {
#pragma unroll
                        for (int st = 0; st < QS; ++st) kk[j][st] = Qk::load_k_global(kr, ((s_lo + j) * 32 + qi) * (int)p.k_pitch, g, st);
                    }
                }
#pragma unroll
                for (int i = 0; i < NSH; ++i) {
                    const int ch = tid + i * PF_THREADS;
                    const int r = ch / CHUNKS, c = ch % CHUNKS;
                    if (r < n_keys) {
                        v8h lo, hi;
                        widen_v<DTYPE, !VS_CONST>(svv[i], svs[i], lo, hi);
                        *(v8h *)(v_short + r * L::V_PITCH + c * 32) = lo;
                        *(v8h *)(v_short + r * L::V_PITCH + c * 32 + 16) = hi;
                    }
                }
                if (tid < n_keys) ks_short[tid] = sks * ads;
                __syncthreads();
#pragma unroll 1
                for (int j = 0; s_lo + j <= s_hi; ++j) {
                    const int sub = s_lo + j;
                    typename Qk::kop_t kop[QS];
#pragma unroll
                    for (int st = 0; st < QS; ++st) { // the operands requested up front, or (long ranges) fetched now
                        if (j == 0) kop[st] = kk[0][st];
                        else if (j == 1) kop[st] = kk[1][st];
                        else if (j == 2) kop[st] = kk[2][st];
                        else kop[st] = Qk::load_k_global(kr, (sub * 32 + qi) * (int)p.k_pitch, g, st);
                    }
                    typename Qk::acc_t acc = {0};
#pragma unroll
                    for (int st = 0; st < QS; ++st) acc = qk.step(kop[st], st, acc);
                    sub_tile(acc, ks_short + 32 * sub, v_short + 32 * sub * L::V_PITCH, kb_first + 32 * sub);
                }
            }
        }
        if (!short_done) {
        load_tile();
        store_tile(0);
        if (n_tiles > 1) load_tile();
        __syncthreads();
        // Tiles in key order are: not needed by this wave, partly inside its spans, fully inside, partly
        // inside (the diagonal), not needed.  The fully-inside run [f0, f1) takes the common-tile path (never
        // the last tile of the workgroup, which has no successor to stage); everything else the general one.
        int f0 = n_tiles, f1 = n_tiles;
        if (FAST_LOOP && w_all_have_keys) {
            f0 = max(0, (w_max_a - kb_first + PF_BN - 1) / PF_BN);
            f1 = min(n_tiles - 1, (w_min_b + 1 - kb_first) / PF_BN); // tiles [.., f1) end at or before the smallest span end
            if (f1 < f0) f1 = f0;
            f0 = min(f0, n_tiles);
            f1 = max(f1, f0);
        }
        f0 = __builtin_amdgcn_readfirstlane(f0);
        f1 = __builtin_amdgcn_readfirstlane(f1);
        int it = 0;
        for (int pass = 0; pass < 2; ++pass) {
            const int end = pass == 0 ? f0 : n_tiles;
            for (; it < end; ++it) {
                const int buf = it & 1;
                const int kb = kb_first + it * PF_BN;
                // does this wave need the tile at all?
                if (!(kb + PF_BN - 1 < w_min_a || kb > w_max_b)) compute_tile(buf, kb);
                if (it + 1 < n_tiles) store_tile(buf ^ 1);
                if (it + 2 < n_tiles) load_tile();
                __syncthreads();
            }
            if constexpr (FAST_LOOP) {
                if (pass == 0) {
                    for (; it < f1; ++it) {
                        fast_tile(it & 1, kb_first + it * PF_BN);
                        if (it + 2 < n_tiles) load_tile();
                        __syncthreads();
                    }
                }
            }
        }
        } // tile loop
    }
    if (MULTI && part + 1 < n_parts) __syncthreads(); // the next part stages its tiles into the same LDS (and reduces into red_lds)
    } // parts

    // ---- epilogue: add the zero vector's weight, normalise, store -----------------------------------
    l += l2;
    float l_all = l + __shfl_xor(l, 32, WAVE);
    l_all += fast_exp2(-m_ref);
    const float inv = (VS_CONST ? p.vs_const : 1.0f) / l_all;
    if constexpr (KV_FUSED) if (p.kv_out) {
        // Fused consumer: KVProduct (gpt/train/cpu_infer.cpp:320-337) of the result, which is in registers, with the
        // rows of kv_k: kv[head][blk][x] = int8((k[x ^ blk] * value[x]) * mult).  x ^ blk stays inside an aligned group
        // of four and a lane holds such groups, so the products are lane-local.  The bytes of two blk at a time go
        // through this wave's corner of LDS (32 rows x D bytes each) so that they leave as whole rows of D bytes,
        // 16 bytes per lane.
        constexpr int KV_PITCH = D + 16;
        static_assert(PF_WAVES * 2 * 32 * KV_PITCH <= LDS_BYTES, "the KVProduct rows of all waves fit into the tiles' LDS");
        __syncthreads(); // every wave is done with the K and V tiles
        // (what follows is computed from these copies, which the compiler cannot trace back: nothing of it is
        // prepared before the tile loop and kept in registers through it)
        int qi = lane & 31, g = lane >> 5, q0 = tile * PF_BM + wave * 32;
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("" : "+v"(qi), "+v"(g), "+v"(q0));
#endif
        const int from = q0 + qi;
        const bool row_ok = from < p.n_tokens;
        uint8_t *const stage = lds_raw + (q0 / 32 % PF_WAVES) * (2 * 32 * KV_PITCH);
        uint32_t kw[DT][4];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int c4 = 0; c4 < 4; ++c4)
                kw[dt][c4] = row_ok ? *(const uint32_t *)(p.kv_k + (int64_t)from * p.kv_k_pitch + hoff + dt * 32 + 8 * c4 + 4 * g) : 0u;
        for (int hb = 0; 2 * hb < p.kv_rep; ++hb) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
#pragma unroll
                for (int c4 = 0; c4 < 4; ++c4) {
                    float o[4], key[4];
#pragma unroll
                    for (int j = 0; j < 4; ++j) {
                        o[j] = o_acc[dt][c4 * 4 + j] * inv;
                        key[j] = (float)(int8_t)((kw[dt][c4] >> (8 * j)) & 0xff);
                    }
#pragma unroll
                    for (int bb = 0; bb < 2; ++bb) {
                        const int blk = 2 * hb + bb; // (x ^ blk) % 4 = j ^ bb ^ 2 hb
                        const float *const kx = key;
                        const int s0 = (0 ^ bb), s1 = (1 ^ bb), s2 = (2 ^ bb), s3 = (3 ^ bb);
                        uint32_t word;
                        if (hb == 0)
                            word = pack_i8x4((kx[s0] * o[0]) * p.kv_mult, (kx[s1] * o[1]) * p.kv_mult, (kx[s2] * o[2]) * p.kv_mult,
                                             (kx[s3] * o[3]) * p.kv_mult, -127.0f);
                        else
                            word = pack_i8x4((kx[s0 ^ 2] * o[0]) * p.kv_mult, (kx[s1 ^ 2] * o[1]) * p.kv_mult, (kx[s2 ^ 2] * o[2]) * p.kv_mult,
                                             (kx[s3 ^ 2] * o[3]) * p.kv_mult, -127.0f);
                        if (blk < p.kv_rep) *(uint32_t *)(stage + (bb * 32 + qi) * KV_PITCH + dt * 32 + 8 * c4 + 4 * g) = word;
                    }
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // this wave's bytes are in LDS (nobody else reads them)
#pragma unroll
            for (int it = 0; it < 2 * 32 * CHUNKS / WAVE; ++it) {
                const int id = it * WAVE + g * 32 + qi;
                const int c = id % CHUNKS, r = (id / CHUNKS) % 32, bb = id / (CHUNKS * 32);
                const int blk = 2 * hb + bb;
                const v4i w = *(const v4i *)(stage + (bb * 32 + r) * KV_PITCH + c * 16);
                if (q0 + r < p.n_tokens && blk < p.kv_rep)
                    *(v4i *)(p.kv_out + (int64_t)(q0 + r) * p.kv_out_pitch + ((int64_t)head * p.kv_rep + blk) * D + c * 16) = w;
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // read before the next two blk overwrite it
        }
    }
    if constexpr (OUT_F16) {
        if (p.out) {
            // The result leaves through this wave's corner of LDS: a lane holds one query's row in pieces of four
            // values, which stored directly would touch 32 rows per instruction, 16 bytes in each; staged, every store
            // instruction writes four whole rows of the head (16 bytes per lane, consecutive), half as many of them.
            constexpr int OUT_PITCH = D * 2 + 16;
            static_assert(PF_WAVES * 32 * OUT_PITCH <= LDS_BYTES, "the waves' result rows fit into the tiles' LDS");
            __syncthreads(); // every wave is done with the K and V tiles
            // (computed from these copies, which the compiler cannot trace back: nothing of it is prepared before the
            // tile loop and kept in registers through it)
            int qi = lane & 31, g = lane >> 5, q0 = tile * PF_BM + wave * 32;
#if defined(__HIP_DEVICE_COMPILE__)
            asm volatile("" : "+v"(qi), "+v"(g), "+v"(q0));
#endif
            uint8_t *const stage = lds_raw + (q0 / 32 % PF_WAVES) * (32 * OUT_PITCH);
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
                const int id = it * WAVE + g * 32 + qi;
                const int c = id % ROW_CHUNKS, r = id / ROW_CHUNKS;
                const v4i w = *(const v4i *)(stage + r * OUT_PITCH + c * 16);
                if (q0 + r < p.n_tokens) *(v4i *)((uint8_t *)p.out + (int64_t)(q0 + r) * p.out_pitch + hoff * 2 + c * 16) = w;
            }
        }
    } else if (p.out) {
        // the same for an f32 result, half of the head's columns at a time (a wave's corner of LDS holds 32 half rows)
        constexpr int HALF = D / 2, OUT_PITCH = HALF * 4 + 16;
        static_assert(PF_WAVES * 32 * OUT_PITCH <= LDS_BYTES, "the waves' result rows fit into the tiles' LDS");
        __syncthreads(); // every wave is done with the K and V tiles (and with the rows a fused KVProduct staged)
        int qi = lane & 31, g = lane >> 5, q0 = tile * PF_BM + wave * 32;
#if defined(__HIP_DEVICE_COMPILE__)
        asm volatile("" : "+v"(qi), "+v"(g), "+v"(q0));
#endif
        uint8_t *const stage = lds_raw + (q0 / 32 % PF_WAVES) * (32 * OUT_PITCH);
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
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // this wave's values are in LDS (nobody else reads them)
#pragma unroll
            for (int it = 0; it < 32 * ROW_CHUNKS / WAVE; ++it) {
                const int id = it * WAVE + g * 32 + qi;
                const int c = id % ROW_CHUNKS, r = id / ROW_CHUNKS;
                const v4i w = *(const v4i *)(stage + r * OUT_PITCH + c * 16);
                if (q0 + r < p.n_tokens) *(v4i *)((uint8_t *)p.out + (int64_t)(q0 + r) * p.out_pitch + (hoff + half * HALF) * 4 + c * 16) = w;
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); // read before the second half overwrites it
        }
    }
    if constexpr (!MULTI) {
        if (p.sum_weight_log) {
            // (the row's index from opaque copies again: kept in registers through the tile loops it costs the ALiBi
            // kernels a spill; the kernels with a loop over parts around the tile loops fare better as they are)
            int qi_e = lane & 31, g_e = lane >> 5, q0_e = tile * PF_BM + wave * 32;
#if defined(__HIP_DEVICE_COMPILE__)
            asm volatile("" : "+v"(qi_e), "+v"(g_e), "+v"(q0_e));
#endif
            const int from_e = q0_e + qi_e;
            if (from_e < p.n_tokens && g_e == 0) p.sum_weight_log[(int64_t)head * p.scale_pitch + from_e] = m_ref + __log2f(l_all);
        }
    } else {
        if (row_ok && p.sum_weight_log && g == 0) p.sum_weight_log[(int64_t)head * p.scale_pitch + from] = m_ref + __log2f(l_all);
    }
}

template <int DTYPE, int D, bool OUT_F16>
static void launch_prefill_do(const PrefillParams &p_in, dim3 grid2, hipStream_t st)
{
    const int n_qtiles = (int)grid2.x;
    dim3 grid(grid2.x * grid2.y);
    PrefillParams p = p_in;
    p.map = wg_plan(n_qtiles, p.n_heads, D, PF_BM, p.period_tiles);
    const bool dump = p.dbg != nullptr;
    const bool slope = p.slope != 0.0f;
    dim3 block(PF_THREADS);
    const bool multi = p.n_parts > 1;
    // 0: scales per row; 1: one query scale; 2: one query scale and one value scale (the rarer kernels exist in the general form only)
    const int consts = (p.qs == nullptr && !dump && !multi) ? (p.vs == nullptr ? 2 : 1) : 0;
    if (dump) {
        // the debug variant always takes the general (slope) path
        if (multi) hipLaunchKernelGGL((prefill_kernel<DTYPE, D, OUT_F16, true, true, true, 0>), grid, block, 0, st, p, n_qtiles);
        else hipLaunchKernelGGL((prefill_kernel<DTYPE, D, OUT_F16, true, true, false, 0>), grid, block, 0, st, p, n_qtiles);
    } else if (slope) {
        if (multi) hipLaunchKernelGGL((prefill_kernel<DTYPE, D, OUT_F16, true, false, true, 0>), grid, block, 0, st, p, n_qtiles);
        else if (consts == 2) hipLaunchKernelGGL((prefill_kernel<DTYPE, D, OUT_F16, true, false, false, 2>), grid, block, 0, st, p, n_qtiles);
        else if (consts == 1) hipLaunchKernelGGL((prefill_kernel<DTYPE, D, OUT_F16, true, false, false, 1>), grid, block, 0, st, p, n_qtiles);
        else hipLaunchKernelGGL((prefill_kernel<DTYPE, D, OUT_F16, true, false, false, 0>), grid, block, 0, st, p, n_qtiles);
    } else {
        if (multi) hipLaunchKernelGGL((prefill_kernel<DTYPE, D, OUT_F16, false, false, true, 0>), grid, block, 0, st, p, n_qtiles);
        else if (consts == 2) hipLaunchKernelGGL((prefill_kernel<DTYPE, D, OUT_F16, false, false, false, 2>), grid, block, 0, st, p, n_qtiles);
        else if (consts == 1) hipLaunchKernelGGL((prefill_kernel<DTYPE, D, OUT_F16, false, false, false, 1>), grid, block, 0, st, p, n_qtiles);
        else hipLaunchKernelGGL((prefill_kernel<DTYPE, D, OUT_F16, false, false, false, 0>), grid, block, 0, st, p, n_qtiles);
    }
}

template <int DTYPE, int D>
static void launch_prefill_dd(const PrefillParams &p, int out_dtype, dim3 grid, hipStream_t st)
{
    if (out_dtype == TSATTN_OUT_F16) launch_prefill_do<DTYPE, D, true>(p, grid, st);
    else launch_prefill_do<DTYPE, D, false>(p, grid, st);
}

hipError_t launch_prefill(const PrefillParams &p, int dtype, int head_dim, int out_dtype, hipStream_t st)
{
    if (p.n_tokens <= 0) return hipSuccess;
    if (p.vt && head_dim == 128 && p.slope == 0.0f && !p.dbg && !p.kv_out) return launch_prefill_long(p, dtype, out_dtype, st);
    dim3 grid((unsigned)((p.n_tokens + PF_BM - 1) / PF_BM), (unsigned)p.n_heads);
    if (dtype == TSATTN_E4M3 && head_dim == 128) launch_prefill_dd<TSATTN_E4M3, 128>(p, out_dtype, grid, st);
    else if (dtype == TSATTN_E4M3 && head_dim == 64) launch_prefill_dd<TSATTN_E4M3, 64>(p, out_dtype, grid, st);
    else if (dtype == TSATTN_I8 && head_dim == 128) launch_prefill_dd<TSATTN_I8, 128>(p, out_dtype, grid, st);
    else if (dtype == TSATTN_I8 && head_dim == 64) launch_prefill_dd<TSATTN_I8, 64>(p, out_dtype, grid, st);
    else return hipErrorInvalidValue;
    return hipGetLastError();
}

} // namespace tsattn
