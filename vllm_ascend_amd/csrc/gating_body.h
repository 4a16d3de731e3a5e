// Group-limited top-k gating of one token row by one wavefront (shared by the gating kernel and the fused
// small-batch routing kernel).
//
// Lane l holds experts l, l+64, l+128, ... (PER of them) in registers, so the
// logits row is read with coalesced loads and the softmax sum follows the
// contract order: strided per-lane partials, then a butterfly.  Group scores
// go through a per-wavefront LDS copy of the selection scores (a group's
// experts are spread over lanes); group and expert selection are repeated
// wavefront arg-max reductions with the "larger value, then lower index" order.
#pragma once

#include "moe355_common.h"

namespace moe355 {

// DPP step: combine every lane with the lane `ctrl` names (row shift / row broadcast).  Lanes
// without a source keep their own value, which is harmless for max.
#define MOE355_DPP(v, ctrl, rmask) __builtin_amdgcn_update_dpp((int)(v), (int)(v), ctrl, rmask, 0xf, false)

// Maximum of an unsigned value over the wavefront; every lane returns it.  Six DPP steps, each one v_max_u32 that
// reads its first operand through the lane permutation (the compiler keeps the permutation and the maximum apart:
// copy, v_mov_dpp, compare, select).  A lane without a source in a step (shifted in from outside its row, or a row
// outside the row mask) is left as it is.  The s_nop in front of every step is the wait that a DPP read of a
// register needs after a vector instruction has written it.
__device__ __forceinline__ unsigned wave_max_u32(unsigned v)
{
    asm volatile(
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_shr:1 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_shr:2 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_shr:4 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_shr:8 row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "s_nop 1\n\tv_max_u32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(v));
    return (unsigned)__builtin_amdgcn_readlane((int)v, 63);
}

// Maximum of a 64-bit key over the wavefront; every lane returns it: the largest high word, and the largest low
// word among the lanes that hold it.
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v)
{
    const unsigned hi = (unsigned)(v >> 32);
    const unsigned m = wave_max_u32(hi);
    const unsigned lo = wave_max_u32(hi == m ? (unsigned)v : 0u);
    return ((unsigned long long)m << 32) | lo;
}

__device__ __forceinline__ float wave_max_dpp(float v)
{
#define MOE355_STEP(ctrl, rmask)                                                 \
    {                                                                            \
        float o = __int_as_float(MOE355_DPP(__float_as_int(v), ctrl, rmask));    \
        v = o > v ? o : v;                                                       \
    }
    MOE355_STEP(0x111, 0xf)
    MOE355_STEP(0x112, 0xf)
    MOE355_STEP(0x114, 0xf)
    MOE355_STEP(0x118, 0xf)
    MOE355_STEP(0x142, 0xa)
    MOE355_STEP(0x143, 0xc)
#undef MOE355_STEP
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// Selection key: larger score first, ties to the lower index.  The float is mapped to an
// unsigned integer with the same order (-0 is folded into +0 first, so equal scores compare
// equal), the index is stored inverted in the low word.  0 never occurs as a key of a real
// candidate and stands for "none".
__device__ __forceinline__ unsigned long long make_key(float score, int index)
{
    score = score + 0.0f;
    unsigned u = __float_as_uint(score);
    u = (u & 0x80000000u) ? ~u : (u | 0x80000000u);
    return ((unsigned long long)u << 32) | (unsigned)(0xffffffffu - (unsigned)index);
}

__device__ __forceinline__ int key_index(unsigned long long key) { return (int)(0xffffffffu - (unsigned)key); }

// Score of one expert group from its gs selection scores: the best one (mode 0) or the sum of the best two, best
// first ("larger value, then lower index").  One pass that keeps the two leaders.
__device__ __forceinline__ float group_score(const float* s, int gs, int mode)
{
    int i1 = 0, i2 = -1;
    float v1 = s[0], v2 = 0.0f;
    for (int j = 1; j < gs; ++j) {
        const float v = s[j];
        if (ranks_before(v, j, v1, i1)) {
            v2 = v1;
            i2 = i1;
            v1 = v;
            i1 = j;
        } else if (i2 < 0 || ranks_before(v, j, v2, i2)) {
            v2 = v;
            i2 = j;
        }
    }
    return (mode != 0 && gs >= 2) ? v1 + v2 : v1;
}

// The scores of all groups of one row at once, for groups of a power of two of at most 64 experts: such a group is
// a run of gs lanes in one of the row's registers (expert e = lane + 64 i), so a butterfly over the lanes of the
// run leaves the group's two largest selection scores in every one of them.  The same two values as the pass of
// group_score (a tie is two equal values either way; the order of a +0 and a -0 does not change their sum), the
// same sum; a row that holds a NaN takes group_score instead, whose treatment of it depends on the position.
// Lane g (< G) returns the score of group g, the other lanes anything.
template <int PER>
__device__ __forceinline__ float group_scores_butterfly(const float (&sel)[PER], int gs, int mode, int lane)
{
    float t1[PER], t2[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        t1[i] = sel[i];
        t2[i] = -__builtin_inff();
    }
    for (int m = 1; m < gs; m <<= 1) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const float p1 = __shfl_xor(t1[i], m);
            const float p2 = __shfl_xor(t2[i], m);
            const bool gt = t1[i] > p1;
            const float hi = gt ? t1[i] : p1;
            const float lo = gt ? p1 : t1[i];
            const float second = t2[i] > p2 ? t2[i] : p2;
            t1[i] = hi;
            t2[i] = lo > second ? lo : second;
        }
    }
    const int runs = 64 / gs;  // groups per register
    const int src = (lane % runs) * gs;
    float out = 0.0f;
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        const float sc = (mode != 0 && gs >= 2) ? t1[i] + t2[i] : t1[i];
        const float v = __shfl(sc, src);
        if (lane / runs == i) out = v;
    }
    return out;
}

template <int PER>
__device__ __forceinline__ bool butterfly_groups(const float (&sel)[PER], int gs)
{
    if (gs > 64 || (gs & (gs - 1)) != 0) return false;
    bool nan = false;
#pragma unroll
    for (int i = 0; i < PER; ++i) nan = nan || (sel[i] != sel[i]);
    return __ballot(nan) == 0ull;
}

// One token row by one wavefront.  Every wavefront of the workgroup calls this the same number of times (it
// contains workgroup barriers); a call with live == false computes a valid row and stores nothing.
// sc_lds: E floats, w_lds: 64 floats, both private to the wavefront.  y may be null (only y_alt wanted);
// idx_lds (LDS, may be null) receives the k chosen experts as well.
template <int DT, int PER>
__device__ __forceinline__ void gate_row(const void* __restrict__ x, const void* __restrict__ bias, int64_t row,
                                         bool live, int E, int k, int k_group, int G, int mode, int renorm,
                                         int norm_type, float rsf, float eps, void* __restrict__ y,
                                         int32_t* __restrict__ idx, float* __restrict__ out, int out_flag,
                                         void* __restrict__ y_alt, int y_alt_dtype, float* sc_lds, float* w_lds,
                                         int32_t* idx_lds, int lane)
{
    float p[PER];
    float sel[PER];
    // ---- normalise
    float m = -__builtin_inff();
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        int e = lane + 64 * i;
        p[i] = (e < E) ? load_as_f32<DT>(x, row * E + e) : -__builtin_inff();
        m = p[i] > m ? p[i] : m;
    }
    if (norm_type == 0) {
        m = wave_max_dpp(m);
        float part = 0.0f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            int e = lane + 64 * i;
            if (e < E) {
                p[i] = m_expf(p[i] - m);
                part = part + p[i];
            }
        }
        float s = wave_tree_sum(part);
        float inv = 1.0f / s;
#pragma unroll
        for (int i = 0; i < PER; ++i) p[i] = p[i] * inv;
    } else {
#pragma unroll
        for (int i = 0; i < PER; ++i) p[i] = 1.0f / (1.0f + m_expf(-p[i]));
    }
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        int e = lane + 64 * i;
        if (e < E) {
            if (out_flag && live) out[row * E + e] = p[i];
            sel[i] = bias ? p[i] + load_as_f32<DT>(bias, e) : p[i];
        } else {
            sel[i] = -__builtin_inff();
        }
    }

    // ---- group limit
    if (G > 1) {
        const int gs = E / G;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            int e = lane + 64 * i;
            if (e < E) sc_lds[e] = sel[i];
        }
        __syncthreads();
        unsigned long long gkey = 0ull;
        if (butterfly_groups<PER>(sel, gs)) {
            const float sc = group_scores_butterfly<PER>(sel, gs, mode, lane);
            if (lane < G) gkey = make_key(sc, lane);
        } else if (lane < G) {
            const float* s = sc_lds + lane * gs;
            gkey = make_key(group_score(s, gs, mode), lane);
        }
        unsigned long long keep = 0ull;
        for (int c = 0; c < k_group; ++c) {
            const int g = key_index(wave_max_u64(gkey));
            keep |= 1ull << g;
            if (lane == g) gkey = 0ull;
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            int e = lane + 64 * i;
            if (e < E && !((keep >> (e / gs)) & 1ull)) sel[i] = -__builtin_inff();
        }
        __syncthreads();
    }

    // ---- top-k over the (masked) selection scores; the unbiased scores wait in LDS
    unsigned long long key[PER];
#pragma unroll
    for (int i = 0; i < PER; ++i) {
        int e = lane + 64 * i;
        key[i] = (e < E) ? make_key(sel[i], e) : 0ull;
        if (e < E) sc_lds[e] = p[i];
    }
    int my_i = 0;
    for (int c = 0; c < k; ++c) {
        unsigned long long best = 0ull;
#pragma unroll
        for (int i = 0; i < PER; ++i) best = key[i] > best ? key[i] : best;
        const int win = key_index(wave_max_u64(best));
        if ((win & 63) == lane) {
#pragma unroll
            for (int i = 0; i < PER; ++i)
                if (i == (win >> 6)) key[i] = 0ull;
        }
        if (lane == c) my_i = win;
    }
    __syncthreads();
    float my_p = (lane < k) ? sc_lds[my_i] : 0.0f;
    if (norm_type == 1 || renorm == 1) {
        if (lane < k) w_lds[lane] = my_p;
        __syncthreads();
        float wsum = 0.0f;
        for (int c = 0; c < k; ++c) wsum = wsum + w_lds[c];
        float d = wsum + eps;
        my_p = my_p / d;
    }
    my_p = my_p * rsf;
    if (idx_lds && lane < k) idx_lds[lane] = my_i;
    if (live && lane < k) {
        if (y) store_from_f32<DT>(y, row * k + lane, my_p);
        idx[row * k + lane] = my_i;
        if (y_alt) {
            // second copy of the weights in another dtype: the value stored in y, narrowed again
            float stored = my_p;
            if constexpr (DT == MOE355_DT_BF16) stored = bf16_to_f32(f32_to_bf16(my_p));
            if constexpr (DT == MOE355_DT_F16) stored = f16_to_f32(f32_to_f16(my_p));
            if (y_alt_dtype == MOE355_DT_BF16) ((uint16_t*)y_alt)[row * k + lane] = f32_to_bf16(stored);
            else if (y_alt_dtype == MOE355_DT_F16) ((uint16_t*)y_alt)[row * k + lane] = f32_to_f16(stored);
            else ((float*)y_alt)[row * k + lane] = stored;
        }
    }
}

// NR token rows by one wavefront at the same time: the arithmetic of gate_row for every row, with the steps of
// the rows interleaved so that the long dependent chains of one row (wavefront reductions, the k selection
// rounds) run in the shadow of the others'.  No workgroup barrier: what a row needs from other lanes travels by
// lane reads, the group scores through grp_lds (NR x E floats private to the wavefront; only touched when G > 1).
// Weights are written to `weights` in w_dtype after rounding to DT (the cast chain of the reference's caller:
// gate output in the logits dtype, then .to(hidden dtype)); ids to idx and, when given, to idx_lds.
template <int DT, int PER, int NR>
__device__ __forceinline__ void gate_rows(const void* __restrict__ x, const void* __restrict__ bias,
                                          const int (&row)[NR], const bool (&live)[NR], int E, int k, int k_group,
                                          int G, int mode, int renorm, int norm_type, float rsf, float eps,
                                          void* __restrict__ weights, int w_dtype, int32_t* __restrict__ idx,
                                          float* grp_lds, int32_t* idx_lds, int lane)
{
    float p[NR][PER], sel[NR][PER];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        float m = -__builtin_inff();
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = lane + 64 * i;
            p[r][i] = (e < E) ? load_as_f32<DT>(x, (int64_t)row[r] * E + e) : -__builtin_inff();
            m = p[r][i] > m ? p[r][i] : m;
        }
        if (norm_type == 0) {
            m = wave_max_dpp(m);
            float part = 0.0f;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                if (lane + 64 * i < E) {
                    p[r][i] = m_expf(p[r][i] - m);
                    part = part + p[r][i];
                }
            }
            const float inv = 1.0f / wave_tree_sum(part);
#pragma unroll
            for (int i = 0; i < PER; ++i) p[r][i] = p[r][i] * inv;
        } else {
#pragma unroll
            for (int i = 0; i < PER; ++i) p[r][i] = 1.0f / (1.0f + m_expf(-p[r][i]));
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int e = lane + 64 * i;
            if (e < E) sel[r][i] = bias ? p[r][i] + load_as_f32<DT>(bias, e) : p[r][i];
            else sel[r][i] = -__builtin_inff();
        }
    }
    if (G > 1) {
        const int gs = E / G;
#pragma unroll
        for (int r = 0; r < NR; ++r)
#pragma unroll
            for (int i = 0; i < PER; ++i)
                if (lane + 64 * i < E) grp_lds[r * E + lane + 64 * i] = sel[r][i];
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        unsigned long long gkey[NR];
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            gkey[r] = 0ull;
            if (butterfly_groups<PER>(sel[r], gs)) {
                const float sc = group_scores_butterfly<PER>(sel[r], gs, mode, lane);
                if (lane < G) gkey[r] = make_key(sc, lane);
            } else if (lane < G) {
                gkey[r] = make_key(group_score(grp_lds + r * E + lane * gs, gs, mode), lane);
            }
        }
        unsigned long long keep[NR];
#pragma unroll
        for (int r = 0; r < NR; ++r) keep[r] = 0ull;
        for (int c = 0; c < k_group; ++c) {
#pragma unroll
            for (int r = 0; r < NR; ++r) {
                const int g = key_index(wave_max_u64(gkey[r]));
                keep[r] |= 1ull << g;
                if (lane == g) gkey[r] = 0ull;
            }
        }
#pragma unroll
        for (int r = 0; r < NR; ++r)
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                const int e = lane + 64 * i;
                if (e < E && !((keep[r] >> (e / gs)) & 1ull)) sel[r][i] = -__builtin_inff();
            }
    }
    // ---- top-k over the (masked) selection scores; the weight of a chosen expert is its unbiased score
    unsigned long long key[NR][PER];
#pragma unroll
    for (int r = 0; r < NR; ++r)
#pragma unroll
        for (int i = 0; i < PER; ++i) key[r][i] = (lane + 64 * i < E) ? make_key(sel[r][i], lane + 64 * i) : 0ull;
    int my_i[NR];
    float my_p[NR];
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        my_i[r] = 0;
        my_p[r] = 0.0f;
    }
    for (int c = 0; c < k; ++c) {
#pragma unroll
        for (int r = 0; r < NR; ++r) {
            unsigned long long best = 0ull;
#pragma unroll
            for (int i = 0; i < PER; ++i) best = key[r][i] > best ? key[r][i] : best;
            const int win = key_index(wave_max_u64(best));
            float cand = 0.0f;
#pragma unroll
            for (int i = 0; i < PER; ++i) {
                if (i == (win >> 6)) {
                    cand = p[r][i];
                    if ((win & 63) == lane) key[r][i] = 0ull;
                }
            }
            const float pw = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(cand), win & 63));
            if (lane == c) {
                my_i[r] = win;
                my_p[r] = pw;
            }
        }
    }
#pragma unroll
    for (int r = 0; r < NR; ++r) {
        if (norm_type == 1 || renorm == 1) {
            float wsum = 0.0f;
            for (int c = 0; c < k; ++c)
                wsum = wsum + __int_as_float(__builtin_amdgcn_readlane(__float_as_int(my_p[r]), c));
            const float d = wsum + eps;
            my_p[r] = my_p[r] / d;
        }
        my_p[r] = my_p[r] * rsf;
        if (idx_lds && live[r] && lane < k) idx_lds[row[r] * k + lane] = my_i[r];
        if (live[r] && lane < k) {
            // a store that is visible to the whole device when it completes (a workgroup on another part of the
            // chip may be the one that sorts the pairs)
            __hip_atomic_store(idx + (int64_t)row[r] * k + lane, my_i[r], __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            float stored = my_p[r];
            if constexpr (DT == MOE355_DT_BF16) stored = bf16_to_f32(f32_to_bf16(stored));
            if constexpr (DT == MOE355_DT_F16) stored = f16_to_f32(f32_to_f16(stored));
            const int64_t o = (int64_t)row[r] * k + lane;
            if (w_dtype == MOE355_DT_BF16) ((uint16_t*)weights)[o] = f32_to_bf16(stored);
            else if (w_dtype == MOE355_DT_F16) ((uint16_t*)weights)[o] = f32_to_f16(stored);
            else ((float*)weights)[o] = stored;
        }
    }
}

}  // namespace moe355
