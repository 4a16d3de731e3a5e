// Group-limited top-k gating: one wavefront per token row.
//
// Lane l holds experts l, l+64, l+128, ... (PER of them) in registers, so the
// logits row is read with coalesced loads and the softmax sum follows the
// contract order: strided per-lane partials, then a butterfly.  Group scores
// go through a per-wavefront LDS copy of the selection scores (a group's
// experts are spread over lanes); group and expert selection are repeated
// wavefront arg-max reductions with the "larger value, then lower index" order.
#include "moe355_common.h"

namespace moe355 {

// DPP step: combine every lane with the lane `ctrl` names (row shift / row broadcast).  Lanes
// without a source keep their own value, which is harmless for max.
#define MOE355_DPP(v, ctrl, rmask) __builtin_amdgcn_update_dpp((int)(v), (int)(v), ctrl, rmask, 0xf, false)

// Maximum of a 64-bit key over the wavefront; every lane returns it.
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v)
{
#define MOE355_STEP(ctrl, rmask)                                                             \
    {                                                                                        \
        unsigned lo = (unsigned)MOE355_DPP((unsigned)v, ctrl, rmask);                        \
        unsigned hi = (unsigned)MOE355_DPP((unsigned)(v >> 32), ctrl, rmask);                \
        unsigned long long o = ((unsigned long long)hi << 32) | lo;                          \
        v = o > v ? o : v;                                                                   \
    }
    MOE355_STEP(0x111, 0xf)  // row_shr:1
    MOE355_STEP(0x112, 0xf)  // row_shr:2
    MOE355_STEP(0x114, 0xf)  // row_shr:4
    MOE355_STEP(0x118, 0xf)  // row_shr:8
    MOE355_STEP(0x142, 0xa)  // row_bcast:15
    MOE355_STEP(0x143, 0xc)  // row_bcast:31
#undef MOE355_STEP
    unsigned lo = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)v, 63);
    unsigned hi = (unsigned)__builtin_amdgcn_readlane((int)(unsigned)(v >> 32), 63);
    return ((unsigned long long)hi << 32) | lo;
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

template <int DT, int PER>
__global__ __launch_bounds__(256) void gating_top_k_kernel(const void* __restrict__ x, const void* __restrict__ bias,
                                                           int64_t rows, int E, int k, int k_group, int G, int mode,
                                                           int renorm, int norm_type, float rsf, float eps,
                                                           void* __restrict__ y, int32_t* __restrict__ idx,
                                                           float* __restrict__ out, int out_flag,
                                                           void* __restrict__ y_alt, int y_alt_dtype)
{
    extern __shared__ float lds[];  // per wavefront: [E] scores, [64] selected weights
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    int64_t row = (int64_t)blockIdx.x * 4 + wave;
    const bool live = row < rows;
    if (!live) row = rows - 1;  // keep every wavefront in the barriers; stores are masked
    float* sc_lds = lds + (size_t)wave * (E + 64);
    float* w_lds = sc_lds + E;

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
        if (lane < G) {
            const float* s = sc_lds + lane * gs;
            int i1 = 0;
            for (int j = 1; j < gs; ++j)
                if (ranks_before(s[j], j, s[i1], i1)) i1 = j;
            float score = s[i1];
            if (mode != 0 && gs >= 2) {
                int i2 = (i1 == 0) ? 1 : 0;
                for (int j = 0; j < gs; ++j)
                    if (j != i1 && ranks_before(s[j], j, s[i2], i2)) i2 = j;
                score = s[i1] + s[i2];
            }
            gkey = make_key(score, lane);
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
    if (live && lane < k) {
        store_from_f32<DT>(y, row * k + lane, my_p);
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

template <int DT>
static int launch_gating(int per, dim3 grid, size_t lds_bytes, hipStream_t st, const void* x, const void* bias,
                         int64_t rows, int E, int k, int k_group, int G, int mode, int renorm, int norm_type, float rsf,
                         float eps, void* y, int32_t* idx, float* out, int out_flag, void* y_alt, int y_alt_dtype)
{
#define MOE355_GATING_CASE(P)                                                                                   \
    case P:                                                                                                     \
        hipLaunchKernelGGL((gating_top_k_kernel<DT, P>), grid, dim3(256), lds_bytes, st, x, bias, rows, E, k,   \
                           k_group, G, mode, renorm, norm_type, rsf, eps, y, idx, out, out_flag, y_alt,        \
                           y_alt_dtype);                                                                        \
        break;
    switch (per) {
        MOE355_GATING_CASE(1)
        MOE355_GATING_CASE(2)
        MOE355_GATING_CASE(4)
        MOE355_GATING_CASE(8)
        MOE355_GATING_CASE(16)
        MOE355_GATING_CASE(32)
        default:
            return MOE355_E_SHAPE;
    }
#undef MOE355_GATING_CASE
    return launch_status();
}

}  // namespace moe355

using namespace moe355;

extern "C" int moe355_gating_top_k(const void* x, int x_dtype, const void* bias, int64_t rows, int64_t num_experts,
                                   int k, int k_group, int group_count, int group_select_mode, int renorm,
                                   int norm_type, int out_flag, float routed_scaling_factor, float eps, void* y,
                                   int32_t* expert_idx, float* out, void* y_alt, int y_alt_dtype, void* stream)
{
    if (rows < 0 || num_experts <= 0 || k <= 0) return MOE355_E_ARG;
    if (norm_type != 0 && norm_type != 1) return MOE355_E_ARG;
    if (group_select_mode != 0 && group_select_mode != 1) return MOE355_E_ARG;
    if (group_count <= 0 || k_group <= 0 || k_group > group_count) return MOE355_E_ARG;
    if (num_experts > 2048 || k > 64 || k > num_experts || group_count > 64) return MOE355_E_SHAPE;
    if (num_experts % group_count != 0) return MOE355_E_SHAPE;
    if (rows == 0) return MOE355_OK;
    if (!x || !y || !expert_idx || (out_flag && !out)) return MOE355_E_ARG;
    if (y_alt && (y_alt_dtype < MOE355_DT_F32 || y_alt_dtype > MOE355_DT_F16)) return MOE355_E_ARG;
    if ((rows + 3) / 4 > 0x7fffffffLL) return MOE355_E_SHAPE;
    const int E = (int)num_experts;
    int per = 1;
    while (64 * per < E) per *= 2;
    dim3 grid((unsigned)((rows + 3) / 4));
    size_t lds_bytes = (size_t)4 * (E + 64) * sizeof(float);
    hipStream_t st = (hipStream_t)stream;
    switch (x_dtype) {
        case MOE355_DT_F32:
            return launch_gating<MOE355_DT_F32>(per, grid, lds_bytes, st, x, bias, rows, E, k, k_group, group_count,
                                                group_select_mode, renorm, norm_type, routed_scaling_factor, eps, y,
                                                expert_idx, out, out_flag, y_alt, y_alt_dtype);
        case MOE355_DT_BF16:
            return launch_gating<MOE355_DT_BF16>(per, grid, lds_bytes, st, x, bias, rows, E, k, k_group, group_count,
                                                 group_select_mode, renorm, norm_type, routed_scaling_factor, eps, y,
                                                 expert_idx, out, out_flag, y_alt, y_alt_dtype);
        case MOE355_DT_F16:
            return launch_gating<MOE355_DT_F16>(per, grid, lds_bytes, st, x, bias, rows, E, k, k_group, group_count,
                                                group_select_mode, renorm, norm_type, routed_scaling_factor, eps, y,
                                                expert_idx, out, out_flag, y_alt, y_alt_dtype);
        default:
            return MOE355_E_ARG;
    }
}
