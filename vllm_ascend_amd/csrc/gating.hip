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

struct Cand {
    float v;   // selection score
    int i;     // expert (or group) index, INT_MAX when empty
    float p;   // unbiased normalised score carried along
};

__device__ __forceinline__ Cand wave_best(Cand c)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        float ov = __shfl_xor(c.v, off, 64);
        int oi = __shfl_xor(c.i, off, 64);
        float op = __shfl_xor(c.p, off, 64);
        // an empty candidate (index INT_MAX) never wins against a real one
        bool take = (c.i == 0x7fffffff) ? (oi != 0x7fffffff)
                                        : (oi != 0x7fffffff && ranks_before(ov, oi, c.v, c.i));
        if (take) {
            c.v = ov;
            c.i = oi;
            c.p = op;
        }
    }
    return c;
}

template <int DT, int PER>
__global__ __launch_bounds__(256) void gating_top_k_kernel(const void* __restrict__ x, const void* __restrict__ bias,
                                                           int64_t rows, int E, int k, int k_group, int G, int mode,
                                                           int renorm, int norm_type, float rsf, float eps,
                                                           void* __restrict__ y, int32_t* __restrict__ idx,
                                                           float* __restrict__ out, int out_flag)
{
    extern __shared__ float lds[];  // [4][E] selection scores
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    int64_t row = (int64_t)blockIdx.x * 4 + wave;
    const bool live = row < rows;
    if (!live) row = rows - 1;  // keep every wavefront in the barriers; stores are masked
    float* sel_lds = lds + (size_t)wave * E;

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
        m = wave_max(m);
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
            if (e < E) sel_lds[e] = sel[i];
        }
        __syncthreads();
        Cand gc;
        gc.v = 0.0f;
        gc.i = 0x7fffffff;
        gc.p = 0.0f;
        if (lane < G) {
            const float* s = sel_lds + lane * gs;
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
            gc.v = score;
            gc.i = lane;
        }
        unsigned long long keep = 0ull;
        for (int c = 0; c < k_group; ++c) {
            Cand b = wave_best(gc);
            keep |= 1ull << b.i;
            if (lane == b.i) gc.i = 0x7fffffff;
        }
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            int e = lane + 64 * i;
            if (e < E && !((keep >> (e / gs)) & 1ull)) sel[i] = -__builtin_inff();
        }
        __syncthreads();
    }

    // ---- top-k over the (masked) selection scores
    unsigned taken = 0u;
    float my_p = 0.0f;
    int my_i = 0;
    for (int c = 0; c < k; ++c) {
        Cand b;
        b.v = 0.0f;
        b.i = 0x7fffffff;
        b.p = 0.0f;
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            int e = lane + 64 * i;
            if (e < E && !((taken >> i) & 1u)) {
                if (b.i == 0x7fffffff || ranks_before(sel[i], e, b.v, b.i)) {
                    b.v = sel[i];
                    b.i = e;
                    b.p = p[i];
                }
            }
        }
        b = wave_best(b);
        if ((b.i & 63) == lane) taken |= 1u << (b.i >> 6);
        if (lane == c) {
            my_p = b.p;
            my_i = b.i;
        }
    }
    if (norm_type == 1 || renorm == 1) {
        float wsum = 0.0f;
        for (int c = 0; c < k; ++c) wsum = wsum + __shfl(my_p, c, 64);
        float d = wsum + eps;
        my_p = my_p / d;
    }
    my_p = my_p * rsf;
    if (live && lane < k) {
        store_from_f32<DT>(y, row * k + lane, my_p);
        idx[row * k + lane] = my_i;
    }
}

template <int DT>
static int launch_gating(int per, dim3 grid, size_t lds_bytes, hipStream_t st, const void* x, const void* bias,
                         int64_t rows, int E, int k, int k_group, int G, int mode, int renorm, int norm_type, float rsf,
                         float eps, void* y, int32_t* idx, float* out, int out_flag)
{
#define MOE355_GATING_CASE(P)                                                                                   \
    case P:                                                                                                     \
        hipLaunchKernelGGL((gating_top_k_kernel<DT, P>), grid, dim3(256), lds_bytes, st, x, bias, rows, E, k,   \
                           k_group, G, mode, renorm, norm_type, rsf, eps, y, idx, out, out_flag);               \
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
                                   int32_t* expert_idx, float* out, void* stream)
{
    if (rows < 0 || num_experts <= 0 || k <= 0) return MOE355_E_ARG;
    if (norm_type != 0 && norm_type != 1) return MOE355_E_ARG;
    if (group_select_mode != 0 && group_select_mode != 1) return MOE355_E_ARG;
    if (group_count <= 0 || k_group <= 0 || k_group > group_count) return MOE355_E_ARG;
    if (num_experts > 2048 || k > 64 || k > num_experts || group_count > 64) return MOE355_E_SHAPE;
    if (num_experts % group_count != 0) return MOE355_E_SHAPE;
    if (rows == 0) return MOE355_OK;
    if (!x || !y || !expert_idx || (out_flag && !out)) return MOE355_E_ARG;
    if ((rows + 3) / 4 > 0x7fffffffLL) return MOE355_E_SHAPE;
    const int E = (int)num_experts;
    int per = 1;
    while (64 * per < E) per *= 2;
    dim3 grid((unsigned)((rows + 3) / 4));
    size_t lds_bytes = (size_t)4 * E * sizeof(float);
    hipStream_t st = (hipStream_t)stream;
    switch (x_dtype) {
        case MOE355_DT_F32:
            return launch_gating<MOE355_DT_F32>(per, grid, lds_bytes, st, x, bias, rows, E, k, k_group, group_count,
                                                group_select_mode, renorm, norm_type, routed_scaling_factor, eps, y,
                                                expert_idx, out, out_flag);
        case MOE355_DT_BF16:
            return launch_gating<MOE355_DT_BF16>(per, grid, lds_bytes, st, x, bias, rows, E, k, k_group, group_count,
                                                 group_select_mode, renorm, norm_type, routed_scaling_factor, eps, y,
                                                 expert_idx, out, out_flag);
        case MOE355_DT_F16:
            return launch_gating<MOE355_DT_F16>(per, grid, lds_bytes, st, x, bias, rows, E, k, k_group, group_count,
                                                group_select_mode, renorm, norm_type, routed_scaling_factor, eps, y,
                                                expert_idx, out, out_flag);
        default:
            return MOE355_E_ARG;
    }
}
