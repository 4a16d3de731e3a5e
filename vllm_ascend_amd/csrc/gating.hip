// Group-limited top-k gating: one wavefront per token row (the row's arithmetic is in gating_body.h).
#include "gating_body.h"

namespace moe355 {

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
    gate_row<DT, PER>(x, bias, row, live, E, k, k_group, G, mode, renorm, norm_type, rsf, eps, y, idx, out, out_flag,
                      y_alt, y_alt_dtype, sc_lds, sc_lds + E, nullptr, lane);
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
