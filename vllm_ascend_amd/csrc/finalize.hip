// Weighted un-permute (finalize routing): one workgroup per token, each lane
// owns runs of 8 hidden elements (16-byte loads), accumulating the k expert
// rows in fp32 in slot order.
#include "moe355_common.h"

namespace moe355 {

// TOPK > 0: the slot loop is unrolled and all TOPK row loads are issued before the first add,
// so their latencies overlap; TOPK == 0: generic loop.
// DT: bf16 or fp16 (rows, weights, residual and result share it).
constexpr int kHistMaxExperts = 2048;

// idx == nullptr: the rows lie in pair order (row of token t, slot s = t * top_k + s).  hist_ids != nullptr: one
// more workgroup (the last of the grid's x range) counts the pairs of every expert into hist_out [hist_experts]
// (int64), next to the others instead of in a launch of its own.
template <int TOPK, int DT = MOE355_DT_BF16>
__global__ __launch_bounds__(256) void token_unpermute_kernel(const uint16_t* __restrict__ permuted,
                                                              const int32_t* __restrict__ idx,
                                                              const uint16_t* __restrict__ probs, int top_k_rt,
                                                              int64_t H, int64_t permuted_rows,
                                                              const uint16_t* __restrict__ residual,
                                                              uint16_t* __restrict__ out,
                                                              const int32_t* __restrict__ hist_ids, int hist_experts,
                                                              int64_t* __restrict__ hist_out)
{
    __shared__ int32_t srow[64];
    __shared__ float sw[64];
    const int top_k = TOPK > 0 ? TOPK : top_k_rt;
    if (hist_ids && blockIdx.x == gridDim.x - 1) {
        __shared__ int32_t hcnt[kHistMaxExperts];
        if (blockIdx.y != 0) return;
        for (int e = threadIdx.x; e < hist_experts; e += 256) hcnt[e] = 0;
        __syncthreads();
        for (int64_t f = threadIdx.x; f < permuted_rows; f += 256) {
            const int32_t e = hist_ids[f];
            if (e >= 0 && e < hist_experts) atomicAdd(&hcnt[e], 1);
        }
        __syncthreads();
        for (int e = threadIdx.x; e < hist_experts; e += 256) hist_out[e] = (int64_t)hcnt[e];
        return;
    }
    const int64_t t = blockIdx.x;
    if (threadIdx.x < top_k) {
        int32_t d = idx ? idx[t * top_k + threadIdx.x] : (int32_t)(t * top_k + threadIdx.x);
        d = d < 0 ? -d : d;
        if (!idx && hist_ids) {  // pair order: a pair whose expert id is out of range was computed by nobody
            const int32_t e = hist_ids[t * top_k + threadIdx.x];
            if (e < 0 || e >= hist_experts) d = 0x7fffffff;
        }
        srow[threadIdx.x] = ((int64_t)d < permuted_rows) ? d : -1;
        sw[threadIdx.x] = probs ? half_to_f32<DT>(probs[t * top_k + threadIdx.x]) : 1.0f;
    }
    __syncthreads();
    const int64_t nv = H >> 3;
    // few tokens: a row is cut into gridDim.y pieces, one workgroup each
    for (int64_t i = (int64_t)blockIdx.y * 256 + threadIdx.x; i < nv; i += 256 * (int64_t)gridDim.y) {
        float acc[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) acc[j] = 0.0f;
        if constexpr (TOPK > 0) {
            v8u16 v[TOPK];
#pragma unroll
            for (int s = 0; s < TOPK; ++s) {
                const int32_t d = srow[s];
                v[s] = (d >= 0) ? ((const v8u16*)(permuted + (int64_t)d * H))[i] : (v8u16){0, 0, 0, 0, 0, 0, 0, 0};
            }
#pragma unroll
            for (int s = 0; s < TOPK; ++s) {
                if (srow[s] < 0) continue;
                const float w = sw[s];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    float pr = w * half_to_f32<DT>(v[s][j]);
                    acc[j] = acc[j] + pr;
                }
            }
        } else {
            for (int s = 0; s < top_k; ++s) {
                const int32_t d = srow[s];
                if (d < 0) continue;
                const float w = sw[s];
                const v8u16 v = ((const v8u16*)(permuted + (int64_t)d * H))[i];
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    float pr = w * half_to_f32<DT>(v[j]);
                    acc[j] = acc[j] + pr;
                }
            }
        }
        if (residual) {
            const v8u16 r = ((const v8u16*)(residual + t * H))[i];
#pragma unroll
            for (int j = 0; j < 8; ++j) acc[j] = acc[j] + half_to_f32<DT>(r[j]);
        }
        v8u16 o;
#pragma unroll
        for (int j = 0; j < 8; ++j) o[j] = f32_to_half<DT>(acc[j]);
        ((v8u16*)(out + t * H))[i] = o;
    }
}

}  // namespace moe355

using namespace moe355;

static int unpermute_impl(const void* permuted, int dtype, const int32_t* sorted_indices, const void* probs,
                          int64_t num_tokens, int top_k, int64_t hidden, int64_t permuted_rows, const void* residual,
                          void* out, const int32_t* hist_ids, int hist_experts, int64_t* hist_out, void* stream)
{
    if (num_tokens < 0 || top_k <= 0 || hidden <= 0 || permuted_rows < 0) return MOE355_E_ARG;
    if (dtype != MOE355_DT_BF16 && dtype != MOE355_DT_F16) return MOE355_E_UNSUPPORTED;
    if (top_k > 64 || hidden % 8 != 0 || num_tokens > 0x7ffffffeLL) return MOE355_E_SHAPE;
    if (num_tokens == 0) return MOE355_OK;
    if (!permuted || (!sorted_indices && !hist_ids) || !out) return MOE355_E_ARG;
    if (((uintptr_t)permuted & 15) || ((uintptr_t)out & 15) || ((uintptr_t)residual & 15)) return MOE355_E_SHAPE;
    // one workgroup per token when the tokens alone fill the chip; otherwise the rows are cut into pieces of 256
    // 16-byte vectors until there are about 1024 workgroups
    unsigned pieces = 1;
    if (num_tokens < 512) {
        const int64_t per_row = (hidden / 8 + 255) / 256;
        const int64_t want = (1024 + num_tokens - 1) / num_tokens;
        pieces = (unsigned)(per_row < want ? per_row : want);
        if (pieces < 1) pieces = 1;
    }
#define MOE355_UNPERMUTE(K, D)                                                                                    \
    hipLaunchKernelGGL((token_unpermute_kernel<K, D>), dim3((unsigned)num_tokens + (hist_ids ? 1u : 0u), pieces), dim3(256), 0, (hipStream_t)stream, \
                       (const uint16_t*)permuted, sorted_indices, (const uint16_t*)probs, top_k, hidden,             \
                       permuted_rows, (const uint16_t*)residual, (uint16_t*)out, hist_ids, hist_experts, hist_out)
    if (dtype == MOE355_DT_F16) {
        // fp16 models: the common fan-outs unrolled, the rest through the generic loop
        if (top_k == 8) MOE355_UNPERMUTE(8, MOE355_DT_F16);
        else if (top_k == 2) MOE355_UNPERMUTE(2, MOE355_DT_F16);
        else MOE355_UNPERMUTE(0, MOE355_DT_F16);
        return launch_status();
    }
    switch (top_k) {
        case 1: MOE355_UNPERMUTE(1, MOE355_DT_BF16); break;
        case 2: MOE355_UNPERMUTE(2, MOE355_DT_BF16); break;
        case 4: MOE355_UNPERMUTE(4, MOE355_DT_BF16); break;
        case 6: MOE355_UNPERMUTE(6, MOE355_DT_BF16); break;
        case 8: MOE355_UNPERMUTE(8, MOE355_DT_BF16); break;
        default: MOE355_UNPERMUTE(0, MOE355_DT_BF16); break;
    }
#undef MOE355_UNPERMUTE
    return launch_status();
}

extern "C" int moe355_token_unpermute(const void* permuted, int dtype, const int32_t* sorted_indices,
                                      const void* probs, int64_t num_tokens, int top_k, int64_t hidden,
                                      int64_t permuted_rows, const void* residual, void* out, void* stream)
{
    if (num_tokens > 0 && !sorted_indices) return MOE355_E_ARG;
    return unpermute_impl(permuted, dtype, sorted_indices, probs, num_tokens, top_k, hidden, permuted_rows, residual, out,
                          nullptr, 0, nullptr, stream);
}

extern "C" int moe355_token_unpermute_pairs(const void* rows, int dtype, const void* probs, const int32_t* topk_ids,
                                            int64_t num_tokens, int top_k, int64_t hidden, int num_experts,
                                            const void* residual, void* out, int64_t* expert_tokens, void* stream)
{
    if (num_experts <= 0) return MOE355_E_ARG;
    if (num_experts > kHistMaxExperts) return MOE355_E_SHAPE;
    if (num_tokens > 0 && (!topk_ids || !expert_tokens)) return MOE355_E_ARG;
    return unpermute_impl(rows, dtype, nullptr, probs, num_tokens, top_k, hidden, num_tokens * top_k, residual, out,
                          topk_ids, num_experts, expert_tokens, stream);
}

extern "C" int moe355_abi_version(void) { return MOE355_ABI_VERSION; }

extern "C" const char* moe355_strerror(int code)
{
    switch (code) {
        case MOE355_OK: return "ok";
        case MOE355_E_ARG: return "invalid argument (null pointer, negative size or unknown enum value)";
        case MOE355_E_SHAPE: return "shape or alignment outside what the kernels support";
        case MOE355_E_WORKSPACE: return "workspace missing, misaligned or too small";
        case MOE355_E_LAUNCH: return "the HIP runtime refused the kernel launch";
        case MOE355_E_UNSUPPORTED: return "option not supported by this build";
        default: return "unknown error code";
    }
}
