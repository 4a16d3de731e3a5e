// Small batches (decode): router and dispatch in one launch.
//
// The reference runs the gating op, then the init-routing op (histogram, stable sort, gather with the first int8
// quantisation), and the expert GEMM reads the gathered copy.  For a few hundred (token, slot) pairs that is two
// launches of a few microseconds each in front of a weight stream of some tens of microseconds.  Here one launch
// does both:
//   - ceil(T / 4) workgroups (every fifth of the grid) gate four token rows each (one per wavefront, the arithmetic of the gating
//     kernel) and then count themselves on a counter; the one that finds all the others done sorts the T * k pairs
//     by expert, stably: per-chunk histograms in LDS (a chunk = 64 consecutive pairs), a scan over (chunk, expert),
//     ballot-matched ranks inside a chunk.  Nobody waits for anybody: a workgroup that is not the last one ends;
//   - the other T workgroups quantise one token row each, ONCE, in token order.  The rows are not copied k times
//     into the expert-sorted order: the expert GEMM reads row r of that order through row_token[r].
// The results are the ones the two separate ops give: topk weights and ids, expanded_row_idx, the per-expert
// counts, and (through row_token) the int8 rows and scales of the expert-sorted activation.
// The counter is one int32 that the caller keeps at zero between calls (the sorting workgroup puts it back).
#include <type_traits>

#include "gating_body.h"

namespace moe355 {

constexpr int kSmallThreads = 256;
constexpr int kSmallWaves = kSmallThreads / 64;
constexpr int kSmallMaxPairs = 1024;
constexpr int kSmallChunks = kSmallMaxPairs / 64;
constexpr int kSmallMaxExperts = 256;  // the sorting workgroup's tables stay well below 64 KiB of LDS

struct SmallRouteArgs {
    const void* x;        // [T, H] bf16 / fp16
    const void* logits;   // [T, E]
    const void* bias;     // [E] or null (logits dtype)
    int T, H, E, k, k_group, G, mode, renorm, norm_type;
    float rsf, eps;
    int tokens_num_type;
    void* topk_weights;   // [T, k] in the dtype of x
    int x_dtype;
    int32_t* topk_ids;    // [T, k]
    int8_t* xq;           // [T, H]
    float* x_scale;       // [T]
    int32_t* dst;         // [T * k] expanded_row_idx
    int32_t* row_token;   // [T * k] token of every expert-sorted row
    int64_t* expert_tokens;  // [E]
    int32_t* arrived;     // one int32, zero between calls
};

// the quantiser of the layer on one row, by the whole workgroup
template <int DT>
__device__ __forceinline__ void quantise_token_row(const SmallRouteArgs& a, int t, float* lds16)
{
    const int tid = threadIdx.x;
    const int64_t nv = a.H >> 3;
    const v8u16* xv = (const v8u16*)((const uint16_t*)a.x + (int64_t)t * a.H);
    v8u16 held = {0, 0, 0, 0, 0, 0, 0, 0};
    if (tid < nv) held = xv[tid];
    float amax = 0.0f;
    for (int64_t i = tid; i < nv; i += kSmallThreads) {
        const v8u16 v = i < kSmallThreads ? held : xv[i];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            const float f = __builtin_fabsf(half_to_f32<DT>(v[j]));
            amax = f > amax ? f : amax;
        }
    }
    amax = wave_max(amax);
    if ((tid & 63) == 0) lds16[tid >> 6] = amax;
    __syncthreads();
    amax = lds16[0];
#pragma unroll
    for (int w = 1; w < kSmallWaves; ++w) amax = lds16[w] > amax ? lds16[w] : amax;
    const float s = amax / 127.0f;
    const RowDivisor d = row_divisor(s);
    if (tid == 0) a.x_scale[t] = (amax == 0.0f) ? 0.0f : s;
    uint2* qv = (uint2*)(a.xq + (int64_t)t * a.H);
    auto emit = [&](auto fast) {
        for (int64_t i = tid; i < nv; i += kSmallThreads) {
            const v8u16 v = i < kSmallThreads ? held : xv[i];
            uint32_t w[2] = {0u, 0u};
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int8_t b = (amax == 0.0f) ? (int8_t)0
                                                : quantise_by_row<decltype(fast)::value>(half_to_f32<DT>(v[j]), d);
                w[j >> 2] |= (uint32_t)(uint8_t)b << (8 * (j & 3));
            }
            qv[i] = make_uint2(w[0], w[1]);
        }
    };
    if (d.fast) emit(std::true_type{});
    else emit(std::false_type{});
}

// LDT: dtype of the logits; XDT: dtype of the hidden states (and of the weights that are returned)
template <int LDT, int PER, int XDT>
__global__ __launch_bounds__(kSmallThreads) void route_quant_small_kernel(SmallRouteArgs a)
{
    extern __shared__ float lds[];
    const int gate_wgs = (a.T + kSmallWaves - 1) / kSmallWaves;
    if ((int)blockIdx.x >= gate_wgs) {
        quantise_token_row<XDT>(a, (int)blockIdx.x - gate_wgs, lds);
        return;
    }
    const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
    const int E = a.E, k = a.k, R = a.T * a.k;
    // ---------------- gating: one row per wavefront
    {
        int row[1] = {(int)blockIdx.x * kSmallWaves + wave};
        bool live[1] = {row[0] < a.T};
        if (!live[0]) row[0] = a.T - 1;
        gate_rows<LDT, PER, 1>(a.logits, a.bias, row, live, E, k, a.k_group, a.G, a.mode, a.renorm, a.norm_type, a.rsf,
                               a.eps, a.topk_weights, a.x_dtype, a.topk_ids, lds + (size_t)wave * E, nullptr, lane);
    }
    if (!a.arrived) return;  // gating and quantisation only (moe355_gate_quant): the maps come from another launch
    // This workgroup's ids have reached memory before it is counted: every thread waits for its own stores, the
    // barrier collects the workgroup, and the counting thread issues a device-scope release fence in front of the
    // atomic (the ids are written with device-scope stores already; the fence is what the memory model asks for,
    // so that the hand-off does not rest on how those stores happen to be compiled).
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
    int32_t* flag = (int32_t*)lds;
    if (tid == 0) {
        __threadfence();
        *flag = atomicAdd(a.arrived, 1) == gate_wgs - 1;
    }
    __syncthreads();
    if (!*flag) return;
    __threadfence();  // acquire side: the reads below come after the count that this workgroup has observed
    __syncthreads();
    // ---------------- the last gating workgroup sorts the R pairs (stable counting sort by expert)
    int32_t* ids_l = (int32_t*)lds;             // [kSmallMaxPairs]
    int32_t* hist = ids_l + kSmallMaxPairs;     // [16][E]: chunk histograms, then rows of the expert in earlier chunks
    int32_t* total = hist + kSmallChunks * E;   // [E]: rows of each expert, then its first row
    int32_t* partial = total + E;               // [16] scan scratch
    for (int i = tid; i < kSmallChunks * E; i += kSmallThreads) hist[i] = 0;
    for (int f = tid; f < R; f += kSmallThreads)
        ids_l[f] = __hip_atomic_load(a.topk_ids + f, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    const int passes = (R + kSmallThreads - 1) / kSmallThreads;  // pair f = pass * 256 + tid, chunk = f / 64
    for (int ps = 0; ps < passes; ++ps) {
        const int f = ps * kSmallThreads + tid;
        if (f < R) {
            const int e = ids_l[f];
            if (e >= 0 && e < E) atomicAdd(&hist[(f >> 6) * E + e], 1);
        }
    }
    __syncthreads();
    for (int e = tid; e < E; e += kSmallThreads) {
        int32_t run = 0;
#pragma unroll
        for (int c = 0; c < kSmallChunks; ++c) {
            const int32_t n = hist[c * E + e];
            hist[c * E + e] = run;
            run += n;
        }
        total[e] = run;
    }
    __syncthreads();
    const int32_t mine = tid < E ? total[tid] : 0;  // E <= 256 = the number of threads
    int32_t all;
    const int32_t first = block_scan_exclusive_i32(mine, partial, all);
    if (tid < E) {
        total[tid] = first;
        a.expert_tokens[tid] = a.tokens_num_type == 1 ? (int64_t)mine : (int64_t)(first + mine);
    }
    __syncthreads();
    // rank inside the chunk: lanes with the same expert find each other with ballots
    int nbits = 0;
    while ((1 << nbits) < E) ++nbits;
    const unsigned long long below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    for (int ps = 0; ps < passes; ++ps) {
        const int f = ps * kSmallThreads + tid;
        int e = -1;
        if (f < R) {
            e = ids_l[f];
            if (e < 0 || e >= E) e = -1;  // cannot happen for ids that the gate chose; kept for symmetry with the op
        }
        const bool valid = e >= 0;
        unsigned long long same = __ballot(valid);
        for (int b = 0; b < nbits; ++b) {
            const bool bit = (e >> b) & 1;
            const unsigned long long bal = __ballot(valid && bit);
            same &= bit ? bal : ~bal;
        }
        if (f < R) {
            int32_t d = R;  // a dropped pair points one past the last row
            if (valid) {
                d = total[e] + hist[(f >> 6) * E + e] + __popcll(same & below);
                a.row_token[d] = f / k;
            }
            a.dst[f] = d;
        }
    }
    if (tid == 0) *a.arrived = 0;  // ready for the next call
}

}  // namespace moe355

using namespace moe355;

extern "C" int moe355_gate_quant_supported(int64_t num_tokens, int top_k, int num_experts)
{
    return num_tokens > 0 && num_tokens < (1 << 30) && top_k > 0 && top_k <= 64 && num_experts > 0 &&
           num_experts <= kSmallMaxExperts && top_k <= num_experts;
}

extern "C" int moe355_route_quant_small_supported(int64_t num_tokens, int top_k, int num_experts)
{
    return num_tokens > 0 && top_k > 0 && top_k <= 64 && num_tokens * top_k <= kSmallMaxPairs && num_experts > 0 &&
           num_experts <= kSmallMaxExperts && top_k <= num_experts;
}

// sort: the whole of moe355_route_quant_small; otherwise gating and quantisation only (any number of tokens)
static int gate_quant_impl(bool sort, const void* x, int x_dtype, const void* logits, int logits_dtype,
                           const void* bias, int64_t num_tokens, int64_t hidden, int num_experts, int k, int k_group,
                           int group_count, int group_select_mode, int renorm, int norm_type,
                           float routed_scaling_factor, float eps, int tokens_num_type, void* topk_weights,
                           int32_t* topk_ids, int8_t* xq, float* x_scale, int32_t* expanded_row_idx,
                           int32_t* row_token, int64_t* expert_tokens, int32_t* sync_counter, void* stream)
{
    if (num_tokens < 0 || hidden <= 0 || num_experts <= 0 || k <= 0) return MOE355_E_ARG;
    if (norm_type != 0 && norm_type != 1) return MOE355_E_ARG;
    if (group_select_mode != 0 && group_select_mode != 1) return MOE355_E_ARG;
    if (group_count <= 0 || k_group <= 0 || k_group > group_count) return MOE355_E_ARG;
    if (tokens_num_type != 0 && tokens_num_type != 1) return MOE355_E_UNSUPPORTED;
    if (x_dtype != MOE355_DT_BF16 && x_dtype != MOE355_DT_F16) return MOE355_E_UNSUPPORTED;
    if (logits_dtype < MOE355_DT_F32 || logits_dtype > MOE355_DT_F16) return MOE355_E_ARG;
    if (num_tokens == 0) return MOE355_OK;
    if (sort && !moe355_route_quant_small_supported(num_tokens, k, num_experts)) return MOE355_E_SHAPE;
    if (!sort && !moe355_gate_quant_supported(num_tokens, k, num_experts)) return MOE355_E_SHAPE;
    if (group_count > 64 || num_experts % group_count != 0) return MOE355_E_SHAPE;
    if (hidden % 8 != 0 || ((uintptr_t)x & 15) || ((uintptr_t)xq & 7)) return MOE355_E_SHAPE;
    if (!x || !logits || !topk_weights || !topk_ids || !xq || !x_scale) return MOE355_E_ARG;
    if (sort && (!expanded_row_idx || !row_token || !expert_tokens || !sync_counter)) return MOE355_E_ARG;
    SmallRouteArgs a = {};
    a.x = x;
    a.logits = logits;
    a.bias = bias;
    a.T = (int)num_tokens;
    a.H = (int)hidden;
    a.E = num_experts;
    a.k = k;
    a.k_group = k_group;
    a.G = group_count;
    a.mode = group_select_mode;
    a.renorm = renorm;
    a.norm_type = norm_type;
    a.rsf = routed_scaling_factor;
    a.eps = eps;
    a.tokens_num_type = tokens_num_type;
    a.topk_weights = topk_weights;
    a.x_dtype = x_dtype;
    a.topk_ids = topk_ids;
    a.xq = xq;
    a.x_scale = x_scale;
    a.dst = expanded_row_idx;
    a.row_token = row_token;
    a.expert_tokens = expert_tokens;
    a.arrived = sort ? sync_counter : nullptr;
    const int E = num_experts;
    int per = 1;
    while (64 * per < E) per *= 2;
    // LDS: the sorting tables; the gating rows need E floats per wavefront and the quantiser 4 floats (less)
    const size_t lds_bytes = sort ? ((size_t)kSmallMaxPairs + (size_t)kSmallChunks * E + E + 16) * 4
                                  : ((size_t)kSmallWaves * E + 16) * 4;
    const dim3 grid((unsigned)((num_tokens + kSmallWaves - 1) / kSmallWaves + num_tokens));
    hipStream_t st = (hipStream_t)stream;
#define MOE355_SMALL(L_, P_, X_)                                                                                  \
    hipLaunchKernelGGL((route_quant_small_kernel<L_, P_, X_>), grid, dim3(kSmallThreads), lds_bytes, st, a)
#define MOE355_SMALL_PER(L_, X_)                    \
    switch (per) {                                  \
        case 1: MOE355_SMALL(L_, 1, X_); break;     \
        case 2: MOE355_SMALL(L_, 2, X_); break;     \
        default: MOE355_SMALL(L_, 4, X_); break;    \
    }
#define MOE355_SMALL_X(L_)                                             \
    if (x_dtype == MOE355_DT_F16) { MOE355_SMALL_PER(L_, MOE355_DT_F16) } \
    else { MOE355_SMALL_PER(L_, MOE355_DT_BF16) }
    if (logits_dtype == MOE355_DT_F32) { MOE355_SMALL_X(MOE355_DT_F32) }
    else if (logits_dtype == MOE355_DT_BF16) { MOE355_SMALL_X(MOE355_DT_BF16) }
    else { MOE355_SMALL_X(MOE355_DT_F16) }
#undef MOE355_SMALL_X
#undef MOE355_SMALL_PER
#undef MOE355_SMALL
    return launch_status();
}

extern "C" int moe355_route_quant_small(const void* x, int x_dtype, const void* logits, int logits_dtype,
                                        const void* bias, int64_t num_tokens, int64_t hidden, int num_experts, int k,
                                        int k_group, int group_count, int group_select_mode, int renorm,
                                        int norm_type, float routed_scaling_factor, float eps, int tokens_num_type,
                                        void* topk_weights, int32_t* topk_ids, int8_t* xq, float* x_scale,
                                        int32_t* expanded_row_idx, int32_t* row_token, int64_t* expert_tokens,
                                        int32_t* sync_counter, void* stream)
{
    return gate_quant_impl(true, x, x_dtype, logits, logits_dtype, bias, num_tokens, hidden, num_experts, k, k_group,
                           group_count, group_select_mode, renorm, norm_type, routed_scaling_factor, eps,
                           tokens_num_type, topk_weights, topk_ids, xq, x_scale, expanded_row_idx, row_token,
                           expert_tokens, sync_counter, stream);
}

extern "C" int moe355_gate_quant(const void* x, int x_dtype, const void* logits, int logits_dtype, const void* bias,
                                 int64_t num_tokens, int64_t hidden, int num_experts, int k, int k_group,
                                 int group_count, int group_select_mode, int renorm, int norm_type,
                                 float routed_scaling_factor, float eps, void* topk_weights, int32_t* topk_ids,
                                 int8_t* xq, float* x_scale, void* stream)
{
    return gate_quant_impl(false, x, x_dtype, logits, logits_dtype, bias, num_tokens, hidden, num_experts, k, k_group,
                           group_count, group_select_mode, renorm, norm_type, routed_scaling_factor, eps, 1,
                           topk_weights, topk_ids, xq, x_scale, nullptr, nullptr, nullptr, nullptr, stream);
}
