// Token dispatch: expert histogram, prefix-scan offsets, stable counting-sort
// permutation of the flattened (token, slot) pairs, and the token gather with
// fused per-row int8 quantisation.
//
// The flat index space [0, R) is cut into chunks of 256.  Stability needs
//   dst[f] = off[e] + #{f' < f : ids[f'] == e},
// which is built in three launches:
//   1. per-chunk expert histograms (LDS atomics; counts are order independent);
//   2. one workgroup turns them into per-(chunk, expert) start rows and the
//      per-expert offsets (exclusive scans);
//   3. one wavefront per chunk walks its 256 indices in order, 64 at a time:
//      lanes with equal expert ids find each other with ballots, rank
//      themselves by lane number, and the lowest lane advances the running
//      per-expert cursor kept in LDS.
// A fourth launch quantises every token row once and writes it to its k
// destination rows.  Batches of at most 2048 pairs take one launch for all of it
// (route_gather_small_kernel).
#include <mutex>
#include <type_traits>

#include "moe355_common.h"

namespace moe355 {

constexpr int kChunk = 256;

struct RouteWs {
    int32_t* chunk_hist;  // [nchunks][E]   histogram, then start row of (chunk, expert)
    int32_t* off;         // [E + 1]        first row of each expert
    int32_t* pbase;       // [parts][E]     rows of expert e in the chunk partitions before part p (scan kernel)
};

__host__ __device__ inline size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

__global__ __launch_bounds__(256) void route_hist_kernel(const int32_t* __restrict__ ids, int64_t R, int E,
                                                         int32_t* __restrict__ chunk_hist)
{
    extern __shared__ int32_t hist[];  // [E]
    for (int e = threadIdx.x; e < E; e += 256) hist[e] = 0;
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kChunk;
    for (int i = threadIdx.x; i < kChunk; i += 256) {
        int64_t f = base + i;
        if (f < R) {
            int e = ids[f];
            if (e >= 0 && e < E) atomicAdd(&hist[e], 1);
        }
    }
    __syncthreads();
    int32_t* dstp = chunk_hist + (int64_t)blockIdx.x * E;
    for (int e = threadIdx.x; e < E; e += 256) dstp[e] = hist[e];
}

// One workgroup of 1024.  The chunks are cut into `parts` contiguous partitions of `cpp` chunks; thread (p, e)
// scans partition p of column e (its loads do not depend on each other, 32 are in flight at a time), so the
// column scan takes nchunks / parts steps instead of nchunks.  chunk_hist[c][e] becomes the number of rows of
// expert e in the earlier chunks of c's partition; pbase[p][e] the number in the partitions before p.
constexpr int kScanThreads = 1024;
__global__ __launch_bounds__(kScanThreads) void route_scan_kernel(int32_t* __restrict__ chunk_hist, int nchunks, int E,
                                                                  int parts, int cpp, int tokens_num_type,
                                                                  int32_t* __restrict__ off,
                                                                  int32_t* __restrict__ pbase,
                                                                  int64_t* __restrict__ expert_tokens)
{
    extern __shared__ int32_t cnt[];  // [E] counts, [256] partials, [parts * E] partition totals
    int32_t* partial = cnt + E;
    int32_t* ptot = partial + 256;
    for (int idx = threadIdx.x; idx < parts * E; idx += kScanThreads) {
        const int p = idx / E, e = idx - p * E;
        const int c_begin = p * cpp;
        const int c_end = c_begin + cpp < nchunks ? c_begin + cpp : nchunks;
        int32_t run = 0;
        for (int c0 = c_begin; c0 < c_end; c0 += 32) {
            int32_t v[32];
#pragma unroll
            for (int j = 0; j < 32; ++j) v[j] = (c0 + j < c_end) ? chunk_hist[(int64_t)(c0 + j) * E + e] : 0;
#pragma unroll
            for (int j = 0; j < 32; ++j) {
                if (c0 + j < c_end) chunk_hist[(int64_t)(c0 + j) * E + e] = run;
                run += v[j];
            }
        }
        ptot[idx] = run;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < parts * E; idx += kScanThreads) {
        const int p = idx / E, e = idx - p * E;
        int32_t before = 0;
        for (int pp = 0; pp < p; ++pp) before += ptot[pp * E + e];
        pbase[idx] = before;
        if (p == parts - 1) cnt[e] = before + ptot[idx];
    }
    __syncthreads();
    // exclusive scan over the experts: thread t owns experts [t * seg, (t + 1) * seg)
    const int seg = (E + kScanThreads - 1) / kScanThreads;
    const int e0 = threadIdx.x * seg;
    int32_t s = 0;
    for (int j = 0; j < seg; ++j)
        if (e0 + j < E) s += cnt[e0 + j];
    int32_t all;
    int32_t run = block_scan_exclusive_i32(s, partial, all);
    for (int j = 0; j < seg; ++j) {
        int e = e0 + j;
        if (e < E) {
            off[e] = run;
            run += cnt[e];
            expert_tokens[e] = (tokens_num_type == 1) ? (int64_t)cnt[e] : (int64_t)run;
            if (e == E - 1) off[E] = run;
        }
    }
}

// One wavefront per chunk.
__global__ __launch_bounds__(64) void route_scatter_kernel(const int32_t* __restrict__ ids, int64_t R, int E,
                                                           int nbits, const int32_t* __restrict__ chunk_start,
                                                           const int32_t* __restrict__ off,
                                                           const int32_t* __restrict__ pbase, int cpp,
                                                           int32_t* __restrict__ dst, int32_t* __restrict__ row_token,
                                                           int top_k)
{
    extern __shared__ int32_t cursor[];  // [E] next free row of each expert for this chunk
    const int lane = threadIdx.x;
    const int32_t* cs = chunk_start + (int64_t)blockIdx.x * E;
    const int32_t* pb = pbase + (int64_t)((int)blockIdx.x / cpp) * E;
    for (int e = lane; e < E; e += 64) cursor[e] = off[e] + pb[e] + cs[e];
    __syncthreads();
    const int64_t base = (int64_t)blockIdx.x * kChunk;
    const unsigned long long below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
    for (int it = 0; it < kChunk / 64; ++it) {
        const int64_t f = base + it * 64 + lane;
        int e = -1;
        if (f < R) {
            e = ids[f];
            if (e < 0 || e >= E) e = -1;
        }
        const bool valid = e >= 0;
        unsigned long long same = __ballot(valid);
        for (int b = 0; b < nbits; ++b) {
            const bool bit = (e >> b) & 1;
            unsigned long long bal = __ballot(valid && bit);
            same &= bit ? bal : ~bal;
        }
        int32_t start = 0;
        if (valid) {
            const int rank = __popcll(same & below);
            const int leader = __ffsll((long long)same) - 1;
            if (lane == leader) {
                start = cursor[e];
                cursor[e] = start + __popcll(same);
            }
            start = __shfl(start, leader, 64);
            dst[f] = start + rank;
            if (row_token) row_token[start + rank] = (int32_t)(f / top_k);
        } else if (f < R) {
            dst[f] = (int32_t)R;  // dropped pair: one past the last row
        }
        __syncthreads();
    }
}

// Small batches (R <= 2048 pairs): routing and gather in ONE launch of num_tokens + 1 workgroups.
// Workgroup t < num_tokens finds the destinations of its own token's k pairs by counting, over all R ids,
// the pairs that a stable sort by expert puts in front of each of them (a smaller expert, or the same expert at a
// smaller flat index), then quantises and writes the token's row; no workgroup waits for another one.
// The last workgroup computes the per-expert counts and their running sum.
constexpr int kSmallMaxIters = 8;  // 8 * 256 = 2048 pairs
constexpr int kInvalidExpert = 0x7fffffff;

__device__ __forceinline__ void small_hist_scan(const int32_t* __restrict__ ids, int R, int E, int tokens_num_type,
                                                int32_t* __restrict__ off, int64_t* __restrict__ expert_tokens,
                                                int32_t* sm)
{
    int32_t* cnt = sm;          // [E]
    int32_t* partial = sm + E;  // [256]
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += 256) cnt[e] = 0;
    __syncthreads();
    for (int f = tid; f < R; f += 256) {
        const int e = ids[f];
        if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
    }
    __syncthreads();
    // exclusive scan of the counts: thread t owns experts [t*seg, (t+1)*seg)
    const int seg = (E + 255) / 256;
    const int e0 = tid * seg;
    int32_t s = 0;
    for (int j = 0; j < seg; ++j)
        if (e0 + j < E) s += cnt[e0 + j];
    int total;
    int32_t run = block_scan_exclusive_i32(s, partial, total);
    for (int j = 0; j < seg; ++j) {
        const int e = e0 + j;
        if (e < E) {
            off[e] = run;
            run += cnt[e];
            expert_tokens[e] = (tokens_num_type == 1) ? (int64_t)cnt[e] : (int64_t)run;
            if (e == E - 1) off[E] = run;
        }
    }
}

// The token's row to its k destinations drow[0..k) (LDS, written before the call; negative = dropped), quantised
// per row when QUANT.  DT: bf16 or fp16 rows (the copy without quantisation moves 16-bit patterns).
// held: the thread's first 16-byte piece of the row (first_piece()), requested by the caller before it worked
// out the destinations; rows of up to 2048 values are then read from memory once.
__device__ __forceinline__ v8u16 first_piece(const uint16_t* __restrict__ xr, int64_t H)
{
    v8u16 v = {0, 0, 0, 0, 0, 0, 0, 0};
    if ((int64_t)threadIdx.x < (H >> 3)) v = ((const v8u16*)xr)[threadIdx.x];
    return v;
}

template <bool QUANT, int DT>
__device__ __forceinline__ void gather_token_row(const uint16_t* __restrict__ xr, int64_t H, int top_k,
                                                 const int32_t* drow, float* lds4, void* __restrict__ xs,
                                                 float* __restrict__ sx, v8u16 held)
{
    const int64_t nv = H >> 3;
    const v8u16* xv = (const v8u16*)xr;
    if constexpr (!QUANT) {
        __syncthreads();
        for (int64_t i = threadIdx.x; i < nv; i += 256) {
            v8u16 v = i < 256 ? held : xv[i];
            for (int j = 0; j < top_k; ++j)
                if (drow[j] >= 0) ((v8u16*)((uint16_t*)xs + (int64_t)drow[j] * H))[i] = v;
        }
        return;
    } else {
        float a = 0.0f;
        for (int64_t i = threadIdx.x; i < nv; i += 256) {
            v8u16 v = i < 256 ? held : xv[i];
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                float f = __builtin_fabsf(half_to_f32<DT>(v[j]));
                a = f > a ? f : a;
            }
        }
        a = wave_max(a);
        if ((threadIdx.x & 63) == 0) lds4[threadIdx.x >> 6] = a;
        __syncthreads();
        a = lds4[0];
        a = lds4[1] > a ? lds4[1] : a;
        a = lds4[2] > a ? lds4[2] : a;
        a = lds4[3] > a ? lds4[3] : a;
        const float s = a / 127.0f;
        const RowDivisor d = row_divisor(s);
        if (threadIdx.x < top_k && drow[threadIdx.x] >= 0) sx[drow[threadIdx.x]] = (a == 0.0f) ? 0.0f : s;
        auto emit = [&](auto fast) {
            for (int64_t i = threadIdx.x; i < nv; i += 256) {
                v8u16 v = i < 256 ? held : xv[i];
                uint32_t w[2] = {0u, 0u};
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    int8_t b = (a == 0.0f) ? (int8_t)0
                                           : quantise_by_row<decltype(fast)::value>(half_to_f32<DT>(v[j]), d);
                    w[j >> 2] |= (uint32_t)(uint8_t)b << (8 * (j & 3));
                }
                const uint2 pk = make_uint2(w[0], w[1]);
                for (int j = 0; j < top_k; ++j)
                    if (drow[j] >= 0) ((uint2*)((int8_t*)xs + (int64_t)drow[j] * H))[i] = pk;
            }
        };
        if (d.fast) emit(std::true_type{});
        else emit(std::false_type{});
    }
}

template <bool QUANT, int DT = MOE355_DT_BF16>
__global__ __launch_bounds__(256) void route_gather_small_kernel(const int32_t* __restrict__ ids, int R, int E,
                                                                 int tokens_num_type, int32_t* __restrict__ off,
                                                                 int64_t* __restrict__ expert_tokens,
                                                                 int32_t* __restrict__ dst,
                                                                 const uint16_t* __restrict__ x, int64_t H, int top_k,
                                                                 void* __restrict__ xs, float* __restrict__ sx)
{
    extern __shared__ int32_t sm[];  // the counting workgroup: [E] counts, [256] scan scratch
    __shared__ float lds4[4];
    __shared__ int32_t drow[64];
    __shared__ int32_t wsum[4][64];
    const int num_tokens = (int)gridDim.x - 1;
    if ((int)blockIdx.x == num_tokens) {
        small_hist_scan(ids, R, E, tokens_num_type, off, expert_tokens, sm);
        return;
    }
    const int t = blockIdx.x;
    const int tid = threadIdx.x;
    const v8u16 held = first_piece(x + (int64_t)t * H, H);
    int my_e[kSmallMaxIters];
#pragma unroll
    for (int it = 0; it < kSmallMaxIters; ++it) {
        const int f = it * 256 + tid;
        int e = kInvalidExpert;
        if (f < R) {
            e = ids[f];
            if (e < 0 || e >= E) e = kInvalidExpert;
        }
        my_e[it] = e;
    }
    const int iters = (R + 255) >> 8;  // 256-pair slices that hold pairs at all
    for (int j = 0; j < top_k; ++j) {
        const int fj = t * top_k + j;
        const int ej = ids[fj];
        int c = 0;
#pragma unroll
        for (int it = 0; it < kSmallMaxIters; ++it) {
            if (it < iters) {
                const int f = it * 256 + tid;
                c += (my_e[it] < ej || (my_e[it] == ej && f < fj)) ? 1 : 0;
            }
        }
        c = wave_sum_i32(c);
        if ((tid & 63) == 0) wsum[tid >> 6][j] = c;
    }
    __syncthreads();
    if (tid < top_k) {
        const int ej = ids[t * top_k + tid];
        const bool valid = ej >= 0 && ej < E;
        const int d = valid ? wsum[0][tid] + wsum[1][tid] + wsum[2][tid] + wsum[3][tid] : -1;
        dst[t * top_k + tid] = valid ? d : R;  // a dropped pair points one past the last row
        drow[tid] = d;
    }
    gather_token_row<QUANT, DT>(x + (int64_t)t * H, H, top_k, drow, lds4, xs, sx, held);
}

// The index maps alone for at most 4096 pairs, in ONE launch of num_tokens + 1 workgroups: workgroup t finds the
// destinations of its token's k pairs by counting (as above) and writes them and the row -> token map; the last
// workgroup the per-expert counts.  Nobody waits for anybody.
constexpr int kMapSmallIters = 16;  // 16 * 256 = 4096 pairs

__global__ __launch_bounds__(256) void route_map_small_kernel(const int32_t* __restrict__ ids, int R, int E,
                                                              int tokens_num_type, int32_t* __restrict__ off,
                                                              int64_t* __restrict__ expert_tokens,
                                                              int32_t* __restrict__ dst, int32_t* __restrict__ row_token,
                                                              int top_k)
{
    extern __shared__ int32_t sm[];  // the counting workgroup: [E] counts, [256] scan scratch
    __shared__ int32_t wsum[4][64];
    const int num_tokens = (int)gridDim.x - 1;
    if ((int)blockIdx.x == num_tokens) {
        small_hist_scan(ids, R, E, tokens_num_type, off, expert_tokens, sm);
        return;
    }
    const int t = blockIdx.x;
    const int tid = threadIdx.x;
    int my_e[kMapSmallIters];
#pragma unroll
    for (int it = 0; it < kMapSmallIters; ++it) {
        const int f = it * 256 + tid;
        int e = kInvalidExpert;
        if (f < R) {
            e = ids[f];
            if (e < 0 || e >= E) e = kInvalidExpert;
        }
        my_e[it] = e;
    }
    const int iters = (R + 255) >> 8;
    for (int j = 0; j < top_k; ++j) {
        const int fj = t * top_k + j;
        const int ej = ids[fj];
        int c = 0;
#pragma unroll
        for (int it = 0; it < kMapSmallIters; ++it) {
            if (it < iters) {
                const int f = it * 256 + tid;
                c += (my_e[it] < ej || (my_e[it] == ej && f < fj)) ? 1 : 0;
            }
        }
        c = wave_sum_i32(c);
        if ((tid & 63) == 0) wsum[tid >> 6][j] = c;
    }
    __syncthreads();
    if (tid < top_k) {
        const int ej = ids[t * top_k + tid];
        const bool valid = ej >= 0 && ej < E;
        const int d = wsum[0][tid] + wsum[1][tid] + wsum[2][tid] + wsum[3][tid];
        dst[t * top_k + tid] = valid ? d : R;  // a dropped pair points one past the last row
        if (valid) row_token[d] = t;
    }
}

// One workgroup per token: quantise the row once, write it to its k destinations.
template <bool QUANT, int DT = MOE355_DT_BF16>
__global__ __launch_bounds__(256) void gather_rows_kernel(const uint16_t* __restrict__ x, int64_t H, int top_k,
                                                          const int32_t* __restrict__ dst, void* __restrict__ xs,
                                                          float* __restrict__ sx)
{
    __shared__ float lds4[4];
    __shared__ int32_t drow[64];
    const int64_t t = blockIdx.x;
    const v8u16 held = first_piece(x + t * H, H);
    if (threadIdx.x < top_k) {
        const int32_t d = dst[t * top_k + threadIdx.x];
        drow[threadIdx.x] = (int64_t)d < (int64_t)gridDim.x * top_k ? d : -1;  // R = tokens * top_k: dropped
    }
    gather_token_row<QUANT, DT>(x + t * H, H, top_k, drow, lds4, xs, sx, held);
}

// expanded_scale[dst[f]] = scale[f / top_k] for every pair that has a row
__global__ __launch_bounds__(256) void gather_scale_kernel(const int32_t* __restrict__ dst,
                                                           const float* __restrict__ scale, int64_t R, int top_k,
                                                           float* __restrict__ expanded_scale)
{
    const int64_t f = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (f >= R) return;
    const int32_t d = dst[f];
    if (d >= 0 && (int64_t)d < R) expanded_scale[d] = scale[f / top_k];
}

}  // namespace moe355

using namespace moe355;

static int nchunks_of(int64_t R) { return (int)((R + kChunk - 1) / kChunk); }

extern "C" size_t moe355_init_routing_workspace(int64_t num_tokens, int top_k, int num_experts)
{
    if (num_tokens < 0 || top_k <= 0 || num_experts <= 0) return 0;
    const int64_t R = num_tokens * top_k;
    size_t n = nchunks_of(R > 0 ? R : 1);
    // chunk histograms, expert offsets, partition bases of the scan (parts * E <= max(1024, E) entries)
    const size_t pb = num_experts > 1024 ? (size_t)num_experts : 1024;
    return align256(n * (size_t)num_experts * 4) + align256(((size_t)num_experts + 1) * 4) + align256(pb * 4);
}

// histogram, scan, stable scatter: destinations of the pairs, optionally the token of every sorted row, counts
static void launch_maps(const int32_t* expert_idx, int64_t R, int E, int top_k, int tokens_num_type, const RouteWs& ws,
                        int nch, int parts, int cpp, int nbits, int32_t* expanded_row_idx, int32_t* row_token,
                        int64_t* expert_tokens, hipStream_t st)
{
    hipLaunchKernelGGL(route_hist_kernel, dim3(nch), dim3(256), (size_t)E * 4, st, expert_idx, R, E, ws.chunk_hist);
    hipLaunchKernelGGL(route_scan_kernel, dim3(1), dim3(kScanThreads), ((size_t)E + 256 + (size_t)parts * E) * 4, st,
                       ws.chunk_hist, nch, E, parts, cpp, tokens_num_type, ws.off, ws.pbase, expert_tokens);
    hipLaunchKernelGGL(route_scatter_kernel, dim3(nch), dim3(64), (size_t)E * 4, st, expert_idx, R, E, nbits,
                       ws.chunk_hist, ws.off, ws.pbase, cpp, expanded_row_idx, row_token, top_k);
}

// the workspace cut into the three arrays of the routing kernels, and how the scan is partitioned
static RouteWs route_ws_of(void* workspace, int64_t R, int E, int& nch, int& parts, int& cpp, int& nbits)
{
    nch = nchunks_of(R > 0 ? R : 1);
    RouteWs ws;
    ws.chunk_hist = (int32_t*)workspace;
    ws.off = (int32_t*)((char*)workspace + align256((size_t)nch * E * 4));
    ws.pbase = (int32_t*)((char*)ws.off + align256(((size_t)E + 1) * 4));
    parts = E < kScanThreads ? kScanThreads / E : 1;
    if (parts > nch) parts = nch;
    cpp = (nch + parts - 1) / parts;
    parts = (nch + cpp - 1) / cpp;  // no empty partition
    nbits = 0;
    while ((1 << nbits) < E) ++nbits;
    return ws;
}

static int init_routing_impl(const void* x, int x_dtype, int64_t num_tokens, int64_t hidden,
                             const int32_t* expert_idx, int top_k, int num_experts, int quant_mode,
                             int tokens_num_type, void* expanded_x, int32_t* expanded_row_idx,
                             int64_t* expert_tokens, float* dynamic_scale, void* workspace, size_t workspace_bytes,
                             void* stream)
{
    if (num_tokens < 0 || hidden <= 0 || top_k <= 0 || num_experts <= 0) return MOE355_E_ARG;
    if (quant_mode != 1 && quant_mode != -1) return MOE355_E_UNSUPPORTED;
    if (tokens_num_type != 0 && tokens_num_type != 1) return MOE355_E_UNSUPPORTED;
    if (x_dtype != MOE355_DT_BF16 && x_dtype != MOE355_DT_F16) return MOE355_E_UNSUPPORTED;
    if (top_k > 64 || num_experts > 2048) return MOE355_E_SHAPE;
    const int64_t R = num_tokens * top_k;
    if (R >= 0x7fffffffLL) return MOE355_E_SHAPE;
    if (hidden % 8 != 0 || ((uintptr_t)x & 15) || ((uintptr_t)expanded_x & 15)) return MOE355_E_SHAPE;
    if (!expert_tokens) return MOE355_E_ARG;
    if (!workspace || ((uintptr_t)workspace & 255) ||
        workspace_bytes < moe355_init_routing_workspace(num_tokens, top_k, num_experts))
        return MOE355_E_WORKSPACE;
    if (R > 0 && (!x || !expert_idx || !expanded_x || !expanded_row_idx)) return MOE355_E_ARG;
    if (R > 0 && quant_mode == 1 && !dynamic_scale) return MOE355_E_ARG;

    hipStream_t st = (hipStream_t)stream;
    const int E = num_experts;
    int nch, parts, cpp, nbits;
    const RouteWs ws = route_ws_of(workspace, R, E, nch, parts, cpp, nbits);

    if (R <= kSmallMaxIters * 256) {
        const dim3 grid((unsigned)num_tokens + 1);
        const size_t lds = ((size_t)E + 256) * 4;
        if (quant_mode == 1 && x_dtype == MOE355_DT_F16)
            hipLaunchKernelGGL((route_gather_small_kernel<true, MOE355_DT_F16>), grid, dim3(256), lds, st, expert_idx,
                               (int)R, E, tokens_num_type, ws.off, expert_tokens, expanded_row_idx,
                               (const uint16_t*)x, hidden, top_k, expanded_x, dynamic_scale);
        else if (quant_mode == 1)
            hipLaunchKernelGGL((route_gather_small_kernel<true>), grid, dim3(256), lds, st, expert_idx, (int)R, E,
                               tokens_num_type, ws.off, expert_tokens, expanded_row_idx, (const uint16_t*)x, hidden,
                               top_k, expanded_x, dynamic_scale);
        else
            hipLaunchKernelGGL((route_gather_small_kernel<false>), grid, dim3(256), lds, st, expert_idx, (int)R, E,
                               tokens_num_type, ws.off, expert_tokens, expanded_row_idx, (const uint16_t*)x, hidden,
                               top_k, expanded_x, dynamic_scale);
        return launch_status();
    }
    launch_maps(expert_idx, R, E, top_k, tokens_num_type, ws, nch, parts, cpp, nbits, expanded_row_idx, nullptr,
                expert_tokens, st);
    if (quant_mode == 1 && x_dtype == MOE355_DT_F16)
        hipLaunchKernelGGL((gather_rows_kernel<true, MOE355_DT_F16>), dim3((unsigned)num_tokens), dim3(256), 0, st,
                           (const uint16_t*)x, hidden, top_k, expanded_row_idx, expanded_x, dynamic_scale);
    else if (quant_mode == 1)
        hipLaunchKernelGGL(gather_rows_kernel<true>, dim3((unsigned)num_tokens), dim3(256), 0, st,
                           (const uint16_t*)x, hidden, top_k, expanded_row_idx, expanded_x, dynamic_scale);
    else
        hipLaunchKernelGGL(gather_rows_kernel<false>, dim3((unsigned)num_tokens), dim3(256), 0, st,
                           (const uint16_t*)x, hidden, top_k, expanded_row_idx, expanded_x, dynamic_scale);
    return launch_status();
}

extern "C" int moe355_init_routing(const void* x, int x_dtype, int64_t num_tokens, int64_t hidden,
                                   const int32_t* expert_idx, int top_k, int num_experts, int quant_mode,
                                   int tokens_num_type, void* expanded_x, int32_t* expanded_row_idx,
                                   int64_t* expert_tokens, float* dynamic_scale, void* workspace,
                                   size_t workspace_bytes, void* stream)
{
    return init_routing_impl(x, x_dtype, num_tokens, hidden, expert_idx, top_k, num_experts, quant_mode,
                             tokens_num_type, expanded_x, expanded_row_idx, expert_tokens, dynamic_scale, workspace,
                             workspace_bytes, stream);
}

extern "C" int moe355_route_map(const int32_t* expert_idx, int64_t num_tokens, int top_k, int num_experts,
                                int tokens_num_type, int32_t* expanded_row_idx, int32_t* row_token,
                                int64_t* expert_tokens, void* workspace, size_t workspace_bytes, void* stream)
{
    if (num_tokens < 0 || top_k <= 0 || num_experts <= 0) return MOE355_E_ARG;
    if (tokens_num_type != 0 && tokens_num_type != 1) return MOE355_E_UNSUPPORTED;
    if (top_k > 64 || num_experts > 2048) return MOE355_E_SHAPE;
    const int64_t R = num_tokens * top_k;
    if (R >= 0x7fffffffLL) return MOE355_E_SHAPE;
    if (!expert_tokens) return MOE355_E_ARG;
    if (!workspace || ((uintptr_t)workspace & 255) ||
        workspace_bytes < moe355_init_routing_workspace(num_tokens, top_k, num_experts))
        return MOE355_E_WORKSPACE;
    if (R > 0 && (!expert_idx || !expanded_row_idx || !row_token)) return MOE355_E_ARG;
    int nch, parts, cpp, nbits;
    const RouteWs ws = route_ws_of(workspace, R, num_experts, nch, parts, cpp, nbits);
    if (R > 0 && R <= kMapSmallIters * 256 && num_tokens <= 1024) {
        // one launch instead of three short ones that wait for each other (every workgroup reads all ids: not for
        // thousands of tokens with one slot each)
        hipLaunchKernelGGL(route_map_small_kernel, dim3((unsigned)num_tokens + 1), dim3(256),
                           ((size_t)num_experts + 256) * 4, (hipStream_t)stream, expert_idx, (int)R, num_experts,
                           tokens_num_type, ws.off, expert_tokens, expanded_row_idx, row_token, top_k);
        return launch_status();
    }
    launch_maps(expert_idx, R, num_experts, top_k, tokens_num_type, ws, nch, parts, cpp, nbits, expanded_row_idx,
                row_token, expert_tokens, (hipStream_t)stream);
    return launch_status();
}

extern "C" int moe355_init_routing_prequant(const int8_t* x, const float* x_scale, int64_t num_tokens, int64_t hidden,
                                            const int32_t* expert_idx, int top_k, int num_experts,
                                            int tokens_num_type, int8_t* expanded_x, int32_t* expanded_row_idx,
                                            int64_t* expert_tokens, float* expanded_scale, void* workspace,
                                            size_t workspace_bytes, void* stream)
{
    if (hidden <= 0 || hidden % 16 != 0) return hidden <= 0 ? MOE355_E_ARG : MOE355_E_SHAPE;
    const int64_t R = num_tokens * (int64_t)top_k;
    if (R > 0 && (!x_scale || !expanded_scale)) return MOE355_E_ARG;
    // an int8 row of `hidden` bytes moves as hidden / 2 16-bit patterns through the copy form of the gather
    const int rc = init_routing_impl(x, MOE355_DT_BF16, num_tokens, hidden / 2, expert_idx, top_k, num_experts, -1,
                                     tokens_num_type, expanded_x, expanded_row_idx, expert_tokens, nullptr, workspace,
                                     workspace_bytes, stream);
    if (rc != MOE355_OK || R == 0) return rc;
    hipLaunchKernelGGL(gather_scale_kernel, dim3((unsigned)((R + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                       expanded_row_idx, x_scale, R, top_k, expanded_scale);
    return launch_status();
}

// ------------------------------------------------------------------ the form that allocates nothing
// The chunk histograms, expert offsets and partition bases of the routing kernels live in a fixed array in
// device memory instead of a caller's workspace.  Every GPU the library runs on holds its own copy of the array
// at its own address; the address is looked up once per device and from then on only that address is used in
// host code (the array's name is a host-side handle, not a device pointer).
static __device__ __align__(256) unsigned char scratch[MOE355_INIT_ROUTING_STATIC_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// device address of `scratch` on the current device; nullptr when the runtime refuses
void* scratch_of_current_device()
{
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        void* p = nullptr;
        if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess || !p) return nullptr;
        g_scratch_ptr[dev] = p;
    }
    return g_scratch_ptr[dev];
}
}  // namespace

extern "C" int moe355_init_routing_static(const void* x, int x_dtype, int64_t num_tokens, int64_t hidden,
                                          const int32_t* expert_idx, int top_k, int num_experts, int quant_mode,
                                          int tokens_num_type, void* expanded_x, int32_t* expanded_row_idx,
                                          int64_t* expert_tokens, float* dynamic_scale, void* stream)
{
    if (num_tokens < 0 || top_k <= 0 || num_experts <= 0) return MOE355_E_ARG;
    const size_t need = moe355_init_routing_workspace(num_tokens, top_k, num_experts);
    if (need > (size_t)MOE355_INIT_ROUTING_STATIC_BYTES) return MOE355_E_WORKSPACE;  // batch too large for the array
    void* ws = scratch_of_current_device();
    if (!ws) return MOE355_E_LAUNCH;
    // Nothing in the array has to start at zero: the histogram kernel writes every entry that is read later.
    return init_routing_impl(x, x_dtype, num_tokens, hidden, expert_idx, top_k, num_experts, quant_mode,
                             tokens_num_type, expanded_x, expanded_row_idx, expert_tokens, dynamic_scale, ws,
                             (size_t)MOE355_INIT_ROUTING_STATIC_BYTES, stream);
}
