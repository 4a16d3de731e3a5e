// Router gate: logits[t][e] = sum_k float(x[t][k]) * w[e][k] in fp32, the linear layer in front of the
// top-k gating (AscendGateLinear, vllm_ascend/ops/fused_moe/gate_linear.py:24-63, and the internal-router
// branch vllm_ascend/ops/fused_moe/fused_moe.py:264-271: F.linear(hidden_states.float(), weight_fp32)).
//
// Arithmetic: K is cut into chunks of 128 (the last one may be 64 long).  Inside a chunk one accumulator
// starts at +0 and takes acc = fma(x_k, w_k, acc) for ascending k; the chunk results are added to a total that
// starts at +0, in ascending chunk order; an optional bias is added last.  That is what a chain of
// v_mfma_f32_32x32x2_f32 computes (each instruction performs the two k steps of its operands as two fused
// multiply-adds, in order), and it does not depend on how the chunks are spread over workgroups: a workgroup
// that owns every chunk keeps the total in registers, a launch that gives every chunk its own workgroup (few
// tokens: decode) writes the chunk results to scratch and a second kernel adds them in the same order.
//
// Tile: 32 tokens x 128 experts per workgroup (one 32 x 32 MFMA tile per wavefront), 64 K values staged
// through LDS at a time: rows are 66 floats apart, so the per-lane reads of the MFMA operands (32 rows at one
// k, the other half-wave at k + 1) fall into 64 different banks.
#include <hip/hip_runtime.h>

#include "moe355_common.h"

namespace moe355 {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f_t __attribute__((ext_vector_type(2)));

constexpr int kGateChunk = 128;
constexpr int kGateStage = 64;
constexpr int kGateStride = kGateStage + 2;

// X_DT: MOE355_DT_BF16, MOE355_DT_F16 or MOE355_DT_F32.  SPLIT: blockIdx.z is the chunk and `out` is the scratch
// [chunks][T][E]; otherwise the workgroup walks all chunks and `out` is logits [T][E] (+ bias).
template <int X_DT, bool SPLIT>
__global__ __launch_bounds__(256) void router_gate_kernel(const void* __restrict__ xv, const float* __restrict__ w,
                                                          const float* __restrict__ bias, float* __restrict__ out,
                                                          int64_t T, int H, int E)
{
    __shared__ __attribute__((aligned(16))) float xs[2][32 * kGateStride];
    __shared__ __attribute__((aligned(16))) float ws[2][4][32 * kGateStride];
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int64_t t0 = (int64_t)blockIdx.x * 32;
    const int e0 = ((int)blockIdx.y * 4 + wave) * 32;
    const bool have = e0 < E;  // the last expert group of a workgroup row may be short of wavefronts
    // stages of 64 K values; a chunk is two stages (the last chunk one, when H is an odd multiple of 64)
    const int n_stages = H / kGateStage;
    const int s_begin = SPLIT ? (int)blockIdx.z * 2 : 0;
    const int s_end = SPLIT ? (s_begin + 2 < n_stages ? s_begin + 2 : n_stages) : n_stages;

    // staging roles.  Tokens: the four wavefronts share the 32 rows; a half-wave covers one row of a stage
    // (bf16: 4 bytes per lane, fp32: 8 bytes per lane).  Experts: every wavefront stages its own 32 rows.
    // The next stage travels global -> registers under the MFMAs of the current one, then into the other
    // LDS buffer.
    const int half = lane >> 5, l32 = lane & 31;
    // A stage's 20 loads per lane (4 token rows, 16 expert rows) travel global -> registers -> LDS two stages
    // ahead of their use.  The MFMAs of one accumulator chain issue 64 cycles apart and block the wavefront
    // while they wait, so everything else (the loads of stage i + 2, the LDS writes of stage i + 1, the operand
    // reads eight MFMAs ahead) is placed in the gaps between the MFMAs of stage i, one or two instructions per
    // gap.
    v2f_t xr[2][4], wr[2][16];
    auto load_one = [&](int set, int stage, int j) {
        const int k0 = stage * kGateStage;
        if (j < 4) {
            int64_t t = t0 + wave * 8 + j * 2 + half;
            if (t > T - 1) t = T - 1;  // rows past the end duplicate the last token (never stored)
            if constexpr (X_DT != MOE355_DT_F32) {
                // two 16-bit values stay packed until the stage is written to LDS
                xr[set][j][0] = __uint_as_float(*(const uint32_t*)((const uint16_t*)xv + t * H + k0 + 2 * l32));
            } else {
                xr[set][j] = *(const v2f_t*)((const float*)xv + t * H + k0 + 2 * l32);
            }
        } else {
            // wavefronts beyond the last expert group (and rows beyond the last expert) repeat the last expert:
            // the loop stays free of branches, their results are never stored
            int e = e0 + (j - 4) * 2 + half;
            if (e > E - 1) e = E - 1;
            wr[set][j - 4] = *(const v2f_t*)(w + (int64_t)e * H + k0 + 2 * l32);
        }
    };
    auto store_one = [&](int set, int buf, int j) {
        if (j < 4) {
            v2f_t v = xr[set][j];
            if constexpr (X_DT == MOE355_DT_BF16) {
                const uint32_t u = __float_as_uint(xr[set][j][0]);
                v[0] = __uint_as_float(u << 16);
                v[1] = __uint_as_float(u & 0xffff0000u);
            } else if constexpr (X_DT == MOE355_DT_F16) {
                const uint32_t u = __float_as_uint(xr[set][j][0]);
                v[0] = f16_to_f32((uint16_t)(u & 0xffffu));
                v[1] = f16_to_f32((uint16_t)(u >> 16));
            }
            *(v2f_t*)&xs[buf][(wave * 8 + j * 2 + half) * kGateStride + 2 * l32] = v;
        } else {
            *(v2f_t*)&ws[buf][wave][((j - 4) * 2 + half) * kGateStride + 2 * l32] = wr[set][j - 4];
        }
    };

    v16f total = {0};
    v16f p = {0};
    const int n_local = s_end - s_begin;
    const int s_last = s_end - 1;
    // loads past the last stage are redirected to it and written to the buffer nobody reads any more, so that
    // every stage issues the same instructions and the compiler's wait counts are exact
#pragma unroll
    for (int j = 0; j < 20; ++j) load_one(0, s_begin, j);
#pragma unroll
    for (int j = 0; j < 20; ++j) store_one(0, 0, j);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 20; ++j) load_one(1, s_begin + 1 < s_last ? s_begin + 1 : s_last, j);
    __syncthreads();

    // stage with local index i (PAR = i % 2, a compile-time constant after inlining)
    auto run_stage = [&](int PAR, int i) {
        const int s = s_begin + i;
        const int s_load = s + 2 < s_last ? s + 2 : s_last;
        const float* xa = &xs[PAR][l32 * kGateStride + half];
        const float* wb = &ws[PAR][wave][l32 * kGateStride + half];
        float xo[2][8], wo[2][8];
#pragma unroll
        for (int j = 0; j < 8; ++j) {
            xo[0][j] = xa[2 * j];
            wo[0][j] = wb[2 * j];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < kGateStage / 2; ++j) {
            const int b = j >> 3, jj = j & 7;
            p = __builtin_amdgcn_mfma_f32_32x32x2f32(xo[b & 1][jj], wo[b & 1][jj], p, 0, 0, 0);
            if (j + 8 < kGateStage / 2) {
                xo[(b + 1) & 1][jj] = xa[2 * (j + 8)];
                wo[(b + 1) & 1][jj] = wb[2 * (j + 8)];
            }
            if (j < 20) load_one(PAR, s_load, j);
            if (j >= 10 && j < 30) store_one(PAR ^ 1, PAR ^ 1, j - 10);
            __builtin_amdgcn_sched_barrier(0);
        }
        if ((s & 1) || s + 1 == n_stages) {  // the chunk ends with this stage
            if constexpr (!SPLIT) {
#pragma unroll
                for (int v = 0; v < 16; ++v) total[v] = total[v] + p[v];
                p = (v16f){0};
            }
        }
        __syncthreads();
    };
    int i = 0;
    for (; i + 2 <= n_local; i += 2) {
        run_stage(0, i);
        run_stage(1, i + 1);
    }
    if (i < n_local) run_stage(0, i);
    if constexpr (SPLIT) total = p;
    if (!have) return;
    // lane l holds expert e0 + l % 32 of tokens 8 (v / 4) + 4 (l / 32) + v % 4
    const int e = e0 + l32;
    if (e >= E) return;
    float b = 0.0f;
    if constexpr (!SPLIT) {
        if (bias) b = bias[e];
    }
    float* dst = SPLIT ? out + (int64_t)blockIdx.z * T * E : out;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int64_t t = t0 + 8 * (v >> 2) + 4 * half + (v & 3);
        if (t < T) dst[t * E + e] = (!SPLIT && bias) ? total[v] + b : total[v];
    }
}

// logits[i] = ((0 + P_0[i]) + P_1[i]) + ... (+ bias)
__global__ __launch_bounds__(256) void router_gate_reduce_kernel(const float* __restrict__ part,
                                                                 const float* __restrict__ bias,
                                                                 float* __restrict__ out, int64_t n, int E,
                                                                 int n_chunks)
{
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= n) return;
    float total = 0.0f;
    // eight loads in flight at a time; the additions keep the ascending chunk order
    int c = 0;
    for (; c + 8 <= n_chunks; c += 8) {
        float v[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) v[j] = part[(int64_t)(c + j) * n + i];
#pragma unroll
        for (int j = 0; j < 8; ++j) total = total + v[j];
    }
    for (; c < n_chunks; ++c) total = total + part[(int64_t)c * n + i];
    if (bias) total = total + bias[i % E];
    out[i] = total;
}

// one workgroup per chunk when the output tiles alone would leave most of the chip idle
static bool gate_splits(int64_t T, int E)
{
    const int64_t tiles = ((T + 31) / 32) * ((E + 127) / 128);
    return tiles < 128;
}

}  // namespace moe355

using namespace moe355;

extern "C" size_t moe355_router_gate_workspace(int64_t num_tokens, int hidden, int num_experts)
{
    if (num_tokens <= 0 || hidden <= 0 || num_experts <= 0) return 0;
    if (!gate_splits(num_tokens, num_experts)) return 0;
    const size_t chunks = (size_t)((hidden + kGateChunk - 1) / kGateChunk);
    return ((chunks * (size_t)num_tokens * (size_t)num_experts * 4 + 255) / 256) * 256;
}

extern "C" int moe355_router_gate(const void* x, int x_dtype, const float* weight, const float* bias, int64_t num_tokens,
                                  int hidden, int num_experts, float* logits, void* workspace, size_t workspace_bytes,
                                  void* stream)
{
    if (num_tokens < 0 || hidden <= 0 || num_experts <= 0) return MOE355_E_ARG;
    if (num_tokens == 0) return MOE355_OK;
    if (!x || !weight || !logits) return MOE355_E_ARG;
    if (x_dtype != MOE355_DT_BF16 && x_dtype != MOE355_DT_F32 && x_dtype != MOE355_DT_F16) return MOE355_E_UNSUPPORTED;
    if (hidden % kGateStage != 0) return MOE355_E_SHAPE;
    if (num_tokens > 0x7fffffffLL / 32 * 32) return MOE355_E_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    const int n_chunks = (hidden + kGateChunk - 1) / kGateChunk;
    const bool split = gate_splits(num_tokens, num_experts);
    const dim3 grid((unsigned)((num_tokens + 31) / 32), (unsigned)((num_experts + 127) / 128), split ? n_chunks : 1);
#define MOE355_GATE(D_, S_, B_, O_)                                                                              \
    hipLaunchKernelGGL((router_gate_kernel<D_, S_>), grid, dim3(256), 0, st, x, weight, B_, O_, num_tokens, hidden, \
                       num_experts)
    if (split) {
        const size_t need = moe355_router_gate_workspace(num_tokens, hidden, num_experts);
        if (!workspace || ((uintptr_t)workspace & 255) || workspace_bytes < need) return MOE355_E_WORKSPACE;
        float* part = (float*)workspace;
        if (x_dtype == MOE355_DT_BF16) MOE355_GATE(MOE355_DT_BF16, true, nullptr, part);
        else if (x_dtype == MOE355_DT_F16) MOE355_GATE(MOE355_DT_F16, true, nullptr, part);
        else MOE355_GATE(MOE355_DT_F32, true, nullptr, part);
        const int64_t n = num_tokens * num_experts;
        hipLaunchKernelGGL(router_gate_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st, part, bias,
                           logits, n, num_experts, n_chunks);
    } else {
        if (x_dtype == MOE355_DT_BF16) MOE355_GATE(MOE355_DT_BF16, false, bias, logits);
        else if (x_dtype == MOE355_DT_F16) MOE355_GATE(MOE355_DT_F16, false, bias, logits);
        else MOE355_GATE(MOE355_DT_F32, false, bias, logits);
    }
#undef MOE355_GATE
    return launch_status();
}
