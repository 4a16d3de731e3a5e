// Router gate: logits[t][e] = sum_k float(x[t][k]) * w[e][k] in fp32, the linear layer in front of the
// top-k gating (AscendGateLinear, vllm_ascend/ops/fused_moe/gate_linear.py:24-63, and the internal-router
// branch vllm_ascend/ops/fused_moe/fused_moe.py:264-271: F.linear(hidden_states.float(), weight_fp32)).
//
// Arithmetic: K is cut into chunks of 128 (the last one may be 64 long).  Inside a chunk one accumulator
// starts at +0 and takes acc = fma(x_k, w_k, acc) for ascending k; the chunk results are added to a total that
// starts at +0, in ascending chunk order; an optional bias is added last.  That is what a chain of
// v_mfma_f32_32x32x2_f32 computes (each instruction performs the two k steps of its operands as two fused
// multiply-adds, in order), and it does not depend on how the chunks are spread over the chip: a wavefront
// that owns every chunk of its 32 x 32 output tile keeps the total in registers; when the tiles alone would
// leave SIMDs idle, two or four wavefronts of a workgroup share a tile, take its chunks in turn and hand the
// chunk results to each other through LDS; and a launch with very few tiles (decode) gives every chunk
// workgroups of its own, writes the chunk results to scratch and adds them in a second kernel.  The order of
// the additions is the same in all three.
//
// Tile: 64 tokens x 64 experts per workgroup (one 32 x 32 MFMA tile per wavefront; 128 x 32 when there are at
// most 32 experts), 64 K values staged through LDS at a time, the even and the odd k of a row in separate
// runs, rows 68 floats apart (16-byte operand reads without bank conflicts).
#include <hip/hip_runtime.h>

#include <type_traits>

#include "moe355_common.h"

namespace moe355 {

typedef float v16f __attribute__((ext_vector_type(16)));
typedef float v2f_t __attribute__((ext_vector_type(2)));

constexpr int kGateChunk = 128;
constexpr int kGateStage = 64;
constexpr int kGateRow = 68;  // floats per staged row: the 32 even k, the 32 odd k, 4 of padding

// X_DT: MOE355_DT_BF16, MOE355_DT_F16 or MOE355_DT_F32.  SPLIT: blockIdx.z is the chunk and `out` is the scratch
// [chunks][T][E]; otherwise the workgroup walks all chunks and `out` is logits [T][E] (+ bias).
// The four wavefronts of a workgroup: EW side by side along the experts, KW sharing one 32 x 32 output tile (they
// take the chunks c = KW g + kw of every group g of KW chunks and exchange the chunk results through LDS, so
// that the total still takes them in ascending order), the other 4 / (EW KW) stacked along the tokens.
template <int X_DT, bool SPLIT, int EW, int KW>
__global__ __launch_bounds__(256) void router_gate_kernel(const void* __restrict__ xv, const float* __restrict__ w,
                                                          const float* __restrict__ bias, float* __restrict__ out,
                                                          int64_t T, int H, int E)
{
    static_assert(!(SPLIT && KW > 1), "a launch splits the chunks over workgroups or over wavefronts, not both");
    constexpr int TW = 4 / (EW * KW);
    constexpr int XB = X_DT == MOE355_DT_F32 ? 4 : 2;  // bytes per token value
    constexpr int XL = TW * KW * XB / 2;                // 16-byte token loads per thread and stage
    constexpr int WL = 2 * EW * KW;                     // 16-byte weight loads per thread and stage
    constexpr int NL = XL + WL;
    constexpr int XROWS = TW * KW * 32;
    constexpr int ROWS = XROWS + EW * KW * 32;
    static_assert(2 * NL <= 24, "the LDS writes of a stage must fit in front of its barrier");
    __shared__ __attribute__((aligned(16))) float lds[2][ROWS * kGateRow];
    __shared__ __attribute__((aligned(16))) v4f px[KW > 1 ? 4 : 1][4][64];
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int lane = tid & 63;
    const int kw = wave % KW, tile = wave / KW;
    const int tw = tile / EW, ew = tile % EW;
    const int half = lane >> 5, l32 = lane & 31;
    const int64_t t0 = (int64_t)blockIdx.x * (32 * TW);
    const int e0 = (int)blockIdx.y * (32 * EW);
    // stages of 64 K values; a chunk is two stages (the last chunk one, when H is an odd multiple of 64).  With
    // KW > 1 a stage of the workgroup is one stage of KW chunks, and every group of chunks has two of them.
    const int n_stages = KW > 1 ? 2 * ((H + kGateChunk * KW - 1) / (kGateChunk * KW)) : H / kGateStage;
    const int s_begin = SPLIT ? (int)blockIdx.z * 2 : 0;
    const int s_end = SPLIT ? (s_begin + 2 < n_stages ? s_begin + 2 : n_stages) : n_stages;
    const int n_local = s_end - s_begin;
    const int s_last = s_end - 1;
    auto stage_k = [&](int s) { return KW > 1 ? (s >> 1) * (kGateChunk * KW) + (s & 1) * kGateStage : s * kGateStage; };

    // Staging: all 256 threads share the rows of a stage, 16 bytes per thread and load.  A thread's values
    // k = 4m .. 4m+3 (fp32) or 8m .. 8m+7 (16-bit) go to LDS split by the parity of k, because lane (row, h) of an
    // MFMA operand holds k = 2j + h of instruction j: with the even and the odd k of a row in two runs, one
    // 16-byte LDS read fetches the operands of four instructions.  Rows past the last token or expert repeat
    // the last one (never stored), so the loop has no branches; K ranges past the end (KW > 1: the last group of
    // chunks may be short) are read from the last 64 columns and written to LDS as zeros.
    const char* xbase = (const char*)xv + t0 * H * XB;
    const char* wbase = (const char*)w;
    uint32_t goff[NL];
    int loff[NL], kwk[NL];
#pragma unroll
    for (int i = 0; i < NL; ++i) {
        if (i < XL) {
            constexpr int LPR = 128 * XB / 2 / 16;  // threads per row: 8 (16-bit) or 16 (fp32)
            const int idx = i * 256 + tid;
            const int vrow = idx / LPR, m = idx % LPR;  // vrow = kw' * 32 TW + row
            const int row = vrow % (32 * TW);
            int64_t t = t0 + row;
            if (t > T - 1) t = T - 1;
            goff[i] = (uint32_t)((t - t0) * H * XB + m * 16);
            loff[i] = vrow * kGateRow + m * (XB == 4 ? 2 : 4);
            kwk[i] = (vrow / (32 * TW)) * kGateChunk;
        } else {
            const int idx = (i - XL) * 256 + tid;
            const int vrow = idx / 16, m = idx % 16;  // vrow = kw' * 32 EW + row
            const int row = vrow % (32 * EW);
            int e = e0 + row;
            if (e > E - 1) e = E - 1;
            goff[i] = (uint32_t)e * (uint32_t)H * 4u + (uint32_t)m * 16u;
            loff[i] = (XROWS + vrow) * kGateRow + m * 2;
            kwk[i] = (vrow / (32 * EW)) * kGateChunk;
        }
    }
    v4f ld[2][NL];
    auto load_one = [&](int set, int stage, int i) {
        int64_t k = stage_k(stage);
        if constexpr (KW > 1) {
            k += kwk[i];
            if (k > H - kGateStage) k = H - kGateStage;
        }
        if (i < XL) ld[set][i] = *(const v4f*)(xbase + k * XB + goff[i]);
        else ld[set][i] = *(const v4f*)(wbase + k * 4 + goff[i]);
    };
    // write wi of a stage: load wi / 2, its even (wi % 2 == 0) or odd values
    auto store_one = [&](int set, int buf, int stage, int wi) {
        const int i = wi >> 1, odd = wi & 1;
        v4f v = ld[set][i];
        if constexpr (KW > 1) {
            if (stage_k(stage) + kwk[i] >= H) v = (v4f){0.0f, 0.0f, 0.0f, 0.0f};
        }
        float* dst = &lds[buf][loff[i] + odd * 32];
        if (i < XL && X_DT != MOE355_DT_F32) {
            v4f o;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const uint32_t u = __float_as_uint(v[q]);  // k = 8m + 2q (low half), 8m + 2q + 1 (high half)
                if constexpr (X_DT == MOE355_DT_BF16) o[q] = __uint_as_float(odd ? (u & 0xffff0000u) : (u << 16));
                else o[q] = f16_to_f32((uint16_t)(odd ? (u >> 16) : (u & 0xffffu)));
            }
            *(v4f*)dst = o;
        } else {
            v2f_t o;
            o[0] = v[odd];
            o[1] = v[2 + odd];
            *(v2f_t*)dst = o;
        }
    };

    v16f total = {0};
    v16f p[2] = {{0}, {0}};
    v4f xo[4], wo[4];  // operands of four instructions each; the reads run two groups ahead of the MFMAs
    const int xrow = ((kw * TW + tw) * 32 + l32) * kGateRow + half * 32;
    const int wrow = (XROWS + (kw * EW + ew) * 32 + l32) * kGateRow + half * 32;

#pragma unroll
    for (int i = 0; i < NL; ++i) load_one(0, s_begin, i);
#pragma unroll
    for (int wi = 0; wi < 2 * NL; ++wi) store_one(0, 0, s_begin, wi);
    __builtin_amdgcn_sched_barrier(0);
    const int s_second = s_begin + 1 < s_last ? s_begin + 1 : s_last;
#pragma unroll
    for (int i = 0; i < NL; ++i) load_one(1, s_second, i);
    __syncthreads();
#pragma unroll
    for (int g = 0; g < 2; ++g) {
        xo[g] = *(const v4f*)&lds[0][xrow + 4 * g];
        wo[g] = *(const v4f*)&lds[0][wrow + 4 * g];
    }

    // One stage: 32 MFMAs of one accumulator chain, which issue 64 cycles apart and block the wavefront while
    // they wait; everything else sits in the gaps between them, one or two instructions per gap: the loads of
    // stage s + 2 (global -> registers), the LDS writes of stage s + 1, the operand reads two groups ahead, the
    // barrier once the last reads of this buffer and the writes of the other are out, then the first reads of
    // the next stage.  BUF: LDS buffer and register set of this stage; PS: accumulator of its chunk (a chunk's
    // first stage has BUF 0 and starts from +0); ADD: accumulator of the chunk before, added to the total here,
    // long after its last MFMA (-1: nothing to add).  With KW > 1 every wavefront posts that accumulator in LDS
    // in front of the barrier and adds the KW results of its tile behind it, in chunk order.
    auto run_stage = [&](auto buf_c, auto ps_c, auto add_c, int s) {
        constexpr int BUF = decltype(buf_c)::value, PS = decltype(ps_c)::value, ADD = decltype(add_c)::value;
        constexpr int AP = ADD < 0 ? 0 : ADD;
        const int s_load = s + 2 < s_last ? s + 2 : s_last;
        const int s_store = s + 1 < s_last ? s + 1 : s_last;
#pragma unroll
        for (int j = 0; j < 32; ++j) {
            const int g = j >> 2, jj = j & 3;
            if (BUF == 0 && j == 0) p[PS] = (v16f){0};
            p[PS] = __builtin_amdgcn_mfma_f32_32x32x2f32(xo[g & 3][jj], wo[g & 3][jj], p[PS], 0, 0, 0);
            if (jj < 2) {
                const int gn = g + 2;  // groups 8 and 9 are groups 0 and 1 of the next stage
                const float* src = &lds[gn < 8 ? BUF : BUF ^ 1][(jj == 0 ? xrow : wrow) + 4 * (gn & 7)];
                if (jj == 0) xo[gn & 3] = *(const v4f*)src;
                else wo[gn & 3] = *(const v4f*)src;
            }
            if (j < NL) load_one(BUF, s_load, j);
            if (j < 2 * NL) store_one(BUF ^ 1, BUF ^ 1, s_store, j);
            if constexpr (ADD >= 0) {
                if constexpr (KW == 1) {
                    if (j >= 8 && j < 12) {
#pragma unroll
                        for (int v = 4 * (j - 8); v < 4 * (j - 8) + 4; ++v) total[v] = total[v] + p[AP][v];
                    }
                } else {
                    if (j >= 8 && j < 12) {
                        const int q = j - 8;
                        px[wave][q][lane] = (v4f){p[AP][4 * q], p[AP][4 * q + 1], p[AP][4 * q + 2], p[AP][4 * q + 3]};
                    }
                    if (j >= 24 && j < 28) {
                        const int q = j - 24;
#pragma unroll
                        for (int c = 0; c < KW; ++c) {
                            const v4f o = px[tile * KW + c][q][lane];
#pragma unroll
                            for (int v = 0; v < 4; ++v) total[4 * q + v] = total[4 * q + v] + o[v];
                        }
                    }
                }
            }
            if (j == 23) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
        }
    };
    // the chunk results still outside the total: accumulator PS, after the last stage
    auto add_last = [&](int ps) {
        if constexpr (KW == 1) {
            total = total + p[ps];
        } else {
            __syncthreads();  // nobody is still reading the results posted during the last stages
#pragma unroll
            for (int q = 0; q < 4; ++q)
                px[wave][q][lane] = (v4f){p[ps][4 * q], p[ps][4 * q + 1], p[ps][4 * q + 2], p[ps][4 * q + 3]};
            __syncthreads();
#pragma unroll
            for (int q = 0; q < 4; ++q) {
#pragma unroll
                for (int c = 0; c < KW; ++c) {
                    const v4f o = px[tile * KW + c][q][lane];
#pragma unroll
                    for (int v = 0; v < 4; ++v) total[4 * q + v] = total[4 * q + v] + o[v];
                }
            }
        }
    };
    using std::integral_constant;
    integral_constant<int, 0> c0;
    integral_constant<int, 1> c1;
    integral_constant<int, -1> cn;
    int i = 0;
    for (; i + 4 <= n_local; i += 4) {
        run_stage(c0, c0, c1, s_begin + i);
        run_stage(c1, c0, cn, s_begin + i + 1);
        run_stage(c0, c1, c0, s_begin + i + 2);
        run_stage(c1, c1, cn, s_begin + i + 3);
    }
    const int rem = n_local - i;
    if (rem == 0) {
        add_last(1);
    } else {
        run_stage(c0, c0, c1, s_begin + i);
        if (rem >= 2) run_stage(c1, c0, cn, s_begin + i + 1);
        if (rem == 3) {
            run_stage(c0, c1, c0, s_begin + i + 2);
            add_last(1);
        } else {
            add_last(0);
        }
    }
    if (kw != 0) return;
    // lane l holds expert e0 + 32 ew + l % 32 of tokens t0 + 32 tw + 8 (v / 4) + 4 (l / 32) + v % 4
    const int e = e0 + ew * 32 + l32;
    if (e >= E) return;
    float b = 0.0f;
    if constexpr (!SPLIT) {
        if (bias) b = bias[e];
    }
    float* dst = SPLIT ? out + (int64_t)blockIdx.z * T * E : out;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
        const int64_t t = t0 + tw * 32 + 8 * (v >> 2) + 4 * half + (v & 3);
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

// How a launch spreads the product over the chip: EW wavefronts of a workgroup side by side along the experts,
// KW sharing a tile, or every chunk with workgroups of its own (split).  One workgroup fits a compute unit, so a
// launch runs in rounds of 256 workgroups; `cost` is its length in rounds of the one-wavefront-per-tile form
// (measured on MI355X, DeepSeek-V3 and Qwen3 gate shapes: a stage of two wavefronts per tile takes 1.2 to 1.45
// times as long, of four 1.5 to 1.7 times, for half and a quarter of the stages).
struct GatePlan {
    int ew, kw;
    bool split;
    int64_t wgs;
    double cost;
    int tw() const { return 4 / (ew * kw); }
};
static GatePlan gate_form(int64_t T, int E, int kw)
{
    GatePlan g;
    g.kw = kw;
    g.ew = kw == 4 ? 1 : (E > 32 ? 2 : 1);
    g.split = false;
    g.wgs = ((T + 32 * g.tw() - 1) / (32 * g.tw())) * ((E + 32 * g.ew - 1) / (32 * g.ew));
    const double stage = kw == 1 ? 1.0 : kw == 2 ? 1.4 : 1.7;
    g.cost = (double)((g.wgs + 255) / 256) * stage / kw;
    return g;
}
// Fewer than 192 output tiles of 32 x 32: the chunk-per-workgroup form (when the caller can take it: it needs
// the scratch).  Otherwise the cheapest of one, two and four wavefronts per tile; sharing a tile pays from four
// chunks per wavefront on, and fp32 tokens are twice the loads, so four wavefronts on one tile would not fit
// their LDS writes in a stage.
static GatePlan gate_plan(int64_t T, int E, int n_chunks, int x_dtype, bool may_split = true)
{
    const int64_t tiles = ((T + 31) / 32) * ((E + 31) / 32);
    GatePlan g = gate_form(T, E, 1);
    if (may_split && tiles < 192) {
        g.split = true;
        return g;
    }
    for (int kw = 2; kw <= 4; kw *= 2) {
        if (n_chunks < 4 * kw || (kw == 4 && x_dtype == MOE355_DT_F32)) break;
        const GatePlan c = gate_form(T, E, kw);
        if (c.cost < g.cost) g = c;
    }
    return g;
}

template <int X_DT>
static void launch_gate(const GatePlan& g, const void* x, const float* weight, const float* bias, float* out, int64_t T,
                        int H, int E, int n_chunks, hipStream_t st)
{
    const int tw = g.tw();
    const dim3 grid((unsigned)((T + 32 * tw - 1) / (32 * tw)), (unsigned)((E + 32 * g.ew - 1) / (32 * g.ew)),
                    g.split ? n_chunks : 1);
#define MOE355_GATE(S_, W_, K_) \
    hipLaunchKernelGGL((router_gate_kernel<X_DT, S_, W_, K_>), grid, dim3(256), 0, st, x, weight, bias, out, T, H, E)
    if (g.split) {
        if (g.ew == 2) MOE355_GATE(true, 2, 1);
        else MOE355_GATE(true, 1, 1);
    } else if (g.kw == 4) {
        if constexpr (X_DT != MOE355_DT_F32) MOE355_GATE(false, 1, 4);
    } else if (g.kw == 2) {
        if (g.ew == 2) MOE355_GATE(false, 2, 2);
        else MOE355_GATE(false, 1, 2);
    } else {
        if (g.ew == 2) MOE355_GATE(false, 2, 1);
        else MOE355_GATE(false, 1, 1);
    }
#undef MOE355_GATE
}

}  // namespace moe355

using namespace moe355;

extern "C" size_t moe355_router_gate_workspace(int64_t num_tokens, int hidden, int num_experts)
{
    if (num_tokens <= 0 || hidden <= 0 || num_experts <= 0) return 0;
    if (!gate_plan(num_tokens, num_experts, 1, MOE355_DT_BF16).split) return 0;  // depends on the tile count alone
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
    if (num_tokens > 0x7fffffffLL / 128 * 128) return MOE355_E_SHAPE;
    // a thread's offsets inside the weight and inside its workgroup's token rows are 32-bit
    if ((int64_t)num_experts * hidden >= (1LL << 30) || hidden >= (1 << 22)) return MOE355_E_SHAPE;
    hipStream_t st = (hipStream_t)stream;
    const int n_chunks = (hidden + kGateChunk - 1) / kGateChunk;
    const GatePlan g = gate_plan(num_tokens, num_experts, n_chunks, x_dtype);
    float* out = logits;
    const float* b = bias;
    if (g.split) {
        const size_t need = moe355_router_gate_workspace(num_tokens, hidden, num_experts);
        if (!workspace || ((uintptr_t)workspace & 255) || workspace_bytes < need) return MOE355_E_WORKSPACE;
        out = (float*)workspace;
        b = nullptr;
    }
    auto launch = [&](const GatePlan& pl, int64_t t_first, int64_t t_count) {
        const int xb = x_dtype == MOE355_DT_F32 ? 4 : 2;
        const void* xp = (const char*)x + t_first * hidden * xb;
        float* op = out + t_first * num_experts;
        if (x_dtype == MOE355_DT_BF16) launch_gate<MOE355_DT_BF16>(pl, xp, weight, b, op, t_count, hidden, num_experts, n_chunks, st);
        else if (x_dtype == MOE355_DT_F16) launch_gate<MOE355_DT_F16>(pl, xp, weight, b, op, t_count, hidden, num_experts, n_chunks, st);
        else launch_gate<MOE355_DT_F32>(pl, xp, weight, b, op, t_count, hidden, num_experts, n_chunks, st);
    };
    // More than one round: the full rounds run one wavefront per tile; a last round that would leave most SIMDs
    // idle becomes a launch of its own over the remaining tokens when sharing its tiles makes it shorter.
    int64_t main_tokens = num_tokens;
    GatePlan first = g, rest = g;
    const GatePlan one = gate_form(num_tokens, num_experts, 1);
    if (!g.split && one.wgs > 256 && one.wgs % 256 != 0) {
        const int64_t wg_cols = (num_experts + 32 * one.ew - 1) / (32 * one.ew);
        const int64_t wg_rows = one.wgs / 256 * 256 / wg_cols;
        const int64_t n_first = wg_rows * 32 * one.tw();
        if (wg_rows > 0 && n_first < num_tokens) {
            const GatePlan r = gate_plan(num_tokens - n_first, num_experts, n_chunks, x_dtype, false);
            if ((double)((wg_rows * wg_cols + 255) / 256) + r.cost < g.cost - 0.05) {
                main_tokens = n_first;
                first = one;
                rest = r;
            }
        }
    }
    // the plan never puts four wavefronts on a tile of fp32 tokens (no such kernel is built)
    if (x_dtype == MOE355_DT_F32 && (first.kw == 4 || rest.kw == 4)) return MOE355_E_UNSUPPORTED;
    launch(first, 0, main_tokens);
    if (main_tokens < num_tokens) launch(rest, main_tokens, num_tokens - main_tokens);
    if (g.split) {
        const int64_t n = num_tokens * num_experts;
        hipLaunchKernelGGL(router_gate_reduce_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, st,
                           (const float*)workspace, bias, logits, n, num_experts, n_chunks);
    }
    return launch_status();
}
