// Pieces shared by the grouped-GEMM kernels: tiled weight addressing, the
// MFMA accumulator <-> (row, channel) mapping and the three epilogues.
//
// MFMA used: v_mfma_i32_32x32x32_i8.  Operand A (4 VGPRs = 16 int8 per lane)
// carries WEIGHTS: lane l supplies channel l%32, K slice 16*(l/32)..+15 of the
// 32-wide K step.  Operand B carries TOKENS with the same K mapping.  The
// 32x32 int32 result sits in 16 VGPRs: lane l, register v holds
//   token   = l % 32
//   channel = 8*(v/4) + 4*(l/32) + v%4
// so every lane owns one token and four runs of four consecutive channels.
#pragma once

#include "moe355_common.h"

namespace moe355 {

enum { EPI_I32 = 0, EPI_SWIGLU = 1, EPI_DEQUANT = 2 };

struct GmmArgs {
    const int8_t* x;        // [R, K]
    const int8_t* w;        // tiled [E][N/32][K/32][1024]
    const int64_t* gl;      // [E]
    int gl_type;
    int64_t R;
    int K, N, E;
    const float* row_scale; // [R]     token scale
    // when set: row r of the expert-sorted activation is row row_src[r] of x, and its scale is
    // row_scale[row_src[r]] (the rows were quantised once, in token order, and never copied)
    const int32_t* row_src;
    const float* ch_scale;  // [E, N]  channel scale
    // per-expert tensors (weights that can be swapped expert by expert): device arrays of E pointers;
    // when set they replace w / ch_scale
    const int8_t* const* w_list;
    const float* const* s_list;
    // Pair order (small batches, streaming kernel only): no group list and no sorted copy.  pair_ids[f] is the
    // expert of pair f = token * pair_k + slot; R pairs.  Every workgroup collects the pairs of its expert itself;
    // row i of the expert is pair f: its values lie in row f / pair_k of x (pair_gather: x and row_scale in token
    // order) or in row f, and its result goes to row f.
    const int32_t* pair_ids;
    int pair_k, pair_gather;
    // > 0: the grid has pair_slots places instead of E, and place s works on the s-th expert that has pairs (fewer
    // pairs than experts: most experts are idle)
    int pair_slots;
    // the same for a sorted activation with fewer rows than experts: place s works on the s-th expert whose group
    // is not empty
    int gl_slots;
    // pair order, down GEMM with the re-quantisation inside (REQ): the SwiGLU values [R, K] fp32 that the gate_up
    // GEMM wrote; the workgroup quantises the rows of its expert itself (x and row_scale are not read)
    const float* y_in;
    float limit;            // swiglu clamp
    // A launch may cover only the experts whose row count lies in [rows_min, rows_max] (rows_max 0: no upper
    // bound): a batch with a skewed histogram is split over kernel families by expert, on the device.
    int rows_min, rows_max;
    // outputs
    int32_t* acc;           // EPI_I32   [R, N]
    int32_t* acc_part;      // EPI_I32 with K cut into slabs: [slabs][R, N] partial sums (or null: atomics into acc)
    float* y;               // EPI_SWIGLU [R, N/2] fp32 SwiGLU values
    uint16_t* out;          // EPI_DEQUANT [R, N] bf16, or fp16 when out_f16 is set
    int out_f16;
};

// tiled weights / channel scales of expert e
__device__ __forceinline__ const int8_t* expert_weights(const GmmArgs& a, int e)
{
    return a.w_list ? a.w_list[e] : a.w + (int64_t)e * a.N * a.K;
}
__device__ __forceinline__ const float* expert_scales(const GmmArgs& a, int e)
{
    return a.s_list ? a.s_list[e] : a.ch_scale + (int64_t)e * a.N;
}

// Loads through pointers that may come out of a per-expert pointer table.  The compiler cannot prove that
// such a pointer is global memory and would emit FLAT loads, which count against the LDS counter as well:
// every s_waitcnt after them becomes a full drain (vmcnt(0) lgkmcnt(0)) and the software pipeline of the
// GEMM kernels collapses to one batch in flight.  Saying "global" keeps the waits partial.
typedef const v4i __attribute__((address_space(1))) * gv4i_ptr;
typedef const v4f __attribute__((address_space(1))) * gv4f_ptr;
__device__ __forceinline__ v4i gload16(const void* p) { return *(gv4i_ptr)(uintptr_t)p; }
__device__ __forceinline__ v4i gload16_nt(const void* p) { return __builtin_nontemporal_load((gv4i_ptr)(uintptr_t)p); }
__device__ __forceinline__ v4f gload4f(const float* p) { return *(gv4f_ptr)(uintptr_t)p; }

__device__ __forceinline__ v16i mfma_i8(v4i a, v4i b, v16i c)
{
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
}

// v_mfma_i32_16x16x64_i8: A = 16 channels x 64 K (lane l: channel l%16, K slice 16*(l/16)..+15),
// B = 16 tokens x 64 K with the same K mapping; result 4 VGPRs: token l%16, channels 4*(l/16)+0..3.
__device__ __forceinline__ v4i mfma_i8_16(v4i a, v4i b, v4i c)
{
    return __builtin_amdgcn_mfma_i32_16x16x64_i8(a, b, c, 0, 0, 0);
}

// One token row, one run of four consecutive channels starting at c0 (tile 0) and c1 (tile 1).
// rs: the row's token scale; s0 / s1: the channel scales of the two runs.  The caller loads them before its
// K loop: a load issued here, behind the stores of an earlier run, would wait for those stores (the memory
// counter retires in order), one store round trip per run.
template <int EPI>
__device__ __forceinline__ void epilogue_run(const GmmArgs& a, int64_t row, bool valid, int c0, int c1, const int* g,
                                             const int* u, float rs, v4f s0, v4f s1)
{
    if (!valid) return;
    if constexpr (EPI == EPI_I32) {
        v4i o0 = {g[0], g[1], g[2], g[3]};
        v4i o1 = {u[0], u[1], u[2], u[3]};
        *(v4i*)(a.acc + row * a.N + c0) = o0;
        *(v4i*)(a.acc + row * a.N + c1) = o1;
    } else if constexpr (EPI == EPI_DEQUANT) {
        v4u16 o0, o1;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const float v0 = ((float)g[j] * rs) * s0[j], v1 = ((float)u[j] * rs) * s1[j];
            o0[j] = a.out_f16 ? f32_to_f16(v0) : f32_to_bf16(v0);
            o1[j] = a.out_f16 ? f32_to_f16(v1) : f32_to_bf16(v1);
        }
        *(v4u16*)(a.out + row * a.N + c0) = o0;
        *(v4u16*)(a.out + row * a.N + c1) = o1;
    } else {
        // tile 0 = gate, tile 1 = the matching up tile (c1 = c0 + N/2)
        const int I = a.N >> 1;
        v4f yv;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            float gg = ((float)g[j] * rs) * s0[j];
            float uu = ((float)u[j] * rs) * s1[j];
            if (a.limit > 0.0f) {
                gg = gg > a.limit ? a.limit : gg;
                uu = uu > a.limit ? a.limit : uu;
                uu = uu < -a.limit ? -a.limit : uu;
            }
            yv[j] = m_silu(gg) * uu;
        }
        *(v4f*)(a.y + row * I + c0) = yv;
    }
}

// First channel, inside a 32-channel tile, of the run that quarter q of a 32x32 accumulator tile holds in
// this lane: 8*q + 4*(lane/32), four consecutive channels.
__device__ __forceinline__ int quad_channel(int q, int lane) { return 8 * q + 4 * (lane >> 5); }

// Whether a launch restricted to [a.rows_min, a.rows_max] covers an expert of m rows.
__device__ __forceinline__ bool expert_in_launch(const GmmArgs& a, int64_t m)
{
    return m >= a.rows_min && (a.rows_max == 0 || m <= a.rows_max);
}

// Measurement hook (gmm.hip): hands out, once, the events that moe355_profile_next_gemm armed on this thread
// (both null when nothing is armed); the caller records them around exactly one kernel launch.
void take_profile_events(hipEvent_t& start, hipEvent_t& stop);

// SwiGLU values y fp32 [R, I] -> per-row absmax -> int8 + scale (defined in gmm.hip).
void launch_swiglu_requant(const float* y, const int64_t* gl, int gl_type, int E, int64_t R, int I, int8_t* q,
                           float* qs, hipStream_t st);

}  // namespace moe355
