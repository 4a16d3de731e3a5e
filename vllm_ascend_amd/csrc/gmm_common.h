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
    const float* ch_scale;  // [E, N]  channel scale
    float limit;            // swiglu clamp
    // outputs
    int32_t* acc;           // EPI_I32   [R, N]
    float* y;               // EPI_SWIGLU [R, N/2] fp32 SwiGLU values
    uint32_t* rowmax;       // EPI_SWIGLU [R] bits(max|y|) + 1, 0 = row untouched
    uint16_t* out;          // EPI_DEQUANT [R, N] bf16
};

__device__ __forceinline__ v16i mfma_i8(v4i a, v4i b, v16i c)
{
    return __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, c, 0, 0, 0);
}

// Epilogue for one pair of 32x32 accumulator tiles held by one wavefront.
// c0/c1: channel tile columns n0/n1 (first channel of each tile); row is the
// lane's token row, valid says whether it exists.
template <int EPI>
__device__ __forceinline__ void epilogue_pair(const GmmArgs& a, int e, int64_t row, bool valid, int n0, int n1,
                                              const v16i& c0, const v16i& c1, int lane)
{
    const int hi = lane >> 5;
    if constexpr (EPI == EPI_I32) {
        if (!valid) return;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int ch = 8 * q + 4 * hi;
            v4i o0 = {c0[4 * q], c0[4 * q + 1], c0[4 * q + 2], c0[4 * q + 3]};
            v4i o1 = {c1[4 * q], c1[4 * q + 1], c1[4 * q + 2], c1[4 * q + 3]};
            *(v4i*)(a.acc + row * a.N + n0 + ch) = o0;
            *(v4i*)(a.acc + row * a.N + n1 + ch) = o1;
        }
    } else if constexpr (EPI == EPI_DEQUANT) {
        if (!valid) return;
        const float rs = a.row_scale[row];
        const float* cs = a.ch_scale + (int64_t)e * a.N;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int ch = 8 * q + 4 * hi;
            const v4f s0 = *(const v4f*)(cs + n0 + ch);
            const v4f s1 = *(const v4f*)(cs + n1 + ch);
            v4u16 o0, o1;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                o0[j] = f32_to_bf16(((float)c0[4 * q + j] * rs) * s0[j]);
                o1[j] = f32_to_bf16(((float)c1[4 * q + j] * rs) * s1[j]);
            }
            *(v4u16*)(a.out + row * a.N + n0 + ch) = o0;
            *(v4u16*)(a.out + row * a.N + n1 + ch) = o1;
        }
    } else {
        // c0 = gate tile, c1 = matching up tile (n1 = n0 + N/2)
        if (!valid) return;
        const int I = a.N >> 1;
        const float rs = a.row_scale[row];
        const float* cs = a.ch_scale + (int64_t)e * a.N;
        float m = 0.0f;
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int ch = 8 * q + 4 * hi;
            const v4f sg = *(const v4f*)(cs + n0 + ch);
            const v4f su = *(const v4f*)(cs + n1 + ch);
            v4f yv;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                float g = ((float)c0[4 * q + j] * rs) * sg[j];
                float u = ((float)c1[4 * q + j] * rs) * su[j];
                if (a.limit > 0.0f) {
                    g = g > a.limit ? a.limit : g;
                    u = u > a.limit ? a.limit : u;
                    u = u < -a.limit ? -a.limit : u;
                }
                float yy = m_silu(g) * u;
                yv[j] = yy;
                float ab = __builtin_fabsf(yy);
                m = ab > m ? ab : m;
            }
            *(v4f*)(a.y + row * I + n0 + ch) = yv;
        }
        // lanes l and l^32 hold the same token (and the same `valid`)
        const float mo = __shfl_xor(m, 32, 64);
        m = mo > m ? mo : m;
        if (hi == 0) atomicMax(a.rowmax + row, __float_as_uint(m) + 1u);
    }
}

}  // namespace moe355
